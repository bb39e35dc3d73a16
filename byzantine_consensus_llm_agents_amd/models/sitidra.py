"""Sitidra: pre-norm decoder over hyper-connection residual streams, with chunked softmax
attention and matrix-memory mixers and sigmoid-scored grouped experts.

The residual is ``streams`` copies ``X [T, S, W]`` (fp32), all equal to the embedding at the start.
Sublayer q of a layer (1: mixer, 2: feed-forward) reads ``u = sum_s in_q[s] X[s]``, runs on the
layer norm of u (a weight, no bias) and writes ``X'[t] = sum_s mix_q[s, t] X[s] + out_q[t] y``, all
streams from the old ones; logits come from the final layer norm of the summed streams and are
soft-capped.  Without streams in the config the same code runs one stream with unit coefficients,
the plain ``x <- x + sublayer(norm(x))``.  The config lists the layers; a layer's mixer is one of

* ``attention``: GQA softmax attention, rotate-half rotary on the first ``rot.dims`` features of
  every q / k head, then q and k divided by their root mean square per head; a chunk mask (a query
  sees the earlier keys of its own ``mask.size``-aligned block of positions); value mixing (every
  ``v_mix`` layer but the first caches ``(1 - lam) v + lam v0`` with v0 the first one's values of the
  token); one sigmoid output gate per head from the mixer's input;
* ``mlstm``: per head a ``dim x vdim`` memory S and a normaliser n with exponential gates kept
  stable by a running maximum m of the log gates: ``m_t = max(f_t + m_(t-1), i_t)``,
  ``S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T`` (n likewise with k alone),
  ``o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)``; per-head unit RMS, a weight over all
  heads and a sigmoid gate of the mixer's input.

Feed-forward: ``top`` of ``experts`` gated experts ``down(silu(gate h) * (up h))`` chosen by
sigmoid score + correction inside the best expert groups, weighted by their normalised scores,
plus an always-on expert of the same form.

State per sequence besides the paged K / V of the attention layers: per matrix-memory layer
``S`` fp32 [rows, heads, dim, vdim + 1] (the last column is n) and ``m`` fp32 [rows, heads], in
tables indexed by the engine's state row; a segment that starts at position 0 starts from zero.

Kernel plan of one layer (HIP backend; the torch backend runs the same ops from ``ops/reference.py``):

    attention     fused GEMM [q | k | v | g] -> rope_norm_kv_write (rotary, unit RMS, value mix, paged
                  write) -> multimap_attention (one map, chunk mask) -> gate_mul (a gate per head) -> o GEMM
    mlstm         fused GEMM [q | k | v | g | i | f] -> exp_gate_prepare (gates, running maximum) ->
                  gated_state_scan (memory and normaliser in one state) -> head_norm_gate -> o GEMM
    feed-forward  moe_route_scored -> grouped expert GEMMs (gated epilogue) -> combine;
                  shared expert: [gate | up] GEMM -> gated_act -> down GEMM
    hyper_update_norm   the streams' update fused with the next sublayer's read and layer norm

No host synchronisation anywhere: a decode step is capturable in a HIP graph.
"""

import math
from typing import Dict, List, Optional

import torch

from .config import SitidraConfig
from .transformer import AttnMeta, TPGroup


class SitidraModel:
    split_single_rows = True
    logits_dtype = torch.float32
    supports_cascade = False
    has_seq_state = True      # matrix memories: a cached prompt prefix cannot stand in for its tokens

    def __init__(self, cfg: SitidraConfig, ops, device, dtype=torch.bfloat16, tp: Optional[TPGroup] = None,
                 quant: Optional[str] = None):
        if quant is not None:
            raise ValueError("Sitidra: quantised weights are not supported")
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Sitidra: tensor parallelism is not supported")
        self.cfg, self.ops, self.device, self.dtype, self.quant = cfg, ops, torch.device(device), dtype, None
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.embed = self.lm_head = self.final_norm = None
        self.S = max(cfg.streams, 1)
        self.n_q = max(l.mixer.heads for l in cfg.layers)
        self.n_kv = 1
        self.hd = max(max(l.mixer.dim, l.mixer.vdim) for l in cfg.layers)
        self.inter = max([2 * l.mlp.ff * l.mlp.top for l in cfg.layers if l.mlp] or [0])
        self.vocab_local = cfg.vocab_size
        self.prefill_tile_rows = 64
        # the first layer that mixes values lends them to the later ones
        mixing = [i for i, l in enumerate(cfg.layers) if l.type == "attention" and l.mixer.v_mix]
        self.v_lender = mixing[0] if mixing else -1

    # ------------------------------------------------------------- KV cache and state
    def kv_block_bytes(self, block_size: int, dtype) -> int:
        item = torch.tensor([], dtype=dtype).element_size()
        return sum(l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim) * block_size * item
                   for l in self.cfg.layers if l.type == "attention")

    def alloc_kv(self, num_blocks: int, block_size: int, dtype, device=None):
        """Per attention layer K [NB, G, BS, dim] and V [NB, G, vdim, BS]; None for the matrix-memory
        layers (block ids are shared by all layers: one block table per sequence)."""
        dev = device or self.device
        ks, vs = [], []
        for l in self.cfg.layers:
            m = l.mixer
            if l.type == "attention":
                ks.append(torch.zeros(num_blocks, m.kv_heads, block_size, m.dim, dtype=dtype, device=dev))
                vs.append(torch.zeros(num_blocks, m.kv_heads, m.vdim, block_size, dtype=dtype, device=dev))
            else:
                ks.append(None)
                vs.append(None)
        return ks, vs

    def alloc_state(self, rows: int, device=None) -> dict:
        """State tables with ``rows`` rows, per matrix-memory layer ``S`` fp32 [rows, heads, dim, vdim + 1]
        (memory, and the normaliser as its last column) and ``m`` fp32 [rows, heads] (running maximum);
        None for the attention layers."""
        dev = device or self.device
        layers = []
        for l in self.cfg.layers:
            m = l.mixer
            if l.type != "mlstm":
                layers.append(None)
                continue
            layers.append({"S": torch.zeros(rows, m.heads, m.dim, m.vdim + 1, dtype=torch.float32, device=dev),
                           "m": torch.zeros(rows, m.heads, dtype=torch.float32, device=dev)})
        return {"layers": layers}

    @staticmethod
    def state_tensors(state: dict) -> List[torch.Tensor]:
        """Every table of `alloc_state` (row-indexed in dimension 0): what the engine moves when
        it moves a row."""
        return [t for L in state["layers"] if L is not None for t in (L["S"], L["m"])]

    def state_row_bytes(self) -> int:
        return sum(4 * l.mixer.heads * (l.mixer.dim * (l.mixer.vdim + 1) + 1) for l in self.cfg.layers if l.type == "mlstm")

    # ------------------------------------------------------------- weights
    def tensor_shapes(self) -> Dict[str, tuple]:
        """Checkpoint tensor names -> shapes."""
        c, W, S = self.cfg, self.cfg.hidden_size, self.cfg.streams
        out = {"embed": (c.vocab_size, W), "head": (c.vocab_size, W), "final.norm": (W,)}
        for i, l in enumerate(c.layers):
            p, m, q = f"l{i}.", l.mixer, f"l{i}.mix."
            out[p + "norm1"] = (W,)
            if l.type == "attention":
                out.update({q + "q": (m.heads * m.dim, W), q + "k": (m.kv_heads * m.dim, W), q + "v": (m.kv_heads * m.vdim, W),
                            q + "g": (m.heads, W), q + "o": (W, m.heads * m.vdim)})
                if m.v_mix:
                    out[q + "vmix"] = ()
            else:
                out.update({q + "q": (m.heads * m.dim, W), q + "k": (m.heads * m.dim, W), q + "v": (m.heads * m.vdim, W),
                            q + "g": (m.heads * m.vdim, W), q + "o": (W, m.heads * m.vdim), q + "norm": (m.heads * m.vdim,),
                            q + "i": (m.heads, W), q + "i.b": (m.heads,), q + "f": (m.heads, W), q + "f.b": (m.heads,)})
            hcs = ["hc1"]
            f = l.mlp
            if f is not None:
                hcs.append("hc2")
                out[p + "norm2"] = (W,)
                for e in range(f.experts):
                    out.update({p + f"mlp.e{e}.gate": (f.ff, W), p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
                out.update({p + "mlp.router": (f.experts, W), p + "mlp.correction": (f.experts,)})
                if f.shared_ff:
                    out.update({p + "mlp.shared.gate": (f.shared_ff, W), p + "mlp.shared.up": (f.shared_ff, W),
                                p + "mlp.shared.down": (W, f.shared_ff)})
            if S:
                for hc in hcs:
                    out.update({p + hc + ".in": (S,), p + hc + ".out": (S,), p + hc + ".mix": (S, S)})
        return out

    def random_state_dict(self, seed: int = 0, std: float = 0.05) -> Dict[str, torch.Tensor]:
        """bf16-representable random weights under the checkpoint names (tests, benchmarks)."""
        gen = torch.Generator().manual_seed(seed)
        S = max(self.cfg.streams, 1)
        sd = {}
        for name, shape in self.tensor_shapes().items():
            r = torch.randn(shape, generator=gen)
            if name.endswith(("norm1", "norm2", "final.norm", "mix.norm")):
                t = 1.0 + 0.2 * r
            elif name.endswith(".vmix"):
                t = 0.3 + 0.2 * torch.rand(shape, generator=gen)
            elif name.endswith((".i.b", ".f.b")):
                t = r + (2.0 if name.endswith(".f.b") else -1.0)
            elif name.endswith("correction"):
                t = r * 0.1
            elif name.endswith("router"):
                t = r * 0.3
            elif name.endswith(".in"):
                t = 1.0 / S + 0.2 * r
            elif name.endswith(".out"):
                t = 1.0 + 0.2 * r
            elif name.endswith(("hc1.mix", "hc2.mix")):
                t = torch.eye(S) + 0.1 * r
            elif name == "embed":
                t = r * 0.7
            elif name.endswith((".mix.i", ".mix.f")):
                t = r * 0.2
            else:
                t = r * (std if name != "head" else 1.0 / math.sqrt(shape[1]))
            sd[name] = t.to(torch.bfloat16)
        return sd

    def init_random(self, seed: int = 0, std: float = 0.05):
        self.load_hf_state_dict(self.random_state_dict(seed, std))

    def load_hf_state_dict(self, sd):
        """Load the checkpoint tensors (names of `tensor_shapes`).  Projections that read the same
        input are stacked into one GEMM weight, every expert's gate and up rows into one
        [E, 2 ff, W] tensor; a checkpoint without stream tensors runs one stream with unit
        coefficients."""
        c, dev, dt, S = self.cfg, self.device, self.dtype, self.S

        def get(name, dtype=None):
            return sd[name].to(device=dev, dtype=dtype or dt).contiguous()

        def f32(name):
            return get(name, torch.float32)

        def hyper(prefix):
            if c.streams:
                return {"in": f32(prefix + ".in"), "mix": f32(prefix + ".mix"), "out": f32(prefix + ".out")}
            one = torch.ones(1, dtype=torch.float32, device=dev)
            return {"in": one, "mix": one.reshape(1, 1), "out": one}

        pair = getattr(self.ops, "moe_pair_rows", None)
        from ..ops.reference import rope_inv_freq
        self.layers = []
        for i, l in enumerate(c.layers):
            p, m, q = f"l{i}.", l.mixer, f"l{i}.mix."
            L = {"norm1": f32(p + "norm1"), "hc1": hyper(p + "hc1"), "o": get(q + "o")}
            if l.type == "attention":
                L["fused"] = torch.cat([get(q + "q"), get(q + "k"), get(q + "v"), get(q + "g")]).contiguous()
                L["inv_freq"] = rope_inv_freq(m.rot_dims, m.rot_base, dev)
                L["lam"] = float(sd[q + "vmix"].float()) if m.v_mix and i != self.v_lender else 0.0
            else:
                L["fused"] = torch.cat([get(q + n) for n in ("q", "k", "v", "g", "i", "f")]).contiguous()
                L["i_bias"], L["f_bias"], L["head_norm"] = f32(q + "i.b"), f32(q + "f.b"), f32(q + "norm")
            f = l.mlp
            if f is not None:
                L["norm2"], L["hc2"] = f32(p + "norm2"), hyper(p + "hc2")
                ups = []
                for e in range(f.experts):
                    g, u = get(p + f"mlp.e{e}.gate"), get(p + f"mlp.e{e}.up")
                    ups.append(pair(g, u) if pair else torch.cat([g, u]))
                L["e_up"] = torch.stack(ups).contiguous()
                L["e_down"] = torch.stack([get(p + f"mlp.e{e}.down") for e in range(f.experts)]).contiguous()
                L["router"] = f32(p + "mlp.router")
                L["correction"] = f32(p + "mlp.correction") if p + "mlp.correction" in sd else None   # (none: the scores choose)
                if f.shared_ff:
                    L["s_up"] = torch.cat([get(p + "mlp.shared.gate"), get(p + "mlp.shared.up")]).contiguous()
                    L["s_down"] = get(p + "mlp.shared.down")
            self.layers.append(L)
        self.embed, self.lm_head, self.final_norm = get("embed"), get("head"), f32("final.norm")
        self.sum_read = torch.ones(S, dtype=torch.float32, device=dev)

    def weight_bytes(self) -> int:
        def size(v):
            if torch.is_tensor(v):
                return v.numel() * v.element_size()
            return sum(size(t) for t in v.values()) if isinstance(v, dict) else 0
        return sum(size(v) for L in self.layers for v in L.values()) + sum(size(t) for t in (self.embed, self.lm_head, self.final_norm))

    # ------------------------------------------------------------- mixers
    def _attention(self, i, m, L, h, meta, k_cache, v_cache, sel, lent):
        ops, eps = self.ops, self.cfg.rms_eps
        y = ops.linear(h, L["fused"])
        qw, kw, vw = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        if i == self.v_lender:
            lent.append(y[:, qw + kw:qw + kw + vw])   # this layer's own values, as later layers blend them in
        v_first = lent[0] if (m.v_mix and i != self.v_lender) else None
        q = ops.rope_norm_kv_write(y, meta.positions, meta.slots, m.heads, m.kv_heads, m.dim, m.vdim, L["inv_freq"], eps,
                                   v_first, L["lam"], k_cache, v_cache)
        att = ops.multimap_attention(q, k_cache, v_cache, meta, m.scale, 1, 0.0, -1.0, 1.0, m.vdim, 0, None, m.chunk)
        gate = y[:, qw + kw + vw:qw + kw + vw + m.heads]
        if sel is not None:
            att, gate = att.index_select(0, sel), gate.index_select(0, sel)
        return ops.linear(ops.gate_mul(att, gate, "sigmoid", m.vdim), L["o"])

    def _mlstm(self, m, L, S, h, meta, sel):
        ops, eps = self.ops, self.cfg.rms_eps
        y = ops.linear(h, L["fused"])
        nk, nv = m.heads * m.dim, m.heads * m.vdim
        off_i = 2 * nk + 2 * nv
        q32, k32, decay, write, floor = ops.exp_gate_prepare(y, 0, nk, off_i, off_i + m.heads, L["i_bias"], L["f_bias"],
                                                             m.gate_cap, m.dim ** -0.5, m.heads, m.dim, meta, S["m"])
        o32 = ops.gated_state_scan(q32, k32, decay, y[:, 2 * nk:2 * nk + nv], write, meta, S["S"], False, True)
        gate = y[:, 2 * nk + nv:2 * nk + 2 * nv]
        if sel is not None:
            o32, floor, gate = o32.index_select(0, sel), floor.index_select(0, sel), gate.index_select(0, sel)
        return ops.linear(ops.head_norm_gate(o32, L["head_norm"], eps, gate, self.dtype, "sigmoid", floor), L["o"])

    def _experts(self, f, L, h):
        """The feed-forward's parts [typed or fp32, ...] whose sum is its output."""
        ops = self.ops
        idx, w = ops.moe_route_scored(h, L["router"], L["correction"], f.top, f.groups, f.keep, f.scale)
        parts = [ops.moe_experts(h, L["e_up"], L["e_down"], idx, w, "silu_gated")]
        if f.shared_ff:
            parts.append(ops.linear(ops.gated_act(ops.linear(h, L["s_up"])), L["s_down"]))
        return parts

    # ------------------------------------------------------------- forward
    def forward(self, tokens: torch.Tensor, meta: AttnMeta, k_cache, v_cache, trace: Optional[list] = None):
        """Logits (fp32) of the rows ``meta.logits_idx`` (all rows when None).  ``meta.state`` holds
        the tables of `alloc_state`, ``meta.state_rows`` every segment's row in them.  ``trace``: a
        list that receives the summed streams after every layer (debugging)."""
        ops, c, dt, eps = self.ops, self.cfg, self.dtype, self.cfg.rms_eps
        st = meta.state
        if st is None or meta.state_rows is None or meta.q_start is None or meta.token_seq is None:
            raise ValueError("Sitidra: the step carries no sequence state (state, state_rows, q_start, token_seq)")
        first = self.layers[0]
        X, h = ops.hyper_embed_norm(tokens, self.embed, self.S, first["hc1"]["in"], first["norm1"], eps, dt)
        n_layers = len(c.layers)
        lent = []
        for i, (spec, L) in enumerate(zip(c.layers, self.layers)):
            last = i == n_layers - 1
            sel = meta.logits_idx if last else None
            if spec.type == "attention":
                y = self._attention(i, spec.mixer, L, h, meta, k_cache[i], v_cache[i], sel, lent)
            else:
                y = self._mlstm(spec.mixer, L, st["layers"][i], h, meta, sel)
            if sel is not None:   # past the last mixer only the rows whose logits are asked for matter
                X = X.index_select(0, sel)
            nxt = (self.sum_read, self.final_norm) if last else (self.layers[i + 1]["hc1"]["in"], self.layers[i + 1]["norm1"])
            hc = L["hc1"]
            if spec.mlp is not None:
                h2 = ops.hyper_update_norm(X, [y], hc["mix"], hc["out"], L["hc2"]["in"], L["norm2"], eps, dt)
                hc = L["hc2"]
                h = ops.hyper_update_norm(X, self._experts(spec.mlp, L, h2), hc["mix"], hc["out"], nxt[0], nxt[1], eps, dt)
            else:
                h = ops.hyper_update_norm(X, [y], hc["mix"], hc["out"], nxt[0], nxt[1], eps, dt)
            if trace is not None:
                trace.append(X.sum(1))
        logits = ops.linear(h, self.lm_head).float()
        return ops.softcap(logits, c.logit_softcap) if c.logit_softcap else logits

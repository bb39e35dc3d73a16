"""Mabivik: sandwich-normed decoder with three kinds of mixer and table-routed experts.

Every layer is ``x <- x + post1(mixer(pre1(x)))``, then ``x <- x + post2(ff(pre2(x)))``, then the
per-layer token input ``x <- x + rms(P (gelu(G x) * e_token)) * w`` (fp32 residual stream x).  All four
norms of a layer are dynamic-tanh norms ``tanh(alpha x) w + b``: elementwise, no row statistic.
The config lists the layers; a layer's mixer is one of

* ``latent_attention``: queries through a normed low-rank latent; keys and values from ONE normed
  latent c per token plus one rotated key part shared by all heads.  The cache holds ``[c | rotated
  part]`` per token and the attention runs in the latent: head h's query becomes ``[W_uk[h]^T q_h |
  rotated q_h]``, the softmax-weighted sum of c is expanded by ``W_uv[h]`` afterwards, so all heads
  read one KV head and nothing per head is cached.  Rotate-half rotary with ramped frequency
  scaling, a sliding window, a sigmoid output gate.  A layer may read an earlier layer's cache
  (``kv_from``) with projections of its own;
* ``delta``: gated delta rule with one decay per head (short convolutions + silu on q / k / v,
  unit-vector q / k, per-head RMS norm times a silu gate);
* ``mamba2``: selective state space with a scalar decay per head (convolution with bias over
  x | B | C, gate before a grouped RMS norm).

Feed-forward: ``top`` experts per token named by a table row of the token id, each
``down(silu(gate h) * (up h))`` with weight 1 / top.

State per sequence besides the paged latent cache: the last ``taps - 1`` inputs of every
convolution and one fp32 matrix per recurrent head, in tables indexed by the engine's state row
(``alloc_state``); a segment that starts at position 0 starts from empty state.

Kernel plan of one layer (HIP backend; the torch backend runs the same ops from
``ops/reference.py``):

    latent_attention  fused GEMM [dq | dkv | g] -> rmsnorm_cols (query latent) -> uq GEMM ->
                      head_linear (W_uk^T q per head, straight into the packed query) + rope_half_tail;
                      latent_kv_write (norm, rotary, paged write) -> multimap_attention (one map,
                      one KV head, window) -> head_linear (W_uv) -> gate_mul -> o GEMM
    delta             fused GEMM [q | k | v | beta | a | g] -> short_conv (silu) -> delta_prepare ->
                      gated_state_scan -> head_norm_gate (silu) -> o GEMM
    mamba2            in GEMM [z | x | B | C | dt] -> short_conv (bias, silu) -> ssm_prepare ->
                      gated_state_scan -> gated_group_norm -> o GEMM
    feed-forward      moe_table_route -> grouped expert GEMMs (gated epilogue) -> combine
    residual_post_norm  x += post(y) fused with the next reader's norm (or a rounded copy of x)
    token input       G GEMM -> gelu_gather_mul -> P GEMM -> residual_post_norm (rms)

No host synchronisation anywhere: a decode step is capturable in a HIP graph.
"""

import math
from typing import Dict, List, Optional

import torch

from .config import MabivikConfig
from .transformer import AttnMeta, TPGroup


class MabivikModel:
    split_single_rows = True
    logits_dtype = torch.float32
    supports_cascade = False
    has_seq_state = True      # recurrent state: a cached prompt prefix cannot stand in for its tokens

    def __init__(self, cfg: MabivikConfig, ops, device, dtype=torch.bfloat16, tp: Optional[TPGroup] = None,
                 quant: Optional[str] = None):
        if quant is not None:
            raise ValueError("Mabivik: quantised weights are not supported")
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Mabivik: tensor parallelism is not supported")
        self.cfg, self.ops, self.device, self.dtype, self.quant = cfg, ops, torch.device(device), dtype, None
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.embed = self.side_embed = self.lm_head = self.final_norm = None
        heads, sizes = [1], [1]
        for l in cfg.layers:
            m = l.mixer
            heads.append(m.heads)
            if l.type == "latent_attention":
                sizes += [m.key_width, m.kv_rank, m.dim + m.rot_dim, m.vdim]
            elif l.type == "delta":
                sizes += [m.dim, m.vdim]
            else:
                sizes += [m.state, m.vdim]
        self.n_q, self.n_kv, self.hd = max(heads), 1, max(sizes)
        self.inter = max([2 * l.mlp.ff * l.mlp.top for l in cfg.layers if l.mlp] or [0])
        self.vocab_local = cfg.vocab_size
        self.prefill_tile_rows = 64

    # ------------------------------------------------------------- KV cache and state
    def _own_cache(self, l) -> bool:
        return l.type == "latent_attention" and l.mixer.kv_from < 0

    def kv_block_bytes(self, block_size: int, dtype) -> int:
        item = torch.tensor([], dtype=dtype).element_size()
        return sum((l.mixer.key_width + l.mixer.kv_rank) * block_size * item for l in self.cfg.layers if self._own_cache(l))

    def alloc_kv(self, num_blocks: int, block_size: int, dtype, device=None):
        """Per latent-attention layer with a cache of its own K [NB, 1, BS, kv_rank + rot_dim] and
        V [NB, 1, kv_rank, BS]; a layer that borrows (``kv_from``) gets the lender's tensors; None
        for the recurrent layers (block ids are shared by all layers: one block table per sequence)."""
        dev = device or self.device
        ks, vs = [], []
        for l in self.cfg.layers:
            m = l.mixer
            if self._own_cache(l):
                ks.append(torch.zeros(num_blocks, 1, block_size, m.key_width, dtype=dtype, device=dev))
                vs.append(torch.zeros(num_blocks, 1, m.kv_rank, block_size, dtype=dtype, device=dev))
            elif l.type == "latent_attention":
                ks.append(ks[m.kv_from])
                vs.append(vs[m.kv_from])
            else:
                ks.append(None)
                vs.append(None)
        return ks, vs

    @staticmethod
    def _state_shape(l):
        """(convolution taps, convolution channels, state heads, state height, state width) of a layer."""
        m = l.mixer
        if l.type == "delta":
            return m.conv, 2 * m.kv_heads * m.dim + m.heads * m.vdim, m.heads, m.dim, m.vdim
        if l.type == "mamba2":
            return m.conv, m.conv_channels, m.heads, m.state, m.vdim
        return 0, 0, 0, 0, 0

    def alloc_state(self, rows: int, device=None) -> dict:
        """State tables with ``rows`` rows, per recurrent layer ``conv`` [rows, taps - 1, channels]
        (activation dtype; None without a convolution) and ``S`` fp32 [rows, heads, height, vdim];
        None for the attention layers."""
        dev = device or self.device
        layers = []
        for l in self.cfg.layers:
            taps, ch, H, d, vd = self._state_shape(l)
            if not H:
                layers.append(None)
                continue
            layers.append({"conv": torch.zeros(rows, taps - 1, ch, dtype=self.dtype, device=dev) if taps > 1 else None,
                           "S": torch.zeros(rows, H, d, vd, dtype=torch.float32, device=dev)})
        return {"layers": layers}

    @staticmethod
    def state_tensors(state: dict) -> List[torch.Tensor]:
        """Every table of `alloc_state` (row-indexed in dimension 0): what the engine moves when
        it moves a row."""
        return [t for L in state["layers"] if L is not None for t in (L["conv"], L["S"]) if t is not None]

    def state_row_bytes(self) -> int:
        item = torch.tensor([], dtype=self.dtype).element_size()
        n = 0
        for l in self.cfg.layers:
            taps, ch, H, d, vd = self._state_shape(l)
            n += max(0, taps - 1) * ch * item + 4 * H * d * vd
        return n

    # ------------------------------------------------------------- weights
    def tensor_shapes(self) -> Dict[str, tuple]:
        """Checkpoint tensor names -> shapes (the expert table is int32)."""
        c, W = self.cfg, self.cfg.hidden_size
        out = {"embed": (c.vocab_size, W), "head": (c.vocab_size, W)}

        def norm(name, n=W):
            out.update({name: (n,), name + ".b": (n,), name + ".alpha": ()})
        norm("final.norm")
        if c.side_dim:
            out["side.embed"] = (c.vocab_size, len(c.layers) * c.side_dim)
        for i, l in enumerate(c.layers):
            p, m, q = f"l{i}.", l.mixer, f"l{i}.mix."
            norm(p + "norm1")
            norm(p + "norm1b")
            if l.type == "latent_attention":
                out.update({q + "dq": (m.q_rank, W), q + "dq.norm": (m.q_rank,), q + "uq": (m.q_width, m.q_rank),
                            q + "uk": (m.heads * m.dim, m.kv_rank), q + "uv": (m.heads * m.vdim, m.kv_rank),
                            q + "g": (m.heads * m.vdim, W), q + "o": (W, m.heads * m.vdim)})
                if m.kv_from < 0:
                    out.update({q + "dkv": (m.key_width, W), q + "dkv.norm": (m.kv_rank,)})
            elif l.type == "delta":
                for n, width in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
                    out[q + n] = (width, W)
                    if m.conv:
                        out[q + n + ".conv"] = (width, m.conv)
                out.update({q + "b": (m.heads, W), q + "a": (m.heads, W), q + "dt_bias": (m.heads,), q + "A_log": (m.heads,),
                            q + "norm": (m.vdim,), q + "g": (m.heads * m.vdim, W), q + "o": (W, m.heads * m.vdim)})
            else:
                out.update({q + "in": (2 * m.inner + 2 * m.groups * m.state + m.heads, W), q + "dt_bias": (m.heads,),
                            q + "A_log": (m.heads,), q + "D": (m.heads,), q + "norm": (m.inner,), q + "o": (W, m.inner)})
                if m.conv:
                    out.update({q + "conv": (m.conv_channels, m.conv), q + "conv.b": (m.conv_channels,)})
            f = l.mlp
            if f is not None:
                norm(p + "norm2")
                norm(p + "norm2b")
                for e in range(f.experts):
                    out.update({p + f"mlp.e{e}.gate": (f.ff, W), p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
                out[p + "mlp.table"] = (c.vocab_size, f.top)
            if c.side_dim:
                out.update({p + "side.gate": (c.side_dim, W), p + "side.proj": (W, c.side_dim), p + "side.norm": (W,)})
        return out

    def random_state_dict(self, seed: int = 0, std: float = 0.05) -> Dict[str, torch.Tensor]:
        """bf16-representable random weights under the checkpoint names (tests, benchmarks)."""
        gen = torch.Generator().manual_seed(seed)
        sd = {}
        for name, shape in self.tensor_shapes().items():
            if name.endswith("mlp.table"):
                E = [l.mlp.experts for i, l in enumerate(self.cfg.layers) if name.startswith(f"l{i}.")][0]
                sd[name] = torch.stack([torch.randperm(E, generator=gen)[:shape[1]] for _ in range(shape[0])]).to(torch.int32)
                continue
            r = torch.randn(shape, generator=gen)
            if name.endswith(".alpha"):
                t = 0.6 + 0.2 * torch.rand(shape, generator=gen)
            elif name.endswith(".norm") or name.endswith(("norm1", "norm2", "norm1b", "norm2b")):
                t = 1.0 + 0.2 * r
            elif name.endswith(("norm1.b", "norm2.b", "norm1b.b", "norm2b.b", "final.norm.b", "conv.b")):
                t = r * 0.1
            elif name.endswith(".conv"):
                t = r * 0.4
            elif name.endswith(("dt_bias", ".D")):
                t = r * 0.5
            elif name.endswith("A_log"):
                t = r * 0.5 - 1.0
            elif name in ("embed", "side.embed"):
                t = r * 0.7
            elif name.endswith((".uq", ".uk", ".uv", "side.proj")):
                t = r * (1.0 / math.sqrt(shape[1]))
            else:
                t = r * (std if name != "head" else 1.0 / math.sqrt(shape[1]))
            sd[name] = t.to(torch.bfloat16)
        return sd

    def init_random(self, seed: int = 0, std: float = 0.05):
        self.load_hf_state_dict(self.random_state_dict(seed, std))

    def load_hf_state_dict(self, sd):
        """Load the checkpoint tensors (names of `tensor_shapes`).  Projections that read the same
        input are stacked into one GEMM weight, the per-head expansions into [H, ...] batches, every
        expert's gate and up rows into one [E, 2 ff, W] tensor."""
        c, dev, dt = self.cfg, self.device, self.dtype
        from ..ops.reference import ramp_inv_freq

        def get(name, dtype=None):
            return sd[name].to(device=dev, dtype=dtype or dt).contiguous()

        def f32(name):
            return get(name, torch.float32)

        def norm(name):
            return ("dyt", float(sd[name + ".alpha"].float()), f32(name), f32(name + ".b"))

        pair = getattr(self.ops, "moe_pair_rows", None)
        self.layers = []
        for i, l in enumerate(c.layers):
            p, m, q = f"l{i}.", l.mixer, f"l{i}.mix."
            L = {"pre1": norm(p + "norm1"), "post1": norm(p + "norm1b")}
            if l.type == "latent_attention":
                parts = [get(q + "dq")] + ([get(q + "dkv")] if m.kv_from < 0 else []) + [get(q + "g")]
                L["fused"] = torch.cat(parts).contiguous()
                L["q_norm"], L["uq"], L["o"] = f32(q + "dq.norm"), get(q + "uq"), get(q + "o")
                if m.kv_from < 0:
                    L["kv_norm"] = f32(q + "dkv.norm")
                # per head: W_uk[h]^T as the weight of a linear (kv_rank outputs from dim inputs), W_uv[h]
                L["uk_t"] = get(q + "uk").reshape(m.heads, m.dim, m.kv_rank).transpose(1, 2).contiguous()
                L["uv"] = get(q + "uv").reshape(m.heads, m.vdim, m.kv_rank).contiguous()
                L["inv_freq"], L["amp"] = ramp_inv_freq(m.rot_dims, m.rot_base, m.rot_scaling, dev)
            elif l.type == "delta":
                names = (q + "q", q + "k", q + "v")
                L["fused"] = torch.cat([get(n) for n in names] + [get(q + "b"), get(q + "a"), get(q + "g")]).contiguous()
                if m.conv:
                    L["conv_w"] = torch.cat([f32(n + ".conv") for n in names]).contiguous()
                L["a_log"], L["dt_bias"], L["head_norm"], L["o"] = f32(q + "A_log"), f32(q + "dt_bias"), f32(q + "norm"), get(q + "o")
            else:
                L["fused"], L["o"] = get(q + "in"), get(q + "o")
                if m.conv:
                    L["conv_w"], L["conv_b"] = f32(q + "conv"), f32(q + "conv.b")
                L["a_log"], L["dt_bias"], L["skip"], L["out_norm"] = f32(q + "A_log"), f32(q + "dt_bias"), f32(q + "D"), f32(q + "norm")
            f = l.mlp
            if f is not None:
                L["pre2"], L["post2"] = norm(p + "norm2"), norm(p + "norm2b")
                ups = []
                for e in range(f.experts):
                    g, u = get(p + f"mlp.e{e}.gate"), get(p + f"mlp.e{e}.up")
                    ups.append(pair(g, u) if pair else torch.cat([g, u]))
                L["e_up"] = torch.stack(ups).contiguous()
                L["e_down"] = torch.stack([get(p + f"mlp.e{e}.down") for e in range(f.experts)]).contiguous()
                L["table"] = sd[p + "mlp.table"].to(device=dev, dtype=torch.int32).contiguous()
            if c.side_dim:
                L["side_gate"], L["side_proj"] = get(p + "side.gate"), get(p + "side.proj")
                L["side_post"] = ("rms", f32(p + "side.norm"), c.rms_eps)
            self.layers.append(L)
        self.embed = get("embed")
        self.side_embed = get("side.embed") if c.side_dim else None
        self.lm_head = get("head")
        self.final_norm = norm("final.norm")

    def weight_bytes(self) -> int:
        def size(v):
            if torch.is_tensor(v):
                return v.numel() * v.element_size()
            return sum(size(t) for t in v) if isinstance(v, tuple) else 0
        n = sum(size(v) for L in self.layers for v in L.values())
        return n + sum(size(t) for t in (self.embed, self.side_embed, self.lm_head, self.final_norm))

    # ------------------------------------------------------------- mixers
    def _latent_attention(self, m, L, h, meta, k_cache, v_cache, sel):
        ops, eps, T = self.ops, self.cfg.rms_eps, h.shape[0]
        y = ops.linear(h, L["fused"])
        off_g = m.q_rank
        if m.kv_from < 0:
            ops.latent_kv_write(y, m.q_rank, m.kv_rank, m.rot_dim, L["kv_norm"], eps, meta.positions, meta.slots,
                                L["inv_freq"], L["amp"], k_cache, v_cache)
            off_g += m.key_width
        q = ops.linear(ops.rmsnorm_cols(y, 0, m.q_rank, L["q_norm"], eps, self.dtype), L["uq"]).view(T, m.heads, m.dim + m.rot_dim)
        qf = torch.empty(T, m.heads, m.key_width, dtype=self.dtype, device=h.device)
        ops.head_linear(q[:, :, :m.dim], L["uk_t"], qf[:, :, :m.kv_rank])
        ops.rope_half_tail(q, m.dim, qf, m.kv_rank, meta.positions, L["inv_freq"], L["amp"])
        lat = ops.multimap_attention(qf, k_cache, v_cache, meta, m.scale, 1, 0.0, -1.0, 1.0, m.kv_rank, m.window, None)
        gate = y[:, off_g:off_g + m.heads * m.vdim]
        if sel is not None:
            lat, gate = lat.index_select(0, sel), gate.index_select(0, sel)
        att = ops.head_linear(lat.view(-1, m.heads, m.kv_rank), L["uv"])
        return ops.linear(ops.gate_mul(att.view(-1, m.heads * m.vdim), gate, "sigmoid"), L["o"])

    def _delta(self, m, L, S, h, meta, sel):
        ops, eps = self.ops, self.cfg.rms_eps
        y = ops.linear(h, L["fused"])
        nqk = m.kv_heads * m.dim
        cw = 2 * nqk + m.heads * m.vdim
        u = ops.short_conv(y, cw, L["conv_w"], meta, S["conv"], "silu") if m.conv else ops.act_fn(y[:, :cw], "silu")
        q32, k32, g32, beta = ops.delta_prepare(u, y, cw, y[:, cw + m.heads:cw + 2 * m.heads], L["a_log"], L["dt_bias"],
                                                m.heads, m.kv_heads, m.dim)
        o32 = ops.gated_state_scan(q32, k32, g32, u[:, 2 * nqk:], beta, meta, S["S"], True)
        gate = y[:, cw + 2 * m.heads:cw + 2 * m.heads + m.heads * m.vdim]
        if sel is not None:
            o32, gate = o32.index_select(0, sel), gate.index_select(0, sel)
        return ops.linear(ops.head_norm_gate(o32, L["head_norm"], eps, gate, self.dtype, "silu"), L["o"])

    def _mamba2(self, m, L, S, h, meta, sel):
        ops, eps = self.ops, self.cfg.rms_eps
        y = ops.linear(h, L["fused"])
        inner, cc = m.inner, m.conv_channels
        xbc = y[:, inner:inner + cc]
        u = ops.short_conv(xbc, cc, L["conv_w"], meta, S["conv"], "silu", L["conv_b"]) if m.conv else ops.act_fn(xbc, "silu")
        q32, k32, g32, dt = ops.ssm_prepare(u, inner, y, inner + cc, L["dt_bias"], L["a_log"], m.heads, m.groups, m.state)
        o32 = ops.gated_state_scan(q32, k32, g32, u[:, :inner], dt, meta, S["S"], False)
        skip, z = u[:, :inner], y[:, :inner]
        if sel is not None:
            o32, skip, z = o32.index_select(0, sel), skip.index_select(0, sel), z.index_select(0, sel)
        return ops.linear(ops.gated_group_norm(o32, skip, L["skip"], z, L["out_norm"], m.norm_groups, eps, self.dtype), L["o"])

    # ------------------------------------------------------------- forward
    def forward(self, tokens: torch.Tensor, meta: AttnMeta, k_cache, v_cache, trace: Optional[list] = None):
        """Logits (fp32) of the rows ``meta.logits_idx`` (all rows when None).  ``meta.state`` holds
        the tables of `alloc_state`, ``meta.state_rows`` every segment's row in them.  ``trace``: a
        list that receives a copy of the residual stream after every layer (debugging)."""
        ops, c, dt = self.ops, self.cfg, self.dtype
        st = meta.state
        if st is None or meta.state_rows is None or meta.q_start is None or meta.token_seq is None:
            raise ValueError("Mabivik: the step carries no sequence state (state, state_rows, q_start, token_seq)")
        x, h = ops.embed_scale_dyt(tokens, self.embed, c.embed_scale, self.layers[0]["pre1"][1:], dt)
        n_layers = len(c.layers)
        for i, (spec, L) in enumerate(zip(c.layers, self.layers)):
            last = i == n_layers - 1
            sel = meta.logits_idx if last else None
            m = spec.mixer
            if spec.type == "latent_attention":
                y = self._latent_attention(m, L, h, meta, k_cache[i], v_cache[i], sel)
            elif spec.type == "delta":
                y = self._delta(m, L, st["layers"][i], h, meta, sel)
            else:
                y = self._mamba2(m, L, st["layers"][i], h, meta, sel)
            if sel is not None:   # past the last mixer only the rows whose logits are asked for matter
                x, tokens = x.index_select(0, sel), tokens.index_select(0, sel)
            nxt = self.final_norm if last else self.layers[i + 1]["pre1"]
            after = ("copy",) if c.side_dim else nxt
            if spec.mlp is not None:
                h2 = ops.residual_post_norm(x, y, L["post1"], L["pre2"], dt)
                idx_e, w_e = ops.moe_table_route(tokens, L["table"], spec.mlp.top)
                h = ops.residual_post_norm(x, ops.moe_experts(h2, L["e_up"], L["e_down"], idx_e, w_e, "silu_gated"),
                                           L["post2"], after, dt)
            else:
                h = ops.residual_post_norm(x, y, L["post1"], after, dt)
            if c.side_dim:
                z = ops.gelu_gather_mul(ops.linear(h, L["side_gate"]), tokens, self.side_embed, i * c.side_dim)
                h = ops.residual_post_norm(x, ops.linear(z, L["side_proj"]), L["side_post"], nxt, dt)
            if trace is not None:
                trace.append(x.clone())
        return ops.linear(h, self.lm_head).float() * c.logit_scale

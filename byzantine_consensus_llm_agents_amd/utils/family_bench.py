"""Prefill / decode throughput of the Mofidra, Padadra, Mabivik and Sitidra families beside the Qwen3-style decoder
at equal layer sizes (random weights, synthetic tokens), and the hot kernels against their
rooflines.  ``bench.py --family-compare`` prints the result as one JSON line.

Equal size: same width, layers, query / KV heads, 128 features per query head (Mofidra: two
64-wide maps), 128 value features, the same feed-forward width (the decoder's SwiGLU has three
matrices, the dense gelu layer two; the MoE variant routes top-2 of 8 experts of ff/4 plus an
always-on expert of ff/2, i.e. the dense layer's active parameters).

Padadra at equal size: the same width, query / KV heads and feed-forward width; the attention
mixer has 128 query / key features and 128 value features per head, a 512-key window and 4-tap
convolutions; the HGRN2 mixer beside it has half as many heads of 64 x 128 state; the gated delta
rule has the query-head count, half as many q / k heads, 128 x 128 state and 4-tap convolutions;
one layer in four is a delta layer.  Its closest relative is Mofidra (the same fp32 stream,
parallel sublayers and attention kernels).

Mabivik at equal size: the same width and head count; four layers (latent attention, state
space, delta rule, a second latent attention that reads the first one's cache); the latent
attention has 128 unrotated + 64 rotated query / key features and 128 value features per head, a
768-wide query latent, a 128-wide key / value latent (a cached row of 192 features, ONE KV head for
all query heads) and a 512-key window; the state-space mixer 2 x width / 128 heads of 128 x 128
state in two groups; the delta rule the query-head count of 128 x 128 states with one decay per
head; 4-tap convolutions; every feed-forward routes top-2 of 8 gated experts of ff/4 by the token id
(Mofidra's MoE variant is its relative there); a 256-wide token input per layer.  Its closest
relative is Padadra (fp32 stream, windowed attention beside recurrences, the same state tables).

Sitidra at equal size: the same width and query / KV head counts; four layers (attention, matrix
memory, attention, matrix memory) over four hyper-connection streams; the attention has 128 query /
key and 128 value features per head, rotary on 64 of them, unit-norm heads, 512-position chunks and
mixed values; the matrix memory has the query-head count of 128 x 128 memories (129 state columns
with the normaliser); every feed-forward routes top-2 of 8 gated experts of ff/4 by sigmoid score
inside 2 of 4 groups, plus a shared expert of ff/2.  Its closest relative is Mabivik (fp32
stream, masked attention beside recurrences on the same scan kernel, the same gated experts).

Rooflines: 2.5 PFLOP/s dense bf16 MFMA, 8 TB/s HBM.  A kernel's ``roof_frac`` is
max(flops / peak, bytes / bandwidth) / measured time.  The recurrence runs on the vector ALUs:
its compute roof is 157 TFLOP/s fp32.
"""

import json
import time

import torch

from ..models.config import MabivikConfig, MofidraConfig, ModelConfig, PadadraConfig, SitidraConfig
from ..models.mabivik import MabivikModel
from ..models.mofidra import MofidraModel
from ..models.padadra import PadadraModel
from ..models.sitidra import SitidraModel
from ..models.transformer import AttnMeta, DecoderModel
from ..ops import get_ops

PEAK_FLOPS, PEAK_BW = 2.5e15, 8.0e12
PEAK_VALU = 157e12
BS = 16

SIZES = {
    "w2048": dict(width=2048, layers=4, heads=16, kv_heads=4, ff=8192, vocab=32768),
    "w4096": dict(width=4096, layers=4, heads=32, kv_heads=8, ff=12288, vocab=32768),
}


def mofidra_config(s, moe: bool) -> MofidraConfig:
    mixer = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": 64, "vdim": 128, "scale": 0.125, "diff": 0.5,
             "rot": {"dims": 64, "base": 1e6}}
    mlp = ({"kind": "moe", "expert": {"ff": s["ff"] // 4}, "router": {"experts": 8, "top": 2}, "shared": {"ff": s["ff"] // 2}}
           if moe else {"kind": "dense", "ff": s["ff"]})
    return MofidraConfig.from_dict({"architecture": "Mofidra", "width": s["width"], "vocab": s["vocab"],
                                    "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
                                    "layers": [{"type": "attention", "mixer": mixer, "mlp": mlp}] * s["layers"]},
                                   "mofidra-bench")


def padadra_config(s) -> PadadraConfig:
    H, G = s["heads"], s["kv_heads"]
    left = {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128, "scale": 0.088, "conv": 4, "mask": {"size": 512},
            "rot": {"dims": 64, "base": 1e6, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    par = {"type": "parallel", "mixer": {"left": left, "right": {"heads": H // 2, "dim": 64, "vdim": 128}},
           "mlp": {"kind": "dense", "ff": s["ff"]}}
    delta = {"type": "channel_delta", "mixer": {"heads": H, "kv_heads": H // 2, "dim": 128, "vdim": 128, "conv": 4,
                                                "decay_rank": 64, "gate_rank": 64}, "mlp": {"kind": "dense", "ff": s["ff"]}}
    layers = [delta if i % 4 == 1 else par for i in range(s["layers"])]
    return PadadraConfig.from_dict({"architecture": "Padadra", "width": s["width"], "vocab": s["vocab"],
                                    "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 1000003, "mul_cur": 31}},
                                    "norm": {"eps": 1e-5}, "residual_mult": 0.5, "layers": layers}, "padadra-bench")


def mabivik_config(s) -> MabivikConfig:
    H, W = s["heads"], s["width"]
    rot = {"dims": 64, "base": 1e6, "scaling": {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}}
    lat = {"heads": H, "dim": 128, "rot_dim": 64, "vdim": 128, "q_rank": 768, "kv_rank": 128, "scale": 0.072, "rot": rot,
           "mask": {"size": 512}}
    mlp = {"kind": "moe", "expert": {"ff": s["ff"] // 4}, "router": {"experts": 8, "top": 2}}
    kinds = [("latent_attention", lat), ("mamba2", {"heads": 2 * W // 128, "vdim": 128, "state": 128, "groups": 2, "norm_groups": 2, "conv": 4}),
             ("delta", {"heads": H, "kv_heads": H // 2, "dim": 128, "vdim": 128, "conv": 4}), ("latent_attention", dict(lat, kv_from=0))]
    layers = []
    for i in range(s["layers"]):
        kind, mixer = kinds[i % 4]
        if kind == "latent_attention" and "kv_from" in mixer:
            mixer = dict(mixer, kv_from=i - 3)
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return MabivikConfig.from_dict({"architecture": "Mabivik", "width": W, "vocab": s["vocab"], "embedding": {"scale": 1.0},
                                    "norm": {"eps": 1e-5}, "logit_scale": 1.0, "token_side": {"dim": 256}, "layers": layers},
                                   "mabivik-bench")


def sitidra_config(s) -> SitidraConfig:
    H, G, W = s["heads"], s["kv_heads"], s["width"]
    att = {"heads": H, "kv_heads": G, "dim": 128, "vdim": 128, "scale": 0.088, "rot": {"dims": 64, "base": 1e6},
           "mask": {"size": 512}, "v_mix": True}
    mem = {"heads": H, "dim": 128, "vdim": 128, "gate_cap": 15.0}
    mlp = {"kind": "moe", "expert": {"ff": s["ff"] // 4},
           "router": {"experts": 8, "top": 2, "scale": 2.0, "groups": {"count": 4, "keep": 2}}, "shared": {"ff": s["ff"] // 2}}
    layers = [{"type": "attention" if i % 2 == 0 else "mlstm", "mixer": att if i % 2 == 0 else mem, "mlp": mlp}
              for i in range(s["layers"])]
    return SitidraConfig.from_dict({"architecture": "Sitidra", "width": W, "vocab": s["vocab"], "norm": {"eps": 1e-5},
                                    "streams": 4, "logit_softcap": 50.0, "layers": layers}, "sitidra-bench")


def decoder_config(s) -> ModelConfig:
    return ModelConfig("decoder-bench", "qwen3", s["width"], s["layers"], s["heads"], s["kv_heads"], 128, s["ff"],
                       s["vocab"], qk_norm=True)


def step_meta(n_seq, ctx, q_len, tile_rows, device, split_single):
    """Packed step: `n_seq` sequences of `ctx` resident tokens, the last `q_len` are this step's."""
    nblk = (ctx + BS - 1) // BS
    tables = (torch.arange(n_seq * nblk, dtype=torch.int32).view(n_seq, nblk) + 1)
    pos = torch.arange(ctx - q_len, ctx).repeat(n_seq)
    seq = torch.arange(n_seq).repeat_interleave(q_len)
    slots = tables[seq, pos // BS].long() * BS + pos % BS
    q_start = torch.arange(n_seq + 1) * q_len
    i32 = torch.int32
    decode = q_len == 1
    tiles, single = [], []
    if not decode:
        for b in range(n_seq):
            for t in range(b * q_len, (b + 1) * q_len, tile_rows):
                tiles.append((ctx - ((b + 1) * q_len - t), b, t, min(t + tile_rows, (b + 1) * q_len)))
        tiles.sort(key=lambda x: -x[0])
    meta = AttnMeta(positions=pos.to(i32).to(device), slots=slots.to(i32).to(device), block_tables=tables.to(device),
                    seq_lens=torch.full((n_seq,), ctx, dtype=i32, device=device), q_start=q_start.to(i32).to(device),
                    max_q_len=q_len, decode=decode, tile_rows=tile_rows,
                    logits_idx=(q_start[1:] - 1).long().to(device),
                    tiles=torch.tensor([t[1:] for t in tiles], dtype=i32, device=device).reshape(-1, 3),
                    single=torch.zeros(0, 2, dtype=i32, device=device) if split_single else None,
                    token_seq=seq.to(i32).to(device), state_rows=torch.arange(n_seq, dtype=i32, device=device))
    return meta, n_seq * nblk + 1


def _time(fn, warmup=3, iters=10):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters


def _graph_time(fn, iters=30):
    fn()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return _time(g.replay, warmup=3, iters=iters)


def model_throughput(model, prefill=(8, 1024), decode=(64, 1024)):
    dev = model.device
    tile_rows = getattr(model, "prefill_tile_rows", None) or model.ops.prefill_tile_rows(model.hd, False, 1024)
    split = getattr(model, "split_single_rows", False)
    out = {}
    n, s = prefill
    meta, nb = step_meta(n, s, s, tile_rows, dev, split)
    k, v = model.alloc_kv(max(nb, decode[0] * ((decode[1] + BS - 1) // BS) + 1), BS, torch.bfloat16)
    tokens = torch.randint(0, model.cfg.vocab_size, (n * s,), dtype=torch.int32, device=dev)
    state = model.alloc_state(max(n, decode[0]) + 1) if hasattr(model, "alloc_state") else None
    meta.state = state
    t = _time(lambda: model.forward(tokens, meta, k, v), iters=5)
    out["prefill_tokens_per_s"] = round(n * s / t)
    out["prefill_ms"] = round(t * 1e3, 3)
    b, ctx = decode
    dmeta, _ = step_meta(b, ctx, 1, tile_rows, dev, split)
    dmeta.logits_idx = None
    dmeta.state = state
    dtok = torch.randint(0, model.cfg.vocab_size, (b,), dtype=torch.int32, device=dev)
    t = _graph_time(lambda: model.forward(dtok, dmeta, k, v))
    out["decode_tokens_per_s"] = round(b / t)
    out["decode_ms"] = round(t * 1e3, 3)
    return out


def _roof(flops, bytes_, t):
    return round(max(flops / PEAK_FLOPS, bytes_ / PEAK_BW) / t, 4)


def kernel_pairs(s, dev):
    """Like kernels of the two families at the same shapes: time and fraction of the roofline."""
    ops = get_ops("hip")
    H, G, W = s["heads"], s["kv_heads"], s["width"]
    bf = torch.bfloat16
    out = {}
    # ---- prefill attention: 8 x 1024 tokens ----
    n, ctx = 8, 1024
    T = n * ctx
    flops = 2 * H * (128 + 128) * n * ctx * ctx / 2   # decoder: QK^T over 128 features + PV over 128 values, causal half
    kv_bytes = n * ctx * G * 256 * 2
    io = T * H * 256 * 2 + kv_bytes
    meta, nb = step_meta(n, ctx, ctx, 64, dev, True)
    q = torch.randn(T, H, 128, device=dev, dtype=bf)
    kc, vc = torch.randn(nb, G, BS, 128, device=dev, dtype=bf), torch.randn(nb, G, 128, BS, device=dev, dtype=bf)
    t = _time(lambda: ops.multimap_attention(q, kc, vc, meta, 0.125, 2, 0.4, 1e-5, 0.5, 128))
    out["prefill_attention"] = {"mofidra_ms": round(t * 1e3, 3), "mofidra_roof_frac": _roof(1.5 * flops, io, t)}  # two maps: PV twice
    rows = ops.prefill_tile_rows(128, False, ctx // BS)
    meta_d, _ = step_meta(n, ctx, ctx, rows, dev, False)
    kd, vd = kc.unsqueeze(0).contiguous(), vc.unsqueeze(0).contiguous()
    t = _time(lambda: ops.paged_attention_prefill(q, kd, vd, 0, meta_d.block_tables, meta_d.q_start, meta_d.seq_lens,
                                                  0.088, ctx, meta_d.tiles, tile_rows=rows))
    out["prefill_attention"].update({"decoder_ms": round(t * 1e3, 3), "decoder_roof_frac": _roof(flops, io, t)})
    # ---- decode attention: 64 rows x 1024 context ----
    b = 64
    dmeta, nb = step_meta(b, ctx, 1, 64, dev, True)
    kc, vc = torch.randn(nb, G, BS, 128, device=dev, dtype=bf), torch.randn(nb, G, 128, BS, device=dev, dtype=bf)
    qd = torch.randn(b, H, 128, device=dev, dtype=bf)
    kv_bytes = b * ctx * G * 256 * 2
    dflops = 2 * H * 256 * b * ctx
    t = _graph_time(lambda: ops.multimap_attention(qd, kc, vc, dmeta, 0.125, 2, 0.4, 1e-5, 0.5, 128), iters=50)
    out["decode_attention"] = {"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(dflops * 1.5, kv_bytes, t)}
    kd, vd = kc.unsqueeze(0).contiguous(), vc.unsqueeze(0).contiguous()
    t = _graph_time(lambda: ops.paged_attention_decode(qd, kd, vd, 0, dmeta.block_tables, dmeta.seq_lens, 0.088), iters=50)
    out["decode_attention"].update({"decoder_ms": round(t * 1e3, 4), "decoder_roof_frac": _roof(dflops, kv_bytes, t)})
    # ---- routed experts (grouped GEMM) beside the dense projection of the same active FLOPs ----
    E, top, ff = 8, 2, s["ff"] // 4
    for name, T in (("prefill", 8192), ("decode", 64)):
        h = torch.randn(T, W, device=dev, dtype=bf)
        up = torch.randn(E, ff, W, device=dev, dtype=bf) * 0.02
        down = torch.randn(E, W, ff, device=dev, dtype=bf) * 0.02
        rw, rb = torch.randn(E, W, device=dev) * 0.02, torch.zeros(E, device=dev)
        idx, wts, _ = ops.moe_route(h, rw, rb, top)
        flops = 2 * 2 * T * top * ff * W
        wbytes = 2 * E * ff * W * 2 + T * W * 2 * (2 + 2 * top)
        t = _time(lambda: ops.moe_experts(h, up, down, idx, wts, "relu2"), iters=20)
        wd_up = torch.randn(top * ff, W, device=dev, dtype=bf) * 0.02
        wd_down = torch.randn(W, top * ff, device=dev, dtype=bf) * 0.02
        t2 = _time(lambda: ops.linear(ops.linear(h, wd_up), wd_down), iters=20)
        out[f"experts_{name}"] = {"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(flops, wbytes, t),
                                  "dense_gemm_ms": round(t2 * 1e3, 4),
                                  "dense_gemm_roof_frac": _roof(flops, 2 * top * ff * W * 2 + T * W * 4, t2)}
    # ---- residual add + norm: fp32 stream against the bf16 stream ----
    T = 8192
    x32, p = torch.randn(T, W, device=dev), torch.randn(T, W, device=dev, dtype=bf)
    w32 = torch.zeros(W, device=dev)
    t = _time(lambda: ops.residual_add_rmsnorm32(x32, [p, p], w32, 1e-5, 1.0, bf), iters=20)
    out["residual_norm"] = {"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(0, T * W * (4 + 4 + 2 + 2 + 2), t)}
    xb, wb = torch.randn(T, W, device=dev, dtype=bf), torch.ones(W, device=dev, dtype=bf)
    t = _time(lambda: ops.add_rmsnorm(p, xb, wb, 1e-5), iters=20)
    out["residual_norm"].update({"decoder_ms": round(t * 1e3, 4), "decoder_roof_frac": _roof(0, T * W * (2 + 2 + 2 + 2), t)})
    return out


def state_kernels(s, dev):
    """The Padadra kernels beside their like kernels of Mofidra at the same shapes (window + sink
    attention: the two-map attention; scalar-gain residual kernel: the weighted one; pair rotary
    with norms: the half-split rotary), and the kernels without a relative (recurrence, convolution)."""
    ops = get_ops("hip")
    H, G, W = s["heads"], s["kv_heads"], s["width"]
    bf = torch.bfloat16
    out = {}
    n, ctx, window = 8, 1024, 512
    T = n * ctx
    # ---- prefill attention, 8 x 1024: one 128-wide map, 512-key window, sink ----
    pairs = sum(min(i + 1, window) for i in range(ctx)) * n
    flops = 2 * H * 256 * pairs
    io = T * H * 256 * 2 + T * G * 256 * 2
    meta, nb = step_meta(n, ctx, ctx, 64, dev, True)
    q = torch.randn(T, H, 128, device=dev, dtype=bf)
    kc, vc = torch.randn(nb, G, BS, 128, device=dev, dtype=bf), torch.randn(nb, G, 128, BS, device=dev, dtype=bf)
    sink = torch.randn(H, device=dev)
    t = _time(lambda: ops.multimap_attention(q, kc, vc, meta, 0.088, 1, 0.0, -1.0, 1.0, 128, window, sink))
    out["prefill_attention"] = {"padadra_ms": round(t * 1e3, 3), "padadra_roof_frac": _roof(flops, io, t)}
    q2 = torch.randn(T, H, 128, device=dev, dtype=bf)
    t = _time(lambda: ops.multimap_attention(q2, kc, vc, meta, 0.125, 2, 0.4, 1e-5, 0.5, 128))
    full = 2 * H * 256 * n * ctx * ctx / 2
    out["prefill_attention"].update({"mofidra_ms": round(t * 1e3, 3), "mofidra_roof_frac": _roof(1.5 * full, io, t)})
    # ---- decode attention, 64 rows x 1024 context ----
    b = 64
    dmeta, nb = step_meta(b, ctx, 1, 64, dev, True)
    kc, vc = torch.randn(nb, G, BS, 128, device=dev, dtype=bf), torch.randn(nb, G, 128, BS, device=dev, dtype=bf)
    qd = torch.randn(b, H, 128, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.multimap_attention(qd, kc, vc, dmeta, 0.088, 1, 0.0, -1.0, 1.0, 128, window, sink), iters=50)
    out["decode_attention"] = {"padadra_ms": round(t * 1e3, 4),
                               "padadra_roof_frac": _roof(2 * H * 256 * b * window, b * window * G * 256 * 2, t)}
    t = _graph_time(lambda: ops.multimap_attention(qd, kc, vc, dmeta, 0.125, 2, 0.4, 1e-5, 0.5, 128), iters=50)
    out["decode_attention"].update({"mofidra_ms": round(t * 1e3, 4),
                                    "mofidra_roof_frac": _roof(2 * H * 256 * b * ctx * 1.5, b * ctx * G * 256 * 2, t)})
    # ---- residual update + next norms, 8192 rows ----
    x32 = torch.randn(T, W, device=dev)
    a, c, p = (torch.randn(T, W, device=dev, dtype=bf) for _ in range(3))
    wa, wb = torch.randn(W, device=dev), torch.randn(W, device=dev)
    t = _time(lambda: ops.residual_mix_norm(x32, [(a, wa), (c, wb)], 0.5, [p], 0.5, 1e-5, (1.0, 0.9), bf), iters=20)
    out["residual_norm"] = {"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, T * W * (4 + 4 + 3 * 2 + 2 * 2), t)}
    w32 = torch.zeros(W, device=dev)
    t = _time(lambda: ops.residual_add_rmsnorm32(x32, [a, p], w32, 1e-5, 1.0, bf), iters=20)
    out["residual_norm"].update({"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(0, T * W * (4 + 4 + 2 + 2 + 2), t)})
    # ---- rotary + cache write, 8192 rows ----
    width = (H + G) * 128 + G * 128
    y = torch.randn(T, width, device=dev, dtype=bf)
    qn, kn = torch.ones(H * 128, device=dev), torch.ones(G * 128, device=dev)
    inv, vinv = torch.rand(32, device=dev), torch.rand(64, device=dev)
    kc, vc = torch.zeros(n * ctx // BS + 1, G, BS, 128, device=dev, dtype=bf), torch.zeros(n * ctx // BS + 1, G, 128, BS, device=dev, dtype=bf)
    t = _time(lambda: ops.rope_pairs_kv_write(y, meta.positions, meta.slots, H, G, 128, 128, qn, kn, 1e-5, inv, vinv, kc, vc), iters=20)
    io = T * width * 2 * 2
    out["rotary_kv_write"] = {"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, io, t)}
    kc2 = torch.zeros(n * ctx // BS + 1, G, BS, 128, device=dev, dtype=bf)
    t = _time(lambda: ops.rope_multi_kv_write(y, meta.positions, meta.slots, H, G, 2, 64, 128, inv, kc2, vc), iters=20)
    out["rotary_kv_write"].update({"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(0, io, t)})
    # ---- short convolution, 8192 rows ----
    cw = torch.randn(width, 4, device=dev)
    cstate = torch.zeros(n + 1, 3, width, device=dev, dtype=bf)
    t = _time(lambda: ops.short_conv(y, width, cw, meta, cstate, "silu"), iters=20)
    out["short_conv"] = {"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, io, t)}
    # ---- the recurrence: gated delta rule, H heads of 128 x 128 state ----
    Gq = max(1, H // 2)
    for name, rows_, m_ in (("prefill", T, meta), ("decode", b, dmeta)):
        q32, k32 = torch.randn(rows_, Gq, 128, device=dev) * 0.1, torch.randn(rows_, Gq, 128, device=dev) * 0.1
        g32, beta = torch.rand(rows_, H, 128, device=dev), torch.rand(rows_, H, device=dev)
        v = torch.randn(rows_, H * 128, device=dev, dtype=bf)
        S = torch.zeros(max(n, b) + 1, H, 128, 128, device=dev)
        m_.state_rows = torch.arange(m_.q_start.numel() - 1, dtype=torch.int32, device=dev)
        fn = lambda: ops.gated_state_scan(q32, k32, g32, v, beta, m_, S, True)  # noqa: E731
        t = _time(fn, iters=10) if name == "prefill" else _graph_time(fn, iters=50)
        flops = rows_ * H * 128 * 128 * 8
        io = rows_ * (2 * Gq * 128 * 4 + H * 128 * 4 + H * 128 * 2 + H * 128 * 4) + (m_.q_start.numel() - 1) * H * 128 * 128 * 4 * 2
        out[f"state_scan_{name}"] = {"padadra_ms": round(t * 1e3, 4),
                                     "padadra_roof_frac": round(max(flops / PEAK_VALU, io / PEAK_BW) / t, 4)}
    # ---- the recurrence: HGRN2, H / 2 heads of 64 x 128 state ----
    Hh = max(1, H // 2)
    q32, k32, g32 = (torch.rand(T, Hh, 64, device=dev) for _ in range(3))
    v = torch.randn(T, Hh * 128, device=dev, dtype=bf)
    S = torch.zeros(n + 1, Hh, 64, 128, device=dev)
    t = _time(lambda: ops.gated_state_scan(q32, k32, g32, v, None, meta, S, False), iters=10)
    io = T * (3 * Hh * 64 * 4 + Hh * 128 * 2 + Hh * 128 * 4)
    out["state_scan_prefill_hgrn2"] = {"padadra_ms": round(t * 1e3, 4),
                                       "padadra_roof_frac": round(max(T * Hh * 64 * 128 * 6 / PEAK_VALU, io / PEAK_BW) / t, 4)}
    return out


def latent_kernels(s, dev):
    """The Mabivik kernels beside their like kernels of Padadra / Mofidra at the same shapes."""
    ops = get_ops("hip")
    H, G, W = s["heads"], s["kv_heads"], s["width"]
    bf = torch.bfloat16
    out = {}
    n, ctx, window = 8, 1024, 512
    T, b = n * ctx, 64
    R, RD = 128, 64
    KD = R + RD
    pairs = sum(min(i + 1, window) for i in range(ctx)) * n
    meta, nb = step_meta(n, ctx, ctx, 64, dev, True)
    dmeta, nbd = step_meta(b, ctx, 1, 64, dev, True)
    nb = max(nb, nbd)
    # ---- prefill attention, 8 x 1024, 512-key window: one KV head of 192 key / 128 value features against GQA heads of 128 / 128 ----
    q = torch.randn(T, H, KD, device=dev, dtype=bf)
    kc, vc = torch.randn(nb, 1, BS, KD, device=dev, dtype=bf), torch.randn(nb, 1, R, BS, device=dev, dtype=bf)
    t = _time(lambda: ops.multimap_attention(q, kc, vc, meta, 0.072, 1, 0.0, -1.0, 1.0, R, window, None))
    out["prefill_attention"] = {"mabivik_ms": round(t * 1e3, 3),
                                "mabivik_roof_frac": _roof(2 * H * (KD + R) * pairs, T * H * (KD + R) * 2 + T * (KD + R) * 2, t)}
    q1 = torch.randn(T, H, 128, device=dev, dtype=bf)
    k1, v1 = torch.randn(nb, G, BS, 128, device=dev, dtype=bf), torch.randn(nb, G, 128, BS, device=dev, dtype=bf)
    sink = torch.randn(H, device=dev)
    t = _time(lambda: ops.multimap_attention(q1, k1, v1, meta, 0.088, 1, 0.0, -1.0, 1.0, 128, window, sink))
    out["prefill_attention"].update({"padadra_ms": round(t * 1e3, 3),
                                     "padadra_roof_frac": _roof(2 * H * 256 * pairs, T * H * 256 * 2 + T * G * 256 * 2, t)})
    # ---- decode attention, 64 rows x 1024 context ----
    qd, qd1 = torch.randn(b, H, KD, device=dev, dtype=bf), torch.randn(b, H, 128, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.multimap_attention(qd, kc, vc, dmeta, 0.072, 1, 0.0, -1.0, 1.0, R, window, None), iters=50)
    out["decode_attention"] = {"mabivik_ms": round(t * 1e3, 4),
                               "mabivik_roof_frac": _roof(2 * H * (KD + R) * b * window, b * window * (KD + R) * 2, t)}
    t = _graph_time(lambda: ops.multimap_attention(qd1, k1, v1, dmeta, 0.088, 1, 0.0, -1.0, 1.0, 128, window, sink), iters=50)
    out["decode_attention"].update({"padadra_ms": round(t * 1e3, 4),
                                    "padadra_roof_frac": _roof(2 * H * 256 * b * window, b * window * G * 256 * 2, t)})
    # ---- decode attention, 512 rows x 1024 context: enough waves to fill the chip with one KV head ----
    b2 = 512
    dmeta2, nb2 = step_meta(b2, ctx, 1, 64, dev, True)
    kc2, vc2 = torch.randn(nb2, 1, BS, KD, device=dev, dtype=bf), torch.randn(nb2, 1, R, BS, device=dev, dtype=bf)
    k12, v12 = torch.randn(nb2, G, BS, 128, device=dev, dtype=bf), torch.randn(nb2, G, 128, BS, device=dev, dtype=bf)
    qd2, qd12 = torch.randn(b2, H, KD, device=dev, dtype=bf), torch.randn(b2, H, 128, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.multimap_attention(qd2, kc2, vc2, dmeta2, 0.072, 1, 0.0, -1.0, 1.0, R, window, None), iters=50)
    out["decode_attention_512_rows"] = {"mabivik_ms": round(t * 1e3, 4),
                                        "mabivik_roof_frac": _roof(2 * H * (KD + R) * b2 * window, b2 * window * (KD + R) * 2, t)}
    t = _graph_time(lambda: ops.multimap_attention(qd12, k12, v12, dmeta2, 0.088, 1, 0.0, -1.0, 1.0, 128, window, sink), iters=50)
    out["decode_attention_512_rows"].update({"padadra_ms": round(t * 1e3, 4),
                                             "padadra_roof_frac": _roof(2 * H * 256 * b2 * window, b2 * window * G * 256 * 2, t)})
    del kc2, vc2, k12, v12
    # ---- residual update + next norm, 8192 rows: dynamic tanh (no reduction) against the RMS kernels ----
    x32 = torch.randn(T, W, device=dev)
    a, c, p = (torch.randn(T, W, device=dev, dtype=bf) for _ in range(3))
    w1, b1, w2, b2 = (torch.randn(W, device=dev) for _ in range(4))
    t = _time(lambda: ops.residual_post_norm(x32, a, ("dyt", 0.5, w1, b1), ("dyt", 0.7, w2, b2), bf), iters=20)
    out["residual_norm"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * W * (4 + 4 + 2 + 2), t)}
    f32part = torch.randn(T, W, device=dev)
    t = _time(lambda: ops.residual_post_norm(x32, f32part, ("rms", w1, 1e-5), ("dyt", 0.7, w2, b2), bf), iters=20)
    out["residual_norm_rms_post"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * W * (4 + 4 + 4 + 2), t)}
    t = _time(lambda: ops.residual_mix_norm(x32, [(a, w1), (c, w2)], 0.5, [p], 0.5, 1e-5, (1.0, 0.9), bf), iters=20)
    out["residual_norm"].update({"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, T * W * (4 + 4 + 3 * 2 + 2 * 2), t)})
    w32 = torch.zeros(W, device=dev)
    t = _time(lambda: ops.residual_add_rmsnorm32(x32, [a, p], w32, 1e-5, 1.0, bf), iters=20)
    out["residual_norm"].update({"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(0, T * W * (4 + 4 + 2 + 2 + 2), t)})
    # ---- cache write, 8192 rows: latent norm + rotary + two slab writes against Padadra's q / k / v rotary write ----
    fused = 768 + KD + H * 128
    y = torch.randn(T, fused, device=dev, dtype=bf)
    inv = torch.rand(RD // 2, device=dev)
    kz, vz = torch.zeros(nb, 1, BS, KD, device=dev, dtype=bf), torch.zeros(nb, 1, R, BS, device=dev, dtype=bf)
    wn = torch.ones(R, device=dev)
    t = _graph_time(lambda: ops.latent_kv_write(y, 768, R, RD, wn, 1e-5, meta.positions, meta.slots, inv, 1.2, kz, vz), iters=50)
    out["cache_write"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * (KD + KD + R) * 2, t)}
    width = (H + G) * 128 + G * 128
    y2 = torch.randn(T, width, device=dev, dtype=bf)
    qn, kn = torch.ones(H * 128, device=dev), torch.ones(G * 128, device=dev)
    inv2, vinv = torch.rand(32, device=dev), torch.rand(64, device=dev)
    kp, vp = torch.zeros(nb, G, BS, 128, device=dev, dtype=bf), torch.zeros(nb, G, 128, BS, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.rope_pairs_kv_write(y2, meta.positions, meta.slots, H, G, 128, 128, qn, kn, 1e-5, inv2, vinv, kp, vp), iters=50)
    out["cache_write"].update({"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, T * width * 2 * 2, t)})
    # ---- query assembly: tail rotary into the packed query (the per-head products are vendor GEMMs) ----
    qsrc, qdst = torch.randn(T, H, 128 + RD, device=dev, dtype=bf), torch.empty(T, H, KD, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.rope_half_tail(qsrc, 128, qdst, R, meta.positions, inv, 1.2), iters=50)
    out["query_tail_rotary"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * H * RD * 2 * 2, t)}
    # ---- routed experts: gated (three matrices, activation in the epilogue) against relu^2 (two matrices) ----
    E, top, ff = 8, 2, s["ff"] // 4
    for name, rows_ in (("prefill", 8192), ("decode", 64)):
        h = torch.randn(rows_, W, device=dev, dtype=bf)
        up2 = torch.randn(E, 2 * ff, W, device=dev, dtype=bf) * 0.02
        up1 = torch.randn(E, ff, W, device=dev, dtype=bf) * 0.02
        down = torch.randn(E, W, ff, device=dev, dtype=bf) * 0.02
        idx = torch.randint(0, E, (rows_, 1), device=dev, dtype=torch.int32)
        idx = torch.cat([idx, (idx + 1 + torch.randint(0, E - 1, (rows_, 1), device=dev, dtype=torch.int32)) % E], 1).contiguous()
        wts = torch.full((rows_, top), 0.5, device=dev)
        act = rows_ * W * 2 * (2 + 2 * top)
        t = _time(lambda: ops.moe_experts(h, up2, down, idx, wts, "silu_gated"), iters=20)
        out[f"experts_{name}"] = {"mabivik_ms": round(t * 1e3, 4),
                                  "mabivik_roof_frac": _roof(2 * 3 * rows_ * top * ff * W, 3 * E * ff * W * 2 + act, t)}
        t = _time(lambda: ops.moe_experts(h, up1, down, idx, wts, "relu2"), iters=20)
        out[f"experts_{name}"].update({"mofidra_ms": round(t * 1e3, 4),
                                       "mofidra_roof_frac": _roof(2 * 2 * rows_ * top * ff * W, 2 * E * ff * W * 2 + act, t)})
    # ---- the recurrences: one decay per head (delta rule; state space with scaled writes) against one per channel ----
    Gq = max(1, H // 2)
    Hs = 2 * W // 128
    for name, rows_, m_ in (("prefill", T, meta), ("decode", b, dmeta)):
        nseq = m_.q_start.numel() - 1
        m_.state_rows = torch.arange(nseq, dtype=torch.int32, device=dev)
        q32, k32 = torch.randn(rows_, Gq, 128, device=dev) * 0.1, torch.randn(rows_, Gq, 128, device=dev) * 0.1
        g1, gc, beta = torch.rand(rows_, H, 1, device=dev), torch.rand(rows_, H, 128, device=dev), torch.rand(rows_, H, device=dev)
        v = torch.randn(rows_, H * 128, device=dev, dtype=bf)
        S = torch.zeros(max(n, b) + 1, H, 128, 128, device=dev)
        timer = (lambda f: _time(f, iters=10)) if name == "prefill" else (lambda f: _graph_time(f, iters=50))
        flops = rows_ * H * 128 * 128 * 8
        io = rows_ * (2 * Gq * 128 * 4 + H * 4 + H * 128 * 2 + H * 128 * 4) + nseq * H * 128 * 128 * 4 * 2
        t = timer(lambda: ops.gated_state_scan(q32, k32, g1, v, beta, m_, S, True))
        entry = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": round(max(flops / PEAK_VALU, io / PEAK_BW) / t, 4)}
        t = timer(lambda: ops.gated_state_scan(q32, k32, gc, v, beta, m_, S, True))
        entry.update({"padadra_ms": round(t * 1e3, 4),
                      "padadra_roof_frac": round(max(flops / PEAK_VALU, (io + rows_ * H * 127 * 4) / PEAK_BW) / t, 4)})
        out[f"delta_scan_{name}"] = entry
        qs, ks = torch.randn(rows_, 2, 128, device=dev) * 0.1, torch.randn(rows_, 2, 128, device=dev) * 0.1
        gs, dts = torch.rand(rows_, Hs, 1, device=dev), torch.rand(rows_, Hs, device=dev)
        vs = torch.randn(rows_, Hs * 128, device=dev, dtype=bf)
        Ss = torch.zeros(max(n, b) + 1, Hs, 128, 128, device=dev)
        t = timer(lambda: ops.gated_state_scan(qs, ks, gs, vs, dts, m_, Ss, False))
        flops = rows_ * Hs * 128 * 128 * 6
        io = rows_ * (2 * 2 * 128 * 4 + Hs * 8 + Hs * 128 * 2 + Hs * 128 * 4) + nseq * Hs * 128 * 128 * 4 * 2
        out[f"ssm_scan_{name}"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": round(max(flops / PEAK_VALU, io / PEAK_BW) / t, 4)}
    # ---- output norms of the recurrent mixers, 8192 rows ----
    o32 = torch.randn(T, Hs, 128, device=dev)
    skip, z = torch.randn(T, Hs * 128, device=dev, dtype=bf), torch.randn(T, Hs * 128, device=dev, dtype=bf)
    D, wg = torch.randn(Hs, device=dev), torch.randn(Hs * 128, device=dev)
    t = _time(lambda: ops.gated_group_norm(o32, skip, D, z, wg, 2, 1e-5, bf), iters=20)
    out["recurrent_out_norm"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * Hs * 128 * (4 + 2 + 2 + 2), t)}
    wh = torch.randn(128, device=dev)
    t = _time(lambda: ops.head_norm_gate(o32, wh, 1e-5, z, bf), iters=20)
    out["recurrent_out_norm"].update({"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, T * Hs * 128 * (4 + 2 + 2), t)})
    # ---- short convolution with bias, 8192 rows ----
    cc = Hs * 128 + 2 * 2 * 128
    yc, cw, cb = torch.randn(T, cc, device=dev, dtype=bf), torch.randn(cc, 4, device=dev), torch.randn(cc, device=dev)
    cstate = torch.zeros(n + 1, 3, cc, device=dev, dtype=bf)
    t = _time(lambda: ops.short_conv(yc, cc, cw, meta, cstate, "silu", cb), iters=20)
    out["short_conv"] = {"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * cc * 2 * 2, t)}
    t = _time(lambda: ops.short_conv(yc, cc, cw, meta, cstate, "silu"), iters=20)
    out["short_conv"].update({"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, T * cc * 2 * 2, t)})
    return out


def hyper_kernels(s, dev):
    """Sitidra's kernels beside the like kernels of Mabivik, Padadra and Mofidra at the same shapes."""
    ops = get_ops("hip")
    H, G, W = s["heads"], s["kv_heads"], s["width"]
    bf = torch.bfloat16
    out = {}
    n, ctx, chunk = 8, 1024, 512
    T, b = n * ctx, 64
    meta, nb = step_meta(n, ctx, ctx, 64, dev, True)
    dmeta, nbd = step_meta(b, ctx, 1, 64, dev, True)
    nb = max(nb, nbd)
    pairs = sum(i % chunk + 1 for i in range(ctx)) * n      # (query, key) pairs under the chunk mask
    pairs_w = sum(min(i + 1, chunk) for i in range(ctx)) * n  # ... under a window of the same size
    # ---- prefill attention, 8 x 1024: 512-position chunks against a 512-key window (one kernel, two masks) ----
    q = torch.randn(T, H, 128, device=dev, dtype=bf)
    kc, vc = torch.randn(nb, G, BS, 128, device=dev, dtype=bf), torch.randn(nb, G, 128, BS, device=dev, dtype=bf)
    io = T * H * 256 * 2 + T * G * 256 * 2
    t = _time(lambda: ops.multimap_attention(q, kc, vc, meta, 0.088, 1, 0.0, -1.0, 1.0, 128, 0, None, chunk))
    out["prefill_attention"] = {"sitidra_ms": round(t * 1e3, 3), "sitidra_roof_frac": _roof(2 * H * 256 * pairs, io, t)}
    sink = torch.randn(H, device=dev)
    t = _time(lambda: ops.multimap_attention(q, kc, vc, meta, 0.088, 1, 0.0, -1.0, 1.0, 128, chunk, sink))
    out["prefill_attention"].update({"padadra_ms": round(t * 1e3, 3), "padadra_roof_frac": _roof(2 * H * 256 * pairs_w, io, t)})
    # ---- decode attention, 64 rows at position 1023: the chunk's 512 keys against the window's ----
    qd = torch.randn(b, H, 128, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.multimap_attention(qd, kc, vc, dmeta, 0.088, 1, 0.0, -1.0, 1.0, 128, 0, None, chunk), iters=50)
    out["decode_attention"] = {"sitidra_ms": round(t * 1e3, 4),
                               "sitidra_roof_frac": _roof(2 * H * 256 * b * chunk, b * chunk * G * 256 * 2, t)}
    t = _graph_time(lambda: ops.multimap_attention(qd, kc, vc, dmeta, 0.088, 1, 0.0, -1.0, 1.0, 128, chunk, sink), iters=50)
    out["decode_attention"].update({"padadra_ms": round(t * 1e3, 4),
                                    "padadra_roof_frac": _roof(2 * H * 256 * b * chunk, b * chunk * G * 256 * 2, t)})
    # ---- stream update + next read + layer norm, 8192 rows x 4 streams, against the one-stream residual kernels ----
    S = 4
    X = torch.randn(T, S, W, device=dev)
    a, p32 = torch.randn(T, W, device=dev, dtype=bf), torch.randn(T, W, device=dev)
    mix, ow, rw, nw = torch.randn(S, S, device=dev) * 0.3, torch.randn(S, device=dev), torch.randn(S, device=dev), torch.randn(W, device=dev)
    t = _time(lambda: ops.hyper_update_norm(X, [a], mix, ow, rw, nw, 1e-5, bf), iters=20)
    out["residual_norm"] = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(0, T * W * (8 * S + 2 + 2), t)}
    t = _time(lambda: ops.hyper_update_norm(X, [a, p32], mix, ow, rw, nw, 1e-5, bf), iters=20)
    out["residual_norm_two_parts"] = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(0, T * W * (8 * S + 2 + 4 + 2), t)}
    x32 = torch.randn(T, W, device=dev)
    w1, b1, w2, b2 = (torch.randn(W, device=dev) for _ in range(4))
    t = _time(lambda: ops.residual_post_norm(x32, a, ("dyt", 0.5, w1, b1), ("dyt", 0.7, w2, b2), bf), iters=20)
    out["residual_norm"].update({"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * W * (4 + 4 + 2 + 2), t)})
    t = _time(lambda: ops.residual_add_rmsnorm32(x32, [a], w1, 1e-5, 1.0, bf), iters=20)
    out["residual_norm"].update({"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(0, T * W * (4 + 4 + 2 + 2), t)})
    del X, x32, p32
    # ---- cache write, 8192 rows: rotary + unit-norm heads + mixed values against Padadra's and Mofidra's rotary writes ----
    width = (H + G) * 128 + G * 128
    y = torch.randn(T, width + H, device=dev, dtype=bf)
    vf = torch.randn(T, G * 128, device=dev, dtype=bf)
    inv = torch.rand(32, device=dev)
    kz, vz = torch.zeros(nb, G, BS, 128, device=dev, dtype=bf), torch.zeros(nb, G, 128, BS, device=dev, dtype=bf)
    t = _graph_time(lambda: ops.rope_norm_kv_write(y, meta.positions, meta.slots, H, G, 128, 128, inv, 1e-5, vf, 0.3, kz, vz), iters=50)
    out["cache_write"] = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(0, T * (width * 2 + G * 128) * 2, t)}
    qn, kn, vinv = torch.ones(H * 128, device=dev), torch.ones(G * 128, device=dev), torch.rand(64, device=dev)
    t = _graph_time(lambda: ops.rope_pairs_kv_write(y, meta.positions, meta.slots, H, G, 128, 128, qn, kn, 1e-5, inv, vinv, kz, vz), iters=50)
    out["cache_write"].update({"padadra_ms": round(t * 1e3, 4), "padadra_roof_frac": _roof(0, T * width * 2 * 2, t)})
    t = _graph_time(lambda: ops.rope_multi_kv_write(y, meta.positions, meta.slots, H, G, 1, 128, 128, inv, kz, vz), iters=50)
    out["cache_write"].update({"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(0, T * width * 2 * 2, t)})
    # ---- output gate: one gate per head against one per feature ----
    att, gh, gf = torch.randn(T, H * 128, device=dev, dtype=bf), torch.randn(T, H, device=dev, dtype=bf), torch.randn(T, H * 128, device=dev, dtype=bf)
    t = _time(lambda: ops.gate_mul(att, gh, "sigmoid", 128), iters=20)
    out["output_gate"] = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(0, T * H * 128 * 2 * 2, t)}
    t = _time(lambda: ops.gate_mul(att, gf, "sigmoid"), iters=20)
    out["output_gate"].update({"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * H * 128 * 2 * 3, t)})
    # ---- the memory: gates + running maximum, the scan with the normaliser column, the output norm ----
    fused = 2 * H * 128 + 2 * H * 128 + 2 * H
    Hs = 2 * W // 128
    for name, rows_, m_ in (("prefill", T, meta), ("decode", b, dmeta)):
        nseq = m_.q_start.numel() - 1
        m_.state_rows = torch.arange(nseq, dtype=torch.int32, device=dev)
        timer = (lambda f: _time(f, iters=10)) if name == "prefill" else (lambda f: _graph_time(f, iters=50))
        yf = torch.randn(rows_, fused, device=dev, dtype=bf)
        ib, fb = torch.zeros(H, device=dev), torch.ones(H, device=dev)
        m_state = torch.zeros(max(n, b) + 1, H, device=dev)
        off_i = 4 * H * 128
        t = timer(lambda: ops.exp_gate_prepare(yf, 0, H * 128, off_i, off_i + H, ib, fb, 15.0, 128 ** -0.5, H, 128, m_, m_state))
        entry = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(0, rows_ * (2 * H * 128 * (2 + 4) + 2 * H * 2 + 3 * H * 4), t)}
        ys = torch.randn(rows_, 2 * Hs * 128 + 2 * 2 * 128 + Hs, device=dev, dtype=bf)
        dtb, al = torch.zeros(Hs, device=dev), torch.zeros(Hs, device=dev)
        t = timer(lambda: ops.ssm_prepare(ys, Hs * 128, ys, 2 * Hs * 128 + 4 * 128, dtb, al, Hs, 2, 128))
        entry.update({"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, rows_ * (4 * 128 * (2 + 4) + Hs * (2 + 8)), t)})
        out[f"gate_prepare_{name}"] = entry
        q32, k32, dec, wr, fl = ops.exp_gate_prepare(yf, 0, H * 128, off_i, off_i + H, ib, fb, 15.0, 128 ** -0.5, H, 128, m_, m_state)
        v = yf[:, 2 * H * 128:3 * H * 128]
        Sm = torch.zeros(max(n, b) + 1, H, 128, 129, device=dev)
        t = timer(lambda: ops.gated_state_scan(q32, k32, dec, v, wr, m_, Sm, False, True))
        flops = rows_ * H * 128 * 129 * 6
        io = rows_ * (2 * H * 128 * 4 + H * 8 + H * 128 * 2 + H * 129 * 4) + nseq * H * 128 * 129 * 4 * 2
        entry = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": round(max(flops / PEAK_VALU, io / PEAK_BW) / t, 4)}
        qs, ks = torch.randn(rows_, 2, 128, device=dev) * 0.1, torch.randn(rows_, 2, 128, device=dev) * 0.1
        gs, dts = torch.rand(rows_, H, 1, device=dev), torch.rand(rows_, H, device=dev)
        Ss = torch.zeros(max(n, b) + 1, H, 128, 128, device=dev)
        t = timer(lambda: ops.gated_state_scan(qs, ks, gs, v, dts, m_, Ss, False))   # the state-space form at the same head count
        flops = rows_ * H * 128 * 128 * 6
        io = rows_ * (2 * 2 * 128 * 4 + H * 8 + H * 128 * 2 + H * 128 * 4) + nseq * H * 128 * 128 * 4 * 2
        entry.update({"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": round(max(flops / PEAK_VALU, io / PEAK_BW) / t, 4)})
        out[f"memory_scan_{name}"] = entry
        del Sm, Ss
    o33 = torch.randn(T, H, 129, device=dev)
    o32 = torch.randn(T, H, 128, device=dev)
    fl, z = torch.rand(T, H, device=dev), torch.randn(T, H * 128, device=dev, dtype=bf)
    wn, wh = torch.randn(H * 128, device=dev), torch.randn(128, device=dev)
    t = _time(lambda: ops.head_norm_gate(o33, wn, 1e-5, z, bf, "sigmoid", fl), iters=20)
    out["recurrent_out_norm"] = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(0, T * H * (129 * 4 + 4 + 128 * 4), t)}
    t = _time(lambda: ops.head_norm_gate(o32, wh, 1e-5, z, bf, "silu"), iters=20)
    out["recurrent_out_norm"].update({"mabivik_ms": round(t * 1e3, 4), "mabivik_roof_frac": _roof(0, T * H * 128 * (4 + 2 + 2), t)})
    # ---- router: sigmoid scores with groups against the softmax over the chosen ----
    E = 8
    h = torch.randn(T, W, device=dev, dtype=bf)
    rw_, corr = torch.randn(E, W, device=dev) * 0.05, torch.randn(E, device=dev) * 0.1
    t = _time(lambda: ops.moe_route_scored(h, rw_, corr, 2, 4, 2, 2.0), iters=20)
    out["router"] = {"sitidra_ms": round(t * 1e3, 4), "sitidra_roof_frac": _roof(2 * T * E * W, T * W * 2, t)}
    t = _time(lambda: ops.moe_route(h, rw_, corr, 2), iters=20)
    out["router"].update({"mofidra_ms": round(t * 1e3, 4), "mofidra_roof_frac": _roof(2 * T * E * W, T * W * 2, t)})
    return out


def run(sizes=("w2048", "w4096"), kernels=True, families=None) -> dict:
    dev = torch.device("cuda", torch.cuda.current_device())
    ops = get_ops("hip")
    ops.prepare_device(dev)
    result = {"metric": "family_compare", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "sizes": {}}
    with torch.no_grad():
        for name in sizes:
            s = SIZES[name]
            entry = {}
            for label, build in (("mofidra_dense", lambda: MofidraModel(mofidra_config(s, False), ops, dev)),
                                 ("mofidra_moe", lambda: MofidraModel(mofidra_config(s, True), ops, dev)),
                                 ("padadra", lambda: PadadraModel(padadra_config(s), ops, dev)),
                                 ("mabivik", lambda: MabivikModel(mabivik_config(s), ops, dev)),
                                 ("sitidra", lambda: SitidraModel(sitidra_config(s), ops, dev)),
                                 ("decoder", lambda: DecoderModel(decoder_config(s), ops, dev))):
                if families and label.split("_")[0] not in families:
                    continue
                model = build()
                model.init_random(seed=1, std=0.02)
                entry[label] = model_throughput(model)
                del model
                torch.cuda.empty_cache()
            groups = (("mofidra", "kernels", kernel_pairs), ("padadra", "state_kernels", state_kernels),
                      ("mabivik", "latent_kernels", latent_kernels), ("sitidra", "hyper_kernels", hyper_kernels))
            for family, key, fn in groups if kernels else ():
                if not families or family in families:
                    entry[key] = fn(s, dev)
            result["sizes"][name] = entry
    return result


if __name__ == "__main__":
    print(json.dumps(run()))

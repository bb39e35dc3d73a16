"""HIP bindings of the dynamic-tanh norm, latent-attention, selective-state-space and token-input
kernels (csrc/kernels/seqmix_latent.hip).

Same conventions as ``seqmix.py`` / ``seqstate.py``: bf16 or fp32 activations (one template
instance each), fp32 residual stream, norms, angles, decays and step sizes; shapes, dtypes and
contiguity are checked on the host before a launch; launches go to the current stream and never
synchronise with the host.  Semantics: the functions of the same names in ``reference.py``.
"""

import torch

from .seqmix import _act, _check, _p, _req, _stream
from .seqstate import _f32, _i32


def _dyt(norm, W):
    alpha, w, b = norm
    _f32(w, W, "dynamic-tanh weight")
    _f32(b, W, "dynamic-tanh bias")
    return float(alpha), _p(w), _p(b)


def seqlatent_ops(lib):
    def embed_scale_dyt(tokens, table, scale, norm, out_dtype):
        _req(tokens.dtype == torch.int32 and tokens.is_contiguous() and tokens.dim() == 1, "tokens int32 [T]")
        _req(table.dim() == 2 and table.is_contiguous() and table.dtype == out_dtype, "table [V, W] in the activation dtype")
        T, W = tokens.numel(), table.shape[1]
        x = torch.empty(T, W, dtype=torch.float32, device=table.device)
        h = torch.empty(T, W, dtype=out_dtype, device=table.device)
        _check(lib.bcg_embed_scale_dyt(_p(tokens), _p(table), scale, *_dyt(norm, W), _p(x), _p(h), T, W, table.shape[0],
                                       _act(table), _stream()), "embed_scale_dyt")
        return x, h

    def residual_post_norm(x, y, post, pre, out_dtype):
        _req(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "residual fp32 [T, W]")
        T, W = x.shape
        _req(y.shape == (T, W) and y.is_contiguous() and y.dtype in (out_dtype, torch.float32),
             "sublayer output [T, W] in the activation dtype or fp32")
        if post[0] == "dyt":
            kind, (pa, pw, pb), eps = 0, _dyt(post[1:], W), 0.0
        elif post[0] == "rms":
            _f32(post[1], W, "norm weight")
            kind, (pa, pw, pb), eps = 1, (0.0, _p(post[1]), None), float(post[2])
        else:
            raise ValueError(f"unknown post norm {post[0]!r}")
        out, pre_kind, (qa, qw, qb) = None, 0, (0.0, None, None)
        if pre is not None:
            out = torch.empty(T, W, dtype=out_dtype, device=x.device)
            if pre[0] == "copy":
                pre_kind = 1
            else:
                pre_kind, (qa, qw, qb) = 2, _dyt(pre[1:], W)
        _check(lib.bcg_residual_post_norm(_p(x), _p(y), int(y.dtype == torch.float32), kind, pa, pw, pb, eps, pre_kind, qa, qw,
                                          qb, _p(out), T, W, int(out_dtype == torch.float32), _stream()), "residual_post_norm")
        return out

    def rmsnorm_cols(y, off, n, w, eps, out_dtype):
        _req(y.dim() == 2 and y.stride(1) == 1 and 0 <= off and off + n <= y.shape[1] and y.dtype == out_dtype,
             "rmsnorm_cols: rows [T, >= off + n] in the activation dtype, unit column stride")
        _f32(w, n, "norm weight")
        T = y.shape[0]
        out = torch.empty(T, n, dtype=out_dtype, device=y.device)
        _check(lib.bcg_rmsnorm_cols(_p(y), y.stride(0), off, n, _p(w), eps, _p(out), T, _act(y), _stream()), "rmsnorm_cols")
        return out

    def latent_kv_write(y, off, kv_rank, rot_dim, w, eps, positions, slots, inv_freq, amp, k_cache, v_cache):
        T = y.shape[0]
        _req(y.dim() == 2 and y.stride(1) == 1 and 0 <= off and off + kv_rank + rot_dim <= y.shape[1],
             "latent_kv_write: rows [T, >= off + kv_rank + rot_dim], unit column stride")
        _f32(w, kv_rank, "latent norm weight")
        _i32(positions, T, "positions")
        _i32(slots, T, "slots")
        half = inv_freq.numel()
        _f32(inv_freq, half, "inv_freq")
        _req(2 * half <= rot_dim, "rotated width <= rot_dim")
        _req(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
             and k_cache.dtype == y.dtype and v_cache.dtype == y.dtype, "latent cache: contiguous, activation dtype")
        NB, G, BS, KD = k_cache.shape
        _req(G == 1 and KD == kv_rank + rot_dim and v_cache.shape == (NB, 1, kv_rank, BS) and BS % 16 == 0,
             "latent cache: K [NB, 1, BS, kv_rank + rot_dim], V [NB, 1, kv_rank, BS], BS % 16 == 0")
        _check(lib.bcg_latent_kv_write(_p(y), y.stride(0), off, kv_rank, rot_dim, _p(w), eps, _p(positions), _p(slots),
                                       _p(inv_freq), half, float(amp), _p(k_cache), _p(v_cache), T, BS, NB, _act(y), _stream()),
               "latent_kv_write")

    def rope_half_tail(src, src_off, dst, dst_off, positions, inv_freq, amp):
        _req(src.dim() == 3 and dst.dim() == 3 and src.is_contiguous() and dst.is_contiguous() and src.dtype == dst.dtype
             and src.shape[:2] == dst.shape[:2], "rope_half_tail: src [T, H, Ds], dst [T, H, Dd] contiguous")
        T, H, Ds = src.shape
        Dd = dst.shape[2]
        _req(0 <= src_off <= Ds and Ds - src_off == Dd - dst_off, "tails of equal width")
        _i32(positions, T, "positions")
        half = inv_freq.numel()
        _f32(inv_freq, half, "inv_freq")
        _req(2 * half <= Ds - src_off, "rotated width <= tail")
        _check(lib.bcg_rope_half_tail(_p(src), Ds, src_off, _p(dst), Dd, dst_off, _p(positions), _p(inv_freq), half, float(amp),
                                      T, H, _act(src), _stream()), "rope_half_tail")
        return dst

    def head_linear(x3, w, out3=None):
        """Per-head products on the vendor's batched GEMM (fp32 accumulation; true fp32 for fp32 operands)."""
        _req(x3.dim() == 3 and w.dim() == 3 and x3.shape[1] == w.shape[0] and x3.shape[2] == w.shape[2] and x3.stride(2) == 1
             and x3.dtype == w.dtype and w.is_contiguous(), "head_linear: x [T, H, K], w [H, N, K]")
        if out3 is None:
            out3 = torch.empty(x3.shape[0], x3.shape[1], w.shape[1], dtype=x3.dtype, device=x3.device)
        _req(out3.shape == (x3.shape[0], x3.shape[1], w.shape[1]) and out3.stride(2) == 1 and out3.dtype == x3.dtype,
             "head_linear: out [T, H, N]")
        if x3.shape[0]:
            torch.bmm(x3.transpose(0, 1), w.transpose(1, 2), out=out3.transpose(0, 1))
        return out3

    def gate_mul(x, gate, kind, group=1):
        _req(x.dim() == 2 and x.is_contiguous() and group >= 1 and gate.shape == (x.shape[0], x.shape[1] // group)
             and x.shape[1] % group == 0 and gate.stride(1) == 1 and gate.dtype == x.dtype,
             "gate_mul: x [T, n] contiguous, gate [T, n / group] with unit column stride")
        out = torch.empty_like(x)
        _check(lib.bcg_gate_mul(_p(x), _p(gate), gate.stride(0), _p(out), x.shape[0], x.shape[1], {"sigmoid": 0, "silu": 1}[kind],
                                group, _act(x), _stream()), "gate_mul")
        return out

    def gated_act(both):
        _req(both.dim() == 2 and both.is_contiguous() and both.shape[1] % 2 == 0, "gated_act: [rows, 2 n] contiguous")
        out = torch.empty(both.shape[0], both.shape[1] // 2, dtype=both.dtype, device=both.device)
        _check(lib.bcg_gated_act(_p(both), _p(out), both.shape[0], both.shape[1] // 2, _act(both), _stream()), "gated_act")
        return out

    def ssm_prepare(c, off_b, y, off_dt, dt_bias, a_log, heads, groups, state):
        T, n = c.shape[0], groups * state
        _req(c.dim() == 2 and c.stride(1) == 1 and c.shape[1] >= off_b + 2 * n and y.dim() == 2 and y.stride(1) == 1
             and y.shape[0] == T and y.shape[1] >= off_dt + heads and c.dtype == y.dtype, "ssm_prepare: rows B | C and dt")
        _f32(dt_bias, heads, "dt_bias")
        _f32(a_log, heads, "A_log")
        dev = c.device
        q = torch.empty(T, groups, state, dtype=torch.float32, device=dev)
        k = torch.empty(T, groups, state, dtype=torch.float32, device=dev)
        g = torch.empty(T, heads, 1, dtype=torch.float32, device=dev)
        dt = torch.empty(T, heads, dtype=torch.float32, device=dev)
        _check(lib.bcg_ssm_prepare(_p(c), c.stride(0), off_b, _p(y), y.stride(0), off_dt, _p(dt_bias), _p(a_log), _p(q), _p(k),
                                   _p(g), _p(dt), T, heads, n, _act(c), _stream()), "ssm_prepare")
        return q, k, g, dt

    def gated_group_norm(o, skip, skip_w, z, w, parts, eps, out_dtype):
        _req(o.dim() == 3 and o.dtype == torch.float32 and o.is_contiguous(), "o fp32 [T, H, vdim]")
        T, H, vdim = o.shape
        inner = H * vdim
        for t, name in ((skip, "skip"), (z, "gate")):
            _req(t.dim() == 2 and t.shape == (T, inner) and t.stride(1) == 1 and t.dtype == out_dtype,
                 f"{name} [T, H vdim] in the activation dtype, unit column stride")
        _f32(skip_w, H, "skip weight")
        _f32(w, inner, "norm weight")
        _req(parts >= 1 and inner % parts == 0, "the row splits into equal parts")
        out = torch.empty(T, inner, dtype=out_dtype, device=o.device)
        _check(lib.bcg_gated_group_norm(_p(o), _p(skip), skip.stride(0), _p(skip_w), _p(z), z.stride(0), _p(w), eps, _p(out), T, H,
                                        vdim, parts, int(out_dtype == torch.float32), _stream()), "gated_group_norm")
        return out

    def moe_table_route(tokens, table, top):
        _req(tokens.dtype == torch.int32 and tokens.dim() == 1 and table.dtype == torch.int32 and table.dim() == 2
             and 1 <= top <= table.shape[1], "moe_table_route: tokens int32 [T], table int32 [vocab, >= top]")
        idx = table.index_select(0, tokens)[:, :top].contiguous()
        return idx, torch.full(idx.shape, 1.0 / top, dtype=torch.float32, device=idx.device)

    def gelu_gather_mul(z, tokens, table, off):
        _req(z.dim() == 2 and z.is_contiguous() and table.dim() == 2 and table.is_contiguous() and table.dtype == z.dtype
             and 0 <= off and off + z.shape[1] <= table.shape[1], "gelu_gather_mul: z [T, n], table [vocab, >= off + n]")
        _i32(tokens, z.shape[0], "tokens")
        out = torch.empty_like(z)
        _check(lib.bcg_gelu_gather_mul(_p(z), _p(tokens), _p(table), table.stride(0), off, _p(out), z.shape[0], z.shape[1],
                                       table.shape[0], _act(z), _stream()), "gelu_gather_mul")
        return out

    return dict(embed_scale_dyt=embed_scale_dyt, residual_post_norm=residual_post_norm, rmsnorm_cols=rmsnorm_cols,
                latent_kv_write=latent_kv_write, rope_half_tail=rope_half_tail, head_linear=head_linear, gate_mul=gate_mul,
                ssm_prepare=ssm_prepare, gated_group_norm=gated_group_norm, moe_table_route=moe_table_route,
                gelu_gather_mul=gelu_gather_mul, gated_act=gated_act)

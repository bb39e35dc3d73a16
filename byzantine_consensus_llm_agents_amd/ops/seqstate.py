"""HIP bindings of the kernels for mixers with per-sequence state (csrc/kernels/seqmix_state.hip).

Same conventions as ``seqmix.py``: bf16 or fp32 activations (one template instance each), fp32
residual stream, norms, recurrences and state; shapes, dtypes and contiguity are checked on the
host before a launch; launches go to the current stream and never synchronise with the host.
Semantics: the functions of the same names in ``reference.py``.
"""

import ctypes

import torch

from .seqmix import _act, _check, _p, _req, _stream


def _i32(t, n, what):
    _req(t is not None and t.dtype == torch.int32 and t.is_contiguous() and t.numel() == n, f"{what}: int32 [{n}]")


def _f32(t, n, what):
    _req(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n, f"{what}: fp32 [{n}]")


def _segments(meta, T):
    """(B, positions, token_seq, q_start, state_rows) of a packed step, checked."""
    _req(meta.q_start is not None and meta.state_rows is not None and meta.token_seq is not None,
         "the step carries no segment tables (q_start, state_rows, token_seq)")
    B = meta.state_rows.numel()
    _i32(meta.positions, T, "positions")
    _i32(meta.token_seq, T, "token_seq")
    _i32(meta.q_start, B + 1, "q_start")
    _i32(meta.state_rows, B, "state_rows")
    return B


def seqstate_ops(lib):
    def embed_hashed_bigram_norm(tokens, meta, prev, table, scale, bigram, hash_mul, eps, gains, out_dtype):
        T, W = tokens.numel(), table.shape[1]
        _req(tokens.dtype == torch.int32 and tokens.is_contiguous() and tokens.dim() == 1, "tokens int32 [T]")
        _req(table.dim() == 2 and table.is_contiguous() and table.dtype == out_dtype, "table [V, W] in the activation dtype")
        B = _segments(meta, T)
        _req(prev.dtype == torch.int32 and prev.is_contiguous() and prev.dim() == 1, "prev int32 [rows]")
        _req(1 <= len(gains) <= 2, "one or two gains")
        buckets = mp = mc = 0
        if bigram is not None:
            _req(bigram.dim() == 2 and bigram.shape[1] == W and bigram.shape[0] >= 2 and bigram.is_contiguous()
                 and bigram.dtype == out_dtype, "bigram [buckets + 1, W] in the activation dtype")
            buckets, (mp, mc) = bigram.shape[0] - 1, hash_mul
        x = torch.empty(T, W, dtype=torch.float32, device=table.device)
        outs = [torch.empty(T, W, dtype=out_dtype, device=table.device) for _ in gains]
        _check(lib.bcg_embed_hashed_bigram(_p(tokens), _p(meta.positions), _p(meta.token_seq), _p(meta.q_start),
                                           _p(meta.state_rows), _p(prev), prev.numel(), _p(table), scale, _p(bigram), buckets,
                                           int(mp), int(mc), eps, float(gains[0]), float(gains[-1]), _p(x), _p(outs[0]),
                                           _p(outs[1]) if len(outs) > 1 else None, T, B, W, table.shape[0], _act(table),
                                           _stream()), "embed_hashed_bigram")
        return x, tuple(outs)

    def residual_mix_norm(x, normed, normed_scale, plain, mult, eps, gains, out_dtype):
        _req(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "residual fp32 [T, W]")
        T, W = x.shape
        _req(len(normed) <= 2 and len(plain) <= 2 and len(gains) <= 2, "at most two normed parts, two plain parts, two gains")
        ptrs = []
        for a, w in normed:
            _req(a.shape == (T, W) and a.is_contiguous() and a.dtype == out_dtype, "normed part [T, W] in the activation dtype")
            _f32(w, W, "out-norm weight")
            ptrs += [_p(a), _p(w)]
        ptrs += [None] * (4 - len(ptrs))
        for p in plain:
            _req(p.shape == (T, W) and p.is_contiguous() and p.dtype == out_dtype, "plain part [T, W] in the activation dtype")
            ptrs.append(_p(p))
        ptrs += [None] * (6 - len(ptrs))
        outs = [torch.empty(T, W, dtype=out_dtype, device=x.device) for _ in gains]
        _check(lib.bcg_residual_mix_norm(_p(x), *ptrs, normed_scale, mult, eps, float(gains[0]) if gains else 1.0,
                                         float(gains[-1]) if gains else 1.0, _p(outs[0]) if outs else None,
                                         _p(outs[1]) if len(outs) > 1 else None, T, W, int(out_dtype == torch.float32), _stream()),
               "residual_mix_norm")
        return tuple(outs)

    def rmsnorm_scalar(x, eps, gains, out_dtype):
        return residual_mix_norm(x, [], 1.0, [], 0.0, eps, gains, out_dtype)

    def short_conv(y, channels, w, meta, state, act=None, bias=None):
        T = y.shape[0]
        _req(y.dim() == 2 and y.stride(1) == 1 and y.shape[1] >= channels, "short_conv: rows [T, >= channels], unit column stride")
        taps = w.shape[1]
        _req(w.dtype == torch.float32 and w.shape == (channels, taps) and w.is_contiguous() and 1 <= taps <= 16,
             "convolution weights fp32 [channels, taps <= 16]")
        B = _segments(meta, T)
        rows = 0
        if taps > 1:
            _req(state is not None and state.dtype == y.dtype and state.is_contiguous() and state.dim() == 3
                 and state.shape[1:] == (taps - 1, channels), "conv state [rows, taps - 1, channels] in the activation dtype")
            rows = state.shape[0]
        if bias is not None:
            _f32(bias, channels, "convolution bias")
        out = torch.empty(T, channels, dtype=y.dtype, device=y.device)
        code = {None: 0, "silu": 1}[act]
        _check(lib.bcg_short_conv(_p(y), y.stride(0), channels, _p(w), taps, _p(meta.positions), _p(meta.token_seq),
                                  _p(meta.q_start), _p(meta.state_rows), _p(state) if taps > 1 else None, rows, _p(out), code,
                                  _p(bias), T, B, _act(y), _stream()), "short_conv")
        return out

    def rope_pairs_kv_write(qkv, positions, slots, n_q, n_kv, dim, vdim, q_norm, k_norm, eps, inv_freq, v_inv_freq,
                            k_cache, v_cache):
        T = qkv.shape[0]
        qw, kw, vw = n_q * dim, n_kv * dim, n_kv * vdim
        _req(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= qw + kw + vw, "row [q | k | v | ...]")
        _i32(positions, T, "positions")
        _i32(slots, T, "slots")
        half = inv_freq.numel()
        _f32(inv_freq, half, "inv_freq")
        _req(2 * half <= dim and (half == 0 or dim % 2 == 0), "rotated width <= dim")
        if q_norm is not None:
            _f32(q_norm, qw, "q norm weight")
        if k_norm is not None:
            _f32(k_norm, kw, "k norm weight")
        if v_inv_freq is not None:
            _f32(v_inv_freq, vdim // 2, "value inv_freq")
            _req(vdim % 2 == 0, "rotated values: even vdim")
        _req(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
             and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "KV cache: contiguous, activation dtype")
        NB, G, BS, KD = k_cache.shape
        _req(G == n_kv and KD == dim and v_cache.shape == (NB, n_kv, vdim, BS) and BS % 16 == 0,
             "KV cache: K [NB, G, BS, dim], V [NB, G, vdim, BS], BS % 16 == 0")
        q = torch.empty(T, n_q, dim, dtype=qkv.dtype, device=qkv.device)
        _check(lib.bcg_rope_pairs_kv_write(_p(qkv), qkv.stride(0), _p(positions), _p(slots), _p(q_norm), _p(k_norm), eps,
                                           _p(inv_freq), half, _p(v_inv_freq), _p(q), _p(k_cache), _p(v_cache), T, n_q, n_kv, dim,
                                           vdim, BS, NB, _act(qkv), _stream()), "rope_pairs_kv_write")
        return q

    def rotate_pairs(x, positions, inv_freq, sign, heads):
        T = x.shape[0]
        _req(x.dim() == 2 and x.is_contiguous() and x.shape[1] % (2 * heads) == 0, "rotate_pairs: [T, heads * 2n] contiguous")
        width = x.shape[1] // heads
        _i32(positions, T, "positions")
        _f32(inv_freq, width // 2, "inv_freq")
        out = torch.empty_like(x)
        _check(lib.bcg_rotate_pairs(_p(x), _p(positions), _p(inv_freq), sign, _p(out), T, heads, width, _act(x), _stream()),
               "rotate_pairs")
        return out

    def hgrn2_prepare(y, off_q, off_f, heads, dim, f_bias, lower):
        T, n = y.shape[0], heads * dim
        _req(y.dim() == 2 and y.stride(1) == 1 and y.shape[1] >= max(off_q, off_f) + n, "hgrn2_prepare: fused projection rows")
        _f32(f_bias, n, "forget-gate bias")
        _f32(lower, n, "lower bound")
        q, k, g = (torch.empty(T, heads, dim, dtype=torch.float32, device=y.device) for _ in range(3))
        _check(lib.bcg_hgrn2_prepare(_p(y), y.stride(0), off_q, off_f, _p(f_bias), _p(lower), _p(q), _p(k), _p(g), T, n, _act(y),
                                     _stream()), "hgrn2_prepare")
        return q, k, g

    def delta_prepare(c, y, off_beta, a, a_log, dt_bias, heads, kv_heads, dim):
        T = c.shape[0]
        _req(c.dim() == 2 and c.stride(1) == 1 and c.shape[1] >= 2 * kv_heads * dim and y.dim() == 2 and y.stride(1) == 1
             and y.shape[0] == T and y.shape[1] >= off_beta + heads and c.dtype == y.dtype, "delta_prepare: rows q | k and beta")
        _req(a.dim() == 2 and a.shape[0] == T and a.shape[1] in (heads, heads * dim) and a.stride(1) == 1 and a.dtype == c.dtype,
             "decay logits [T, heads dim] or [T, heads], unit column stride")
        gd = a.shape[1] // heads
        _f32(a_log, heads, "A_log")
        _f32(dt_bias, heads * gd, "dt_bias")
        _req(heads % kv_heads == 0 and heads <= 256, "heads % kv_heads, heads <= 256")
        dev = c.device
        q = torch.empty(T, kv_heads, dim, dtype=torch.float32, device=dev)
        k = torch.empty(T, kv_heads, dim, dtype=torch.float32, device=dev)
        g = torch.empty(T, heads, gd, dtype=torch.float32, device=dev)
        beta = torch.empty(T, heads, dtype=torch.float32, device=dev)
        _check(lib.bcg_delta_prepare(_p(c), c.stride(0), _p(y), y.stride(0), off_beta, _p(a), a.stride(0), gd, _p(a_log),
                                     _p(dt_bias), _p(q), _p(k), _p(g), _p(beta), T, heads, kv_heads, dim, _act(c), _stream()),
               "delta_prepare")
        return q, k, g, beta

    def gated_state_scan(q, k, g, v, beta, meta, state, delta, unit_last=False):
        T, H, gd = g.shape
        _req(state.dim() == 4 and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] == H,
             "state fp32 [rows, H, dim, vdim]")
        dim = state.shape[2]
        _req(gd in (1, dim), "g fp32 [T, H, dim] or [T, H, 1]")
        vdim = state.shape[3]
        Gq = q.shape[1]
        for t, name in ((q, "q"), (k, "k")):
            _req(t.dtype == torch.float32 and t.is_contiguous() and t.shape == (T, Gq, dim), f"{name} fp32 [T, Gq, dim]")
        _req(g.dtype == torch.float32 and g.is_contiguous() and H % Gq == 0 and 1 <= dim <= 256, "g fp32 [T, H, dim], dim <= 256")
        v_head = vdim - 1 if unit_last else vdim   # the state's last column then reads ones, not v
        _req(v.dim() == 2 and v.stride(1) == 1 and v.shape == (T, H * v_head), "v [T, H vdim], unit column stride")
        _req(beta is not None or not delta, "the delta rule needs beta")
        _req(not unit_last or (not delta and vdim >= 2), "a unit last column: without the delta rule")
        if beta is not None:
            _req(beta.dtype == torch.float32 and beta.is_contiguous() and beta.shape == (T, H), "beta fp32 [T, H]")
        B = _segments(meta, T)
        out = torch.empty(T, H, vdim, dtype=torch.float32, device=g.device)
        _check(lib.bcg_gated_state_scan(_p(q), _p(k), _p(g), _p(v), v.stride(0), _p(beta), _p(meta.positions),
                                        _p(meta.q_start), _p(meta.state_rows), _p(state), state.shape[0], _p(out), B, H, Gq, dim,
                                        vdim, gd, int(bool(delta)), int(bool(unit_last)), _act(v), _stream()), "gated_state_scan")
        return out

    def head_norm_gate(o, w, eps, gate, out_dtype, gate_act="sigmoid", floor=None):
        _req(o.dim() == 3 and o.dtype == torch.float32 and o.is_contiguous(), "o fp32 [T, H, vdim]")
        T, H, vdim = o.shape
        if floor is not None:   # o's last column is a normaliser
            vdim -= 1
            _req(vdim >= 1 and floor.dtype == torch.float32 and floor.shape == (T, H) and floor.is_contiguous(), "floor fp32 [T, H]")
        _req(w.numel() in (vdim, H * vdim), "head norm weight [vdim] or [H vdim]")
        _f32(w, w.numel(), "head norm weight")
        stride = 0
        if gate is not None:
            _req(gate.dim() == 2 and gate.stride(1) == 1 and gate.shape == (T, H * vdim) and gate.dtype == out_dtype,
                 "gate logits [T, H vdim] in the activation dtype")
            stride = gate.stride(0)
        out = torch.empty(T, H * vdim, dtype=out_dtype, device=o.device)
        _check(lib.bcg_head_norm_gate(_p(o), _p(w), eps, _p(gate), stride, _p(out), T, H, vdim,
                                      {"sigmoid": 0, "silu": 1}[gate_act], _p(floor), vdim if w.numel() != vdim else 0,
                                      int(out_dtype == torch.float32), _stream()),
               "head_norm_gate")
        return out

    return dict(embed_hashed_bigram_norm=embed_hashed_bigram_norm, residual_mix_norm=residual_mix_norm,
                rmsnorm_scalar=rmsnorm_scalar, short_conv=short_conv, rope_pairs_kv_write=rope_pairs_kv_write,
                rotate_pairs=rotate_pairs, hgrn2_prepare=hgrn2_prepare, delta_prepare=delta_prepare,
                gated_state_scan=gated_state_scan, head_norm_gate=head_norm_gate)

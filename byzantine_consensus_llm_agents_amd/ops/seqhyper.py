"""HIP bindings of the hyper-connection stream, unit-norm rotary cache write, exponential-gate and
logit-cap kernels (csrc/kernels/seqmix_hyper.hip).

Same conventions as ``seqmix.py`` / ``seqstate.py``: bf16 or fp32 activations (one template
instance each), fp32 streams, norms, angles and gates; shapes, dtypes and contiguity are checked on
the host before a launch; launches go to the current stream and never synchronise with the host.
Semantics: the functions of the same names in ``reference.py``.
"""

import torch

from .seqmix import _act, _check, _p, _req, _stream
from .seqstate import _f32, _i32, _segments

MAX_STREAMS = 16
MAX_NORM_WIDTH = 12288


def seqhyper_ops(lib):
    def hyper_embed_norm(tokens, table, streams, read_w, norm_w, eps, out_dtype):
        _req(tokens.dtype == torch.int32 and tokens.is_contiguous() and tokens.dim() == 1, "tokens int32 [T]")
        _req(table.dim() == 2 and table.is_contiguous() and table.dtype == out_dtype, "table [V, W] in the activation dtype")
        T, W = tokens.numel(), table.shape[1]
        _req(1 <= streams <= MAX_STREAMS and W <= MAX_NORM_WIDTH, "streams <= 16, width <= 12288")
        _f32(read_w, streams, "stream read weights")
        _f32(norm_w, W, "norm weight")
        X = torch.empty(T, streams, W, dtype=torch.float32, device=table.device)
        h = torch.empty(T, W, dtype=out_dtype, device=table.device)
        _check(lib.bcg_hyper_embed_norm(_p(tokens), _p(table), _p(read_w), _p(norm_w), eps, _p(X), _p(h), T, streams, W,
                                        table.shape[0], _act(table), _stream()), "hyper_embed_norm")
        return X, h

    def hyper_update_norm(X, parts, mix, out_w, read_w, norm_w, eps, out_dtype):
        _req(X.dtype == torch.float32 and X.dim() == 3 and X.is_contiguous(), "streams fp32 [T, S, W]")
        T, S, W = X.shape
        _req(1 <= S <= MAX_STREAMS and W <= MAX_NORM_WIDTH, "streams <= 16, width <= 12288")
        typed = f32 = None
        for p in parts if mix is not None else ():
            _req(p.shape == (T, W) and p.is_contiguous(), "sublayer output [T, W] contiguous")
            if p.dtype == torch.float32 and (out_dtype != torch.float32 or typed is not None) and f32 is None:
                f32 = p
            else:
                _req(typed is None and p.dtype == out_dtype, "sublayer outputs: at most one activation-typed and one fp32")
                typed = p
        if mix is not None:
            _req(mix.dtype == torch.float32 and mix.shape == (S, S) and mix.is_contiguous(), "stream mix fp32 [S, S]")
            _f32(out_w, S, "stream write weights")
        h = None
        if read_w is not None:
            _f32(read_w, S, "stream read weights")
            _f32(norm_w, W, "norm weight")
            h = torch.empty(T, W, dtype=out_dtype, device=X.device)
        _check(lib.bcg_hyper_update_norm(_p(X), _p(typed), _p(f32), _p(mix), _p(out_w) if mix is not None else None,
                                         _p(read_w), _p(norm_w) if read_w is not None else None, eps, _p(h), T, S, W,
                                         int(out_dtype == torch.float32), _stream()), "hyper_update_norm")
        return h

    def rope_norm_kv_write(qkv, positions, slots, n_q, n_kv, dim, vdim, inv_freq, qk_eps, v_first, lam, k_cache, v_cache):
        T = qkv.shape[0]
        qw, kw, vw = n_q * dim, n_kv * dim, n_kv * vdim
        _req(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= qw + kw + vw, "fused projection row [q | k | v | ...]")
        _i32(positions, T, "positions")
        _i32(slots, T, "slots")
        half = inv_freq.numel()
        _f32(inv_freq, half, "inv_freq")
        _req(2 * half <= dim <= 512, "rotated width <= dim <= 512")
        _req(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
             and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "KV cache: contiguous, activation dtype")
        NB, G, BS, KD = k_cache.shape
        _req(G == n_kv and KD == dim and v_cache.shape == (NB, n_kv, vdim, BS) and BS % 16 == 0,
             "KV cache: K [NB, G, BS, dim], V [NB, G, vdim, BS], BS % 16 == 0")
        vf_stride = 0
        if v_first is not None:
            _req(v_first.dim() == 2 and v_first.shape == (T, vw) and v_first.stride(1) == 1 and v_first.dtype == qkv.dtype,
                 "lent values [T, n_kv vdim] in the activation dtype, unit column stride")
            vf_stride = v_first.stride(0)
        q = torch.empty(T, n_q, dim, dtype=qkv.dtype, device=qkv.device)
        _check(lib.bcg_rope_norm_kv_write(_p(qkv), qkv.stride(0), _p(positions), _p(slots), _p(inv_freq), half, float(qk_eps),
                                          _p(v_first), vf_stride, float(lam), _p(q), _p(k_cache), _p(v_cache), T, n_q, n_kv,
                                          dim, vdim, BS, NB, _act(qkv), _stream()), "rope_norm_kv_write")
        return q

    def exp_gate_prepare(y, off_q, off_k, off_i, off_f, i_bias, f_bias, cap, q_scale, heads, dim, meta, m_state):
        T, n = y.shape[0], heads * dim
        _req(y.dim() == 2 and y.stride(1) == 1 and min(off_q, off_k, off_i, off_f) >= 0
             and max(off_q + n, off_k + n, off_i + heads, off_f + heads) <= y.shape[1], "exp_gate_prepare: fused projection rows")
        _f32(i_bias, heads, "input-gate bias")
        _f32(f_bias, heads, "forget-gate bias")
        _req(1 <= heads <= 256 and cap > 0, "heads <= 256, positive gate cap")
        _req(m_state.dtype == torch.float32 and m_state.dim() == 2 and m_state.shape[1] == heads and m_state.is_contiguous(),
             "running maximum fp32 [rows, heads]")
        B = _segments(meta, T)
        dev = y.device
        q = torch.empty(T, heads, dim, dtype=torch.float32, device=dev)
        k = torch.empty(T, heads, dim, dtype=torch.float32, device=dev)
        decay = torch.empty(T, heads, 1, dtype=torch.float32, device=dev)
        write = torch.empty(T, heads, dtype=torch.float32, device=dev)
        floor = torch.empty(T, heads, dtype=torch.float32, device=dev)
        _check(lib.bcg_exp_gate_prepare(_p(y), y.stride(0), off_q, off_k, off_i, off_f, _p(i_bias), _p(f_bias), float(cap),
                                        float(q_scale), _p(meta.positions), _p(meta.q_start), _p(meta.state_rows), _p(m_state),
                                        m_state.shape[0], _p(q), _p(k), _p(decay), _p(write), _p(floor), T, B, heads, dim,
                                        _act(y), _stream()), "exp_gate_prepare")
        return q, k, decay, write, floor

    def softcap(logits, cap):
        _req(logits.dtype == torch.float32 and logits.is_contiguous() and cap > 0, "softcap: contiguous fp32 logits, cap > 0")
        _check(lib.bcg_softcap(_p(logits), logits.numel(), float(cap), _stream()), "softcap")
        return logits

    return dict(hyper_embed_norm=hyper_embed_norm, hyper_update_norm=hyper_update_norm, rope_norm_kv_write=rope_norm_kv_write,
                exp_gate_prepare=exp_gate_prepare, softcap=softcap)

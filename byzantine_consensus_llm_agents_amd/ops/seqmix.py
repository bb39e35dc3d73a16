"""HIP bindings of the fp32-stream mixer kernels (csrc/kernels/seqmix_*.hip).

Activations are bf16 or fp32 (one template instance each; fp32 is the exact mode: true-fp32
MFMAs, fp32 vendor GEMMs); the residual stream, norm weights, router and gate are fp32 always.
Every wrapper checks shapes, dtypes and contiguity on the host before it launches, and launches
on the current stream (graph-capturable: no host synchronisation, scratch from the caching
allocator).  Semantics: the functions of the same names in ``reference.py``.
"""

import ctypes

import torch

c_void_p = ctypes.c_void_p


def _p(t):
    return c_void_p(t.data_ptr()) if t is not None else None


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _req(cond, msg):
    if not cond:
        raise ValueError(msg)


def _check(rc, name):
    if rc != 0:
        raise RuntimeError(f"{name} launch failed (rc={rc})")


def _act(t):
    _req(t.dtype in (torch.bfloat16, torch.float32), "activations: bf16 or fp32")
    return int(t.dtype == torch.float32)


def seqmix_ops(lib, linear):
    split_keys = lib.bcg_multimap_split_keys()
    tile_rows = lib.bcg_moe_tile_rows()

    def embed_scale_rmsnorm(tokens, table, scale, w, eps, w_offset, out_dtype):
        _req(tokens.dtype == torch.int32 and tokens.is_contiguous() and tokens.dim() == 1, "tokens int32 [T]")
        _req(table.dim() == 2 and table.is_contiguous() and table.dtype == out_dtype, "table [V, W] in the activation dtype")
        T, W = tokens.numel(), table.shape[1]
        _req(w.dtype == torch.float32 and w.shape == (W,) and w.is_contiguous(), "norm weight fp32 [W]")
        resid = torch.empty(T, W, dtype=torch.float32, device=table.device)
        out = torch.empty(T, W, dtype=out_dtype, device=table.device)
        _check(lib.bcg_embed_scale_rmsnorm(_p(tokens), _p(table), scale, _p(w), eps, w_offset, _p(resid), _p(out), T, W,
                                           table.shape[0], _act(table), _stream()), "embed_scale_rmsnorm")
        return out, resid

    def residual_add_rmsnorm32(residual, parts, w, eps, w_offset, out_dtype, gate=None, gated=None):
        _req(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(), "residual fp32 [T, W]")
        T, W = residual.shape
        typed, f32 = [], []
        for p in parts:
            _req(p.shape == (T, W) and p.is_contiguous(), "residual part [T, W] contiguous")
            (f32 if p.dtype == torch.float32 and out_dtype != torch.float32 else typed).append(p)
        if out_dtype == torch.float32 and len(typed) > 2:
            f32, typed = typed[2:], typed[:2]
        _req(len(typed) <= 2 and len(f32) <= 1 and all(p.dtype == out_dtype for p in typed)
             and all(p.dtype == torch.float32 for p in f32), "residual parts: <= 2 activation-typed + <= 1 fp32")
        if gated is not None:
            _req(gated.shape == (T, W) and gated.is_contiguous() and gated.dtype == out_dtype and gate is not None
                 and gate.dtype == torch.float32 and gate.numel() == T and gate.is_contiguous(), "gated part / gate")
        out = None
        if w is not None:
            _req(w.dtype == torch.float32 and w.shape == (W,) and w.is_contiguous(), "norm weight fp32 [W]")
            out = torch.empty(T, W, dtype=out_dtype, device=residual.device)
        typed = typed + [None, None]
        _check(lib.bcg_residual_add_rmsnorm32(_p(residual), _p(typed[0]), _p(typed[1]), _p(f32[0]) if f32 else None,
                                              _p(gate) if gated is not None else None, _p(gated), _p(w), eps, w_offset,
                                              _p(out), T, W, int(out_dtype == torch.float32), _stream()),
               "residual_add_rmsnorm32")
        return out

    def rmsnorm32(x, w, eps, w_offset, out_dtype):
        return residual_add_rmsnorm32(x, [], w, eps, w_offset, out_dtype)

    def act_fn(x, kind):
        _req(x.dim() == 2 and x.stride(1) == 1, "act_fn: [rows, n] with unit column stride")
        rows, n = x.shape
        out = torch.empty(rows, n, dtype=x.dtype, device=x.device)
        code = {"gelu_tanh": 0, "relu2": 1, "silu": 2}[kind]
        _check(lib.bcg_act_fn(_p(x), _p(out), rows, n, x.stride(0), code, _act(x), _stream()), "act_fn")
        return out

    def _cache_ok(k_cache, v_cache, n_kv, kd, vdim, dtype):
        _req(k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous()
             and k_cache.dtype == dtype and v_cache.dtype == dtype, "KV cache: contiguous, activation dtype")
        NB, G, BS, KD = k_cache.shape
        _req(G == n_kv and KD == kd and v_cache.shape == (NB, n_kv, vdim, BS) and BS % 16 == 0,
             "KV cache: K [NB, G, BS, maps dim], V [NB, G, vdim, BS], BS % 16 == 0")
        return NB, BS

    def kv_from_logical(k, v):
        """The cache tensors the kernels read, from logical K [NB, G, BS, KD] / V [NB, G, vdim, BS]
        (tests, tools): with KD % 4 == 0 every (page, head) slab is stored fragment-major, K as
        [KD / 4][BS][4] and V as [BS / 4][vdim][4]; the shapes stay the logical ones."""
        NB, G, BS, KD = k.shape
        if KD % 4:
            return k.contiguous(), v.contiguous()
        vd = v.shape[2]
        kp = k.reshape(NB, G, BS, KD // 4, 4).permute(0, 1, 3, 2, 4).contiguous().view(NB, G, BS, KD)
        vp = v.reshape(NB, G, vd, BS // 4, 4).permute(0, 1, 3, 2, 4).contiguous().view(NB, G, vd, BS)
        return kp, vp

    def kv_to_logical(k, v):
        """Inverse of `kv_from_logical`."""
        NB, G, BS, KD = k.shape
        if KD % 4:
            return k, v
        vd = v.shape[2]
        kl = k.reshape(NB, G, KD // 4, BS, 4).permute(0, 1, 3, 2, 4).contiguous().view(NB, G, BS, KD)
        vl = v.reshape(NB, G, BS // 4, vd, 4).permute(0, 1, 3, 2, 4).contiguous().view(NB, G, vd, BS)
        return kl, vl

    def rope_multi_kv_write(qkv, positions, slots, n_q, n_kv, maps, dim, vdim, inv_freq, k_cache, v_cache):
        T = qkv.shape[0]
        qw, kw, vw = n_q * maps * dim, n_kv * maps * dim, n_kv * vdim
        _req(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= qw + kw + vw, "fused projection row [q | k | v | ...]")
        _req(positions.dtype == torch.int32 and slots.dtype == torch.int32 and positions.numel() == T
             and slots.numel() == T and positions.is_contiguous() and slots.is_contiguous(), "positions / slots int32 [T]")
        half = inv_freq.numel()
        _req(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous() and 2 * half <= dim, "inv_freq fp32 [rot/2]")
        NB, BS = _cache_ok(k_cache, v_cache, n_kv, maps * dim, vdim, qkv.dtype)
        q = torch.empty(T, n_q, maps * dim, dtype=qkv.dtype, device=qkv.device)
        _check(lib.bcg_rope_multi_kv_write(_p(qkv), qkv.stride(0), _p(positions), _p(slots), _p(inv_freq), half, _p(q),
                                           _p(k_cache), _p(v_cache), T, n_q, n_kv, maps, dim, vdim, BS, NB, _act(qkv),
                                           _stream()), "rope_multi_kv_write")
        return q

    def multimap_tile_rows(dim, vdim):
        """Query rows per prefill tile (the tile table the engine builds) for these head sizes."""
        return 64  # four waves x 16 rows

    def multimap_attention(q, k_cache, v_cache, meta, scale, maps, lam, head_eps, out_scale, vdim, window=0, sink=None,
                           chunk=0):
        """Prefill tiles (``meta.tiles``) on the MFMA kernel, one-token rows (``meta.single``, or
        every row of a decode step) on the split-KV kernel.  ``window`` / ``chunk`` / ``sink``
        (one-map heads): sliding window in keys, or a chunk mask (a query sees the keys of its own
        ``chunk``-aligned block of positions only); fp32 [H] sink logits of the softmax denominator."""
        T, H, qd = q.shape
        _req(q.is_contiguous() and qd % maps == 0, "q [T, H, maps dim] contiguous")
        dim = qd // maps
        G = k_cache.shape[1]
        NB, BS = _cache_ok(k_cache, v_cache, G, qd, vdim, q.dtype)
        _req(H % G == 0 and maps in (1, 2) and dim <= (512 if maps == 1 else 128) and vdim <= 256,
             "multimap attention: maps <= 2, dim <= 128 (one map: 512), vdim <= 256")
        bt = meta.block_tables
        lens = meta.seq_lens if meta.attn_seq_lens is None else meta.attn_seq_lens
        _req(bt.dtype == torch.int32 and bt.dim() == 2 and bt.is_contiguous() and lens.dtype == torch.int32
             and lens.is_contiguous() and lens.numel() == bt.shape[0], "block tables int32 [B, max_blocks], lens int32 [B]")
        out = torch.empty(T, H * vdim, dtype=q.dtype, device=q.device)
        f32 = _act(q)
        tile_rows = meta.tile_rows if not meta.decode else 64
        _req(tile_rows == 64, "prefill tiles: 64 query rows")
        window, chunk = int(window or 0), int(chunk or 0)
        _req(window >= 0 and chunk >= 0 and not (window and chunk)
             and (maps == 1 or (window == 0 and chunk == 0 and sink is None)), "window / chunk / sink: one-map heads, one mask")
        if sink is not None:
            _req(sink.dtype == torch.float32 and sink.numel() == H and sink.is_contiguous(), "sink fp32 [H]")
        common = (H, G, maps, dim, vdim, BS, NB, scale, lam, head_eps, out_scale, tile_rows, f32, window, chunk, _p(sink), _stream())

        def decode(work, n_items):
            n_splits = max(1, (bt.shape[1] * BS + split_keys - 1) // split_keys)
            if window or chunk:  # splits are counted from the window's (chunk's) first: it touches this many at most
                n_splits = min(n_splits, (max(window, chunk) + split_keys - 1) // split_keys + 1)
            ws = torch.empty(n_items * H * n_splits * (2 * maps + maps * vdim), dtype=torch.float32, device=q.device)
            _check(lib.bcg_multimap_attention(1, _p(q), _p(k_cache), _p(v_cache), _p(bt), bt.shape[1], None, _p(lens),
                                              _p(work), n_items, _p(out), _p(ws), n_splits, *common), "multimap decode")

        if meta.decode:
            _req(T == bt.shape[0], "decode step: one row per sequence")
            decode(None, T)
            return out
        tiles, single = meta.tiles, meta.single
        _req(tiles is not None and tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 3
             and tiles.is_contiguous() and meta.q_start.dtype == torch.int32, "prefill tiles int32 [n, 3]")
        if tiles.shape[0]:
            _check(lib.bcg_multimap_attention(0, _p(q), _p(k_cache), _p(v_cache), _p(bt), bt.shape[1], _p(meta.q_start),
                                              _p(lens), _p(tiles), tiles.shape[0], _p(out), None, 0, *common),
                   "multimap prefill")
        if single is not None and single.shape[0]:
            _req(single.dtype == torch.int32 and single.dim() == 2 and single.shape[1] == 2 and single.is_contiguous(),
                 "single rows int32 [n, 2]")
            decode(single, single.shape[0])
        return out

    def moe_route(h, router_w, router_b, top, gate_w=None):
        T, W = h.shape
        E = router_w.shape[0]
        _req(h.is_contiguous() and router_w.dtype == torch.float32 and router_w.shape == (E, W) and router_w.is_contiguous()
             and (router_b is None or (router_b.dtype == torch.float32 and router_b.numel() == E))
             and 1 <= top <= E <= 256, "moe_route: fp32 router [E, W], E <= 256")
        idx = torch.empty(T, top, dtype=torch.int32, device=h.device)
        wts = torch.empty(T, top, dtype=torch.float32, device=h.device)
        gate = None
        if gate_w is not None:
            _req(gate_w.dtype == torch.float32 and gate_w.numel() == W and gate_w.is_contiguous(), "gate fp32 [W]")
            gate = torch.empty(T, dtype=torch.float32, device=h.device)
        _check(lib.bcg_moe_route(_p(h), _p(router_w), _p(router_b), _p(gate_w), _p(idx), _p(wts), _p(gate), T, W, E, top,
                                 _act(h), _stream()), "moe_route")
        return idx, wts, gate

    def moe_route_scored(h, router_w, corr, top, groups, keep, scale):
        T, W = h.shape
        E = router_w.shape[0]
        _req(h.is_contiguous() and router_w.dtype == torch.float32 and router_w.shape == (E, W) and router_w.is_contiguous()
             and (corr is None or (corr.dtype == torch.float32 and corr.numel() == E and corr.is_contiguous()))
             and 1 <= top <= E <= 256, "moe_route_scored: fp32 router [E, W], fp32 correction [E], E <= 256")
        _req(groups >= 1 and E % groups == 0 and 1 <= keep <= groups and top <= keep * (E // groups),
             "moe_route_scored: equal groups, `top` experts inside the kept groups")
        idx = torch.empty(T, top, dtype=torch.int32, device=h.device)
        wts = torch.empty(T, top, dtype=torch.float32, device=h.device)
        _check(lib.bcg_moe_route_scored(_p(h), _p(router_w), _p(corr), _p(idx), _p(wts), T, W, E, top, groups, keep,
                                        float(scale), _act(h), _stream()), "moe_route_scored")
        return idx, wts

    def moe_pair_rows(gate, up):
        """The [2 ff, W] weight of one gated expert as `moe_experts` (kind "silu_gated") reads it:
        gate and up rows in alternating groups of 16 when ff is a multiple of 16 (the product's
        epilogue then forms silu(gate) * up), else [gate; up]."""
        ff, W = gate.shape
        if ff % 16:
            return torch.cat([gate, up])
        return torch.stack([gate.reshape(ff // 16, 16, W), up.reshape(ff // 16, 16, W)], 1).reshape(2 * ff, W)

    def moe_experts(h, up, down, idx, weights, kind="relu2"):
        T, W = h.shape
        E, n_up, _ = up.shape
        top = idx.shape[1]
        _req(kind in ("relu2", "silu_gated"), "moe_experts: relu2 or silu-gated experts")
        gated = kind == "silu_gated"
        _req(not gated or n_up % 2 == 0, "gated experts: [gate; up] rows")
        ff = n_up // 2 if gated else n_up
        _req(h.is_contiguous() and up.shape == (E, n_up, W) and down.shape == (E, W, ff) and up.is_contiguous()
             and down.is_contiguous() and up.dtype == h.dtype and down.dtype == h.dtype, "expert weights [E, ff, W] / [E, W, ff]")
        _req(idx.dtype == torch.int32 and idx.shape == (T, top) and idx.is_contiguous() and weights.dtype == torch.float32
             and weights.shape == (T, top) and weights.is_contiguous(), "routing tables [T, top]")
        n_slots = T * top
        n_tiles = (n_slots + E * (tile_rows - 1) + tile_rows - 1) // tile_rows
        cap = n_tiles * tile_rows
        dev, f32 = h.device, _act(h)
        sorted_ = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_e = torch.empty(n_tiles, dtype=torch.int32, device=dev)
        _check(lib.bcg_moe_align(_p(idx), n_slots, E, _p(sorted_), cap, _p(tile_e), n_tiles, _stream()), "moe_align")
        if gated and ff % 16 == 0:   # rows paired by `moe_pair_rows`: silu(gate) * up in the product's epilogue
            hidden = torch.empty(cap, ff, dtype=h.dtype, device=dev)
            _check(lib.bcg_moe_gemm(_p(h), W, _p(up), _p(hidden), ff, _p(sorted_), _p(tile_e), n_tiles, n_up, W, top, 1, 0, 2,
                                    f32, _stream()), "moe gate / up")
        elif gated:   # the stacked projection, then silu(gate) * up over its halves
            both = torch.empty(cap, n_up, dtype=h.dtype, device=dev)
            _check(lib.bcg_moe_gemm(_p(h), W, _p(up), _p(both), n_up, _p(sorted_), _p(tile_e), n_tiles, n_up, W, top, 1, 0, 0,
                                    f32, _stream()), "moe gate / up")
            hidden = torch.empty(cap, ff, dtype=h.dtype, device=dev)
            _check(lib.bcg_gated_act(_p(both), _p(hidden), cap, ff, f32, _stream()), "gated_act")
        else:
            hidden = torch.empty(cap, ff, dtype=h.dtype, device=dev)
            _check(lib.bcg_moe_gemm(_p(h), W, _p(up), _p(hidden), ff, _p(sorted_), _p(tile_e), n_tiles, ff, W, top, 1, 0, 1,
                                    f32, _stream()), "moe up")
        y = torch.empty(n_slots, W, dtype=h.dtype, device=dev)
        _check(lib.bcg_moe_gemm(_p(hidden), ff, _p(down), _p(y), W, _p(sorted_), _p(tile_e), n_tiles, W, ff, top, 0, 1, 0,
                                f32, _stream()), "moe down")
        out = torch.empty(T, W, dtype=torch.float32, device=dev)
        _check(lib.bcg_moe_combine(_p(y), _p(weights), _p(out), T, W, top, f32, _stream()), "moe_combine")
        return out

    return dict(embed_scale_rmsnorm=embed_scale_rmsnorm, residual_add_rmsnorm32=residual_add_rmsnorm32,
                rmsnorm32=rmsnorm32, act_fn=act_fn, rope_multi_kv_write=rope_multi_kv_write,
                kv_from_logical=kv_from_logical, kv_to_logical=kv_to_logical,
                multimap_attention=multimap_attention, multimap_tile_rows=multimap_tile_rows, moe_route=moe_route, moe_experts=moe_experts,
                moe_pair_rows=moe_pair_rows, moe_route_scored=moe_route_scored)

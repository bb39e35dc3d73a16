"""PyTorch reference implementations of every engine op (fp32 math).

These define the semantics the HIP kernels in ``csrc/kernels`` must match and
run the ``torch`` backend (CPU tests).  Layout conventions shared with the
kernels:

* KV cache: ``k_cache : [L, num_blocks, n_kv, block_size, head_dim]`` and
  ``v_cache : [L, num_blocks, n_kv, head_dim, block_size]`` (V stored
  transposed per block-head: it is the A operand of ``O^T = V^T P^T`` in the
  MFMA attention kernels); bf16; block 0 is a never-allocated scratch block.
* ``block_tables : [B, max_blocks] int32``; ``seq_lens : [B] int32`` = number
  of tokens whose KV is resident *including* the tokens of this step.
* Sampling: Gumbel-max with a counter-based hash (``gumbel_hash``) so the
  HIP kernel and this reference pick identical tokens from identical logits.
"""

import math
from typing import Optional, Tuple

import torch

MASK32 = 0xFFFFFFFF


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(x.dtype)


def add_rmsnorm(x: torch.Tensor, residual: Optional[torch.Tensor], w: torch.Tensor,
                eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """``residual <- residual + x`` (in place, or x itself if None); returns (norm(residual), residual)."""
    if residual is None:
        residual = x.clone()
    else:
        residual.copy_((residual.float() + x.float()).to(residual.dtype))
    return rmsnorm(residual, w, eps), residual


def embed_rmsnorm(tokens: torch.Tensor, table: torch.Tensor, w: torch.Tensor,
                  eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Embedding gather fused with the first RMSNorm: (rmsnorm(E[tokens]) * w, E[tokens])."""
    residual = table.index_select(0, tokens.long())
    return rmsnorm(residual, w, eps), residual


def rope_cache(max_pos: int, head_dim: int, theta: float, device=None) -> torch.Tensor:
    """[max_pos, head_dim] fp32: first half cos, second half sin (neox layout)."""
    half = head_dim // 2
    inv = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float64) * 2 / head_dim))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.cat([ang.cos(), ang.sin()], dim=-1).float().to(device)


def _rope(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    half = x.shape[-1] // 2
    cos, sin = cs[..., :half], cs[..., half:]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


def qk_norm_rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                          n_q: int, n_kv: int, head_dim: int, q_norm: Optional[torch.Tensor],
                          k_norm: Optional[torch.Tensor], eps: float, cos_sin: torch.Tensor,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, layer: int,
                          contiguous: bool = True) -> torch.Tensor:
    """Split fused QKV, (Qwen3) RMSNorm q/k per head, neox RoPE, scatter K/V into the paged cache.

    Returns q as ``[T, n_q, head_dim]`` (activation dtype).
    """
    T = qkv.shape[0]
    q = qkv[:, : n_q * head_dim].float().view(T, n_q, head_dim)
    k = qkv[:, n_q * head_dim:(n_q + n_kv) * head_dim].float().view(T, n_kv, head_dim)
    v = qkv[:, (n_q + n_kv) * head_dim:].view(T, n_kv, head_dim)
    if q_norm is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm.float()
    cs = cos_sin[positions.long()][:, None, :]
    q = _rope(q, cs)
    k = _rope(k, cs)
    bs = k_cache.shape[3]
    blk = (slots // bs).long()
    off = (slots % bs).long()
    if k_cache.dtype == torch.float8_e4m3fn:  # fp8 KV cache: saturate (e4m3fn has no inf)
        k, v = k.clamp(-448.0, 448.0), v.float().clamp(-448.0, 448.0)
    k_cache[layer, blk, :, off] = k.to(k_cache.dtype)
    v_cache[layer, blk, :, :, off] = v.to(v_cache.dtype)
    return q.to(qkv.dtype)


def _gather_kv(cache, layer, table_row, ctx, transposed=False):
    blocks = cache[layer]
    if transposed:                                        # V: [NB, n_kv, hd, bs]
        blocks = blocks.transpose(2, 3)
    bs = blocks.shape[2]
    nblk = (ctx + bs - 1) // bs
    sel = blocks[table_row[:nblk].long()]                  # [nblk, n_kv, bs, hd]
    return sel.permute(1, 0, 2, 3).reshape(sel.shape[1], nblk * bs, sel.shape[3])[:, :ctx]


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, layer: int,
                    block_tables: torch.Tensor, q_start: torch.Tensor, seq_lens: torch.Tensor,
                    scale: float) -> torch.Tensor:
    """Causal GQA attention of packed queries over paged KV.

    ``q : [T, n_q, hd]``; sequence b owns query rows ``q_start[b]:q_start[b+1]``
    which are its LAST rows, i.e. positions ``seq_lens[b]-q_len .. seq_lens[b]-1``.
    Returns ``[T, n_q*hd]``.
    """
    T, n_q, hd = q.shape
    n_kv = k_cache.shape[2]
    group = n_q // n_kv
    out = torch.zeros(T, n_q, hd, dtype=torch.float32, device=q.device)
    for b in range(block_tables.shape[0]):
        s, e = int(q_start[b]), int(q_start[b + 1])
        if e <= s:
            continue
        ctx = int(seq_lens[b])
        k = _gather_kv(k_cache, layer, block_tables[b], ctx).float()   # [n_kv, ctx, hd]
        v = _gather_kv(v_cache, layer, block_tables[b], ctx, transposed=True).float()
        k = k.repeat_interleave(group, 0)
        v = v.repeat_interleave(group, 0)
        qb = q[s:e].float().permute(1, 0, 2)                            # [n_q, qlen, hd]
        scores = torch.matmul(qb, k.transpose(1, 2)) * scale            # [n_q, qlen, ctx]
        qpos = torch.arange(ctx - (e - s), ctx, device=q.device)[:, None]
        kpos = torch.arange(ctx, device=q.device)[None, :]
        scores = scores.masked_fill(kpos > qpos, float("-inf"))
        out[s:e] = torch.matmul(torch.softmax(scores, -1), v).permute(1, 0, 2)
    return out.reshape(T, n_q * hd).to(q.dtype)


def _partial(q, k, v, scale):
    """(O unnormalised, m, l) of q [n_q, hd] over k, v [n_q, n, hd] -- one flash-decoding split."""
    s = torch.einsum("hd,hnd->hn", q, k) * scale
    m = s.max(-1).values
    p = torch.exp(s - m[:, None])
    return torch.einsum("hn,hnd->hd", p, v), m, p.sum(-1)


def paged_attention_decode_cascade(q, k_cache, v_cache, layer, block_tables, seq_lens, scale, cascade):
    """Decode attention the way the HIP cascade computes it, from its tables (fp32).

    A grouped row's tokens [0, kv_begin) come from its group's FIRST member's block table
    (``decode_shared_kernel``, in pieces -- merged here as one); [kv_begin, ctx) from its own
    (``decode_attn_kernel``); the partials merge as flash-decoding splits do.  Equal to
    `paged_attention` exactly when the tables are consistent (every member holds the group's
    block ids) -- what the CPU tests of ``engine/cascade.py`` check.  ``cascade``: CascadeTables (any device)."""
    B, n_q, hd = q.shape
    n_kv = k_cache.shape[2]
    group = n_q // n_kv
    kv_begin = cascade.kv_begin.cpu().tolist()
    lead_of = {}
    desc = cascade.grp_desc.cpu().tolist()
    rows = cascade.grp_rows.cpu().tolist()
    items = cascade.items.cpu().tolist()[:int(cascade.n_items[0])]
    for g, _, _, _ in items:
        first, n, shared = desc[g][:3]
        for m in rows[first:first + n]:
            lead_of[m] = (rows[first], shared * k_cache.shape[3])
    out = torch.zeros(B, n_q, hd, dtype=torch.float32)
    for b in range(B):
        ctx = int(seq_lens[b])
        qb = q[b].float().cpu()
        parts = []
        begin = kv_begin[b]
        if begin:
            lead, shared = lead_of[b]
            assert shared == begin, "kv_begin disagrees with the group table"
            k = _gather_kv(k_cache, layer, block_tables[lead], shared).float().cpu().repeat_interleave(group, 0)
            v = _gather_kv(v_cache, layer, block_tables[lead], shared, True).float().cpu().repeat_interleave(group, 0)
            parts.append(_partial(qb, k, v, scale))
        k = _gather_kv(k_cache, layer, block_tables[b], ctx).float().cpu()[:, begin:].repeat_interleave(group, 0)
        v = _gather_kv(v_cache, layer, block_tables[b], ctx, True).float().cpu()[:, begin:].repeat_interleave(group, 0)
        parts.append(_partial(qb, k, v, scale))
        m = torch.stack([p[1] for p in parts]).max(0).values
        o = sum(p[0] * torch.exp(p[1] - m)[:, None] for p in parts)
        l_sum = sum(p[2] * torch.exp(p[1] - m) for p in parts)
        out[b] = o / l_sum[:, None]
    return out.reshape(B, n_q * hd).to(q.dtype)


def linear_silu(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) with W = [gate; up]: the fused gate_up GEMM epilogue (fp32 math)."""
    gu = x.float() @ w.float().t()
    inter = gu.shape[-1] // 2
    return (torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]).to(x.dtype)


def linear_residual(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
    """residual <- residual + x W^T, rounded once (the fused o/down GEMM epilogue); in place."""
    residual.copy_((residual.float() + x.float() @ w.float().t()).to(residual.dtype))
    return residual


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    inter = gu.shape[-1] // 2
    g, u = gu[..., :inter].float(), gu[..., inter:].float()
    return (g * torch.sigmoid(g) * u).to(gu.dtype)


# ------------------------------------------------------------------ sampling
def _fmix32(h: torch.Tensor) -> torch.Tensor:
    h = h & MASK32
    h = h ^ (h >> 16)
    h = (h * 0x85EBCA6B) & MASK32
    h = h ^ (h >> 13)
    h = (h * 0xC2B2AE35) & MASK32
    return h ^ (h >> 16)


def gumbel_hash(seed: int, row_key: torch.Tensor, step: int, tokens: torch.Tensor) -> torch.Tensor:
    """Uniform (0,1) from (seed, row key, step, token) -- same bits as sample.hip."""
    a = _fmix32((row_key.long() * 0x9E3779B9 + step * 0x632BE5AB + seed) & MASK32)
    h = _fmix32(a[:, None] ^ ((tokens.long()[None, :] * 0x27D4EB2F) & MASK32))
    return ((h >> 8).double() + 0.5) / 16777216.0


def sample_step(logits: torch.Tensor, fsm_next: torch.Tensor, fsm_dist: torch.Tensor,
                fsm_base: torch.Tensor, fsm_state: torch.Tensor, gen_count: torch.Tensor,
                max_new: torch.Tensor, temperature: torch.Tensor, row_keys: torch.Tensor,
                done: torch.Tensor, seq_lens: torch.Tensor, out_tokens: torch.Tensor,
                next_tokens: torch.Tensor, seed: int, budget_aware: bool, n_text_tokens: int,
                eos_id: int, eos_id2: int) -> None:
    """One guided sampling step for every row, updating all per-row state in place.

    Row b is guided when ``fsm_base[b] >= 0`` (allowed tokens: those with
    ``fsm_next[base+state, t] >= 0``; in budget mode additionally
    ``fsm_dist[base+next] <= remaining-1`` whenever some token satisfies it);
    otherwise every text token and the EOS ids are allowed.  The sampled token
    goes to ``out_tokens[b, gen_count[b]]`` and ``next_tokens[b]``;
    ``gen_count`` and ``seq_lens`` advance.  Rows already ``done`` are untouched.
    """
    B, V = logits.shape
    tok_ids = torch.arange(V, device=logits.device)
    for b in range(B):
        if bool(done[b]):
            continue
        base = int(fsm_base[b])
        step = int(gen_count[b])
        rem = int(max_new[b]) - step
        lg = logits[b].float()
        if base >= 0:
            row = base + int(fsm_state[b])
            nxt = fsm_next[row, :V].long()
            ok = nxt >= 0
            if budget_aware:
                dist_next = torch.where(ok, fsm_dist[(base + nxt.clamp(min=0))].long(),
                                        torch.full_like(nxt, 1 << 20))
                tight = ok & (dist_next <= rem - 1)
                if bool(tight.any()):
                    ok = tight
        else:
            ok = (tok_ids < n_text_tokens) | (tok_ids == eos_id) | (tok_ids == eos_id2)
        if not bool(ok.any()):
            done[b] = 1
            continue
        t = float(temperature[b])
        if t <= 0:
            score = lg.double()
        else:
            u = gumbel_hash(seed, row_keys[b:b + 1], step, tok_ids)[0]
            score = lg.double() / t - torch.log(-torch.log(u))
        score = torch.where(ok, score, torch.full_like(score, -math.inf))
        tok = int(torch.argmax(score))
        out_tokens[b, step] = tok
        next_tokens[b] = tok
        gen_count[b] = step + 1
        seq_lens[b] += 1
        finished = rem - 1 <= 0
        if base >= 0:
            ns = int(fsm_next[base + int(fsm_state[b]), tok])
            fsm_state[b] = ns
            finished = finished or int(fsm_dist[base + ns]) == 0
        else:
            finished = finished or tok in (eos_id, eos_id2)
        if finished:
            done[b] = 1


# ------------------------------------------------------------------ fp8 (OCP e4m3fn)
FP8_MAX = 448.0
FP8 = torch.float8_e4m3fn


def quant_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-wise dynamic quantisation: scale = max|x_row| / 448, q = x / scale (fp8 e4m3fn)."""
    xf = x.float()
    scale = xf.abs().amax(dim=-1).clamp(min=1e-12) / FP8_MAX
    q = (xf / scale[:, None]).clamp(-FP8_MAX, FP8_MAX).to(FP8)
    return q, scale


def add_rmsnorm_fp8(x, residual, w, eps):
    """add_rmsnorm (bf16-rounded output, as the bf16 path) then row-wise fp8 quantisation."""
    y, residual = add_rmsnorm(x, residual, w, eps)
    q, s = quant_fp8(y)
    return q, s, residual


def rmsnorm_fp8(x, w, eps):
    """Plain RMSNorm (bf16-rounded, as the bf16 path) then row-wise fp8 quantisation."""
    return quant_fp8(rmsnorm(x, w, eps))


def embed_rmsnorm_fp8(tokens, table, w, eps):
    """(fp8(rmsnorm(table[tokens]) * w), row scales, table[tokens])."""
    y, residual = embed_rmsnorm(tokens, table, w, eps)
    q, s = quant_fp8(y)
    return q, s, residual


def linear_fp8_residual(xq, xs, wq, ws, residual):
    """residual <- residual + dequant(xq . wq^T), rounded once (the fused fp8 epilogue); in place."""
    y = (xq.float() * xs[:, None]) @ (wq.float() * ws[:, None]).t()
    residual.copy_((residual.float() + y).to(residual.dtype))
    return residual


def silu_mul_fp8(gu):
    return quant_fp8(silu_mul(gu))


def quantize_weight_fp8(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-output-channel weight quantisation: w [N, K] -> (fp8 [N, K], scale fp32 [N])."""
    return quant_fp8(w)


def linear_fp8(xq, xs, wq, ws, bias=None, out_dtype=torch.bfloat16):
    """y = (xq * xs[:, None]) @ (wq * ws[:, None])^T (+ bias), fp32 accumulate."""
    y = (xq.float() * xs[:, None]) @ (wq.float() * ws[:, None]).t()
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype)


# ------------------------------------------------------------------ fp32 residual stream, multi-map attention, MoE
# Mechanisms of the parallel-sublayer / differential-attention / mixture-of-experts decoders
# (models/mofidra.py).  Conventions shared with csrc/kernels/seqmix_*.hip:
#
# * the residual stream is fp32 whatever the activation dtype; norms, router, softmax, the
#   map combination and the per-head unit norm are fp32;
# * per layer run the KV cache is ``k : [num_blocks, n_kv, block_size, maps * dim]`` and
#   ``v : [num_blocks, n_kv, vdim, block_size]`` (V transposed per block-head, as above);
# * a q / k head is laid out map after map: ``[map 0 (dim), map 1 (dim), ...]``.

def rope_inv_freq(rot_dims: int, base: float, device=None) -> torch.Tensor:
    """fp32 ``base^(-2i/rot_dims)``, i < rot_dims/2 (empty for rot_dims = 0)."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / max(rot_dims, 1))).float().to(device)


def rmsnorm32(x: torch.Tensor, w: torch.Tensor, eps: float, w_offset: float, out_dtype) -> torch.Tensor:
    """fp32 ``x / sqrt(mean(x^2) + eps) * (w_offset + w)``, rounded once to ``out_dtype``."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * (w_offset + w.float())).to(out_dtype)


def embed_scale_rmsnorm(tokens, table, scale: float, w, eps: float, w_offset: float, out_dtype):
    """(norm(scale * E[tokens]) in ``out_dtype``, scale * E[tokens] in fp32)."""
    residual = table.index_select(0, tokens.long()).float() * scale
    return rmsnorm32(residual, w, eps, w_offset, out_dtype), residual


def residual_add_rmsnorm32(residual, parts, w, eps: float, w_offset: float, out_dtype, gate=None, gated=None):
    """``residual += sum(parts) [+ sigmoid(gate) * gated]`` in fp32, in place (the sublayer
    outputs are summed first, then added); returns the norm of the new residual
    (None when ``w`` is None).  ``gate`` : fp32 [T] logits, ``gated`` : [T, W]."""
    total = None
    for p in parts:
        total = p.float() if total is None else total + p.float()
    if gated is not None:
        g = torch.sigmoid(gate.float())[:, None] * gated.float()
        total = g if total is None else total + g
    if total is not None:
        residual.add_(total)
    return None if w is None else rmsnorm32(residual, w, eps, w_offset, out_dtype)


def rope_multi_kv_write(qkv, positions, slots, n_q: int, n_kv: int, maps: int, dim: int, vdim: int,
                        inv_freq, k_cache, v_cache):
    """Split a fused projection row ``[q | k | v | anything]``, rotate the first
    ``2 * len(inv_freq)`` features of every map of every q / k head (feature i pairs with
    i + rot/2; angle = position * inv_freq[i], fp32), scatter K / V into the paged cache of
    this layer run.  Returns q ``[T, n_q, maps * dim]`` in the activation dtype."""
    T = qkv.shape[0]
    qw, kw = n_q * maps * dim, n_kv * maps * dim
    q = qkv[:, :qw].float().reshape(T, n_q, maps, dim)
    k = qkv[:, qw:qw + kw].float().reshape(T, n_kv, maps, dim)
    v = qkv[:, qw + kw:qw + kw + n_kv * vdim].reshape(T, n_kv, vdim)
    half = inv_freq.numel()
    if half:
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        cos, sin = ang.cos()[:, None, None, :], ang.sin()[:, None, None, :]

        def rot(x):
            a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
            return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)
        q, k = rot(q), rot(k)
    bs = k_cache.shape[2]
    blk, off = (slots // bs).long(), (slots % bs).long()
    k_cache[blk, :, off] = k.reshape(T, n_kv, maps * dim).to(k_cache.dtype)
    v_cache[blk, :, :, off] = v.to(v_cache.dtype)
    return q.reshape(T, n_q, maps * dim).to(qkv.dtype)


def multimap_attention(q, k_cache, v_cache, block_tables, q_start, seq_lens, scale: float, maps: int,
                       lam: float, head_eps: float, out_scale: float, vdim: int, window: int = 0, sink=None,
                       chunk: int = 0):
    """Causal GQA attention with ``maps`` softmax maps per head over shared values:
    ``o = a_0 - lam * a_1`` (maps = 2; maps = 1: ``a_0``), then per head
    ``o / sqrt(mean(o^2) + head_eps) * out_scale`` (``head_eps < 0``: only the scale).
    Sequence b's query rows ``q_start[b]:q_start[b+1]`` are its last positions.  ``window`` > 0:
    position i sees only j with i - j < window.  ``chunk`` > 0: position i sees only j of its own
    chunk, floor(j / chunk) = floor(i / chunk), chunks counted from position 0.  ``sink`` fp32 [n_q]: the softmax denominator of
    head h also holds ``exp(sink[h])`` (no key, no value, not scaled).  Returns
    ``[T, n_q * vdim]``; fp32 math."""
    T, n_q, qd = q.shape
    dim = qd // maps
    n_kv = k_cache.shape[1]
    group = n_q // n_kv
    bs = k_cache.shape[2]
    out = torch.zeros(T, n_q, vdim, dtype=torch.float32, device=q.device)
    for b in range(block_tables.shape[0]):
        s, e = int(q_start[b]), int(q_start[b + 1])
        if e <= s:
            continue
        ctx = int(seq_lens[b])
        nblk = (ctx + bs - 1) // bs
        ids = block_tables[b, :nblk].long()
        k = k_cache[ids].permute(1, 0, 2, 3).reshape(n_kv, nblk * bs, qd)[:, :ctx].float()
        v = v_cache[ids].permute(1, 0, 3, 2).reshape(n_kv, nblk * bs, vdim)[:, :ctx].float()
        k, v = k.repeat_interleave(group, 0), v.repeat_interleave(group, 0)
        qb = q[s:e].float().permute(1, 0, 2)
        qpos = torch.arange(ctx - (e - s), ctx, device=q.device)[:, None]
        kpos = torch.arange(ctx, device=q.device)[None, :]
        hidden = kpos > qpos
        if window > 0:
            hidden = hidden | (kpos < qpos - window + 1)
        if chunk > 0:
            hidden = hidden | (kpos < qpos - qpos % chunk)
        o = None
        for m in range(maps):
            sc = torch.matmul(qb[..., m * dim:(m + 1) * dim], k[..., m * dim:(m + 1) * dim].transpose(1, 2)) * scale
            sc = sc.masked_fill(hidden, float("-inf"))
            if sink is not None:
                col = sink.float()[:, None, None].expand(n_q, e - s, 1)
                a = torch.matmul(torch.softmax(torch.cat([sc, col], -1), -1)[..., :-1], v)
            else:
                a = torch.matmul(torch.softmax(sc, -1), v)
            o = a if m == 0 else o - lam * a
        if head_eps >= 0:
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + head_eps)
        out[s:e] = (o * out_scale).permute(1, 0, 2)
    return out.reshape(T, n_q * vdim).to(q.dtype)


def act_fn(x: torch.Tensor, kind: str) -> torch.Tensor:
    """"gelu_tanh": 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))); "relu2": max(z, 0)^2; "silu": z sigmoid(z)."""
    z = x.float()
    if kind == "gelu_tanh":
        y = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))
    elif kind == "relu2":
        y = torch.relu(z).pow(2)
    elif kind == "silu":
        y = z * torch.sigmoid(z)
    else:
        raise ValueError(f"unknown activation {kind!r}")
    return y.to(x.dtype)


def moe_route(h, router_w, router_b, top: int, gate_w=None):
    """fp32 router: ``z = W h + b``; the ``top`` largest logits (ties: lowest index) and the
    softmax over those only.  Returns (expert ids int32 [T, top], weights fp32 [T, top],
    fp32 [T] logit of the always-on expert's gate ``gate_w . h`` or None)."""
    hf = h.float()
    z = hf @ router_w.float().t()
    if router_b is not None:
        z = z + router_b.float()
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    gate = None if gate_w is None else hf @ gate_w.float().reshape(-1)
    return idx[:, :top].to(torch.int32), torch.softmax(val[:, :top], dim=-1), gate


def moe_experts(h, up, down, idx, weights, kind: str = "relu2"):
    """``sum_j weights[t, j] * down[e] act(up[e] h_t)``, e = idx[t, j]; up [E, ff, W],
    down [E, W, ff].  kind "silu_gated": up is [E, 2 ff, W], rows [gate; up], and the hidden
    activation is ``silu(gate h) * (up h)``.  Hidden activations are rounded to the activation dtype like a
    projection's output; the weighted sum is returned in fp32 (it goes into the fp32 residual)."""
    T, W = h.shape
    out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
    for e in range(up.shape[0]):
        rows, slot = (idx == e).nonzero(as_tuple=True)
        if rows.numel() == 0:
            continue
        x = h.index_select(0, rows)
        z = torch.nn.functional.linear(x, up[e])
        if kind == "silu_gated":
            ff = z.shape[1] // 2
            hid = (act_fn(z[:, :ff], "silu").float() * z[:, ff:].float()).to(z.dtype)
        else:
            hid = act_fn(z, kind)
        y = torch.nn.functional.linear(hid, down[e])
        out.index_add_(0, rows, y.float() * weights[rows, slot][:, None])
    return out


# ------------------------------------------------------------------ per-sequence state: hashed bigram, short convolutions,
# pair rotary with value rotation, gated-state recurrences (models/padadra.py)
#
# A packed step holds B segments; segment b is rows ``q_start[b]:q_start[b+1]`` (consecutive
# positions of one sequence), ``token_seq[t]`` is the segment of row t and ``state_rows[b]`` the
# row of the per-sequence state tables that the segment continues.  A segment that starts at
# position 0 starts from empty state whatever the table holds, so a state row needs no reset
# when it is handed to a new sequence.

def embed_hashed_bigram(tokens, meta, prev, table, scale: float, bigram, hash_mul):
    """fp32 stream ``scale * E[token] + bigram[row]``; row = (previous token * mul_prev + token *
    mul_cur) mod buckets, or the table's last row at position 0 (``bigram`` None: no bigram term).
    ``prev`` int32 [rows]: the last token of every state row; read for a segment's first token,
    then set to the segment's last token."""
    x = table.index_select(0, tokens.long()).float() * scale
    if bigram is None:
        return x
    T = tokens.numel()
    first, last = meta.q_start[:-1].long(), meta.q_start[1:].long() - 1
    before = torch.zeros(T, dtype=torch.int64, device=tokens.device)
    before[1:] = tokens[:-1].long()
    before[first] = prev[meta.state_rows.long()].long()
    buckets = bigram.shape[0] - 1
    row = (before * int(hash_mul[0]) + tokens.long() * int(hash_mul[1])) % buckets
    row = torch.where(meta.positions.long() == 0, torch.full_like(row, buckets), row)
    prev[meta.state_rows.long()] = tokens[last].to(prev.dtype)
    return x + bigram.index_select(0, row).float()


def embed_hashed_bigram_norm(tokens, meta, prev, table, scale: float, bigram, hash_mul, eps: float, gains, out_dtype):
    """(`embed_hashed_bigram` stream, its `rmsnorm_scalar` for ``gains``)."""
    x = embed_hashed_bigram(tokens, meta, prev, table, scale, bigram, hash_mul)
    return x, rmsnorm_scalar(x, eps, gains, out_dtype)


def rmsnorm_scalar(x, eps: float, gains, out_dtype):
    """``x / sqrt(mean(x^2) + eps) * g`` for every scalar g of ``gains`` (fp32 math)."""
    xf = x.float()
    unit = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return tuple((unit * float(g)).to(out_dtype) for g in gains)


def residual_mix_norm(x, normed, normed_scale: float, plain, mult: float, eps: float, gains, out_dtype):
    """``x += mult * (normed_scale * sum_i rms(a_i) * w_i + sum_j p_j)`` in fp32, in place
    (``normed``: [(a_i [T, W], w_i fp32 [W])], every a_i RMS-normed over the row; ``plain``:
    [p_j]); returns `rmsnorm_scalar` of the new x for ``gains``."""
    total = None
    for a, w in normed:
        af = a.float()
        t = af * torch.rsqrt(af.pow(2).mean(-1, keepdim=True) + eps) * w.float() * normed_scale
        total = t if total is None else total + t
    for p in plain:
        total = p.float() if total is None else total + p.float()
    if total is not None:
        x.add_(total * mult)
    return rmsnorm_scalar(x, eps, gains, out_dtype)


def short_conv(y, channels: int, w, meta, state, act=None, bias=None):
    """Causal convolution over time on the first ``channels`` columns of ``y`` [T, >= channels]:
    ``out_t = sum_j w[:, j] u_(t - taps + 1 + j)`` (+ ``bias`` fp32 [channels]; fp32 sum, rounded
    once), zeros before position 0, then ``act`` (None | "silu").  ``state`` [rows, taps - 1, channels]: the last inputs of
    every state row; read where a segment reaches before its first row, then updated."""
    T, taps = y.shape[0], w.shape[1]
    u = y[:, :channels]
    seg = meta.token_seq.long()
    qs = meta.q_start.long()
    t_idx = torch.arange(T, device=y.device)
    off = t_idx - qs[seg]                      # row's offset in its segment
    rows = meta.state_rows.long()
    pos = meta.positions.long()
    acc = torch.zeros(T, channels, dtype=torch.float32, device=y.device)
    for j in range(taps):
        back = taps - 1 - j
        in_seg = off >= back
        val = u[(t_idx - back).clamp(min=0)].float()
        if taps > 1:
            old = state[rows[seg], (j + off).clamp(max=taps - 2)].float()
            val = torch.where(in_seg[:, None], val, torch.where((pos - back >= 0)[:, None], old, torch.zeros_like(old)))
        acc += w[:, j].float()[None, :] * val
    if taps > 1:
        new = torch.zeros(rows.numel(), taps - 1, channels, dtype=torch.float32, device=y.device)
        n = qs[1:] - qs[:-1]
        pos0 = pos[qs[:-1]]
        for i in range(taps - 1):
            b = taps - 1 - i
            fresh = u[(qs[1:] - b).clamp(min=0)].float()
            old = state[rows, (i + n).clamp(max=taps - 2)].float() * (pos0 > 0)[:, None]
            new[:, i] = torch.where((n >= b)[:, None], fresh, old)
        state[rows] = new.to(state.dtype)
    if bias is not None:
        acc = acc + bias.float()[None, :]
    if act == "silu":
        acc = acc * torch.sigmoid(acc)
    elif act is not None:
        raise ValueError(f"unknown activation {act!r}")
    return acc.to(y.dtype)


def scaled_inv_freq(dims: int, base: float, scaling=None, device=None) -> torch.Tensor:
    """fp32 ``base^(-2i/dims)``; with ``scaling`` = (factor, low, high, original) a frequency whose
    wavelength l = 2 pi / f is above original / low is divided by factor, one below original /
    high is kept, and between them s = (original / l - low) / (high - low) blends
    ``(1 - s) f / factor + s f``."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(dims, 1))
    if scaling is not None:
        factor, low, high, orig = (float(v) for v in scaling)
        wl = 2.0 * math.pi / f
        s = ((orig / wl - low) / (high - low)).clamp(0.0, 1.0)
        mid = (1.0 - s) * f / factor + s * f
        f = torch.where(wl < orig / high, f, torch.where(wl > orig / low, f / factor, mid))
    return f.float().to(device)


def _turn_pairs(x, ang):
    """x [..., 2n]: the pair (2i, 2i + 1) turned by ang[..., i]."""
    a, b = x[..., 0::2], x[..., 1::2]
    c, s = ang.cos(), ang.sin()
    return torch.stack([a * c - b * s, b * c + a * s], dim=-1).flatten(-2)


def rope_pairs_kv_write(qkv, positions, slots, n_q: int, n_kv: int, dim: int, vdim: int, q_norm, k_norm, eps: float,
                        inv_freq, v_inv_freq, k_cache, v_cache):
    """Row ``[q | k | v | ...]``: one RMS norm over the whole q part (weight ``q_norm``
    [n_q dim]; None = no norm) and one over the whole k part, then every q / k head's features
    (2i, 2i + 1), i < len(inv_freq), are turned by ``position * inv_freq[i]``; every v head's pairs
    by ``position * v_inv_freq[i]`` (None: values as they are).  K / V go to the paged cache of
    `rope_multi_kv_write`; returns q [T, n_q, dim]."""
    T = qkv.shape[0]
    qw, kw = n_q * dim, n_kv * dim
    q, k = qkv[:, :qw].float(), qkv[:, qw:qw + kw].float()
    v = qkv[:, qw + kw:qw + kw + n_kv * vdim].float().reshape(T, n_kv, vdim)
    if q_norm is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()
    if k_norm is not None:
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm.float()
    q, k = q.reshape(T, n_q, dim), k.reshape(T, n_kv, dim)
    pos = positions.float()[:, None, None]
    r = 2 * inv_freq.numel()
    if r:
        ang = pos * inv_freq.float()[None, None, :]
        q = torch.cat([_turn_pairs(q[..., :r], ang), q[..., r:]], -1)
        k = torch.cat([_turn_pairs(k[..., :r], ang), k[..., r:]], -1)
    if v_inv_freq is not None:
        v = _turn_pairs(v, pos * v_inv_freq.float()[None, None, :])
    bs = k_cache.shape[2]
    blk, off = (slots // bs).long(), (slots % bs).long()
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, :, off] = v.to(v_cache.dtype)
    return q.to(qkv.dtype)


def rotate_pairs(x, positions, inv_freq, sign: float, heads: int):
    """x [T, heads * 2n]: every head's pair (2i, 2i + 1) turned by ``sign * position * inv_freq[i]``."""
    T = x.shape[0]
    xf = x.float().reshape(T, heads, -1)
    ang = sign * positions.float()[:, None, None] * inv_freq.float()[None, None, :]
    return _turn_pairs(xf, ang).reshape(T, -1).to(x.dtype)


def hgrn2_prepare(y, off_q: int, off_f: int, heads: int, dim: int, f_bias, lower):
    """From a fused projection row: ``q = silu(y_q)``, forget gate ``f = l + (1 - l) sigmoid(y_f +
    bias)``; returns fp32 (q, 1 - f, f), each [T, heads, dim]: the read, write and decay vectors of
    `gated_state_scan`."""
    T, n = y.shape[0], heads * dim
    q = y[:, off_q:off_q + n].float()
    q = q * torch.sigmoid(q)
    low = lower.float()
    f = low + (1.0 - low) * torch.sigmoid(y[:, off_f:off_f + n].float() + f_bias.float())
    return q.reshape(T, heads, dim), (1.0 - f).reshape(T, heads, dim), f.reshape(T, heads, dim)


def delta_prepare(c, y, off_beta: int, a, a_log, dt_bias, heads: int, kv_heads: int, dim: int):
    """``c`` [T, >= 2 kv_heads dim]: q | k after convolution and activation; every q / k head
    becomes a unit vector ``x / sqrt(sum x^2 + 1e-6)`` (q also times dim^-1/2); ``beta = sigmoid(y
    [:, off_beta + h])``; decay ``g = exp(-exp(a_log[h]) softplus(a + dt_bias))`` with ``a`` [T,
    heads gd] (unit column stride), gd = dim (one decay per head and key channel) or 1 (one per
    head).  Returns fp32 (q [T, kv_heads, dim], k, g [T, heads, gd], beta [T, heads])."""
    T, n = c.shape[0], kv_heads * dim
    gd = a.shape[1] // heads
    q = c[:, :n].float().reshape(T, kv_heads, dim)
    k = c[:, n:2 * n].float().reshape(T, kv_heads, dim)
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(y[:, off_beta:off_beta + heads].float())
    sp = torch.nn.functional.softplus(a.float() + dt_bias.float()).reshape(T, heads, gd)
    g = torch.exp(-torch.exp(a_log.float())[None, :, None] * sp)
    return q, k, g, beta


def gated_state_scan(q, k, g, v, beta, meta, state, delta: bool, unit_last: bool = False):
    """Per head a ``dim x vdim`` fp32 state S, token after token:

        S <- diag(g_t) S;   u = v_t  (times beta_t when given)   (delta False)
                            u = beta_t (v_t - S^T k_t)           (delta True)
        S <- S + k_t u^T;   o_t = S^T q_t

    q / k [T, Gq, dim] fp32 (head h reads q / k head h // (H / Gq)), g fp32 [T, H, dim] (a decay
    per key channel) or [T, H, 1] (one per head), v [T, H vdim], beta [T, H] fp32 or None;
    ``state`` [rows, H, dim, vdim] fp32 is read (unless the segment starts at position 0) and left
    at the segment's last token.  ``unit_last`` (without the delta rule): v is [T, H (vdim - 1)] and the
    state's last column reads a value of 1 for every token, so it accumulates the written keys alone
    (a normaliser beside the memory); o's last column is then its product with q.  Returns fp32 o [T, H, vdim]."""
    T, H = g.shape[:2]
    vdim = state.shape[3]
    per = H // q.shape[1]
    if unit_last:
        vf = torch.cat([v.float().reshape(T, H, vdim - 1), torch.ones(T, H, 1, device=v.device)], -1)
    else:
        vf = v.float().reshape(T, H, vdim)
    qh, kh = q.repeat_interleave(per, 1), k.repeat_interleave(per, 1)
    out = torch.zeros(T, H, vdim, dtype=torch.float32, device=g.device)
    qs = meta.q_start.tolist()
    rows = meta.state_rows.tolist()
    pos = meta.positions.tolist()
    for b in range(len(rows)):
        s, e = qs[b], qs[b + 1]
        if e <= s:
            continue
        S = state[rows[b]].clone() if pos[s] > 0 else torch.zeros_like(state[rows[b]])
        for t in range(s, e):
            S = S * g[t][:, :, None]
            u = vf[t]
            if delta:
                u = beta[t][:, None] * (u - torch.einsum("hde,hd->he", S, kh[t]))
            elif beta is not None:
                u = beta[t][:, None] * u
            S = S + kh[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hde,hd->he", S, qh[t])
        state[rows[b]] = S
    return out


def head_norm_gate(o, w, eps: float, gate, out_dtype, gate_act: str = "sigmoid", floor=None):
    """o fp32 [T, H, vdim]: every head divided by its root mean square, times ``w`` ([vdim], or
    [H vdim]: a weight per head), times ``sigmoid(gate)`` or ``silu(gate)`` (gate [T, H vdim] logits or
    None; ``gate_act``); returns [T, H vdim] in ``out_dtype``.  ``floor`` fp32 [T, H]: o has one more
    column, a normaliser, and the head is first divided by ``max(|normaliser|, floor) + 1e-6``."""
    if floor is not None:
        o = o[..., :-1] / (torch.maximum(o[..., -1].abs(), floor.float()) + 1e-6)[..., None]
    T, H, vdim = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w.float().reshape(-1, vdim)
    if gate is not None:
        z = gate.float().reshape(T, H, vdim)
        y = y * (torch.sigmoid(z) if gate_act == "sigmoid" else z * torch.sigmoid(z))
    return y.reshape(T, H * vdim).to(out_dtype)


# ------------------------------------------------------------------ dynamic-tanh norms, latent attention, selective state
# space, table-routed gated experts, per-layer token input (models/mabivik.py)
#
# A dynamic-tanh norm is the triple (alpha, w, b): ``tanh(alpha x) w + b`` elementwise (alpha a
# number, w / b fp32 [W]); it takes no statistic of the row.  The latent-attention cache of one
# layer is ``k : [num_blocks, 1, block_size, kv_rank + rot_dim]`` (the normed latent, then the
# rotated shared key part) and ``v : [num_blocks, 1, kv_rank, block_size]`` (the latent again,
# transposed per block): `multimap_attention` with one KV head reads them when every query
# head carries ``W_uk[h]^T q_h`` in front of its rotated part, and its output is the softmax-
# weighted latent, which ``W_uv[h]`` then expands.

def dyt(x, norm, out_dtype):
    """``tanh(alpha x) w + b`` in fp32, rounded once; ``norm`` = (alpha, w, b)."""
    alpha, w, b = norm
    return (torch.tanh(float(alpha) * x.float()) * w.float() + b.float()).to(out_dtype)


def embed_scale_dyt(tokens, table, scale: float, norm, out_dtype):
    """(fp32 stream ``scale * E[tokens]``, its `dyt` in ``out_dtype``)."""
    x = table.index_select(0, tokens.long()).float() * scale
    return x, dyt(x, norm, out_dtype)


def residual_post_norm(x, y, post, pre, out_dtype):
    """``x += post(y)`` in fp32, in place, with ``post`` = ("dyt", alpha, w, b) or ("rms", w, eps)
    (``y / sqrt(mean(y^2) + eps) * w``); then returns what the next reader of x takes: ``pre`` =
    ("dyt", alpha, w, b) -> `dyt` of the new x, ("copy",) -> x rounded to ``out_dtype``, None -> None."""
    yf = y.float()
    if post[0] == "dyt":
        x.add_(torch.tanh(float(post[1]) * yf) * post[2].float() + post[3].float())
    elif post[0] == "rms":
        x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + float(post[2])) * post[1].float())
    else:
        raise ValueError(f"unknown post norm {post[0]!r}")
    if pre is None:
        return None
    if pre[0] == "copy":
        return x.to(out_dtype)
    return dyt(x, pre[1:], out_dtype)


def rmsnorm_cols(y, off: int, n: int, w, eps: float, out_dtype):
    """RMS norm over the columns ``off : off + n`` of ``y`` (fp32), times ``w`` [n]; contiguous [T, n]."""
    z = y[:, off:off + n].float()
    return (z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def ramp_inv_freq(dims: int, base: float, scaling=None, device=None):
    """(fp32 frequencies [dims / 2], amplitude).  Plain: ``base^(-2i/dims)``, 1.  ``scaling`` =
    (factor, original, fast, slow): with ``d(t) = dims ln(original / (2 pi t)) / (2 ln base)``, lo =
    max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1) and the ramp r_i = clamp((i - lo) /
    max(hi - lo, 0.001), 0, 1) the frequency is ``f_i / factor * r_i + f_i (1 - r_i)`` and the
    amplitude of cos and sin ``0.1 ln(factor) + 1``."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(dims, 1))
    amp = 1.0
    if scaling is not None:
        factor, orig, fast, slow = (float(v) for v in scaling)

        def d(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo, hi = max(math.floor(d(fast)), 0), min(math.ceil(d(slow)), dims - 1)
        r = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * r + f * (1.0 - r)
        amp = 0.1 * math.log(factor) + 1.0
    return f.float().to(device), amp


def _turn_half(x, positions, inv_freq, amp: float):
    """x [T, ..., n]: feature i < len(inv_freq) pairs with i + len(inv_freq); cos and sin times amp."""
    half = inv_freq.numel()
    if not half:
        return x
    ang = positions.float().reshape(-1, *([1] * (x.dim() - 1))) * inv_freq.float()
    c, s = ang.cos() * amp, ang.sin() * amp
    a, b = x[..., :half], x[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., 2 * half:]], dim=-1)


def latent_kv_write(y, off: int, kv_rank: int, rot_dim: int, w, eps: float, positions, slots, inv_freq, amp: float,
                    k_cache, v_cache):
    """Columns ``off : off + kv_rank`` of ``y`` are RMS-normed (weight ``w``) into the latent c,
    the next ``rot_dim`` are turned by the position (`_turn_half`, not normed); the token's cache
    row becomes K = [c | turned part], V^T = c."""
    c = rmsnorm_cols(y, off, kv_rank, w, eps, torch.float32)
    kr = _turn_half(y[:, off + kv_rank:off + kv_rank + rot_dim].float(), positions, inv_freq, amp)
    bs = k_cache.shape[2]
    blk, o = (slots // bs).long(), (slots % bs).long()
    k_cache[blk, 0, o] = torch.cat([c, kr], -1).to(k_cache.dtype)
    v_cache[blk, 0, :, o] = c.to(v_cache.dtype)


def rope_half_tail(src, src_off: int, dst, dst_off: int, positions, inv_freq, amp: float):
    """``dst[:, h, dst_off:] = turn(src[:, h, src_off:])`` for every head of src [T, H, Ds] / dst
    [T, H, Dd] (tails of equal width): the first ``2 len(inv_freq)`` features of the tail are turned
    by the position (feature i pairs with i + half), the rest copied."""
    dst[:, :, dst_off:] = _turn_half(src[:, :, src_off:].float(), positions, inv_freq, amp).to(dst.dtype)
    return dst


def head_linear(x3, w, out3=None):
    """``out3[t, h] = w[h] x3[t, h]``: x3 [T, H, K] (any strides with a unit last one), w [H, N, K],
    out3 [T, H, N] (a view to fill, or None: a new contiguous tensor)."""
    if out3 is None:
        out3 = torch.empty(x3.shape[0], x3.shape[1], w.shape[1], dtype=x3.dtype, device=x3.device)
    torch.bmm(x3.transpose(0, 1), w.transpose(1, 2), out=out3.transpose(0, 1))
    return out3


def gate_mul(x, gate, kind: str, group: int = 1):
    """``x * sigmoid(gate)`` or ``x * silu(gate)`` (fp32, rounded once); gate [T, n / group] with any
    row stride: one gate column serves ``group`` neighbouring columns of x (one gate per head)."""
    z = gate.float().repeat_interleave(group, 1) if group > 1 else gate.float()
    return (x.float() * (torch.sigmoid(z) if kind == "sigmoid" else z * torch.sigmoid(z))).to(x.dtype)


def ssm_prepare(c, off_b: int, y, off_dt: int, dt_bias, a_log, heads: int, groups: int, state: int):
    """``c`` [T, >= off_b + 2 groups state]: B | C after convolution and activation at ``off_b``;
    ``dt = softplus(y[:, off_dt + h] + dt_bias[h])``, decay ``g = exp(-exp(a_log[h]) dt)``.  Returns
    fp32 (C [T, groups, state], B [T, groups, state], g [T, heads, 1], dt [T, heads]): the read,
    write and decay vectors of `gated_state_scan` and the scale of its written value."""
    T, n = c.shape[0], groups * state
    B = c[:, off_b:off_b + n].float().reshape(T, groups, state)
    C = c[:, off_b + n:off_b + 2 * n].float().reshape(T, groups, state)
    dt = torch.nn.functional.softplus(y[:, off_dt:off_dt + heads].float() + dt_bias.float())
    g = torch.exp(-torch.exp(a_log.float())[None, :] * dt)
    return C.contiguous(), B.contiguous(), g[:, :, None].contiguous(), dt.contiguous()


def gated_group_norm(o, skip, skip_w, z, w, parts: int, eps: float, out_dtype):
    """``u = (o + skip_w[h] skip) * silu(z)`` over o fp32 [T, H, vdim] (skip, z [T, H vdim], any row
    stride), then u in ``parts`` equal pieces of the row, each divided by its own root mean
    square, times ``w`` [H vdim]; returns [T, H vdim] in ``out_dtype``."""
    T, H, vdim = o.shape
    zf = z.float()
    u = (o + skip_w.float()[None, :, None] * skip.float().reshape(T, H, vdim)).reshape(T, H * vdim) * (zf * torch.sigmoid(zf))
    u = u.reshape(T, parts, -1)
    u = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    return (u.reshape(T, H * vdim) * w.float()).to(out_dtype)


def moe_table_route(tokens, table, top: int):
    """Experts by token id: (``table[token, :top]`` int32 [T, top], weights fp32 [T, top] = 1 / top)."""
    idx = table.index_select(0, tokens.long())[:, :top].to(torch.int32).contiguous()
    return idx, torch.full(idx.shape, 1.0 / top, dtype=torch.float32, device=idx.device)


def gelu_gather_mul(z, tokens, table, off: int):
    """``gelu_tanh(z) * table[token, off : off + n]`` for z [T, n] (fp32 math, rounded once)."""
    e = table.index_select(0, tokens.long())[:, off:off + z.shape[1]].float()
    return (act_fn(z.float(), "gelu_tanh") * e).to(z.dtype)


def gated_act(both):
    """``silu(both[:, :n]) * both[:, n:]`` for a stacked [gate | up] projection [rows, 2 n]; the
    activation is rounded like a projection's output before the product."""
    n = both.shape[1] // 2
    return (act_fn(both[:, :n], "silu").float() * both[:, n:].float()).to(both.dtype)


# ------------------------------------------------------------------ hyper-connection streams, layer norms, unit-norm rotary
# heads with value mixing, exponential-gate matrix memory, sigmoid-scored grouped routing (models/sitidra.py)
#
# The residual is S streams X [T, S, W] fp32.  A sublayer reads ``u = sum_s read[s] X[s]`` through a
# layer norm and its output y is written back as ``X'[t] = sum_s mix[s, t] X[s] + out[t] y``, all
# streams from the old ones.  S = 1 with read = mix = out = 1 is the plain residual sum.

def layer_norm32(u, w, eps: float, out_dtype):
    """fp32 ``(u - mean) / sqrt(var + eps) * w`` (biased variance, no bias), rounded once."""
    uf = u.float()
    d = uf - uf.mean(-1, keepdim=True)
    return (d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def hyper_embed_norm(tokens, table, streams: int, read_w, norm_w, eps: float, out_dtype):
    """(X fp32 [T, streams, W] with every stream = table[token], layer norm of ``sum_s read_w[s] X[s]``)."""
    x = table.index_select(0, tokens.long()).float()
    X = x[:, None, :].repeat(1, streams, 1).contiguous()
    return X, layer_norm32(torch.einsum("s,nsw->nw", read_w.float(), X), norm_w, eps, out_dtype)


def hyper_update_norm(X, parts, mix, out_w, read_w, norm_w, eps: float, out_dtype):
    """In place ``X[:, t] <- sum_s mix[s, t] X[:, s] + out_w[t] y`` with y the fp32 sum of ``parts``
    (``mix`` None: X stays); returns the layer norm of ``sum_s read_w[s] X[:, s]`` (``read_w`` None: None)."""
    if mix is not None:
        y = None
        for p in parts:
            y = p.float() if y is None else y + p.float()
        new = torch.einsum("sd,nsw->ndw", mix.float(), X)
        if y is not None:
            new = new + out_w.float()[None, :, None] * y[:, None, :]
        X.copy_(new)
    if read_w is None:
        return None
    return layer_norm32(torch.einsum("s,nsw->nw", read_w.float(), X), norm_w, eps, out_dtype)


def rope_norm_kv_write(qkv, positions, slots, n_q: int, n_kv: int, dim: int, vdim: int, inv_freq, qk_eps: float,
                       v_first, lam: float, k_cache, v_cache):
    """Split a fused projection row ``[q | k | v | anything]``; rotate the first ``2 * len(inv_freq)``
    features of every q / k head (feature i pairs with i + rot/2; angle = position * inv_freq[i], fp32);
    divide every head by its root mean square over ``dim`` (``qk_eps`` < 0: not); blend the values,
    ``v <- (1 - lam) v + lam v_first`` (``v_first`` [T, n_kv vdim], any row stride; None: v as it is);
    scatter K / V into the paged cache.  Returns q ``[T, n_q, dim]`` in the activation dtype."""
    T = qkv.shape[0]
    qw, kw = n_q * dim, n_kv * dim
    q = qkv[:, :qw].float().reshape(T, n_q, dim)
    k = qkv[:, qw:qw + kw].float().reshape(T, n_kv, dim)
    v = qkv[:, qw + kw:qw + kw + n_kv * vdim].float()
    half = inv_freq.numel()
    if half:
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]

        def rot(x):
            a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
            return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)
        q, k = rot(q), rot(k)
    if qk_eps >= 0:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + qk_eps)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + qk_eps)
    if v_first is not None:
        v = (1.0 - lam) * v + lam * v_first.float()
    bs = k_cache.shape[2]
    blk, off = (slots // bs).long(), (slots % bs).long()
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, :, off] = v.reshape(T, n_kv, vdim).to(v_cache.dtype)
    return q.to(qkv.dtype)


def exp_gate_prepare(y, off_q: int, off_k: int, off_i: int, off_f: int, i_bias, f_bias, cap: float, q_scale: float,
                     heads: int, dim: int, meta, m_state):
    """Gates of a matrix memory from the fused projection ``y``: per head the log input gate
    ``i = cap tanh((y_i + b_i) / cap)`` and the log forget gate ``f = logsigmoid(cap tanh((y_f + b_f) / cap))``,
    the running maximum ``m_t = max(f_t + m_(t-1), i_t)`` (``m_state`` fp32 [rows, heads], read unless
    the segment starts at position 0 -- it then starts at 0 -- and left at the segment's last token).
    Returns fp32 (q_scale * q [T, heads, dim], k [T, heads, dim], decay ``exp(f_t + m_(t-1) - m_t)``
    [T, heads, 1], write scale ``exp(i_t - m_t)`` [T, heads], floor ``exp(-m_t)`` [T, heads])."""
    T, n = y.shape[0], heads * dim
    q = (y[:, off_q:off_q + n].float() * q_scale).reshape(T, heads, dim).contiguous()
    k = y[:, off_k:off_k + n].float().reshape(T, heads, dim).contiguous()
    gi = cap * torch.tanh((y[:, off_i:off_i + heads].float() + i_bias.float()) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((y[:, off_f:off_f + heads].float() + f_bias.float()) / cap))
    decay = torch.empty(T, heads, dtype=torch.float32, device=y.device)
    write, floor = torch.empty_like(decay), torch.empty_like(decay)
    qs, rows, pos = meta.q_start.tolist(), meta.state_rows.tolist(), meta.positions.tolist()
    for b in range(len(rows)):
        s, e = qs[b], qs[b + 1]
        if e <= s:
            continue
        m = m_state[rows[b]].clone() if pos[s] > 0 else torch.zeros(heads, dtype=torch.float32, device=y.device)
        for t in range(s, e):
            new = torch.maximum(gf[t] + m, gi[t])
            decay[t], write[t], floor[t] = torch.exp(gf[t] + m - new), torch.exp(gi[t] - new), torch.exp(-new)
            m = new
        m_state[rows[b]] = m
    return q, k, decay[:, :, None].contiguous(), write, floor


def moe_route_scored(h, router_w, corr, top: int, groups: int, keep: int, scale: float):
    """fp32 router with sigmoid scores ``s = sigmoid(W h)``.  The ``top`` experts with the largest choice
    score ``s + corr`` (ties: lowest index) among the ``keep`` best of ``groups`` equal groups of neighbouring
    experts (a group's score: the sum of its two largest choice scores; ties: lowest group); the others
    cannot be chosen.  Weights: the chosen ``s`` over their sum (+ 1e-20), times ``scale``.  Returns
    (expert ids int32 [T, top], weights fp32 [T, top])."""
    sc = torch.sigmoid(h.float() @ router_w.float().t())
    choice = sc if corr is None else sc + corr.float()
    T, E = choice.shape
    if groups > 1 and keep < groups:
        per = E // groups
        g = choice.reshape(T, groups, per)
        gs = g.topk(min(2, per), dim=-1).values.sum(-1)
        order = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
        allowed = torch.zeros(T, groups, dtype=torch.bool, device=h.device).scatter_(1, order, True)
        choice = g.masked_fill(~allowed[:, :, None], float("-inf")).reshape(T, E)
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    w = sc.gather(1, idx)
    return idx.to(torch.int32), w / (w.sum(-1, keepdim=True) + 1e-20) * scale


def softcap(logits, cap: float):
    """``cap tanh(logits / cap)`` on fp32 logits, in place."""
    return logits.copy_(cap * torch.tanh(logits / cap))

"""Op dispatch: ``get_ops("hip")`` -> HIP/CDNA4 kernels, ``get_ops("torch")`` -> references.

Both namespaces expose the same functions (see ``reference.py`` for the
semantics).  The HIP namespace raises at import when ``libbcg_kernels.so``
is missing instead of silently falling back.
"""

from types import SimpleNamespace

import torch

from . import reference as _ref


def _torch_ops() -> SimpleNamespace:
    def decode(q, k_cache, v_cache, layer, block_tables, seq_lens, scale, workspace=None, cascade=None):
        # the shared-prefix cascade changes how the kernel walks the KV, not the result
        B = q.shape[0]
        q_start = torch.arange(B + 1, dtype=torch.int32, device=q.device)
        return _ref.paged_attention(q, k_cache, v_cache, layer, block_tables, q_start, seq_lens, scale)

    def prefill(q, k_cache, v_cache, layer, block_tables, q_start, seq_lens, scale, max_q_len=None, tiles=None,
                tile_rows=64):
        return _ref.paged_attention(q, k_cache, v_cache, layer, block_tables, q_start, seq_lens, scale)

    def multimap_attention(q, k_cache, v_cache, meta, scale, maps, lam, head_eps, out_scale, vdim, window=0, sink=None,
                           chunk=0):
        # tiles / single-row lists only tell the HIP kernels how to walk the batch
        q_start = meta.q_start
        if q_start is None:  # decode: one row per sequence
            q_start = torch.arange(q.shape[0] + 1, dtype=torch.int32, device=q.device)
        lens = meta.seq_lens if meta.attn_seq_lens is None else meta.attn_seq_lens
        return _ref.multimap_attention(q, k_cache, v_cache, meta.block_tables, q_start, lens, scale, maps,
                                       lam, head_eps, out_scale, vdim, window, sink, chunk)

    return SimpleNamespace(
        name="torch",
        rmsnorm32=_ref.rmsnorm32,
        embed_scale_rmsnorm=_ref.embed_scale_rmsnorm,
        residual_add_rmsnorm32=_ref.residual_add_rmsnorm32,
        rope_multi_kv_write=_ref.rope_multi_kv_write,
        multimap_attention=multimap_attention,
        act_fn=_ref.act_fn,
        moe_route=_ref.moe_route,
        moe_experts=_ref.moe_experts,
        embed_hashed_bigram_norm=_ref.embed_hashed_bigram_norm,
        rmsnorm_scalar=_ref.rmsnorm_scalar,
        residual_mix_norm=_ref.residual_mix_norm,
        short_conv=_ref.short_conv,
        rope_pairs_kv_write=_ref.rope_pairs_kv_write,
        rotate_pairs=_ref.rotate_pairs,
        hgrn2_prepare=_ref.hgrn2_prepare,
        delta_prepare=_ref.delta_prepare,
        gated_state_scan=_ref.gated_state_scan,
        head_norm_gate=_ref.head_norm_gate,
        embed_scale_dyt=_ref.embed_scale_dyt,
        residual_post_norm=_ref.residual_post_norm,
        rmsnorm_cols=_ref.rmsnorm_cols,
        latent_kv_write=_ref.latent_kv_write,
        rope_half_tail=_ref.rope_half_tail,
        head_linear=_ref.head_linear,
        gate_mul=_ref.gate_mul,
        ssm_prepare=_ref.ssm_prepare,
        gated_group_norm=_ref.gated_group_norm,
        moe_table_route=_ref.moe_table_route,
        gelu_gather_mul=_ref.gelu_gather_mul,
        gated_act=_ref.gated_act,
        hyper_embed_norm=_ref.hyper_embed_norm,
        hyper_update_norm=_ref.hyper_update_norm,
        rope_norm_kv_write=_ref.rope_norm_kv_write,
        exp_gate_prepare=_ref.exp_gate_prepare,
        moe_route_scored=_ref.moe_route_scored,
        softcap=_ref.softcap,
        linear=torch.nn.functional.linear,
        rmsnorm=_ref.rmsnorm,
        add_rmsnorm=_ref.add_rmsnorm,
        embed_rmsnorm=_ref.embed_rmsnorm,
        qk_norm_rope_kv_write=_ref.qk_norm_rope_kv_write,
        paged_attention_decode=decode,
        paged_attention_prefill=prefill,
        prefill_tile_rows=lambda hd, kv_fp8=False, max_blocks=0: 64,
        silu_mul=_ref.silu_mul,
        linear_silu=_ref.linear_silu,
        linear_residual=_ref.linear_residual,
        sample_step=_ref.sample_step,
        quant_fp8=_ref.quant_fp8,
        add_rmsnorm_fp8=_ref.add_rmsnorm_fp8,
        silu_mul_fp8=_ref.silu_mul_fp8,
        linear_fp8=_ref.linear_fp8,
        rmsnorm_fp8=_ref.rmsnorm_fp8,
        embed_rmsnorm_fp8=_ref.embed_rmsnorm_fp8,
        linear_fp8_residual=_ref.linear_fp8_residual,
    )


_CACHE = {}


def get_ops(backend: str) -> SimpleNamespace:
    if backend not in _CACHE:
        if backend == "torch":
            _CACHE[backend] = _torch_ops()
        elif backend == "hip":
            from .hip import hip_ops
            _CACHE[backend] = hip_ops()
        else:
            raise ValueError(f"unknown ops backend {backend!r}")
    return _CACHE[backend]

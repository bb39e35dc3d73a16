"""Sitidra on the HIP backend against the float64 oracle: every mechanism's kernels alone (fp32 and
bf16), the new HIP ops against their PyTorch fp32 references at larger shapes, packed steps of
the engine (prompt portions beside single tokens, page and state-row reuse), and greedy
generation through the scheduler with captured decode graphs."""
import numpy as np
import pytest
import torch

import sitidra_cases as C
import sitidra_checks as K
import sitidra_oracle as O
from byzantine_consensus_llm_agents_amd.ops import reference as ref
from test_sitidra_cpu import ATTENTION

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


@pytest.fixture(params=DTYPES)
def env(request):
    e = K.Env("hip", "cuda", getattr(torch, request.param))
    assert e.ops.name == "hip"
    return e


# ------------------------------------------------------------------ mechanisms
@pytest.mark.parametrize("S", [1, 2, 3, 4, 7, 11, 16])
def test_streams_read_write_and_layer_norm(env, S):
    K.check_streams(env, S)
    K.check_streams(env, S, W=1000)
    K.check_streams(env, S, W=50)    # off the 4-column grid: one column per thread
    K.check_streams(env, S, W=333)


@pytest.mark.parametrize("name", list(ATTENTION))
def test_attention_whole_and_in_portions(env, name):
    for cuts in (None, [2, 14, 1, 1, 17, 2, 8]):
        got, want = K.run_mixer(env, ATTENTION[name], 45, cuts, seed=3)
        env.close(got, want)


def test_attention_exact_and_wide_shapes(env):
    """Heads on the 16-wide MFMA grid (the straight-line instances) and off it, GQA groups above
    the 16 MFMA columns, chunks longer than a decode split, several 64-row tiles."""
    for heads, kv, dim, vdim, chunk, rot in [(4, 2, 32, 32, 70, 16), (8, 4, 128, 64, 80, 32), (3, 1, 48, 32, 0, 48),
                                             (17, 1, 16, 16, 40, 8), (2, 2, 64, 128, 150, 32), (4, 4, 128, 128, 130, 0)]:
        layers = [C.layer("attention", C.attn(heads, kv, dim, vdim, chunk, rot, scale=0.2), 0)]
        got, want = K.run_mixer(env, layers, 200, [150, 1, 1, 40, 1, 1, 1, 1, 1, 1, 1, 1], seed=heads, width=48)
        env.close(got, want)


def test_chunk_edge_shows_with_one_loud_value(env):
    whole = K.check_chunk_edge(env)
    steps = K.check_chunk_edge(env, cuts=[19] + [1] * 21)
    if env.dtype == torch.float32:
        env.close(steps, whole.double().cpu().numpy(), 1e-4)
    K.check_chunk_edge(env, chunk=16, T=60, cuts=[3, 2, 11, 17] + [1] * 27)      # the edges fall on page borders
    K.check_chunk_edge(env, chunk=23, T=80, cuts=[45, 2, 22, 1, 1, 1, 8])        # a portion starts inside a chunk
    K.check_chunk_edge(env, chunk=140, T=430, cuts=[270] + [1] * 160)            # ... and chunks longer than a decode split


def test_far_value_inside_a_long_chunk(env):
    m = C.attn(2, 1, 16, 16, 0, 8, scale=0.05)
    layers = [C.layer("attention", m, 0)]
    got, want = K.run_mixer(env, layers, 300, [290] + [1] * 10, K.loud_value(3), seed=6)
    env.close(got, want)
    _, without = K.run_mixer(env, layers, 300, None, None, seed=6)
    assert np.abs(want[295:] - without[295:]).max() > 0.05


@pytest.mark.parametrize("H,d,e,cap", [(3, 12, 20, 15.0), (1, 5, 3, 2.0), (2, 72, 70, 8.0), (5, 20, 33, 50.0), (4, 16, 16, 0.5),
                                       (4, 128, 64, 15.0), (8, 64, 128, 15.0)])
def test_matrix_memory_in_portions(env, H, d, e, cap):
    layers = [C.layer("mlstm", C.mlstm(H, d, e, cap), 0)]
    for cuts in (None, [1, 1, 2, 9, 1, 16, 10]):
        got, want = K.run_mixer(env, layers, 40, cuts, seed=H)
        env.close(got, want)


@pytest.mark.parametrize("i_bias,f_bias", [(6.0, -4.0), (-9.0, 5.0), (0.0, 0.0)])
def test_matrix_memory_gate_regimes(env, i_bias, f_bias):
    def craft(sd, hs):
        sd["l0.mix.i.b"] = torch.full_like(sd["l0.mix.i.b"], i_bias)
        sd["l0.mix.f.b"] = torch.full_like(sd["l0.mix.f.b"], f_bias)
    layers = [C.layer("mlstm", C.mlstm(2, 8, 12, 12.0), 0)]
    whole, want = K.run_mixer(env, layers, 120, None, craft, seed=2)
    env.close(whole, want)
    steps, _ = K.run_mixer(env, layers, 120, [50] + [1] * 70, craft, seed=2)
    env.close(steps, want)


@pytest.mark.parametrize("E,top,groups,keep,shift", [(12, 2, 2, 1, 0.0), (6, 2, 3, 2, -2.0), (8, 3, 0, 0, 0.0), (8, 5, 8, 5, -1.5),
                                                     (9, 3, 3, 1, 0.3), (4, 4, 2, 2, 0.0), (1, 1, 1, 1, 0.0), (10, 1, 5, 2, -3.0),
                                                     (256, 8, 8, 4, 0.0)])
def test_grouped_sigmoid_router(env, E, top, groups, keep, shift):
    K.check_router(env, E, top, groups, keep, 1.7, corr_shift=shift)


@pytest.mark.parametrize("E,top,groups,keep,ff,shared", [(6, 2, 3, 2, 24, 20), (1, 1, 0, 0, 8, 0), (4, 4, 2, 2, 16, 7), (9, 3, 3, 1, 72, 40),
                                                         (8, 2, 4, 2, 64, 128)])
def test_routed_and_shared_experts(env, E, top, groups, keep, ff, shared):
    K.check_experts(env, E, top, groups, keep, ff, shared)
    K.check_experts(env, E, top, groups, keep, ff, shared, W=64, T=150)


# ------------------------------------------------------------------ HIP ops against their fp32 references
def _tol(dtype):
    return dict(atol=2e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("S,W", [(4, 2048), (1, 96), (8, 1000), (2, 12288), (3, 1001), (4, 250)])
def test_stream_kernels_at_model_widths(dtype, S, W):
    ops = K.Env("hip", "cuda").ops
    g = torch.Generator().manual_seed(S + W)
    T, V = 37, 50
    table = torch.randn(V, W, generator=g).to(dtype).cuda()
    toks = torch.randint(0, V, (T,), generator=g, dtype=torch.int32).cuda()
    r1, r2, o1 = (torch.randn(S, generator=g).cuda() for _ in range(3))
    mix = torch.randn(S, S, generator=g).cuda()
    w = (1 + 0.1 * torch.randn(W, generator=g)).cuda()
    X, h = ops.hyper_embed_norm(toks, table, S, r1, w, 1e-5, dtype)
    Xr, hr = ref.hyper_embed_norm(toks, table, S, r1, w, 1e-5, dtype)
    torch.testing.assert_close(X, Xr, atol=0, rtol=0)
    torch.testing.assert_close(h.float(), hr.float(), **_tol(dtype))
    ya, yb = torch.randn(T, W, generator=g).to(dtype).cuda(), torch.randn(T, W, generator=g).cuda()
    h2 = ops.hyper_update_norm(X, [ya, yb], mix, o1, r2, w, 1e-5, dtype)
    h2r = ref.hyper_update_norm(Xr, [ya, yb], mix, o1, r2, w, 1e-5, dtype)
    torch.testing.assert_close(X, Xr, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(h2.float(), h2r.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gate_prepare_many_segments(dtype):
    """Segments of 1 to 300 tokens, some continuing a state row, some starting at position 0 over a
    stale row; the maximum chain equals the token-by-token reference bit for bit in its inputs."""
    ops = K.Env("hip", "cuda").ops
    g = torch.Generator().manual_seed(5)
    H, dim = 6, 20
    parts = [(0, 300), (17, 1), (0, 1), (40, 33), (5, 64), (0, 16)]
    T = sum(n for _, n in parts)
    width = 2 * H * dim + 2 * H + 3
    y = (torch.randn(T, width, generator=g) * 2).to(dtype).cuda()
    ib, fb = torch.randn(H, generator=g).cuda(), (torch.randn(H, generator=g) + 1).cuda()
    meta = C.segments(parts, [0, 1, 2, 3, 4, 5], "cuda")
    m0 = torch.randn(7, H, generator=g).cuda()
    m_hip, m_ref = m0.clone(), m0.clone()
    args = (y, 3, 3 + H * dim, 3 + 2 * H * dim, 3 + 2 * H * dim + H, ib, fb, 6.0, 0.25, H, dim, meta)
    got = ops.exp_gate_prepare(*args, m_hip)
    want = ref.exp_gate_prepare(*args, m_ref)
    for a, b in zip(got, want):
        assert a.shape == b.shape
        torch.testing.assert_close(a, b, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(m_hip, m_ref, atol=2e-5, rtol=2e-5)


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module", params=[(n, d) for n in C.CASES for d in DTYPES], ids=lambda p: f"{p[0]}-{p[1]}")
def case(request, tmp_path_factory):
    name, dtype = request.param
    path = str(tmp_path_factory.mktemp(name))
    cfg = C.CASES[name]
    sd = O.to_f64(C.checkpoint(cfg, path, seed=len(name)))
    e = K.Env("hip", "cuda", getattr(torch, dtype))
    e.measure_noise(path, cfg, sd)
    eng = C.engine(path, backend="hip", dtype=e.dtype, pool_tokens=320)
    assert eng.ops.name == "hip"
    yield e, cfg, sd, eng
    eng.shutdown()


def test_whole_prompt_every_position(case):
    K.whole_prompt(*case, n=150)


def test_summed_streams_after_every_layer(case):
    K.stream_after_every_layer(*case)


def test_prefill_then_token_by_token(case):
    K.prefill_then_token_by_token(*case, n=140, first=75)


def test_first_tokens_one_by_one(case):
    K.first_tokens_one_by_one(*case)


@pytest.mark.parametrize("sizes", [[2, 2, 3, 17, 16, 1, 31, 2, 5], [15, 1, 1, 16, 33, 11], [2, 3, 64, 1, 17, 2, 1, 70]])
def test_portions_of_changing_size(case, sizes):
    K.portions(*case, sizes)


def test_mixed_batches_and_reuse(case):
    K.mixed_batches_and_reuse(*case)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation(tmp_path, graphs):
    """Captured decode graphs: replays advance the memories exactly once per step (the capture's
    warm-up runs are rolled back), finished rows write the scratch state row."""
    cfg = C.CASES["mixed"]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=2))
    eng = C.engine(path, backend="hip", dtype=torch.float32, rows=4, use_hip_graphs=graphs, precapture_graphs=False)
    try:
        K.greedy_generation(K.Env("hip", "cuda"), cfg, sd, eng, tie=0.05)
    finally:
        eng.shutdown()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed, dtype):
    K.drawn_configuration(K.Env("hip", "cuda", getattr(torch, dtype)), tmp_path, seed)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(C.ONE_KIND))
def test_models_of_one_kind_of_mixer(tmp_path, name, dtype):
    K.drawn_configuration(K.Env("hip", "cuda", getattr(torch, dtype)), tmp_path, 3, cfg=C.ONE_KIND[name])


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_context_chunks_across_decode_splits(tmp_path, dtype):
    """Chunks longer than a decode split and a context several chunks long: the decode kernel starts
    at the chunk's first split, the memories run hundreds of tokens."""
    cfg = C.config([C.layer("attention", C.attn(4, 2, 32, 32, 200, 16, 50000.0, 0.2, True)),
                    C.layer("mlstm", C.mlstm(4, 32, 16)), C.layer("mlstm", C.mlstm(2, 16, 32, 3.0), 0),
                    C.layer("attention", C.attn(2, 2, 16, 32, 131, 16, 50000.0, 0.3, True), 0)],
                   width=64, vocab=80, streams=4)
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=11))
    e = K.Env("hip", "cuda", getattr(torch, dtype))
    e.measure_noise(path, cfg, sd)
    eng = C.engine(path, backend="hip", dtype=e.dtype, pool_tokens=1024, max_len=1024)
    try:
        toks = C.tokens(700, cfg["vocab"], 3)
        want = O.forward(sd, cfg, toks)
        idx = list(range(0, 520, 7)) + [519]
        e.close(eng.stream_step([("x", toks[:520], idx)]), want[idx])
        got = [eng.stream_step([("x", toks[p:p + 1], [0])]) for p in range(520, 600)]
        e.close(torch.cat(got), want[520:600])
        e.close(eng.stream_step([("x", toks[600:], list(range(100)))], end=["x"]), want[600:])
    finally:
        eng.shutdown()

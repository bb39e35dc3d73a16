"""Mabivik on the HIP backend against the float64 oracle: every mechanism's kernels alone (fp32 and
bf16), packed steps of the engine (prompt portions beside single tokens, page and state-row
reuse), and greedy generation through the scheduler with captured decode graphs."""
import numpy as np
import pytest
import torch

import mabivik_cases as C
import mabivik_checks as K
import mabivik_oracle as O
from test_mabivik_cpu import LATENT

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


@pytest.fixture(params=DTYPES)
def env(request):
    e = K.Env("hip", "cuda", getattr(torch, request.param))
    assert e.ops.name == "hip"
    return e


# ------------------------------------------------------------------ mechanisms
def test_dynamic_tanh_norms_around_the_stream(env):
    K.check_norms(env)


@pytest.mark.parametrize("taps,cuts", [(4, [1, 1, 2, 5, 1, 3]), (2, [3, 1, 9]), (5, [2, 2, 2, 7]), (1, [6, 7]), (3, [13])])
def test_convolution_with_bias_continues_from_its_state_row(env, taps, cuts):
    K.check_conv_bias(env, taps, cuts)


@pytest.mark.parametrize("name", list(LATENT))
def test_latent_attention_whole_and_in_portions(env, name):
    for cuts in (None, [2, 14, 1, 1, 17, 2, 8]):
        got, want = K.run_mixer(env, LATENT[name], 45, cuts, seed=3)
        env.close(got, want)


def test_latent_attention_exact_and_wide_shapes(env):
    """Cached rows on the 16-wide MFMA grid (the straight-line instances), of 160 and 256 features
    (the wide one-map instance) and of 320 (the widest), several 64-row tiles and decode splits."""
    for heads, dim, rot, vdim, rank, window in [(4, 32, 32, 32, 64, 70), (2, 64, 32, 48, 128, 150), (3, 48, 64, 32, 192, 0),
                                                (17, 16, 16, 16, 32, 40), (2, 32, 64, 24, 256, 90)]:
        layers = [C.layer("latent_attention", C.latent(heads, dim, rot, vdim, 24, rank, window), 0)]
        got, want = K.run_mixer(env, layers, 200, [150, 1, 1, 40, 1, 1, 1, 1, 1, 1, 1, 1], seed=heads, width=48)
        env.close(got, want)


def test_window_edge_shows_with_one_loud_key(env):
    whole = K.check_window_edge(env)
    steps = K.check_window_edge(env, cuts=[10] + [1] * 20)
    if env.dtype == torch.float32:
        env.close(steps, whole.double().cpu().numpy(), 1e-4)
    K.check_window_edge(env, window=16, T=40, loud=15, cuts=[3, 2, 11] + [1] * 24)   # the edge falls on a page border
    K.check_window_edge(env, window=130, T=300, loud=100, cuts=[200] + [1] * 100)    # ... and past a decode split


def test_far_key_among_hundreds(env):
    m = C.latent(2, 16, 8, 16, 12, 16, 0, 10000.0, None)
    layers = [C.layer("latent_attention", m, 0)]
    got, want = K.run_mixer(env, layers, 300, [290] + [1] * 10, K.loud_key(3), seed=6)
    env.close(got, want)
    _, without = K.run_mixer(env, layers, 300, None, None, seed=6)
    assert np.abs(want[295:] - without[295:]).max() > 0.05


@pytest.mark.parametrize("H,G,d,e,taps", [(4, 2, 16, 12, 4), (3, 3, 20, 18, 2), (2, 1, 8, 8, 0), (6, 2, 70, 33, 3), (1, 1, 5, 3, 5),
                                          (4, 1, 128, 64, 4)])
def test_delta_rule_per_head_decay_in_portions(env, H, G, d, e, taps):
    layers = [C.layer("delta", C.delta(H, G, d, e, taps), 0)]
    for cuts in (None, [1, 1, 2, 9, 1, 16, 10]):
        got, want = K.run_mixer(env, layers, 40, cuts, seed=H)
        env.close(got, want)


@pytest.mark.parametrize("H,e,N,G,taps,parts", [(4, 12, 16, 2, 3, 2), (2, 8, 8, 1, 0, 1), (6, 22, 72, 3, 5, 3), (3, 5, 7, 3, 2, 1),
                                                (4, 6, 10, 1, 4, 4), (8, 64, 128, 2, 4, 2)])
def test_state_space_mixer_in_portions(env, H, e, N, G, taps, parts):
    layers = [C.layer("mamba2", C.mamba2(H, e, N, G, taps, parts), 0)]
    for cuts in (None, [1, 1, 2, 9, 1, 16, 10]):
        got, want = K.run_mixer(env, layers, 40, cuts, seed=H + e)
        env.close(got, want)


@pytest.mark.parametrize("E,top,ff", [(5, 2, 24), (1, 1, 8), (4, 4, 16), (9, 3, 72), (3, 1, 7), (6, 2, 64)])
def test_table_routed_gated_experts(env, E, top, ff):
    K.check_experts(env, E, top, ff)
    K.check_experts(env, E, top, ff, W=64, T=150)


def test_token_input_after_the_feed_forward(env):
    K.check_token_side(env)


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


def test_residual_stream_after_every_layer(case):
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
    """Captured decode graphs: replays advance the recurrent state exactly once per step (the
    capture's warm-up runs are rolled back), finished rows write the scratch state row."""
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
def test_long_context_window_across_decode_splits(tmp_path, dtype):
    """A window longer than a decode split and a context several windows long: the decode kernel
    starts at the window's first split, the recurrences run hundreds of tokens."""
    cfg = C.config([C.layer("latent_attention", C.latent(4, 32, 16, 32, 24, 48, 200, 50000.0, (4.0, 128, 16.0, 1.0))),
                    C.layer("mamba2", C.mamba2(4, 16, 32, 2, 4, 2)), C.layer("delta", C.delta(2, 2, 32, 16, 4)),
                    C.layer("latent_attention", C.latent(2, 16, 16, 24, 12, 48, 131, 50000.0, (4.0, 128, 16.0, 1.0), kv_from=0), 0)],
                   width=64, vocab=80)
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=11))
    e = K.Env("hip", "cuda", getattr(torch, dtype))
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

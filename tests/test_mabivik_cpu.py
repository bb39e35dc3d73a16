"""Mabivik on the torch backend (CPU, fp32) against the float64 oracle (tests/mabivik_oracle.py):
mechanisms one by one, then the engine's packed steps, paging, state-row reuse and generation."""
import numpy as np
import pytest
import torch

import mabivik_cases as C
import mabivik_checks as K
import mabivik_oracle as O
from byzantine_consensus_llm_agents_amd.models.config import MabivikConfig, from_hf_config
from byzantine_consensus_llm_agents_amd.ops import reference as ref

ENV = K.Env("torch", "cpu")


# ------------------------------------------------------------------ mechanisms
def test_dynamic_tanh_norms_around_the_stream():
    K.check_norms(ENV)


@pytest.mark.parametrize("taps,cuts", [(4, [1, 1, 2, 5, 1, 3]), (2, [3, 1, 9]), (5, [2, 2, 2, 7]), (1, [6, 7]), (3, [13])])
def test_convolution_with_bias_continues_from_its_state_row(taps, cuts):
    K.check_conv_bias(ENV, taps, cuts)


def test_ramped_frequencies():
    for dims, base, sc in [(32, 1e6, (4.0, 512, 32.0, 1.0)), (8, 5000.0, (3.0, 48, 8.0, 1.0)), (64, 1e4, (16.0, 4096, 32.0, 1.0)),
                           (6, 100.0, (2.0, 16, 2.0, 4.0)), (16, 1e4, None), (24, 300.0, (8.0, 32, 4.0, 0.5))]:
        scaling = dict(zip(("factor", "original", "fast", "slow"), sc)) if sc else None
        want, amp = O.ramp_freqs(dims, base, scaling)
        got, got_amp = ref.ramp_inv_freq(dims, base, sc)
        np.testing.assert_allclose(got.double().numpy(), want, rtol=1e-6)
        assert abs(amp - got_amp) < 1e-12
    # the ramp does something: low frequencies are divided by the factor, high ones kept
    f, _ = O.ramp_freqs(32, 1e6, {"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0})
    plain = np.array([1e6 ** (-2.0 * i / 32) for i in range(16)])
    assert f[0] == plain[0] and abs(f[-1] - plain[-1] / 4.0) < 1e-12 and np.any((f < plain * 0.999) & (f > plain / 4.0 * 1.001))


LATENT = {
    "plain": [C.layer("latent_attention", C.latent(), 0)],
    "no-window-half-rot": [C.layer("latent_attention", C.latent(2, 16, 16, 16, 16, 16, 0, 10000.0, None, rot_dims=8), 0)],
    "one-head-window-1": [C.layer("latent_attention", C.latent(1, 5, 6, 7, 3, 9, 1, 100.0, (2.0, 16, 2.0, 4.0), 0.3), 0)],
    "wide-row": [C.layer("latent_attention", C.latent(3, 24, 20, 10, 30, 120, 17), 0)],
    "borrowed": [C.layer("latent_attention", C.latent(), 0), C.layer("delta", C.delta(), 0),
                 C.layer("latent_attention", C.latent(5, 10, 8, 6, 7, 24, 6, kv_from=0), 0)],
}


@pytest.mark.parametrize("name", list(LATENT))
def test_latent_attention_whole_and_in_portions(name):
    for cuts in (None, [2, 14, 1, 1, 17, 2, 8]):
        got, want = K.run_mixer(ENV, LATENT[name], 45, cuts, seed=3)
        ENV.close(got, want)


def test_window_edge_shows_with_one_loud_key():
    whole = K.check_window_edge(ENV)
    steps = K.check_window_edge(ENV, cuts=[10] + [1] * 20)
    ENV.close(steps, whole.double().numpy(), 1e-4)
    K.check_window_edge(ENV, window=16, T=40, loud=15, cuts=[3, 2, 11] + [1] * 24)   # the edge falls on a page border


def test_far_key_among_hundreds():
    m = C.latent(2, 16, 8, 16, 12, 16, 0, 10000.0, None)
    layers = [C.layer("latent_attention", m, 0)]
    got, want = K.run_mixer(ENV, layers, 300, [290] + [1] * 10, K.loud_key(3), seed=6)
    ENV.close(got, want)
    _, without = K.run_mixer(ENV, layers, 300, None, None, seed=6)
    assert np.abs(want[295:] - without[295:]).max() > 0.05   # the far key carries weight at the end


@pytest.mark.parametrize("H,G,d,e,taps", [(4, 2, 16, 12, 4), (3, 3, 20, 18, 2), (2, 1, 8, 8, 0), (6, 2, 70, 33, 3), (1, 1, 5, 3, 5)])
def test_delta_rule_per_head_decay_in_portions(H, G, d, e, taps):
    layers = [C.layer("delta", C.delta(H, G, d, e, taps), 0)]
    for cuts in (None, [1, 1, 2, 9, 1, 16, 10]):
        got, want = K.run_mixer(ENV, layers, 40, cuts, seed=H)
        ENV.close(got, want)


@pytest.mark.parametrize("H,e,N,G,taps,parts", [(4, 12, 16, 2, 3, 2), (2, 8, 8, 1, 0, 1), (6, 22, 72, 3, 5, 3), (3, 5, 7, 3, 2, 1),
                                                (4, 6, 10, 1, 4, 4)])
def test_state_space_mixer_in_portions(H, e, N, G, taps, parts):
    layers = [C.layer("mamba2", C.mamba2(H, e, N, G, taps, parts), 0)]
    for cuts in (None, [1, 1, 2, 9, 1, 16, 10]):
        got, want = K.run_mixer(ENV, layers, 40, cuts, seed=H + e)
        ENV.close(got, want)


@pytest.mark.parametrize("E,top,ff", [(5, 2, 24), (1, 1, 8), (4, 4, 16), (9, 3, 72), (3, 1, 7)])
def test_table_routed_gated_experts(E, top, ff):
    K.check_experts(ENV, E, top, ff)


def test_token_input_after_the_feed_forward():
    K.check_token_side(ENV)


def test_config_round_trip(tmp_path):
    for name, cfg in C.CASES.items():
        path = str(tmp_path / name)
        C.checkpoint(cfg, path)
        read = from_hf_config(path)
        assert isinstance(read, MabivikConfig) and read.family == "mabivik"
        assert MabivikConfig.from_dict(read.to_dict(), "x").layers == read.layers
        assert read.logit_scale == cfg["logit_scale"] and read.side_dim == (cfg.get("token_side") or {}).get("dim", 0)
    bad = C.config([C.layer("latent_attention", C.latent(kv_from=0))])
    with pytest.raises(ValueError):
        MabivikConfig.from_dict(bad)   # a layer cannot borrow from itself


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module", params=list(C.CASES))
def case(request, tmp_path_factory):
    path = str(tmp_path_factory.mktemp(request.param))
    cfg = C.CASES[request.param]
    sd = O.to_f64(C.checkpoint(cfg, path, seed=len(request.param)))
    eng = C.engine(path, pool_tokens=320)
    yield cfg, sd, eng
    eng.shutdown()


def test_whole_prompt_every_position(case):
    K.whole_prompt(ENV, *case)


def test_residual_stream_after_every_layer(case):
    K.stream_after_every_layer(ENV, *case)


def test_prefill_then_token_by_token(case):
    K.prefill_then_token_by_token(ENV, *case)


def test_first_tokens_one_by_one(case):
    K.first_tokens_one_by_one(ENV, *case)


@pytest.mark.parametrize("sizes", [[2, 2, 3, 17, 16, 1, 31, 2, 5], [15, 1, 1, 16, 33, 11]])
def test_portions_of_changing_size(case, sizes):
    K.portions(ENV, *case, sizes)


def test_mixed_batches_equal_each_alone_and_reuse_pages_and_rows(case):
    K.mixed_batches_and_reuse(ENV, *case)


def test_long_decoding(case):
    cfg, sd, eng = case
    toks = C.tokens(150, cfg["vocab"], 6)
    want = O.forward(sd, cfg, toks)
    eng.stream_step([("l", toks[:4], [])])
    for p in range(4, 150):
        got = eng.stream_step([("l", toks[p:p + 1], [0])], end=["l"] if p == 149 else [])
        if p % 9 == 0 or p > 140:
            ENV.close(got, want[p:p + 1])


def test_greedy_generation_through_the_scheduler(case):
    K.greedy_generation(ENV, *case)


def test_generate_command_line(tmp_path, capsys):
    from byzantine_consensus_llm_agents_amd.engine.generate import main
    cfg = C.CASES["mixed"]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=6))
    prompts = [C.tokens(7, cfg["vocab"], 1), C.tokens(20, cfg["vocab"], 2)]
    argv = ["--weights", path, "--backend", "torch", "--dtype", "float32", "--max-tokens", "3", "--max-model-len", "64"]
    for p in prompts:
        argv += ["--prompt", " ".join(map(str, p))]
    assert main(argv) == 0
    lines = [l for l in capsys.readouterr().out.strip().splitlines() if l.strip()]
    assert len(lines) == 2
    for p, line in zip(prompts, lines):
        ids = [int(t) for t in line.split()]
        assert len(ids) == 3 and ids[0] == int(O.forward(sd, cfg, p)[-1].argmax())


@pytest.mark.parametrize("seed", range(8, 14))
def test_drawn_configurations(tmp_path, seed):
    K.drawn_configuration(ENV, tmp_path, seed)


def test_text_entry_point_with_id_prompts(tmp_path):
    from byzantine_consensus_llm_agents_amd.engine import LLM, SamplingParams
    cfg = C.CASES["plain"]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=4))
    llm = LLM(path, backend="torch", weights=path, seed=1, max_model_len=128, kv_cache_gb=0.01, max_batch_seqs=4, dtype=torch.float32)
    try:
        prompt = C.tokens(12, cfg["vocab"], 8)
        out = llm.generate(" ".join(map(str, prompt)), SamplingParams(temperature=0.0, max_tokens=5))[0].outputs[0].text
        ids = [int(t) for t in out.split()]
        assert len(ids) == 5 and ids[0] == int(O.forward(sd, cfg, prompt)[-1].argmax())
    finally:
        llm.shutdown()

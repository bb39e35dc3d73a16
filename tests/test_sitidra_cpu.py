"""Sitidra on the torch backend (CPU, fp32) against the float64 oracle (tests/sitidra_oracle.py):
mechanisms one by one, then the engine's packed steps, paging, state-row reuse and generation."""
import numpy as np
import pytest
import torch

import sitidra_cases as C
import sitidra_checks as K
import sitidra_oracle as O
from byzantine_consensus_llm_agents_amd.models.config import SitidraConfig, from_hf_config

ENV = K.Env("torch", "cpu")


# ------------------------------------------------------------------ mechanisms
@pytest.mark.parametrize("S", [1, 2, 3, 4, 7, 16])
def test_streams_read_write_and_layer_norm(S):
    K.check_streams(ENV, S)
    K.check_streams(ENV, S, W=50)


ATTENTION = {
    "gqa-partial-rotary": [C.layer("attention", C.attn(), 0)],
    "mha-full-rotary-chunk-7": [C.layer("attention", C.attn(2, 2, 24, 12, 7, 24), 0)],
    "no-mask-no-rotary": [C.layer("attention", C.attn(3, 1, 8, 16, 0, 0), 0)],
    "chunk-1": [C.layer("attention", C.attn(2, 1, 16, 8, 1, 4), 0)],
    "off-grid-chunk-37": [C.layer("attention", C.attn(5, 1, 40, 36, 37, 18, 20000.0, 0.3), 0)],
    "wide-head": [C.layer("attention", C.attn(2, 2, 70, 18, 16, 70, 300.0, 0.11), 0)],
    "lender-alone": [C.layer("attention", C.attn(v_mix=True), 0)],
    "mixed-values": [C.layer("attention", C.attn(v_mix=True), 0), C.layer("mlstm", C.mlstm(), 0),
                     C.layer("attention", C.attn(6, 2, 10, 12, 9, 6, v_mix=True), 0)],
}


@pytest.mark.parametrize("name", list(ATTENTION))
def test_attention_whole_and_in_portions(name):
    for cuts in (None, [2, 14, 1, 1, 17, 2, 8]):
        got, want = K.run_mixer(ENV, ATTENTION[name], 45, cuts, seed=3)
        ENV.close(got, want)


def test_value_mixing_uses_the_first_layers_values():
    layers = ATTENTION["mixed-values"]
    _, want = K.run_mixer(ENV, layers, 20, None, seed=3)

    def no_mix(sd, hs):
        sd["l2.mix.vmix"] = torch.zeros((), dtype=torch.bfloat16)
    _, plain = K.run_mixer(ENV, layers, 20, None, no_mix, seed=3)
    assert np.abs(want - plain).max() > 0.05


def test_chunk_edge_shows_with_one_loud_value():
    whole = K.check_chunk_edge(ENV)
    steps = K.check_chunk_edge(ENV, cuts=[19] + [1] * 21)   # the loud row and both edges are decoded alone
    ENV.close(steps, whole.double().numpy(), 1e-4)
    K.check_chunk_edge(ENV, chunk=16, T=60, cuts=[3, 2, 11, 17] + [1] * 27)   # the edges fall on page borders
    K.check_chunk_edge(ENV, chunk=23, T=80, cuts=[45, 2, 22, 1, 1, 1, 8])     # a portion starts inside a chunk


def test_far_value_inside_a_long_chunk():
    m = C.attn(2, 1, 16, 16, 0, 8, scale=0.05)
    layers = [C.layer("attention", m, 0)]
    got, want = K.run_mixer(ENV, layers, 300, [290] + [1] * 10, K.loud_value(3), seed=6)
    ENV.close(got, want)
    _, without = K.run_mixer(ENV, layers, 300, None, None, seed=6)
    assert np.abs(want[295:] - without[295:]).max() > 0.05   # the far key carries weight at the end


@pytest.mark.parametrize("H,d,e,cap", [(3, 12, 20, 15.0), (1, 5, 3, 2.0), (2, 72, 70, 8.0), (5, 20, 33, 50.0), (4, 16, 16, 0.5)])
def test_matrix_memory_in_portions(H, d, e, cap):
    layers = [C.layer("mlstm", C.mlstm(H, d, e, cap), 0)]
    for cuts in (None, [1, 1, 2, 9, 1, 16, 10]):
        got, want = K.run_mixer(ENV, layers, 40, cuts, seed=H)
        ENV.close(got, want)


@pytest.mark.parametrize("i_bias,f_bias", [(6.0, -4.0), (-9.0, 5.0), (0.0, 0.0)])
def test_matrix_memory_gate_regimes(i_bias, f_bias):
    """Open input gates (the running maximum grows and the floor of the denominator vanishes), closed
    ones (the maximum stays at its start and the floor decides) and the middle."""
    def craft(sd, hs):
        sd["l0.mix.i.b"] = torch.full_like(sd["l0.mix.i.b"], i_bias)
        sd["l0.mix.f.b"] = torch.full_like(sd["l0.mix.f.b"], f_bias)
    layers = [C.layer("mlstm", C.mlstm(2, 8, 12, 12.0), 0)]
    whole, want = K.run_mixer(ENV, layers, 120, None, craft, seed=2)
    ENV.close(whole, want)
    steps, _ = K.run_mixer(ENV, layers, 120, [50] + [1] * 70, craft, seed=2)
    ENV.close(steps, want)


@pytest.mark.parametrize("E,top,groups,keep,shift", [(12, 2, 2, 1, 0.0), (6, 2, 3, 2, -2.0), (8, 3, 0, 0, 0.0), (8, 5, 8, 5, -1.5),
                                                     (9, 3, 3, 1, 0.3), (4, 4, 2, 2, 0.0), (1, 1, 1, 1, 0.0), (10, 1, 5, 2, -3.0)])
def test_grouped_sigmoid_router(E, top, groups, keep, shift):
    K.check_router(ENV, E, top, groups, keep, 1.7, corr_shift=shift)


@pytest.mark.parametrize("E,top,groups,keep,ff,shared", [(6, 2, 3, 2, 24, 20), (1, 1, 0, 0, 8, 0), (4, 4, 2, 2, 16, 7), (9, 3, 3, 1, 72, 40)])
def test_routed_and_shared_experts(E, top, groups, keep, ff, shared):
    K.check_experts(ENV, E, top, groups, keep, ff, shared)


def test_config_round_trip(tmp_path):
    for name, cfg in C.CASES.items():
        path = str(tmp_path / name)
        C.checkpoint(cfg, path)
        read = from_hf_config(path)
        assert isinstance(read, SitidraConfig) and read.family == "sitidra"
        assert SitidraConfig.from_dict(read.to_dict(), "x") == SitidraConfig.from_dict(cfg, "x")
        assert read.streams == cfg.get("streams", 0) and read.logit_softcap == cfg.get("logit_softcap", 0.0)
    with pytest.raises(ValueError):   # more experts asked for than the kept groups hold
        SitidraConfig.from_dict(C.config([C.layer("mlstm", C.mlstm(), 8, 6, 3, (3, 1))]))
    with pytest.raises(ValueError):   # mixed values of two shapes
        SitidraConfig.from_dict(C.config([C.layer("attention", C.attn(v_mix=True)), C.layer("attention", C.attn(vdim=8, v_mix=True))]))


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


def test_summed_streams_after_every_layer(case):
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


@pytest.mark.parametrize("name", list(C.ONE_KIND))
def test_models_of_one_kind_of_mixer(tmp_path, name):
    K.drawn_configuration(ENV, tmp_path, 3, cfg=C.ONE_KIND[name])


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

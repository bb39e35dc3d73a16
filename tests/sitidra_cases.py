"""Small Sitidra configurations, random checkpoints on disk and engines for the tests."""
import json
import os

import torch

from byzantine_consensus_llm_agents_amd.models.config import SitidraConfig
from byzantine_consensus_llm_agents_amd.models.sitidra import SitidraModel
from mabivik_cases import Pages, segments, tokens  # noqa: F401  (page tables and segment tables of a packed step)


def attn(heads=4, kv_heads=2, dim=16, vdim=12, chunk=20, rot=8, base=5000.0, scale=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 0.6}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    if chunk:
        m["mask"] = {"size": chunk}
    if v_mix:
        m["v_mix"] = True
    return m


def mlstm(heads=3, dim=12, vdim=20, cap=15.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def layer(kind, mixer, ff=24, experts=6, top=2, groups=(3, 2), scale=1.5, shared=20):
    mlp = None
    if ff:
        router = {"experts": experts, "top": top, "scale": scale}
        if groups:
            router["groups"] = {"count": groups[0], "keep": groups[1]}
        mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
        if shared:
            mlp["shared"] = {"ff": shared}
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=48, vocab=53, streams=3, eps=1e-5, softcap=8.0):
    c = {"architecture": "Sitidra", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if streams:
        c["streams"] = streams
    if softcap:
        c["logit_softcap"] = softcap
    return c


# every branch: a lender of values and two borrowers, layers without feed-forward, attention without
# mask / rotary / value mixing, full and partial rotary, GQA / MHA / one KV head, chunks shorter than a
# page, across pages and off the 16-key tiles, no streams (the plain residual) and one stream with
# coefficients, no logit cap, routing without groups, one expert per group, every allowed expert
# chosen, no shared expert, sizes off the 16-wide MFMA grid and off the 4-element grid
CASES = {
    "mixed": config([layer("attention", attn(v_mix=True)), layer("mlstm", mlstm()), layer("mlstm", mlstm(2, 16, 8, 4.0), ff=0),
                     layer("attention", attn(2, 2, 24, 12, 7, 24, v_mix=True), 16, 4, 1, (2, 1)),
                     layer("attention", attn(3, 1, 8, 16, 0, 4), 40, 3, 3, None, 1.0, 0),
                     layer("attention", attn(6, 2, 16, 12, 33, 0, v_mix=True), 0)]),
    "plain": config([layer("mlstm", mlstm(2, 8, 8, 30.0), 16, 2, 1, None, 1.0, 0), layer("attention", attn(2, 2, 16, 16, 0, 0), 0),
                     layer("attention", attn(2, 1, 16, 16, 5, 16), 16, 4, 2, (4, 3), 2.5, 8)],
                    width=32, vocab=37, streams=0, softcap=0),
    "wide": config([layer("mlstm", mlstm(2, 72, 70, 8.0), 56, 9, 3, (3, 1), 0.7, 44),
                    layer("attention", attn(5, 1, 40, 36, 37, 18, 20000.0, 0.3), 24, 6, 4, (3, 2)),
                    layer("mlstm", mlstm(5, 20, 33), 0),
                    layer("attention", attn(2, 2, 70, 18, 64, 70, 300.0, 0.11), 40, 8, 2, (8, 5))],
                   width=72, vocab=45, streams=4, eps=1e-6, softcap=25.0),
    "one_stream": config([layer("attention", attn(2, 1, 32, 32, 16, 32)), layer("mlstm", mlstm(1, 32, 32))], width=40, streams=1),
}


# models of one kind of mixer: no K / V pages at all, no state tables at all
ONE_KIND = {
    "memories": config([layer("mlstm", mlstm(2, 16, 12)), layer("mlstm", mlstm(3, 8, 20, 3.0), 0)], width=40, streams=2),
    "attention": config([layer("attention", attn(4, 4, 16, 16, 24, 8, v_mix=True), 0), layer("attention", attn(2, 1, 32, 8, 0, 32))],
                        width=40, streams=2, softcap=0),
}


def checkpoint(cfg_dict, path, seed=0):
    """Write config.json + model.safetensors (bf16) under `path`; returns the tensors."""
    from safetensors.torch import save_file
    cfg = SitidraConfig.from_dict(cfg_dict, "test")
    sd = SitidraModel(cfg, None, "cpu").random_state_dict(seed, std=0.12)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg_dict, fh)
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    return sd


def engine(path, backend="torch", dtype=torch.float32, pool_tokens=512, rows=4, max_len=512, **kw):
    from byzantine_consensus_llm_agents_amd.engine.engine import EngineArgs, InferenceEngine
    args = EngineArgs.from_configs(path, backend=backend, weights=path, seed=0, dtype=dtype, kv_block_size=16,
                                   max_batch_seqs=rows, max_model_len=max_len, kv_pool_tokens=pool_tokens,
                                   use_hip_graphs=kw.pop("use_hip_graphs", False), prefix_caching=kw.pop("prefix_caching", False),
                                   **kw)
    return InferenceEngine(args)


def random_config(seed):
    """A configuration drawn from a seed: sizes, head counts, layer order, chunks, routing, constants."""
    import random
    r = random.Random(seed)
    even = lambda lo, hi: 2 * r.randint(lo // 2, hi // 2)  # noqa: E731
    layers = []
    mix_shape = (r.choice([1, 2, 3]), r.randint(3, 40))   # KV heads and value width of the layers that mix values
    for _ in range(r.randint(2, 6)):
        kind = r.choice(["attention", "mlstm"])
        if kind == "attention":
            v_mix = r.random() < 0.5
            kv, vdim = mix_shape if v_mix else (r.choice([1, 2, 3]), r.randint(3, 72))
            dim = r.randint(3, 72)
            m = attn(kv * r.choice([1, 2, 4]), kv, dim, vdim, r.choice([0, 1, 5, 16, 23, 64]), r.choice([0, even(2, dim)]),
                     r.choice([100.0, 10000.0, 1000000.0]), r.choice([0.05, 0.3, 1.0]), v_mix)
        else:
            m = mlstm(r.randint(1, 5), r.randint(3, 80), r.randint(3, 72), r.choice([1.5, 15.0, 50.0]))
        ff = r.choice([0, 8, 24, 40, 72])
        groups = r.choice([1, 2, 3])
        per = r.randint(1, 4)
        keep = r.randint(1, groups)
        layers.append(layer(kind, m, ff, groups * per, r.randint(1, keep * per), r.choice([None, (groups, keep)]) if keep == groups
                            else (groups, keep), r.choice([1.0, 2.5]), r.choice([0, 8, 33])))
    return config(layers, width=even(24, 96), vocab=r.randint(20, 90), streams=r.choice([0, 1, 2, 4, 5]),
                  eps=r.choice([1e-5, 1e-6]), softcap=r.choice([0, 5.0, 20.0]))

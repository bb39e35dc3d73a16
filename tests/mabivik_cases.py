"""Small Mabivik configurations, random checkpoints on disk and engines for the tests."""
import json
import os

import torch

from byzantine_consensus_llm_agents_amd.models.config import MabivikConfig
from byzantine_consensus_llm_agents_amd.models.mabivik import MabivikModel


def latent(heads=3, dim=16, rot_dim=8, vdim=12, q_rank=20, kv_rank=24, window=20, base=5000.0, scaling=(3.0, 48, 8.0, 1.0),
           scale=None, kv_from=None, rot_dims=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
         "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def delta(heads=4, kv_heads=2, dim=16, vdim=12, conv=4):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim}
    if conv:
        m["conv"] = conv
    return m


def mamba2(heads=4, vdim=12, state=16, groups=2, conv=3, norm_groups=2):
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups}
    if conv:
        m["conv"] = conv
    return m


def layer(kind, mixer, ff=24, experts=5, top=2):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}} if ff else None
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=48, vocab=53, scale=2.0, eps=1e-5, logit_scale=0.5, side=6):
    c = {"architecture": "Mabivik", "width": width, "vocab": vocab, "embedding": {"scale": scale}, "norm": {"eps": eps},
         "logit_scale": logit_scale, "layers": layers}
    if side:
        c["token_side"] = {"dim": side}
    return c


# every branch: a cache lent to a later layer (twice), layers without feed-forward, no token input,
# no window, no frequency scaling, fewer rotated features than the rotated part, GQA and MHA in the
# delta rule, one and several groups / norm parts, no convolution, taps 2 .. 5, one expert per
# token and all of them, sizes off the 16-wide MFMA grid and off the 4-element grid, a cached row
# wider than 128 features, windows shorter than a page and across pages
CASES = {
    "mixed": config([layer("latent_attention", latent()), layer("mamba2", mamba2()), layer("delta", delta(), ff=0),
                     layer("latent_attention", latent(2, 12, 8, 20, 9, 24, 7, kv_from=0), 16, 4, 1),
                     layer("delta", delta(3, 3, 20, 18, 2), 40, 3, 3),
                     layer("latent_attention", latent(4, 8, 8, 8, 16, 24, 33, kv_from=0), 0)]),
    "plain": config([layer("mamba2", mamba2(2, 8, 8, 1, 0, 1), 16, 2, 1), layer("delta", delta(2, 1, 8, 8, 0), 0),
                     layer("latent_attention", latent(2, 16, 16, 16, 16, 16, 0, 10000.0, None, rot_dims=8), 16, 3, 2)],
                    width=32, vocab=37, scale=1.0, logit_scale=1.0, side=0),
    "wide": config([layer("delta", delta(2, 1, 80, 72, 3), 56, 7, 2),
                    layer("latent_attention", latent(5, 40, 36, 44, 50, 108, 37, 20000.0, (4.0, 64, 16.0, 2.0)), 24, 6, 4),
                    layer("mamba2", mamba2(6, 22, 72, 3, 5, 3), 0),
                    layer("latent_attention", latent(2, 70, 30, 18, 24, 13, 5, 300.0, (8.0, 32, 4.0, 0.5)), 40, 9, 2)],
                   width=64, vocab=45, eps=1e-6, logit_scale=2.0, side=3),
}


def checkpoint(cfg_dict, path, seed=0):
    """Write config.json + model.safetensors (bf16, int32 expert tables) under `path`; returns the tensors."""
    from safetensors.torch import save_file
    cfg = MabivikConfig.from_dict(cfg_dict, "test")
    sd = MabivikModel(cfg, None, "cpu").random_state_dict(seed, std=0.12)
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


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def segments(parts, rows, device="cpu"):
    """AttnMeta of a packed step over segments ``parts`` = [(first position, count)] that continue
    the state rows ``rows`` (no KV fields: for ops that only read the segment tables)."""
    from byzantine_consensus_llm_agents_amd.models.transformer import AttnMeta
    pos, seg, qs = [], [], [0]
    for i, (a, n) in enumerate(parts):
        pos += list(range(a, a + n))
        seg += [i] * n
        qs.append(qs[-1] + n)
    i32 = dict(dtype=torch.int32, device=device)
    return AttnMeta(positions=torch.tensor(pos, **i32), slots=None, block_tables=None, seq_lens=None,
                    q_start=torch.tensor(qs, **i32), state_rows=torch.tensor(rows, **i32), token_seq=torch.tensor(seg, **i32))


class Pages:
    """Shuffled pages for sequences of the final lengths ``lens``; ``meta(parts)`` is the AttnMeta
    of a packed step over ``parts`` = [(sequence, first position, count)] (sequence i continues
    state row i)."""

    def __init__(self, lens, block_size=16, seed=0, device="cpu"):
        import random
        self.bs, self.device = block_size, device
        need = [(n + block_size - 1) // block_size for n in lens]
        ids = list(range(1, sum(need) + 1))
        random.Random(seed).shuffle(ids)
        self.pages = []
        for n in need:
            self.pages.append(ids[:n])
            ids = ids[n:]
        self.num_blocks = sum(need) + 1   # + scratch block 0

    def meta(self, parts):
        from byzantine_consensus_llm_agents_amd.models.transformer import AttnMeta
        bs = self.bs
        width = max(len(p) for p in self.pages)
        table = torch.zeros(len(parts), width, dtype=torch.int32)
        pos, slots, seg, qs, tiles, single, rows, lens = [], [], [], [0], [], [], [], []
        for i, (s, a, n) in enumerate(parts):
            table[i, :len(self.pages[s])] = torch.tensor(self.pages[s], dtype=torch.int32)
            for q in range(a, a + n):
                pos.append(q)
                slots.append(self.pages[s][q // bs] * bs + q % bs)
                seg.append(i)
            if n == 1 and a > 0:
                single.append([qs[-1], i])
            else:
                tiles += [[i, r, min(r + 64, qs[-1] + n)] for r in range(qs[-1], qs[-1] + n, 64)]
            qs.append(qs[-1] + n)
            rows.append(s)
            lens.append(a + n)
        i32 = dict(dtype=torch.int32, device=self.device)
        return AttnMeta(positions=torch.tensor(pos, **i32), slots=torch.tensor(slots, **i32), block_tables=table.to(self.device),
                        seq_lens=torch.tensor(lens, **i32), q_start=torch.tensor(qs, **i32),
                        tiles=torch.tensor(tiles, **i32).reshape(-1, 3), single=torch.tensor(single, **i32).reshape(-1, 2),
                        state_rows=torch.tensor(rows, **i32), token_seq=torch.tensor(seg, **i32))


def random_config(seed):
    """A configuration drawn from a seed: sizes, head counts, layer order, windows, taps, constants."""
    import random
    r = random.Random(seed)
    even = lambda lo, hi: 2 * r.randint(lo // 2, hi // 2)  # noqa: E731
    layers, lenders = [], []
    for i in range(r.randint(2, 6)):
        kind = r.choice(["latent_attention", "delta", "mamba2"])
        experts = r.randint(1, 9)
        ff = r.choice([0, 8, 24, 40, 72])
        if kind == "latent_attention":
            rot_dim = even(2, 40)
            scaling = r.choice([None, (r.choice([2.0, 4.0, 8.0]), r.choice([16, 64, 256]), r.choice([8.0, 32.0]), r.choice([0.5, 1.0, 2.0]))])
            src = r.choice(lenders) if lenders and r.random() < 0.4 else None
            kv_rank, rd = (layers[src]["mixer"]["kv_rank"], layers[src]["mixer"]["rot_dim"]) if src is not None else (r.randint(3, 140), rot_dim)
            m = latent(r.randint(1, 6), r.randint(3, 72), rd, r.randint(3, 72), r.randint(3, 60), kv_rank,
                       r.choice([0, 1, 5, 16, 23, 64]), r.choice([100.0, 10000.0, 1000000.0]), scaling, r.choice([None, 0.2, 0.05]),
                       src, r.choice([None, even(2, rd)]))
            if src is None:
                lenders.append(i)
            else:   # a borrowed cache holds keys turned the lender's way: the queries turn the same way
                m["rot"] = json.loads(json.dumps(layers[src]["mixer"]["rot"]))
        elif kind == "delta":
            kv = r.choice([1, 2, 3])
            m = delta(kv * r.choice([1, 2, 3]), kv, r.randint(3, 100), r.randint(3, 72), r.choice([0, 2, 3, 4]))
        else:
            groups = r.choice([1, 2, 3])
            heads = groups * r.choice([1, 2, 3])
            vdim = r.randint(2, 40)
            parts = r.choice([p for p in (1, 2, 3, heads) if (heads * vdim) % p == 0])
            m = mamba2(heads, vdim, r.randint(3, 80), groups, r.choice([0, 2, 4, 5]), parts)
        layers.append(layer(kind, m, ff, experts, r.randint(1, experts)))
    return config(layers, width=even(24, 96), vocab=r.randint(20, 90), scale=r.choice([1.0, 3.0]), eps=r.choice([1e-5, 1e-6]),
                  logit_scale=r.choice([1.0, 0.3]), side=r.choice([0, 1, 5, 16]))

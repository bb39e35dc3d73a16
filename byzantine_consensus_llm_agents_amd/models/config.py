"""Decoder architectures served by the engine (shapes from SURVEY.md §2.3).

One ``ModelConfig`` describes every family the reference can select
(``bcg/config.py:20-25``) plus the plumbing model of BASELINE config 1:

* Qwen3 8B/14B/32B - GQA, per-head QK-RMSNorm, no QKV bias, untied head;
* Qwen2.5-0.5B     - QKV bias, tied embeddings, no QK-norm;
* Mistral-Small-Instruct-2409 (22B) - GQA, no bias, no QK-norm, 32k vocab.

Tiny variants exist for CPU tests.  A model directory with an HF
``config.json`` overrides the preset (``from_hf_config``).
"""

import json
import os
from dataclasses import asdict, dataclass, replace
from typing import Optional


@dataclass(frozen=True)
class ModelConfig:
    name: str
    family: str                 # "qwen3" | "qwen2" | "mistral"
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int             # embedding / lm-head rows
    rope_theta: float = 1_000_000.0
    rms_eps: float = 1e-6
    qk_norm: bool = False
    qkv_bias: bool = False
    tie_embeddings: bool = False
    max_position: int = 32768

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        h, i = self.hidden_size, self.intermediate_size
        per_layer = h * (self.q_size + 2 * self.kv_size) + self.q_size * h + 3 * h * i + 2 * h
        if self.qk_norm:
            per_layer += 2 * self.head_dim
        if self.qkv_bias:
            per_layer += self.q_size + 2 * self.kv_size
        emb = self.vocab_size * h * (1 if self.tie_embeddings else 2)
        return per_layer * self.num_layers + emb + h

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.num_layers * self.kv_size * dtype_bytes

    def to_dict(self):
        return asdict(self)


@dataclass(frozen=True)
class MixerSpec:
    """One differential-attention mixer: ``heads`` query heads over ``kv_heads`` key/value
    heads, ``maps`` softmax maps per head (each with its own ``dim``-wide q/k slice, all over
    the same ``vdim``-wide values), rotary on the first ``rot_dims`` features of every map."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    rot_dims: int
    rot_base: float
    maps: int = 2

    @property
    def q_width(self) -> int:
        return self.heads * self.maps * self.dim

    @property
    def k_width(self) -> int:
        return self.kv_heads * self.maps * self.dim

    @property
    def v_width(self) -> int:
        return self.kv_heads * self.vdim


@dataclass(frozen=True)
class FeedForwardSpec:
    """kind "dense": one ``ff``-wide layer.  kind "moe": ``experts`` layers of width ``ff`` of
    which a token uses ``top``, plus an always-on gated expert of width ``shared_ff`` (0 = none)."""
    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    shared_ff: int = 0


@dataclass(frozen=True)
class LayerSpec:
    type: str
    mixer: MixerSpec
    mlp: Optional[FeedForwardSpec]


@dataclass(frozen=True)
class MofidraConfig:
    """Mofidra: parallel-sublayer decoder (one norm feeds the mixer and the feed-forward),
    differential attention, dense or mixture-of-experts feed-forwards, a weight-shared loop
    over a span of layers.  Everything is read from the model directory's config.json; the
    attributes the engine asks every model for (sizes, ``num_layers`` = cache-holding layer
    runs) are derived."""
    name: str
    hidden_size: int
    vocab_size: int
    layers: tuple
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    rms_eps: float = 1e-6
    embed_scale: float = 1.0
    family: str = "mofidra"
    max_position: int = 1 << 20
    tie_embeddings: bool = False

    @classmethod
    def from_dict(cls, c: dict, name: str = "mofidra") -> "MofidraConfig":
        layers = []
        for entry in c["layers"]:
            if entry["type"] != "attention":
                raise ValueError(f"Mofidra: unknown mixer type {entry['type']!r}")
            m = entry["mixer"]
            rot = m.get("rot") or {"dims": 0, "base": 10000.0}
            mixer = MixerSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                              vdim=int(m["vdim"]), scale=float(m["scale"]), diff=float(m["diff"]),
                              rot_dims=int(rot["dims"]), rot_base=float(rot["base"]))
            if mixer.heads % mixer.kv_heads or mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
                raise ValueError("Mofidra: heads must be a multiple of kv_heads, rot.dims even and <= dim")
            f = entry.get("mlp")
            mlp = None
            if f is not None and f["kind"] == "dense":
                mlp = FeedForwardSpec("dense", int(f["ff"]))
            elif f is not None and f["kind"] == "moe":
                shared = f.get("shared") or {}
                mlp = FeedForwardSpec("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]),
                                      int(f["router"]["top"]), int(shared.get("ff", 0)))
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError("Mofidra: router.top must be in [1, experts]")
            elif f is not None:
                raise ValueError(f"Mofidra: unknown feed-forward kind {f['kind']!r}")
            layers.append(LayerSpec(entry["type"], mixer, mlp))
        loop = c.get("loop") or {}
        start, stop = int(loop.get("start", 0)), int(loop.get("stop", 0))
        times = int(loop.get("times", 1))
        if not 0 <= start <= max(start, stop) <= len(layers) or times < 1:
            raise ValueError("Mofidra: loop span outside the layer list")
        return cls(name=name, hidden_size=int(c["width"]), vocab_size=int(c["vocab"]), layers=tuple(layers),
                   loop_start=start, loop_stop=max(start, stop), loop_times=times,
                   rms_eps=float(c["norm"]["eps"]), embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)))

    def to_dict(self) -> dict:
        """The config.json form (inverse of `from_dict`)."""
        out = []
        for l in self.layers:
            m = l.mixer
            entry = {"type": l.type, "mixer": {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                                               "scale": m.scale, "diff": m.diff,
                                               "rot": {"dims": m.rot_dims, "base": m.rot_base}}, "mlp": None}
            if l.mlp is not None and l.mlp.kind == "dense":
                entry["mlp"] = {"kind": "dense", "ff": l.mlp.ff}
            elif l.mlp is not None:
                entry["mlp"] = {"kind": "moe", "expert": {"ff": l.mlp.ff},
                                "router": {"experts": l.mlp.experts, "top": l.mlp.top}}
                if l.mlp.shared_ff:
                    entry["mlp"]["shared"] = {"ff": l.mlp.shared_ff}
            out.append(entry)
        return {"architecture": "Mofidra", "width": self.hidden_size, "vocab": self.vocab_size,
                "embedding": {"scale": self.embed_scale}, "norm": {"eps": self.rms_eps}, "layers": out,
                "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}}

    @property
    def layer_runs(self) -> tuple:
        """Layer index of every layer run, in execution order: the loop span repeats
        ``loop_times`` times with the same weights; every run keeps a KV cache of its own."""
        n = len(self.layers)
        span = tuple(range(self.loop_start, self.loop_stop))
        return tuple(range(self.loop_start)) + span * self.loop_times + tuple(range(self.loop_stop, n))

    @property
    def num_layers(self) -> int:
        return len(self.layer_runs)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size + self.hidden_size
        for l in self.layers:
            m = l.mixer
            n += W * (m.q_width + m.k_width + m.v_width) + W * m.heads * m.vdim + W + 4 * m.dim
            f = l.mlp
            if f is not None and f.kind == "dense":
                n += 2 * W * f.ff
            elif f is not None:
                n += f.experts * (2 * W * f.ff + W + 1) + (2 * W * f.shared_ff + W if f.shared_ff else 0)
        return n



@dataclass(frozen=True)
class SinkAttentionSpec:
    """Softmax attention with a learned per-head sink in the denominator, an optional sliding
    window (``window`` keys: the query's own position and the ``window - 1`` before it; 0 = all),
    an optional short causal convolution over time on q / k / v (``conv`` taps; 0 = none), one
    RMS norm over the whole q (and k) projection, interleaved-pair rotary on the first
    ``rot_dims`` features of every head (``rot_scaling`` = (factor, low, high, original): the
    wavelength-dependent frequency scaling; None = plain) and values that are rotated by their
    own position over all ``vdim`` features (the head output is turned back by the query's)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0
    window: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[tuple] = None

    @property
    def q_width(self) -> int:
        return self.heads * self.dim

    @property
    def k_width(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_width(self) -> int:
        return self.kv_heads * self.vdim


@dataclass(frozen=True)
class GatedStateSpec:
    """A recurrent mixer whose state is one ``dim x vdim`` matrix per head with a decay per key
    channel.  kind "hgrn2": the forget gate also weights the write (``heads`` q heads, no keys).
    kind "delta": gated delta rule with ``kv_heads`` q / k heads, a short convolution of ``conv``
    taps on q / k / v, low-rank decay and output-gate projections (``decay_rank`` / ``gate_rank``
    are taken from the checkpoint's tensor shapes when one is loaded)."""
    kind: str
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0
    conv: int = 0
    decay_rank: int = 0
    gate_rank: int = 0


@dataclass(frozen=True)
class PadadraLayer:
    type: str                              # "parallel" | "channel_delta"
    attn: Optional[SinkAttentionSpec]      # parallel: the left mixer
    state: GatedStateSpec                  # parallel: the right mixer (hgrn2); channel_delta: the mixer
    mlp: Optional[FeedForwardSpec]


@dataclass(frozen=True)
class PadadraConfig:
    """Padadra: every layer is ``x <- x + m (mixer(norm1 x) + ff(norm2 x))`` with scalar-weight
    norms; the mixer is either a windowed sink attention beside an HGRN2 recurrence ("parallel")
    or a gated delta rule with per-channel decay ("channel_delta").  The embedding adds a hashed
    bigram row.  Everything is read from the model directory's config.json."""
    name: str
    hidden_size: int
    vocab_size: int
    layers: tuple
    rms_eps: float = 1e-6
    embed_scale: float = 1.0
    residual_mult: float = 1.0
    bigram: Optional[tuple] = None         # (buckets, mul_prev, mul_cur)
    family: str = "padadra"
    max_position: int = 1 << 20
    tie_embeddings: bool = False

    @staticmethod
    def _attn(m: dict) -> SinkAttentionSpec:
        rot = m.get("rot") or {}
        sc = rot.get("scaling")
        spec = SinkAttentionSpec(
            heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m["vdim"]),
            scale=float(m["scale"]), conv=int(m.get("conv") or 0), window=int((m.get("mask") or {}).get("size", 0)),
            rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
            rot_scaling=None if not sc else tuple(float(sc[k]) for k in ("factor", "low", "high", "original")))
        if spec.heads % spec.kv_heads or spec.rot_dims % 2 or spec.rot_dims > spec.dim or spec.vdim % 2:
            raise ValueError("Padadra: heads % kv_heads, rot.dims even and <= dim, vdim even")
        return spec

    @classmethod
    def from_dict(cls, c: dict, name: str = "padadra") -> "PadadraConfig":
        layers = []
        for entry in c["layers"]:
            m, kind = entry["mixer"], entry["type"]
            if kind == "parallel":
                r = m["right"]
                attn = cls._attn(m["left"])
                state = GatedStateSpec("hgrn2", int(r["heads"]), int(r["dim"]), int(r["vdim"]))
            elif kind == "channel_delta":
                attn = None
                state = GatedStateSpec("delta", int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                       kv_heads=int(m.get("kv_heads", m["heads"])), conv=int(m.get("conv") or 0),
                                       decay_rank=int(m.get("decay_rank", 0)), gate_rank=int(m.get("gate_rank", 0)))
                if state.heads % state.kv_heads:
                    raise ValueError("Padadra: heads must be a multiple of kv_heads")
            else:
                raise ValueError(f"Padadra: unknown layer type {kind!r}")
            f = entry.get("mlp")
            if f is not None and f["kind"] != "dense":
                raise ValueError(f"Padadra: unknown feed-forward kind {f['kind']!r}")
            layers.append(PadadraLayer(kind, attn, state, FeedForwardSpec("dense", int(f["ff"])) if f else None))
        emb = c.get("embedding") or {}
        bg = emb.get("bigram")
        return cls(name=name, hidden_size=int(c["width"]), vocab_size=int(c["vocab"]), layers=tuple(layers),
                   rms_eps=float(c["norm"]["eps"]), embed_scale=float(emb.get("scale", 1.0)),
                   residual_mult=float(c.get("residual_mult", 1.0)),
                   bigram=(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None)

    def to_dict(self) -> dict:
        """The config.json form (inverse of `from_dict`)."""
        out = []
        for l in self.layers:
            s = l.state
            if l.type == "parallel":
                a = l.attn
                left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
                if a.conv:
                    left["conv"] = a.conv
                if a.window:
                    left["mask"] = {"size": a.window}
                if a.rot_dims:
                    left["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
                    if a.rot_scaling:
                        left["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), a.rot_scaling))
                else:
                    left["rot"] = {"dims": 0, "base": a.rot_base}
                mixer = {"left": left, "right": {"heads": s.heads, "dim": s.dim, "vdim": s.vdim}}
            else:
                mixer = {"heads": s.heads, "kv_heads": s.kv_heads, "dim": s.dim, "vdim": s.vdim}
                if s.conv:
                    mixer["conv"] = s.conv
                if s.decay_rank:
                    mixer["decay_rank"] = s.decay_rank
                if s.gate_rank:
                    mixer["gate_rank"] = s.gate_rank
            out.append({"type": l.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": l.mlp.ff} if l.mlp else None})
        emb = {"scale": self.embed_scale}
        if self.bigram:
            emb["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))
        return {"architecture": "Padadra", "width": self.hidden_size, "vocab": self.vocab_size, "embedding": emb,
                "norm": {"eps": self.rms_eps}, "residual_mult": self.residual_mult, "layers": out}

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            s = l.state
            if l.attn is not None:
                a = l.attn
                n += W * (a.q_width + a.k_width + a.v_width) + W * a.heads * a.vdim
                n += W * (2 * s.heads * s.dim + s.heads * s.vdim) + W * s.heads * s.vdim
            else:
                n += W * (2 * s.kv_heads * s.dim + 2 * s.heads * s.vdim)
            if l.mlp is not None:
                n += 2 * W * l.mlp.ff
        return n


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Softmax attention whose keys and values are read from one low-rank latent per token: the
    cache holds the RMS-normed latent ``c`` (``kv_rank``) and one rotated key part (``rot_dim``)
    shared by all heads; head h's unrotated key is ``W_uk[h] c`` (``dim``), its value ``W_uv[h] c``
    (``vdim``).  Queries pass a latent of their own (``q_rank``).  Rotary (feature i pairs with
    i + rot_dims / 2) acts on the first ``rot_dims`` features of the rotated part; ``rot_scaling``
    = (factor, original, fast, slow) ramps the frequencies between two turn counts and multiplies
    cos and sin by ``0.1 ln(factor) + 1``.  ``window`` keys are visible (0 = all); ``kv_from``: the
    layer whose cache this one reads instead of holding one (-1 = its own)."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[tuple] = None
    kv_from: int = -1

    @property
    def q_width(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def key_width(self) -> int:
        """Cached key features per token: the latent and the shared rotated part."""
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class HeadDeltaSpec:
    """Gated delta rule with ONE decay per head: ``kv_heads`` q / k heads of ``dim``, ``heads``
    value heads of ``vdim``, a short causal convolution of ``conv`` taps (0 = none) and silu on
    q / k / v, a full-width silu output gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int = 0


@dataclass(frozen=True)
class SelectiveStateSpec:
    """State-space mixer with a scalar decay per head (state ``state x vdim`` per head): one input
    projection ``[z | x | B | C | dt]``, B and C shared by the heads of a group, a short causal
    convolution with bias over x | B | C, the gated output RMS-normed in ``norm_groups`` parts."""
    heads: int
    vdim: int
    state: int
    groups: int = 1
    conv: int = 0
    norm_groups: int = 1

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass(frozen=True)
class MabivikLayer:
    type: str                    # "latent_attention" | "delta" | "mamba2"
    mixer: object                # LatentAttentionSpec | HeadDeltaSpec | SelectiveStateSpec
    mlp: Optional[FeedForwardSpec]


@dataclass(frozen=True)
class MabivikConfig:
    """Mabivik: ``x <- x + post(mixer(pre(x)))`` then ``x <- x + post(ff(pre(x)))`` with dynamic-tanh
    norms before and after every sublayer, a per-layer token input after the feed-forward
    (``side_dim`` columns of a second embedding table per layer; 0 = none), mixers of three kinds
    (latent attention, gated delta rule, selective state space) in the order the config lists,
    mixture-of-experts feed-forwards whose experts come from a table row of the token id.
    Everything is read from the model directory's config.json."""
    name: str
    hidden_size: int
    vocab_size: int
    layers: tuple
    rms_eps: float = 1e-6
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    side_dim: int = 0
    family: str = "mabivik"
    max_position: int = 1 << 20
    tie_embeddings: bool = False

    @staticmethod
    def _latent(m: dict, layers: list) -> LatentAttentionSpec:
        rot = m.get("rot") or {}
        sc = rot.get("scaling")
        rot_dim = int(m.get("rot_dim", 0))
        spec = LatentAttentionSpec(
            heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim, vdim=int(m["vdim"]), q_rank=int(m["q_rank"]),
            kv_rank=int(m["kv_rank"]), scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size", 0)),
            rot_dims=int(rot.get("dims", rot_dim)), rot_base=float(rot.get("base", 10000.0)),
            rot_scaling=None if not sc else tuple(float(sc[k]) for k in ("factor", "original", "fast", "slow")),
            kv_from=-1 if m.get("kv_from") is None else int(m["kv_from"]))
        if spec.rot_dims % 2 or spec.rot_dims > spec.rot_dim:
            raise ValueError("Mabivik: rot.dims even and <= rot_dim")
        if spec.kv_from >= 0:
            src = layers[spec.kv_from].mixer if spec.kv_from < len(layers) else None
            if not isinstance(src, LatentAttentionSpec) or src.kv_from >= 0 or (src.kv_rank, src.rot_dim) != (spec.kv_rank, spec.rot_dim):
                raise ValueError("Mabivik: kv_from names an earlier latent-attention layer with a cache of the same shape")
        return spec

    @classmethod
    def from_dict(cls, c: dict, name: str = "mabivik") -> "MabivikConfig":
        layers = []
        for entry in c["layers"]:
            m, kind = entry["mixer"], entry["type"]
            if kind == "latent_attention":
                mixer = cls._latent(m, layers)
            elif kind == "delta":
                mixer = HeadDeltaSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]),
                                      int(m.get("conv") or 0))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError("Mabivik: heads must be a multiple of kv_heads")
            elif kind == "mamba2":
                mixer = SelectiveStateSpec(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1)),
                                           int(m.get("conv") or 0), int(m.get("norm_groups", 1)))
                if mixer.heads % mixer.groups or mixer.inner % mixer.norm_groups:
                    raise ValueError("Mabivik: heads % groups, heads * vdim % norm_groups")
            else:
                raise ValueError(f"Mabivik: unknown layer type {kind!r}")
            f = entry.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"Mabivik: unknown feed-forward kind {f['kind']!r}")
                mlp = FeedForwardSpec("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]))
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError("Mabivik: router.top must be in [1, experts]")
            layers.append(MabivikLayer(kind, mixer, mlp))
        return cls(name=name, hidden_size=int(c["width"]), vocab_size=int(c["vocab"]), layers=tuple(layers),
                   rms_eps=float(c["norm"]["eps"]), embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                   logit_scale=float(c.get("logit_scale", 1.0)), side_dim=int((c.get("token_side") or {}).get("dim", 0)))

    def to_dict(self) -> dict:
        """The config.json form (inverse of `from_dict`)."""
        out = []
        for l in self.layers:
            m = l.mixer
            if l.type == "latent_attention":
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "q_rank": m.q_rank,
                         "kv_rank": m.kv_rank, "scale": m.scale, "rot": {"dims": m.rot_dims, "base": m.rot_base}}
                if m.rot_scaling:
                    mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rot_scaling))
                if m.window:
                    mixer["mask"] = {"size": m.window}
                if m.kv_from >= 0:
                    mixer["kv_from"] = m.kv_from
            elif l.type == "delta":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim}
                if m.conv:
                    mixer["conv"] = m.conv
            else:
                mixer = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "norm_groups": m.norm_groups}
                if m.conv:
                    mixer["conv"] = m.conv
            mlp = None
            if l.mlp is not None:
                mlp = {"kind": "moe", "expert": {"ff": l.mlp.ff}, "router": {"experts": l.mlp.experts, "top": l.mlp.top}}
            out.append({"type": l.type, "mixer": mixer, "mlp": mlp})
        d = {"architecture": "Mabivik", "width": self.hidden_size, "vocab": self.vocab_size,
             "embedding": {"scale": self.embed_scale}, "norm": {"eps": self.rms_eps}, "logit_scale": self.logit_scale,
             "layers": out}
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        return d

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            m = l.mixer
            if l.type == "latent_attention":
                n += W * m.q_rank + m.q_rank * m.q_width + m.heads * m.kv_rank * (m.dim + m.vdim) + 2 * W * m.heads * m.vdim
                n += W * m.key_width if m.kv_from < 0 else 0
            elif l.type == "delta":
                n += W * (2 * m.kv_heads * m.dim + 3 * m.heads * m.vdim + 2 * m.heads)
            else:
                n += W * (2 * m.inner + 2 * m.groups * m.state + m.heads) + W * m.inner
            if l.mlp is not None:
                n += l.mlp.experts * 3 * W * l.mlp.ff
            n += self.side_dim * (2 * W + self.vocab_size)
        return n


@dataclass(frozen=True)
class ChunkAttentionSpec:
    """Softmax attention with GQA, rotate-half rotary on the first ``rot_dims`` features of every
    q / k head (0 = none), q and k divided by their root mean square per head after the rotation,
    a configured score scale, a chunk mask (``chunk`` > 0: position i sees j <= i only when
    floor(i / chunk) = floor(j / chunk); 0 = plain causal), optional value mixing (``v_mix``: every
    such layer but the first blends its values with the first one's values of the same token) and
    one sigmoid output gate per head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    v_mix: bool = False


@dataclass(frozen=True)
class MatrixMemorySpec:
    """Matrix memory with exponential gating (mLSTM): per head a ``dim x vdim`` memory, a
    ``dim`` normaliser and a running maximum of the log gates; input and forget gate logits
    are soft-capped at ``gate_cap``."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class ScoredRouterSpec:
    """Mixture of gated experts whose router scores are sigmoids: ``top`` of ``experts`` experts of
    width ``ff`` per token, chosen by score + correction among the ``keep`` best of ``groups``
    groups of neighbouring experts; weights are the chosen scores over their sum, times ``scale``;
    ``shared_ff`` > 0: an always-on expert of that width is added."""
    ff: int
    experts: int
    top: int
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0


@dataclass(frozen=True)
class SitidraLayer:
    type: str                    # "attention" | "mlstm"
    mixer: object                # ChunkAttentionSpec | MatrixMemorySpec
    mlp: Optional[ScoredRouterSpec]


@dataclass(frozen=True)
class SitidraConfig:
    """Sitidra: pre-norm decoder (layer norms with a weight and no bias) over ``streams``
    hyper-connection residual streams (0 = one plain residual stream), mixers of two kinds (chunked
    softmax attention, matrix memory) in the order the config lists, mixture-of-experts
    feed-forwards with sigmoid-scored grouped routing and a shared expert, soft-capped logits
    (``logit_softcap`` 0 = none).  Everything is read from the model directory's config.json."""
    name: str
    hidden_size: int
    vocab_size: int
    layers: tuple
    streams: int = 0
    rms_eps: float = 1e-6
    logit_softcap: float = 0.0
    family: str = "sitidra"
    max_position: int = 1 << 20
    tie_embeddings: bool = False

    @classmethod
    def from_dict(cls, c: dict, name: str = "sitidra") -> "SitidraConfig":
        layers = []
        for entry in c["layers"]:
            m, kind = entry["mixer"], entry["type"]
            if kind == "attention":
                rot = m.get("rot") or {}
                mixer = ChunkAttentionSpec(
                    heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                    vdim=int(m.get("vdim") or m["dim"]), scale=float(m["scale"]), chunk=int((m.get("mask") or {}).get("size", 0)),
                    rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), v_mix=bool(m.get("v_mix", False)))
                if mixer.heads % mixer.kv_heads or mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim or mixer.chunk < 0:
                    raise ValueError("Sitidra: heads must be a multiple of kv_heads, rot.dims even and <= dim")
            elif kind == "mlstm":
                mixer = MatrixMemorySpec(int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"]), float(m["gate_cap"]))
                if not mixer.gate_cap > 0:
                    raise ValueError("Sitidra: gate_cap must be positive")
            else:
                raise ValueError(f"Sitidra: unknown layer type {kind!r}")
            f = entry.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"Sitidra: unknown feed-forward kind {f['kind']!r}")
                r = f["router"]
                grp = r.get("groups") or {}
                mlp = ScoredRouterSpec(ff=int(f["expert"]["ff"]), experts=int(r["experts"]), top=int(r["top"]),
                                       groups=int(grp.get("count", 1)), keep=int(grp.get("keep", grp.get("count", 1))),
                                       scale=float(r.get("scale", 1.0)), shared_ff=int((f.get("shared") or {}).get("ff", 0)))
                if (not 1 <= mlp.top <= mlp.experts or mlp.groups < 1 or mlp.experts % mlp.groups
                        or not 1 <= mlp.keep <= mlp.groups or mlp.top > mlp.keep * (mlp.experts // mlp.groups)):
                    raise ValueError("Sitidra: router.top in [1, experts], equal groups, top experts within the kept groups")
            layers.append(SitidraLayer(kind, mixer, mlp))
        mixers = [l.mixer for l in layers if l.type == "attention" and l.mixer.v_mix]
        if any((a.kv_heads, a.vdim) != (mixers[0].kv_heads, mixers[0].vdim) for a in mixers):
            raise ValueError("Sitidra: layers that mix values need values of one shape")
        return cls(name=name, hidden_size=int(c["width"]), vocab_size=int(c["vocab"]), layers=tuple(layers),
                   streams=int(c.get("streams") or 0), rms_eps=float(c["norm"]["eps"]),
                   logit_softcap=float(c.get("logit_softcap") or 0.0))

    def to_dict(self) -> dict:
        """The config.json form (inverse of `from_dict`)."""
        out = []
        for l in self.layers:
            m = l.mixer
            if l.type == "attention":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.rot_dims:
                    mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
                if m.chunk:
                    mixer["mask"] = {"size": m.chunk}
                if m.v_mix:
                    mixer["v_mix"] = True
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap}
            mlp = None
            if l.mlp is not None:
                f = l.mlp
                mlp = {"kind": "moe", "expert": {"ff": f.ff},
                       "router": {"experts": f.experts, "top": f.top, "scale": f.scale,
                                  "groups": {"count": f.groups, "keep": f.keep}}}
                if f.shared_ff:
                    mlp["shared"] = {"ff": f.shared_ff}
            out.append({"type": l.type, "mixer": mixer, "mlp": mlp})
        d = {"architecture": "Sitidra", "width": self.hidden_size, "vocab": self.vocab_size, "norm": {"eps": self.rms_eps},
             "layers": out}
        if self.streams:
            d["streams"] = self.streams
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        return d

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def num_params(self) -> int:
        W, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size + self.hidden_size
        for l in self.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim) + m.heads) + W * m.heads * m.vdim
            else:
                n += W * (2 * m.heads * m.dim + 3 * m.heads * m.vdim + 2 * m.heads)
            if l.mlp is not None:
                n += l.mlp.experts * (3 * W * l.mlp.ff + W) + 3 * W * l.mlp.shared_ff
        return n


PRESETS = {
    "Qwen/Qwen3-8B": ModelConfig("Qwen/Qwen3-8B", "qwen3", 4096, 36, 32, 8, 128, 12288, 151936,
                                 qk_norm=True, max_position=40960),
    "Qwen/Qwen3-14B": ModelConfig("Qwen/Qwen3-14B", "qwen3", 5120, 40, 40, 8, 128, 17408, 151936,
                                  qk_norm=True, max_position=40960),
    "Qwen/Qwen3-32B": ModelConfig("Qwen/Qwen3-32B", "qwen3", 5120, 64, 64, 8, 128, 25600, 151936,
                                  qk_norm=True, max_position=40960),
    "mistralai/Mistral-Small-Instruct-2409": ModelConfig(
        "mistralai/Mistral-Small-Instruct-2409", "mistral", 6144, 56, 48, 8, 128, 16384, 32768,
        rms_eps=1e-5, max_position=32768),
    "Qwen/Qwen2.5-0.5B-Instruct": ModelConfig("Qwen/Qwen2.5-0.5B-Instruct", "qwen2", 896, 24, 14, 2, 64,
                                              4864, 151936, qkv_bias=True, tie_embeddings=True,
                                              max_position=32768),
    # CPU-test sized variants (same code paths, real tokenizer vocab)
    # (head_dim 64/128 only: the HIP attention kernels are specialised for those)
    "bcg/tiny-qwen3": ModelConfig("bcg/tiny-qwen3", "qwen3", 256, 2, 4, 2, 64, 512, 151936, qk_norm=True),
    "bcg/tiny-qwen2": ModelConfig("bcg/tiny-qwen2", "qwen2", 256, 2, 4, 2, 64, 512, 151936,
                                  qkv_bias=True, tie_embeddings=True),
    "bcg/tiny-mistral": ModelConfig("bcg/tiny-mistral", "mistral", 256, 2, 8, 2, 128, 512, 32768, rms_eps=1e-5),
}

ALIASES = {
    "qwen3-8b": "Qwen/Qwen3-8B",
    "qwen3-14b": "Qwen/Qwen3-14B",
    "qwen3-32b": "Qwen/Qwen3-32B",
    "mistral-22b": "mistralai/Mistral-Small-Instruct-2409",
    "qwen2.5-0.5b": "Qwen/Qwen2.5-0.5B-Instruct",
}


def from_hf_config(path: str, name: Optional[str] = None):
    with open(os.path.join(path, "config.json")) as fh:
        c = json.load(fh)
    if str(c.get("architecture", "")).lower() == "mofidra":
        return MofidraConfig.from_dict(c, name or path)
    if str(c.get("architecture", "")).lower() == "padadra":
        return PadadraConfig.from_dict(c, name or path)
    if str(c.get("architecture", "")).lower() == "mabivik":
        return MabivikConfig.from_dict(c, name or path)
    if str(c.get("architecture", "")).lower() == "sitidra":
        return SitidraConfig.from_dict(c, name or path)
    arch = (c.get("model_type") or "").lower()
    family = "qwen3" if arch == "qwen3" else ("qwen2" if arch == "qwen2" else "mistral")
    heads = c["num_attention_heads"]
    return ModelConfig(
        name=name or path, family=family, hidden_size=c["hidden_size"],
        num_layers=c["num_hidden_layers"], num_heads=heads,
        num_kv_heads=c.get("num_key_value_heads", heads),
        head_dim=c.get("head_dim") or c["hidden_size"] // heads,
        intermediate_size=c["intermediate_size"], vocab_size=c["vocab_size"],
        rope_theta=float(c.get("rope_theta", 10000.0)), rms_eps=float(c.get("rms_norm_eps", 1e-6)),
        qk_norm=family == "qwen3", qkv_bias=family == "qwen2" or bool(c.get("attention_bias", False)),
        tie_embeddings=bool(c.get("tie_word_embeddings", False)),
        max_position=int(c.get("max_position_embeddings", 32768)))


def get_model_config(name: str, model_dir: Optional[str] = None) -> ModelConfig:
    if model_dir and os.path.exists(os.path.join(model_dir, "config.json")):
        return from_hf_config(model_dir, name)
    key = ALIASES.get(name, name)
    if key in PRESETS:
        return PRESETS[key]
    low = key.lower()
    for preset_name, cfg in PRESETS.items():
        if preset_name.lower() == low:
            return cfg
    raise KeyError(f"unknown model {name!r}; known: {sorted(PRESETS)}")


def with_vocab(cfg: ModelConfig, vocab: int) -> ModelConfig:
    return replace(cfg, vocab_size=vocab)

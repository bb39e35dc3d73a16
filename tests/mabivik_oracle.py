"""Plain float64 implementation of the Mabivik equations: one function per mechanism, a loop per
token, no cache, no batching, no state carried between calls.  It shares no code with the
package; the tests compare the engine with it.

Notation: ``sd`` maps checkpoint names to float64 arrays (integer tables stay integers), ``cfg``
is the config.json dictionary, ``h`` is a mixer's input [T, W] for ONE sequence that starts at
position 0, ``p`` a tensor-name prefix such as ``"l3.mix."``.
"""
import math

import numpy as np


def to_f64(sd):
    import torch
    return {k: (v.double().numpy() if v.dtype.is_floating_point else v.numpy().astype(np.int64)) for k, v in sd.items()}


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def dyt(sd, name, x):
    """Dynamic tanh: tanh(alpha x) w + b; no statistic of x."""
    return np.tanh(float(sd[name + ".alpha"]) * x) * sd[name] + sd[name + ".b"]


def short_conv(u, w, bias=None):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j) (+ bias); u [T, C], w [C, taps]; zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
        if bias is not None:
            y[t] += bias
    return y


# ------------------------------------------------------------------ rotary with ramped frequency scaling
def ramp_freqs(dims, base, scaling):
    """(frequencies [dims / 2], amplitude).  Without scaling: base^(-2i/dims), 1."""
    f = np.array([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    out = np.zeros_like(f)
    for i in range(dims // 2):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / factor * r + f[i] * (1.0 - r)
    return out, 0.1 * math.log(factor) + 1.0


def rotate_half(x, pos, freqs, amp):
    """x [..., dims]: feature i pairs with i + dims / 2; both cos and sin carry ``amp``."""
    n = freqs.shape[0]
    a, b = x[..., :n], x[..., n:2 * n]
    c, s = np.cos(pos * freqs) * amp, np.sin(pos * freqs) * amp
    return np.concatenate([a * c - b * s, b * c + a * s, x[..., 2 * n:]], axis=-1)


# ------------------------------------------------------------------ latent attention
def latent_kv(sd, p, m, h, eps):
    """What a latent-attention layer caches for every token: (c [T, kv_rank], rotated shared key
    part [T, rot_dim])."""
    r, rd = int(m["kv_rank"]), int(m["rot_dim"])
    rot = m.get("rot") or {}
    freqs, amp = ramp_freqs(int(rot.get("dims", rd)), float(rot.get("base", 10000.0)), rot.get("scaling"))
    y = h @ sd[p + "dkv"].T
    c = unit_rms(y[:, :r], eps) * sd[p + "dkv.norm"]
    kr = np.stack([rotate_half(y[t, r:r + rd], t, freqs, amp) for t in range(h.shape[0])])
    return c, kr


def latent_attention(sd, p, m, h, eps, kv):
    """``kv`` = (c, kr) of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, d, rd, vd = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    r = int(m["kv_rank"])
    rot = m.get("rot") or {}
    freqs, amp = ramp_freqs(int(rot.get("dims", rd)), float(rot.get("base", 10000.0)), rot.get("scaling"))
    window = int((m.get("mask") or {}).get("size", 0))
    scale = float(m["scale"])
    c, kr = kv
    cq = unit_rms(h @ sd[p + "dq"].T, eps) * sd[p + "dq.norm"]
    q = (cq @ sd[p + "uq"].T).reshape(T, H, d + rd)
    k_nr = (c @ sd[p + "uk"].T).reshape(T, H, d)
    v = (c @ sd[p + "uv"].T).reshape(T, H, vd)
    gate = sigmoid(h @ sd[p + "g"].T)
    out = np.zeros((T, H * vd))
    for t in range(T):
        first = max(0, t - window + 1) if window > 0 else 0
        for hh in range(H):
            qn = q[t, hh, :d]
            qr = rotate_half(q[t, hh, d:], t, freqs, amp)
            s = np.array([(qn @ k_nr[j, hh] + qr @ kr[j]) * scale for j in range(first, t + 1)])
            w = np.exp(s - s.max())
            w /= w.sum()
            out[t, hh * vd:(hh + 1) * vd] = w @ v[first:t + 1, hh]
    return (out * gate) @ sd[p + "o"].T


# ------------------------------------------------------------------ gated delta rule, one decay per head
def delta_mixer(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, d, vd = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])

    def branch(name):
        y = h @ sd[p + name].T
        if (p + name + ".conv") in sd:
            y = short_conv(y, sd[p + name + ".conv"])
        return silu(y)
    q = branch("q").reshape(T, G, d)
    k = branch("k").reshape(T, G, d)
    v = branch("v").reshape(T, H, vd)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ sd[p + "b"].T)
    g = np.exp(-np.exp(sd[p + "A_log"]) * softplus(h @ sd[p + "a"].T + sd[p + "dt_bias"]))
    gate = silu(h @ sd[p + "g"].T).reshape(T, H, vd)
    out = np.zeros((T, H, vd))
    for hh in range(H):
        kh = hh // (H // G)
        S = np.zeros((d, vd))
        for t in range(T):
            S = g[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + np.outer(k[t, kh], u)
            out[t, hh] = S.T @ q[t, kh]
    out = unit_rms(out, eps) * sd[p + "norm"] * gate
    return out.reshape(T, H * vd) @ sd[p + "o"].T


# ------------------------------------------------------------------ selective state space (scalar decay per head)
def mamba2_mixer(sd, p, m, h, eps):
    T = h.shape[0]
    H, vd, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1))
    parts = int(m.get("norm_groups", 1))
    inner = H * vd
    y = h @ sd[p + "in"].T
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    if (p + "conv") in sd:
        xbc = short_conv(xbc, sd[p + "conv"], sd.get(p + "conv.b"))
    xbc = silu(xbc)
    x = xbc[:, :inner].reshape(T, H, vd)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + sd[p + "dt_bias"])
    out = np.zeros((T, H, vd))
    for hh in range(H):
        gg = hh // (H // G)
        S = np.zeros((N, vd))
        for t in range(T):
            S = math.exp(-math.exp(sd[p + "A_log"][hh]) * dt[t, hh]) * S + dt[t, hh] * np.outer(B[t, gg], x[t, hh])
            out[t, hh] = S.T @ C[t, gg] + sd[p + "D"][hh] * x[t, hh]
    yg = (out.reshape(T, inner) * silu(z)).reshape(T, parts, inner // parts)
    yn = unit_rms(yg, eps).reshape(T, inner) * sd[p + "norm"]
    return yn @ sd[p + "o"].T


# ------------------------------------------------------------------ feed-forward and the per-layer token input
def table_experts(sd, p, f, h, tokens):
    """Experts chosen by a table row of the token id, each with weight 1 / top."""
    top = int(f["router"]["top"])
    out = np.zeros_like(h)
    for t, tok in enumerate(tokens):
        for e in sd[p + "table"][int(tok)][:top]:
            q = f"{p}e{int(e)}."
            out[t] += (sd[q + "down"] @ (silu(sd[q + "gate"] @ h[t]) * (sd[q + "up"] @ h[t]))) / top
    return out


def token_side(sd, cfg, i, x, tokens, eps):
    dim = int(cfg["token_side"]["dim"])
    p = f"l{i}.side."
    e = sd["side.embed"][np.asarray(tokens)][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ sd[p + "gate"].T) * e) @ sd[p + "proj"].T
    return unit_rms(y, eps) * sd[p + "norm"]


def forward(sd, cfg, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out``: a list that receives the stream after
    every layer."""
    eps = float(cfg["norm"]["eps"])
    x = sd["embed"][np.asarray(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    kv = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = dyt(sd, p + "norm1", x)
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = latent_kv(sd, p + "mix.", m, h, eps)
            y = latent_attention(sd, p + "mix.", m, h, eps, kv[i if src is None else int(src)])
        elif layer["type"] == "delta":
            y = delta_mixer(sd, p + "mix.", m, h, eps)
        elif layer["type"] == "mamba2":
            y = mamba2_mixer(sd, p + "mix.", m, h, eps)
        else:
            raise ValueError(layer["type"])
        x = x + dyt(sd, p + "norm1b", y)
        if layer.get("mlp") is not None:
            x = x + dyt(sd, p + "norm2b", table_experts(sd, p + "mlp.", layer["mlp"], dyt(sd, p + "norm2", x), tokens))
        if cfg.get("token_side"):
            x = x + token_side(sd, cfg, i, x, tokens, eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return (dyt(sd, "final.norm", x) @ sd["head"].T) * float(cfg.get("logit_scale", 1.0))

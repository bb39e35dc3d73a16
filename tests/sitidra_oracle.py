"""Plain float64 implementation of the Sitidra equations: one function per mechanism, a loop per
token, no cache, no batching, no state carried between calls.  It shares no code with the
package; the tests compare the engine with it.

Notation: ``sd`` maps checkpoint names to float64 arrays, ``cfg`` is the config.json dictionary,
``h`` is a mixer's input [T, W] for ONE sequence that starts at position 0, ``p`` a tensor-name
prefix such as ``"l3.mix."``.
"""
import math

import numpy as np


def to_f64(sd):
    return {k: (v.double().numpy() if v.dtype.is_floating_point else v.numpy().astype(np.int64)) for k, v in sd.items()}


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, biased variance, no bias."""
    mu = x.mean(-1, keepdims=True)
    d = x - mu
    return d / np.sqrt((d * d).mean(-1, keepdims=True) + eps) * w


# ------------------------------------------------------------------ rotary, chunked softmax attention
def rotate_half(x, pos, dims, base):
    """x [dim] at position pos: feature i < dims/2 pairs with i + dims/2; the rest unchanged."""
    out = x.copy()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = x[i], x[i + half]
        out[i] = u * math.cos(a) - v * math.sin(a)
        out[i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def attention_values(sd, p, m, h):
    """The layer's own values W_v h, [T, kv_heads, vdim] (before any mixing)."""
    return (h @ sd[p + "v"].T).reshape(h.shape[0], m.get("kv_heads", m["heads"]), m["vdim"])


def attention(sd, p, m, h, eps, v_first=None):
    """Chunked causal GQA attention with partial rotate-half rotary, unit-RMS q / k after the
    rotation, value mixing with ``v_first`` [T, G, vdim] (None: this layer's values as they are)
    and one sigmoid output gate per head."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = (h @ sd[p + "q"].T).reshape(T, H, d)
    k = (h @ sd[p + "k"].T).reshape(T, G, d)
    v = attention_values(sd, p, m, h)
    if v_first is not None:
        lam = float(sd[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    rot = m.get("rot")
    chunk = (m.get("mask") or {}).get("size", 0)
    for t in range(T):
        for a, n in ((q, H), (k, G)):
            for j in range(n):
                x = a[t, j]
                if rot and rot["dims"]:
                    x = rotate_half(x, t, rot["dims"], rot["base"])
                a[t, j] = unit_rms(x, eps)
    gate = sigmoid(h @ sd[p + "g"].T)           # [T, H]
    out = np.zeros((T, H, vd))
    for t in range(T):
        first = (t // chunk) * chunk if chunk else 0
        for j in range(H):
            g = j // (H // G)
            sc = np.array([q[t, j] @ k[s, g] for s in range(first, t + 1)]) * m["scale"]
            w = np.exp(sc - sc.max())
            w /= w.sum()
            out[t, j] = (w[:, None] * v[first:t + 1, g]).sum(0) * gate[t, j]
    return out.reshape(T, H * vd) @ sd[p + "o"].T


# ------------------------------------------------------------------ matrix memory with exponential gates
def mlstm(sd, p, m, h, eps):
    T = h.shape[0]
    H, d, vd, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ sd[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ sd[p + "k"].T).reshape(T, H, d)
    v = (h @ sd[p + "v"].T).reshape(T, H, vd)
    ig = cap * np.tanh((h @ sd[p + "i"].T + sd[p + "i.b"]) / cap)
    fg = log_sigmoid(cap * np.tanh((h @ sd[p + "f"].T + sd[p + "f.b"]) / cap))
    o = np.zeros((T, H, vd))
    for j in range(H):
        S, n, mx = np.zeros((d, vd)), np.zeros(d), 0.0
        for t in range(T):
            new = max(fg[t, j] + mx, ig[t, j])
            keep, write = math.exp(fg[t, j] + mx - new), math.exp(ig[t, j] - new)
            S = keep * S + write * np.outer(k[t, j], v[t, j])
            n = keep * n + write * k[t, j]
            mx = new
            o[t, j] = (S.T @ q[t, j]) / (max(abs(n @ q[t, j]), math.exp(-mx)) + 1e-6)
    o = unit_rms(o, eps).reshape(T, H * vd) * sd[p + "norm"] * sigmoid(h @ sd[p + "g"].T)
    return o @ sd[p + "o"].T


# ------------------------------------------------------------------ routed experts
def gated_expert(sd, p, h):
    return (silu(h @ sd[p + "gate"].T) * (h @ sd[p + "up"].T)) @ sd[p + "down"].T


def route(sd, p, f, h):
    """Per token (chosen experts, weights): sigmoid scores; the choice adds the correction and is
    limited to the best groups (a group's score: its two largest choice scores)."""
    r = f["router"]
    E, top = r["experts"], r["top"]
    s = sigmoid(h @ sd[p + "router"].T)
    choice = s + sd[p + "correction"]
    grp = r.get("groups")
    out = []
    for t in range(h.shape[0]):
        c = choice[t].copy()
        if grp and grp["count"] > 1:
            per = E // grp["count"]
            score = [np.sort(c[g * per:(g + 1) * per])[-2:].sum() for g in range(grp["count"])]
            best = sorted(range(grp["count"]), key=lambda g: (-score[g], g))[:grp["keep"]]
            for g in range(grp["count"]):
                if g not in best:
                    c[g * per:(g + 1) * per] = -np.inf
        ids = sorted(range(E), key=lambda e: (-c[e], e))[:top]
        w = s[t, ids]
        out.append((ids, w / (w.sum() + 1e-20) * r["scale"]))
    return out


def feed_forward(sd, p, f, h):
    y = np.zeros_like(h)
    for t, (ids, w) in enumerate(route(sd, p, f, h)):
        for e, we in zip(ids, w):
            y[t] += we * gated_expert(sd, f"{p}e{e}.", h[t])
    if f.get("shared"):
        y += gated_expert(sd, p + "shared.", h)
    return y


# ------------------------------------------------------------------ hyper-connections and the model
def hyper_sublayer(sd, p, xs, fn):
    """xs [S, T, W]: read ``u = sum in[s] x_s``, run ``fn`` on it, write every stream from the old ones."""
    u = np.tensordot(sd[p + "in"], xs, 1)
    y = fn(u)
    return np.tensordot(sd[p + "mix"].T, xs, 1) + sd[p + "out"][:, None, None] * y


def forward(sd, cfg, tokens, trace=None):
    """Logits [T, vocab] of one sequence; ``trace`` receives the summed streams after every layer."""
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams", 0)
    x = sd["embed"][np.asarray(tokens)]
    xs = np.stack([x] * max(S, 1))
    v_first = None
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]

        def mixer(u, p=p, m=m, kind=l["type"]):
            nonlocal v_first
            hn = layer_norm(u, sd[p + "norm1"], eps)
            if kind == "mlstm":
                return mlstm(sd, p + "mix.", m, hn, eps)
            if not m.get("v_mix"):
                return attention(sd, p + "mix.", m, hn, eps)
            if v_first is None:
                v_first = attention_values(sd, p + "mix.", m, hn)
                return attention(sd, p + "mix.", m, hn, eps)
            return attention(sd, p + "mix.", m, hn, eps, v_first)

        def ff(u, p=p, f=l["mlp"]):
            return feed_forward(sd, p + "mlp.", f, layer_norm(u, sd[p + "norm2"], eps))

        if S:
            xs = hyper_sublayer(sd, p + "hc1.", xs, mixer)
            if l["mlp"] is not None:
                xs = hyper_sublayer(sd, p + "hc2.", xs, ff)
        else:
            xs = xs + mixer(xs[0])
            if l["mlp"] is not None:
                xs = xs + ff(xs[0])
        if trace is not None:
            trace.append(xs.sum(0))
    z = layer_norm(xs.sum(0), sd["final.norm"], eps) @ sd["head"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z

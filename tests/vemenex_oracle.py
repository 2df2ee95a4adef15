"""A slow float64 implementation of the Vemenex equations, one function per
mechanism.  It imports nothing from the package: the tests compare the
engine's kernels, caches and scheduler against it.

Notation: T tokens of ONE sequence, positions 0..T-1; W model width; a linear
map stored [out, in] is applied as x @ M.T; S residual streams.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np

F = np.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is ONE number for all coordinates."""
    return rms(x, eps) * float(g)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotary_freqs(base: float, dims: int, factor: float = 1.0):
    """f_i = base^(-2i/dims) / factor, i < dims/2 (linear position scaling
    divides every frequency)."""
    return np.array([base ** (-2.0 * i / dims) / factor for i in range(dims // 2)], dtype=F)


def rotate(x, pos, freqs, layout: str):
    """x [T, heads, dim].  The first 2*len(freqs) entries of a head turn, the
    rest pass.  layout "interleaved": entry 2i pairs with 2i+1; "half": entry
    i pairs with i + len(freqs).  The pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a), a = p * f_i."""
    out = x.copy()
    n = len(freqs)
    for i in range(n):
        a = pos.astype(F) * freqs[i]
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        iu, iv = (2 * i, 2 * i + 1) if layout == "interleaved" else (i, i + n)
        u, v = x[:, :, iu], x[:, :, iv]
        out[:, :, iu] = u * c - v * s
        out[:, :, iv] = v * c + u * s
    return out


def window_visible(i: int, j: int, size: int) -> bool:
    """Query i sees key j: itself and the size - 1 tokens before it."""
    return 0 <= i - j < size


def window_mask(T: int, size: int):
    return np.array([[window_visible(i, j, size) for j in range(T)] for i in range(T)])


def sigmoid_weights(s, visible, bias):
    """Unnormalised weights: sigmoid(score + bias) on visible keys, 0 elsewhere."""
    return np.where(visible, sigmoid(s + bias), 0.0)


def sink_softmax(s, visible):
    """Softmax over the visible keys with one more in the denominator: a key
    of score 0 that carries no value."""
    s = np.where(visible, s, -np.inf)
    m = np.maximum(s.max(axis=-1, keepdims=True), 0.0)
    e = np.exp(s - m)
    return e / (np.exp(-m) + e.sum(axis=-1, keepdims=True))


def windowed_attention(q, k, v, scale: float, window: int, weights: str, bias=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv].  Query head h
    reads key/value head h // (H/G).  weights "sigmoid": per-key logistic of
    score + bias[h], not normalised; "sink": softmax with a zero-score sink."""
    T, H, _ = q.shape
    G = k.shape[1]
    vis = window_mask(T, window)
    out = np.zeros((T, H, v.shape[2]), dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if weights == "sigmoid":
            p = sigmoid_weights(s, vis, float(bias[h]))
        else:
            p = sink_softmax(s, vis)
        out[:, h] = p @ v[:, g]
    return out


def attention_mixer(h, pos, w: Dict[str, np.ndarray], m: dict, eps: float, kind: str):
    """Either attention mixer.  kind "attention": interleaved rotation, sigmoid
    weights with a per-head bias `pb`.  kind "attention_2": rotate-half
    rotation, sink softmax, one sigmoid output gate per head from `g`.
    q and k are divided by their per-head root mean square AFTER rotation."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D)
    k = (h @ w["k"].T).reshape(T, G, D)
    v = (h @ w["v"].T).reshape(T, G, Dv)
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    if dims > 0:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        fr = rotary_freqs(float(rot["base"]), dims, factor)
        layout = "interleaved" if kind == "attention" else "half"
        q, k = rotate(q, pos, fr, layout), rotate(k, pos, fr, layout)
    q, k = rms(q, eps), rms(k, eps)
    window = int(m["mask"]["size"])
    if kind == "attention":
        o = windowed_attention(q, k, v, m["scale"], window, "sigmoid", w["pb"])
    else:
        o = windowed_attention(q, k, v, m["scale"], window, "sink")
        o = o * sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * Dv) @ w["o"].T


def dense_ff(h, w):
    """down(relu(gate h) * (up h))."""
    return (np.maximum(h @ w["gate"].T, 0.0) * (h @ w["up"].T)) @ w["down"].T


def clamped_expert(h, w, limit: float):
    g = np.minimum(h @ w["gate"].T, limit)
    u = np.clip(h @ w["up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def route(z, correction, top: int, groups: int, keep: int):
    """z [T, N] router logits over N = experts + identity experts.  Returns
    (chosen [T, top] indices, weights [T, top]).  Scores are a softmax over
    all N; the choice uses score + correction, restricted to the `keep`
    groups (of N/groups neighbours) whose largest choice score is largest;
    the weights are the chosen plain scores over their sum."""
    T, N = z.shape
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    s = e / e.sum(axis=-1, keepdims=True)
    c = s + correction[None, :]
    per = N // groups
    gs = c.reshape(T, groups, per).max(axis=-1)
    chosen = np.zeros((T, top), dtype=np.int64)
    weights = np.zeros((T, top), dtype=F)
    for t in range(T):
        kept = np.argsort(-gs[t], kind="stable")[:keep]
        allowed = np.full(N, -np.inf)
        for g in kept:
            allowed[g * per : (g + 1) * per] = c[t, g * per : (g + 1) * per]
        idx = np.argsort(-allowed, kind="stable")[:top]
        chosen[t] = idx
        weights[t] = s[t, idx] / (s[t, idx].sum() + 1e-20)
    return chosen, weights


def moe_ff(h, w, mlp: dict):
    """Routed experts; the last `identity` router outputs are experts whose
    output is their input."""
    r = mlp["router"]
    E, ident = int(r["experts"]), int(r.get("identity", 0))
    grp = r.get("groups") or {}
    z = h @ w["router"].T
    corr = w["correction"] if "correction" in w else np.zeros(E + ident)
    chosen, weights = route(z, corr, int(r["top"]), int(grp.get("count", 1)), int(grp.get("keep", 1)))
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t], weights[t]):
            if e >= E:
                out[t] += wt * h[t]
            else:
                ew = {n: w[f"e{e}.{n}"] for n in ("gate", "up", "down")}
                out[t] += wt * clamped_expert(h[t : t + 1], ew, float(mlp["expert"]["limit"]))[0]
    return out


def feed_forward(h, w, mlp: dict):
    return dense_ff(h, w) if mlp.get("kind", "dense") == "dense" else moe_ff(h, w, mlp)


def hyper_read(xs, w_in):
    """xs [S, T, W] -> the sub-layer's input sum_s in[s] x_s."""
    return np.tensordot(w_in, xs, axes=(0, 0))


def hyper_write(xs, y, mix, out, m: float):
    """All streams at once from the old ones:
    x_t <- sum_s mix[s, t] x_s + m * out[t] * y."""
    return np.tensordot(mix.T, xs, axes=(1, 0)) + m * out[:, None, None] * y[None]


def sub(tensors: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {k[len(prefix):]: v.astype(F) for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg: dict, tensors: Dict[str, np.ndarray], tokens: List[int], residuals: Optional[list] = None):
    """Logits [T, vocab] of one sequence; `residuals` collects the sum of the
    streams after every layer."""
    eps = float(cfg["norm"]["eps"])
    m = float(cfg.get("residual_mult", 1.0))
    S = int(cfg.get("streams", 1))
    T = len(tokens)
    pos = np.arange(T)
    x0 = scalar_norm(tensors["embed"].astype(F)[np.asarray(tokens)], tensors["embed.norm"], eps)
    hyper = any(k.endswith(".hc1.in") for k in tensors)
    xs = np.stack([x0] * S) if hyper else x0[None]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        subs = [(1, lambda u: attention_mixer(u, pos, sub(tensors, p + "mix."), layer["mixer"], eps, layer["type"]))]
        if layer.get("mlp") is not None:
            subs.append((2, lambda u: feed_forward(u, sub(tensors, p + "mlp."), layer["mlp"])))
        for qn, fn in subs:
            g = tensors[f"{p}norm{qn}"]
            if hyper:
                hc = sub(tensors, f"{p}hc{qn}.")
                y = fn(scalar_norm(hyper_read(xs, hc["in"]), g, eps))
                xs = hyper_write(xs, y, hc["mix"], hc["out"], m)
            else:
                xs = xs + m * fn(scalar_norm(xs[0], g, eps))[None]
        if residuals is not None:
            residuals.append(xs.sum(axis=0))
    x = xs.sum(axis=0)
    return scalar_norm(x, tensors["final.norm"], eps) @ tensors["head"].astype(F).T

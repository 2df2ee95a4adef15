"""A slow float64 implementation of the Potatar equations, one function per
mechanism.  It imports nothing from the package: the tests compare the
engine's kernels, caches and scheduler against it.

Notation: T tokens of ONE sequence, positions 0..T-1; W model width; a linear
map stored [out, in] is applied as x @ M.T.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np

F = np.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotate_half(x, pos, base, dims):
    """x [T, heads, dim]: entry i of a head is paired with entry i + dims/2,
    i < dims/2; the pair turns by pos * base^(-2i/dims).  Entries from `dims`
    on pass unchanged."""
    out = x.copy()
    half = dims // 2
    for i in range(half):
        f = base ** (-2.0 * i / dims)
        a = pos.astype(F) * f
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[:, :, i], x[:, :, i + half]
        out[:, :, i] = u * c - v * s
        out[:, :, i + half] = v * c + u * s
    return out


def chunk_visible(i: int, j: int, size: int) -> bool:
    return j <= i and i // size == j // size


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance table for distance n >= 0: exact below rows/2,
    logarithmic steps up to `far` above, the last row beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def softmax_rows(s, visible):
    """s [T, T] scores, visible [T, T] bool -> weights (rows sum to one)."""
    s = np.where(visible, s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=-1, keepdims=True)


def visibility(T: int, size: int):
    return np.array([[chunk_visible(i, j, size) for j in range(T)] for i in range(T)])


def chunked_attention(q, k, v, scale: float, chunk: int, bias=None, talk=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] of one sequence -> [T, H, Dv].
    Scores (q . k) * scale, plus bias [T, T, H] if given, then mixed across
    heads with talk [H, H] if given; softmax over the keys of the query's
    own chunk up to the query."""
    T, H, _ = q.shape
    G = k.shape[1]
    s = np.zeros((H, T, T), F)
    for hh in range(H):
        s[hh] = q[:, hh] @ k[:, hh // (H // G)].T * scale
        if bias is not None:
            s[hh] += bias[:, :, hh]
    if talk is not None:
        s = np.einsum("hg,gij->hij", talk, s)
    vis = visibility(T, chunk) if chunk > 0 else np.tril(np.ones((T, T), bool))
    out = np.zeros((T, H, v.shape[2]), F)
    for hh in range(H):
        out[:, hh] = softmax_rows(s[hh], vis) @ v[:, hh // (H // G)]
    return out


def distance_bias(rel, T: int, far: float):
    """bias[i, j, h] = rel[bucket(i - j), h] for j <= i."""
    bias = np.zeros((T, T, rel.shape[1]), F)
    for i in range(T):
        for j in range(i + 1):
            bias[i, j] = rel[distance_bucket(i - j, rel.shape[0], far)]
    return bias


def bonus_recurrence(r, k, v, w, u, S0=None):
    """r, k, w [T, D], v [T, Dv], u [D] of one head: o_t = (S + diag(u) k_t
    v_t^T)^T r_t, then S <- diag(w_t) S + k_t v_t^T.  Returns (o, S)."""
    T, D = k.shape
    S = np.zeros((D, v.shape[1]), F) if S0 is None else S0.copy()
    o = np.zeros((T, v.shape[1]), F)
    for i in range(T):
        kv = np.outer(k[i], v[i])
        o[i] = (S + u[:, None] * kv).T @ r[i]
        S = w[i][:, None] * S + kv
    return o, S


def decay_recurrence(q, k, v, d: float, S0=None):
    """S <- d S + k_t v_t^T, then o_t = S^T q_t.  Returns (o, S)."""
    T, D = k.shape
    S = np.zeros((D, v.shape[1]), F) if S0 is None else S0.copy()
    o = np.zeros((T, v.shape[1]), F)
    for i in range(T):
        S = d * S + np.outer(k[i], v[i])
        o[i] = S.T @ q[i]
    return o, S


def attention_mixer(h, t: Dict[str, np.ndarray], m: dict, eps: float, v_first: Optional[np.ndarray]):
    """Softmax attention with whole-projection query/key norms, partial
    rotate-half rotation, unit-RMS values, optional value mixing with the
    values of the first such layer.  Returns (output, values as cached)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ t["q"].T + t["q.b"]
    k = h @ t["k"].T + t["k.b"]
    v = h @ t["v"].T + t["v.b"]
    q = rms(q, eps) * t["q.norm"]
    k = rms(k, eps) * t["k.norm"]
    pos = np.arange(T)
    q = q.reshape(T, H, D)
    k = k.reshape(T, G, D)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, pos, rot["base"], rot["dims"])
        k = rotate_half(k, pos, rot["base"], rot["dims"])
    v = rms(v.reshape(T, G, Dv), eps)
    if m.get("v_mix") and v_first is not None:
        lam = float(t["vmix"])
        v = (1.0 - lam) * v + lam * v_first
    out = chunked_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size", 0))
    return out.reshape(T, H * Dv) @ t["o"].T + t["o.b"], v


def token_shift(h, mu):
    """h + (h_prev - h) * mu, h_prev the row before (zeros ahead of the first)."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]], axis=0)
    return h + (prev - h) * mu


def wkv_mixer(h, t: Dict[str, np.ndarray], m: dict, eps: float):
    """Matrix-state recurrence with a per-channel, per-token decay and a
    bonus for the current token."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (token_shift(h, t["mu.r"]) @ t["r"].T).reshape(T, H, D)
    k = (token_shift(h, t["mu.k"]) @ t["k"].T).reshape(T, H, D)
    v = (token_shift(h, t["mu.v"]) @ t["v"].T).reshape(T, H, D)
    gate = silu(token_shift(h, t["mu.g"]) @ t["g"].T)
    lw = np.tanh(token_shift(h, t["mu.w"]) @ t["w1"].T) @ t["w2"].T + t["w0"]
    w = np.exp(-np.exp(lw)).reshape(T, H, D)
    u = t["u"].reshape(H, D)
    o = np.zeros((T, H, D), F)
    for hh in range(H):
        o[:, hh], _ = bonus_recurrence(r[:, hh], k[:, hh], v[:, hh], w[:, hh], u[hh])
    o = rms(o, eps).reshape(T, H * D) * t["norm"] * gate
    return o @ t["o"].T


def shared_kv_attention(h, t: Dict[str, np.ndarray], m: dict, eps: float):
    """Softmax attention whose values are the keys as projected: per-head
    query/key norms with one shared weight, no rotation, a learned distance
    bias per head, scores mixed across heads before the softmax."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ t["q"].T + t["q.b"]).reshape(T, H, D)
    k = (h @ t["k"].T + t["k.b"]).reshape(T, G, D)
    v = k
    q = rms(q, eps) * t["q.norm"]
    k = rms(k, eps) * t["k.norm"]
    out = chunked_attention(
        q, k, v, m["scale"], (m.get("mask") or {}).get("size", 0),
        bias=distance_bias(t["rel"], T, m["bias_max"]), talk=t["talk"],
    )
    return out.reshape(T, H * D) @ t["o"].T + t["o.b"]


def decay_mixer(h, t: Dict[str, np.ndarray], m: dict, eps: float):
    """Linear attention with one constant decay per head."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ t["q"].T).reshape(T, H, D)
    k = silu(h @ t["k"].T).reshape(T, H, D)
    v = silu(h @ t["v"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv), F)
    for hh in range(H):
        o[:, hh], _ = decay_recurrence(q[:, hh], k[:, hh], v[:, hh], m["decay"][hh])
    o = rms(o.reshape(T, H * Dv), eps) * t["norm"] * sigmoid(h @ t["g"].T)
    return o @ t["o"].T


def parallel_mixer(h, t: Dict[str, np.ndarray], m: dict, eps: float):
    left = shared_kv_attention(h, sub(t, "left."), m["left"], eps)
    right = decay_mixer(h, sub(t, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def feed_forward(h, t: Dict[str, np.ndarray]):
    return gelu_erf(h @ t["up"].T) @ t["down"].T


def sub(t: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {k[len(prefix):]: v for k, v in t.items() if k.startswith(prefix)}


def forward(cfg: dict, tensors: Dict[str, np.ndarray], tokens: List[int]):
    """Logits [T, vocab] and the residual stream after every layer
    [layers, T, W] of one sequence run from its first token."""
    t = {k: np.asarray(v, F) for k, v in tensors.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = t["embed"][np.asarray(tokens)]
    v_first = None
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        lt = sub(t, f"l{i}.")
        mt = sub(lt, "mix.")
        m = layer["mixer"]
        if layer["type"] == "attention":
            y, v = attention_mixer(x, mt, m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif layer["type"] == "wkv":
            y = wkv_mixer(x, mt, m, eps)
        elif layer["type"] == "parallel":
            y = parallel_mixer(x, mt, m, eps)
        else:
            raise ValueError(layer["type"])
        x = rms(alpha * x + y, eps) * lt["norm1"]
        if layer.get("mlp") is not None:
            x = rms(alpha * x + feed_forward(x, sub(lt, "mlp.")), eps) * lt["norm2"]
        streams.append(x.copy())
    z = (rms(x, eps) * t["final.norm"]) @ t["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * np.tanh(z / cap)
    return z, np.stack(streams)

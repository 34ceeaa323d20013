"""A plain, slow implementation of the Miterax decoder: whole sequences, no cache, no state
carried between calls, one function per mechanism, numpy float64.  It shares no code with the
engine: the tests compare the two.

The design in short.  Token table plus a sinusoidal position vector.  Every layer is parallel:
one scalar-gain RMS norm feeds a mixer and (optionally) a dense feed-forward, whose results
are each scaled per channel and added to the residual together.  A mixer is either causal
grouped-query attention without rotation (a position-dependent query temperature, tanh
soft-capped scores, separate key and value sizes) or an mLSTM cell (matrix memory with a
stabilised exponential input gate).  A run of layers may be looped with the same weights, a
learned vector being added to the residual before each pass.

`config` is the model's config.json as a dict, `w` maps tensor names to arrays.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import numpy as np


def softplus(z):
    z = np.asarray(z, dtype=np.float64)
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def logsigmoid(z):
    return -softplus(-np.asarray(z, dtype=np.float64))


def sigmoid(z):
    return np.exp(logsigmoid(z))


def rms_unit(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) along the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def scalar_rmsnorm(x: np.ndarray, gain: float, eps: float) -> np.ndarray:
    return rms_unit(x, eps) * float(gain)


def sinusoid(positions: Sequence[int], width: int, base: float = 10000.0) -> np.ndarray:
    """Entry 2i: sin(p * base^(-2i/width)); entry 2i+1: the cosine of the same angle."""
    out = np.zeros((len(positions), width))
    p = np.asarray(positions, dtype=np.float64)[:, None]
    for c in range(width):
        i = c // 2
        angle = p[:, 0] * base ** (-2.0 * i / width)
        out[:, c] = np.sin(angle) if c % 2 == 0 else np.cos(angle)
    return out


def xielu(z: np.ndarray, p: float, q: float) -> np.ndarray:
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    ap = float(softplus(p))
    an = 0.5 + float(softplus(q))
    zn = np.minimum(z, 0.0)
    return np.where(z > 0, ap * z * z + 0.5 * z, an * (np.expm1(zn) - zn) + 0.5 * z)


def dense_ffn(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str) -> np.ndarray:
    act = w[prefix + ".act"]
    return xielu(h @ w[prefix + ".up"].T, act[0], act[1]) @ w[prefix + ".down"].T


def query_temperature(position: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((position + 1) // every + 1)


def attention(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, m: dict, start: int = 0) -> np.ndarray:
    """Causal softmax attention over the rows of h (positions start, start + 1, ...)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + ".q"].T).reshape(T, H, d)
    k = (h @ w[prefix + ".k"].T).reshape(T, G, d)
    v = (h @ w[prefix + ".v"].T).reshape(T, G, dv)
    qt = m.get("q_temp")
    if qt:
        temp = np.array([query_temperature(start + t, qt["coef"], qt["every"]) for t in range(T)])
        q = q * temp[:, None, None]
    cap = m.get("softcap")
    out = np.zeros((T, H, dv))
    per = H // G
    for hd in range(H):
        g = hd // per
        s = (q[:, hd, :] @ k[:, g, :].T) * m["scale"]
        if cap:
            s = cap * np.tanh(s / cap)
        s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p = p / p.sum(axis=1, keepdims=True)
        out[:, hd, :] = p @ v[:, g, :]
    return out.reshape(T, H * dv) @ w[prefix + ".o"].T


def mlstm(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, m: dict, eps: float) -> np.ndarray:
    """The mLSTM cell token by token from an empty memory (S = 0, n = 0, m = 0)."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[prefix + ".q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[prefix + ".k"].T).reshape(T, H, d)
    v = (h @ w[prefix + ".v"].T).reshape(T, H, dv)
    ig = cap * np.tanh((h @ w[prefix + ".i"].T + w[prefix + ".i.b"]) / cap)
    fg = logsigmoid(cap * np.tanh((h @ w[prefix + ".f"].T + w[prefix + ".f.b"]) / cap))
    o = np.zeros((T, H, dv))
    for hd in range(H):
        S = np.zeros((d, dv))
        n = np.zeros(d)
        mm = 0.0
        for t in range(T):
            m_new = max(fg[t, hd] + mm, ig[t, hd])
            decay = math.exp(fg[t, hd] + mm - m_new)
            take = math.exp(ig[t, hd] - m_new)
            S = decay * S + take * np.outer(k[t, hd], v[t, hd])
            n = decay * n + take * k[t, hd]
            mm = m_new
            o[t, hd] = (S.T @ q[t, hd]) / (max(abs(float(n @ q[t, hd])), math.exp(-mm)) + 1e-6)
    o = rms_unit(o, eps).reshape(T, H * dv) * w[prefix + ".norm"]
    return (o * sigmoid(h @ w[prefix + ".g"].T)) @ w[prefix + ".o"].T


def run_order(config: dict) -> List[tuple]:
    """[(layer index, pass number or None)]: pass number where a pass of the loop begins."""
    L = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(L)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            order.append((i, t if i == loop["start"] else None))
    order += [(i, None) for i in range(loop["stop"], L)]
    return order


def forward(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int], layers_out: Optional[list] = None) -> np.ndarray:
    """Logits [T, vocab] of a whole sequence from position 0."""
    width, eps = config["width"], config["norm"]["eps"]
    T = len(tokens)
    x = w["embed"][np.asarray(tokens)] + sinusoid(range(T), width)
    for i, begins in run_order(config):
        if begins is not None:
            x = x + w["loop.step"][begins]
        layer = config["layers"][i]
        pre = f"l{i}"
        h = scalar_rmsnorm(x, w[pre + ".norm1"], eps)
        if layer["type"] == "attention":
            y = attention(h, w, pre + ".mix", layer["mixer"])
        elif layer["type"] == "mlstm":
            y = mlstm(h, w, pre + ".mix", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        add = y * w[pre + ".ls1"]
        if layer.get("mlp"):
            add = add + dense_ffn(h, w, pre + ".mlp") * w[pre + ".ls2"]
        x = x + add
        if layers_out is not None:
            layers_out.append(x.copy())
    return scalar_rmsnorm(x, w["final.norm"], eps) @ w["head"].T

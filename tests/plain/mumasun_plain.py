"""A plain, slow implementation of the Mumasun decoder: whole sequences, no cache, no state
carried between calls, one function per mechanism, numpy float64.  It shares no code with the
engine: the tests compare the two.

The design in short.  x = N(E[token]) with the model's norm N (weight kept around zero: the
gain is 1 + w).  A layer normalises what a sublayer returns, not what it reads:
x += N1(mixer(x)), x += N2(ff(x)).  The mixer is differential attention: every query head
holds two maps (two queries, two keys, one value), each an ordinary softmax attention; the
second map's result is subtracted lambda times, the difference is divided by its root mean
square and scaled by 1 - diff.  Queries, keys and values pass a short causal convolution
over time right behind their projections; queries and keys are then normed per head and map
and partly rotated (frequencies interpolated as YaRN does).  A position sees only earlier
positions of its own block of `mask.size` positions.  The feed-forward is a mixture of
experts with sigmoid scores that scale the chosen experts' inputs.  The logits are
E N(x) * logit_scale.

`config` is the model's config.json as a dict, `w` maps tensor names to arrays.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import numpy as np


def rms_unit(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) along the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_one_plus(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    return rms_unit(x, eps) * (1.0 + weight)


def short_conv(u: np.ndarray, taps: np.ndarray) -> np.ndarray:
    """u [T, C], taps [C, K]: y_t = sum_j taps[:, j] u_(t - K + 1 + j), zeros before the start."""
    T, C = u.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C)), u], axis=0)
    y = np.zeros((T, C))
    for j in range(K):
        y += padded[j:j + T] * taps[:, j][None, :]
    return y


def yarn_frequencies(rot: dict) -> tuple:
    """(frequency per pair, factor on cos and sin)."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def turns_to_dim(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turns_to_dim(sc["fast"])), 0)
    hi = min(math.ceil(turns_to_dim(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(half) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half_partial(x: np.ndarray, positions: Sequence[int], rot: dict) -> np.ndarray:
    """x [T, ..., d]: the first rot.dims entries of the last axis are turned, entry i with entry i + dims/2."""
    dims = rot["dims"]
    half = dims // 2
    f, mag = yarn_frequencies(rot)
    out = x.copy()
    for t, p in enumerate(positions):
        a = p * f
        c, s = np.cos(a) * mag, np.sin(a) * mag
        u, v = x[t, ..., :half], x[t, ..., half:dims]
        out[t, ..., :half] = u * c - v * s
        out[t, ..., half:dims] = v * c + u * s
    return out


def block_mask(T: int, size: int) -> np.ndarray:
    """visible[i, j]: j <= i and both in the same block of `size` positions counted from 0."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def softmax_rows(s: np.ndarray, visible: np.ndarray) -> np.ndarray:
    s = np.where(visible, s, -np.inf)
    s = s - s.max(axis=1, keepdims=True)
    p = np.exp(s)
    return p / p.sum(axis=1, keepdims=True)


def differential_lambda(w: Dict[str, np.ndarray], prefix: str, diff: float) -> float:
    return (math.exp(float(np.sum(w[prefix + ".lq1"] * w[prefix + ".lk1"])))
            - math.exp(float(np.sum(w[prefix + ".lq2"] * w[prefix + ".lk2"]))) + diff)


def diff_attention(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, m: dict, eps: float) -> np.ndarray:
    """The mixer over a whole sequence from position 0."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[prefix + ".q"].T
    k = h @ w[prefix + ".k"].T
    v = h @ w[prefix + ".v"].T
    if m.get("conv"):
        q, k, v = (short_conv(u, w[f"{prefix}.{n}.conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q, k, v = q.reshape(T, H, 2, d), k.reshape(T, G, 2, d), v.reshape(T, G, dv)
    q = rms_unit(q, eps) * w[prefix + ".q.norm"]
    k = rms_unit(k, eps) * w[prefix + ".k.norm"]
    if m.get("rot"):
        q = rotate_half_partial(q, range(T), m["rot"])
        k = rotate_half_partial(k, range(T), m["rot"])
    visible = block_mask(T, m["mask"]["size"] if m.get("mask") else T)
    lam = differential_lambda(w, prefix, m["diff"])
    per = H // G
    out = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // per
        a = []
        for mp in range(2):
            s = (q[:, hd, mp, :] @ k[:, g, mp, :].T) * m["scale"]
            a.append(softmax_rows(s, visible) @ v[:, g, :])
        o = a[0] - lam * a[1]
        out[:, hd, :] = rms_unit(o, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ w[prefix + ".o"].T


def router_choice(h: np.ndarray, w_router: np.ndarray, top: int) -> tuple:
    """(indices [T, top], scores [T, top]): the experts with the largest sigmoid scores (ties: the lower index)."""
    s = 1.0 / (1.0 + np.exp(-(h @ w_router.T)))
    idx = np.argsort(-s, axis=1, kind="stable")[:, :top]
    return idx, np.take_along_axis(s, idx, axis=1)


def relu_squared(z: np.ndarray) -> np.ndarray:
    r = np.maximum(z, 0.0)
    return r * r


def moe(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, mlp: dict) -> np.ndarray:
    idx, score = router_choice(h, w[prefix + ".router"], mlp["router"]["top"])
    out = np.zeros((h.shape[0], w[prefix + ".e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, s in zip(idx[t], score[t]):
            out[t] += relu_squared((s * h[t]) @ w[f"{prefix}.e{e}.up"].T) @ w[f"{prefix}.e{e}.down"].T
    return out


def forward(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int], layers_out: Optional[list] = None) -> np.ndarray:
    """Logits [T, vocab] of a whole sequence from position 0."""
    eps = config["norm"]["eps"]
    x = norm_one_plus(w["embed"][np.asarray(tokens)], w["embed.norm"], eps)
    for i, layer in enumerate(config["layers"]):
        pre = f"l{i}"
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        x = x + norm_one_plus(diff_attention(x, w, pre + ".mix", layer["mixer"], eps), w[pre + ".norm1"], eps)
        if layer.get("mlp"):
            x = x + norm_one_plus(moe(x, w, pre + ".mlp", layer["mlp"]), w[pre + ".norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return (norm_one_plus(x, w["final.norm"], eps) @ w["embed"].T) * config["logit_scale"]

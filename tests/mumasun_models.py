"""Small Mumasun configurations and random weights for the tests.  The weights are drawn here with numpy
(not by the framework's own generator), rounded to bfloat16 and written with the safetensors package, so
that the engine and the plain implementation read the same numbers.  Scales are chosen so that activations
stay of order one, attention is far from uniform, the two maps of a head differ and lambda is of order one."""
import json
import os

import numpy as np


def layer(heads, kv_heads, dim, vdim, conv, diff, scale, mask, rot_dims, base=10000.0, scaling=None, experts=None, top=None, ff=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, diff=diff, scale=scale, mask=dict(size=mask),
             rot=dict(base=base, dims=rot_dims, scaling=scaling))
    mlp = None if experts is None else dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    return dict(type="attention", mixer=m, mlp=mlp)


def yarn(factor, original, fast, slow):
    return dict(factor=factor, original=original, fast=fast, slow=slow)


CONFIGS = {
    # three query heads over one kv head, the rotation on half of a map only, a block of 24 positions (three pages of 8),
    # two experts of five per token, a layer without a feed-forward, four taps
    "mixed": dict(architecture="Mumasun", width=48, vocab=89, logit_scale=0.7, norm=dict(eps=1e-5),
                  layers=[layer(3, 1, 16, 24, 4, 0.3, 0.25, 24, 8, 1000.0, yarn(4.0, 64, 16.0, 2.0), experts=5, top=2, ff=40),
                          layer(2, 2, 12, 8, 2, 0.6, 0.3, 50, 12, 500.0, None),
                          layer(4, 2, 8, 8, 3, 0.2, 0.35, 24, 4, 100.0, yarn(1.5, 32, 8.0, 1.0), experts=3, top=3, ff=16)]),
    # sizes that are no multiples of 4 or 16; a block that is no multiple of a page; a block longer than every request
    # (no block edge at all) beside a block of 7; one expert of one; every head its own kv head; one tap (a factor per channel)
    "odd": dict(architecture="Mumasun", width=50, vocab=61, logit_scale=1.3, norm=dict(eps=3e-6),
                layers=[layer(2, 2, 10, 7, 1, 0.45, 0.4, 7, 10, 10000.0, yarn(8.0, 16, 4.0, 0.5), experts=1, top=1, ff=9),
                        layer(1, 1, 18, 33, 5, 0.8, 0.2, 1000, 6, 50.0, None, experts=7, top=4, ff=21),
                        layer(5, 5, 6, 10, 2, 0.1, 0.5, 33, 0, 10000.0, None, experts=4, top=1, ff=30)]),
    # widths the matrix-core kernels serve: keys of 32 and 64, values of 64 and 32, pages of 16 under blocks of 64 and 48
    "wide": dict(architecture="Mumasun", width=128, vocab=320, logit_scale=0.5, norm=dict(eps=1e-6),
                 layers=[layer(6, 2, 32, 64, 2, 0.4, 0.18, 64, 32, 20000.0, yarn(3.0, 128, 16.0, 1.0), experts=8, top=2, ff=96),
                         layer(2, 1, 64, 32, 4, 0.25, 0.125, 48, 16, 10000.0, None, experts=6, top=1, ff=128)]),
}


def to_bf16(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(np.asarray(a, dtype=np.float32))).to(torch.bfloat16)


def draw_weights(config, seed):
    """{name: torch bfloat16 tensor} for every tensor the configuration's model holds."""
    rng = np.random.default_rng(seed)
    W, V = config["width"], config["vocab"]
    t = {}

    def mat(rows, cols, gain=1.0):
        return rng.normal(0.0, gain / np.sqrt(cols), size=(rows, cols))

    t["embed"] = rng.normal(0.0, 1.0, size=(V, W))
    t["embed.norm"] = rng.normal(0.0, 0.2, size=W)
    t["final.norm"] = rng.normal(0.0, 0.2, size=W)
    for i, lay in enumerate(config["layers"]):
        p, m = f"l{i}", lay["mixer"]
        H, G, d, dv, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        t[p + ".norm1"] = rng.normal(0.0, 0.2, size=W)
        t[p + ".mix.q"] = mat(H * 2 * d, W, 2.0)
        t[p + ".mix.k"] = mat(G * 2 * d, W, 2.0)
        t[p + ".mix.v"] = mat(G * dv, W)
        t[p + ".mix.o"] = mat(W, H * dv)
        t[p + ".mix.q.norm"] = 1.0 + rng.normal(0.0, 0.3, size=d)
        t[p + ".mix.k.norm"] = 1.0 + rng.normal(0.0, 0.3, size=d)
        if K:
            for name, ch in (("q", H * 2 * d), ("k", G * 2 * d), ("v", G * dv)):
                taps = rng.normal(0.0, 0.4, size=(ch, K))
                taps[:, -1] += 1.0                      # the token itself weighs most, the ones before it clearly
                t[f"{p}.mix.{name}.conv"] = taps
        for name in ("lq1", "lk1", "lq2", "lk2"):
            t[f"{p}.mix.{name}"] = rng.normal(0.0, 0.6 / np.sqrt(d) ** 0.5, size=d)
        if lay.get("mlp"):
            E, F = lay["mlp"]["router"]["experts"], lay["mlp"]["expert"]["ff"]
            t[p + ".norm2"] = rng.normal(0.0, 0.2, size=W)
            t[p + ".mlp.router"] = mat(E, W, 2.0)
            for e in range(E):
                t[f"{p}.mlp.e{e}.up"] = mat(F, W, 1.5)
                t[f"{p}.mlp.e{e}.down"] = mat(W, F)
    return {k: to_bf16(v) for k, v in t.items()}


def write_folder(path, config, seed, weights=None):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    w = weights if weights is not None else draw_weights(config, seed)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_float64(weights):
    import torch
    return {k: v.to(torch.float64).numpy() for k, v in weights.items()}

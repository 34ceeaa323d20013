"""Small Miterax configurations and random weights for the tests.  The weights are drawn here with numpy
(not by the framework's own generator), rounded to bfloat16 and written with the safetensors package, so
that the engine and the plain implementation read the same numbers.  Scales are chosen so that activations
stay of order one and attention and gates are far from uniform."""
import json
import os

import numpy as np


def attention(heads, kv_heads, dim, vdim, scale, softcap=None, coef=None, every=None, ff=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap is not None:
        m["softcap"] = softcap
    if coef is not None:
        m["q_temp"] = dict(coef=coef, every=every)
    return dict(type="attention", mixer=m, mlp=None if ff is None else dict(kind="dense", ff=ff))


def mlstm(heads, dim, vdim, cap, ff=None):
    return dict(type="mlstm", mixer=dict(heads=heads, dim=dim, vdim=vdim, gate_cap=cap),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


CONFIGS = {
    # keys and values of different sizes everywhere, three kv groups of two, a layer without a feed-forward, the first two
    # layers looped three times
    "loop3": dict(architecture="Miterax", width=64, vocab=131, norm=dict(eps=1e-6),
                  layers=[attention(4, 2, 16, 24, 0.25, softcap=8.0, coef=0.25, every=8, ff=96),
                          mlstm(2, 16, 24, 6.0, ff=80),
                          attention(3, 3, 20, 12, 0.2, softcap=30.0, coef=0.5, every=5)],
                  loop=dict(start=0, stop=2, times=3)),
    # no loop at all; an mLSTM first and last, one of a single head; one kv head under six query heads; a temperature
    # that changes at every position
    "noloop": dict(architecture="Miterax", width=72, vocab=97, norm=dict(eps=1e-5),
                   layers=[mlstm(3, 40, 20, 15.0),
                           attention(6, 1, 32, 32, 0.18, softcap=5.0, coef=0.1, every=1, ff=100),
                           mlstm(1, 8, 72, 3.0, ff=56)]),
    # widths the matrix-core products and the norm inside a product serve (multiples of 64); the whole model is one
    # loop of a single pass; heads each their own group
    "wide": dict(architecture="Miterax", width=128, vocab=320, norm=dict(eps=1e-5),
                 layers=[attention(2, 2, 64, 64, 0.125, softcap=12.0, coef=0.3, every=16, ff=256),
                         mlstm(2, 64, 64, 10.0, ff=192)],
                 loop=dict(start=0, stop=2, times=1)),
    # odd sizes: nothing is a multiple of 16, key sizes that fill their registers only in part, more value columns than
    # one pass of the scan holds, a loop that ends with the model
    "odd": dict(architecture="Miterax", width=40, vocab=53, norm=dict(eps=3e-6),
                layers=[attention(5, 5, 12, 5, 0.3, softcap=2.5, coef=1.0, every=3, ff=24),
                        mlstm(2, 33, 17, 9.0, ff=31),
                        mlstm(1, 130, 70, 20.0),
                        attention(2, 1, 7, 9, 0.4, softcap=50.0, coef=0.05, every=100, ff=8)],
                loop=dict(start=1, stop=4, times=2)),
    # a width that is no multiple of four (no 16-byte rows anywhere), tiny heads, an odd feed-forward, a loop over one layer
    "width50": dict(architecture="Miterax", width=50, vocab=71, norm=dict(eps=1e-5),
                    layers=[attention(2, 1, 10, 6, 0.31, softcap=7.0, coef=0.2, every=2, ff=30),
                            mlstm(1, 5, 3, 4.0, ff=17),
                            attention(4, 2, 3, 11, 0.5, softcap=1.5, coef=0.7, every=9)],
                    loop=dict(start=1, stop=2, times=2)),
}


def to_bf16(a):
    import torch
    a = np.asarray(a, dtype=np.float32)
    if a.ndim == 0:
        return torch.tensor(float(a), dtype=torch.float32).to(torch.bfloat16)       # a single number keeps the shape []
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16)


def draw_weights(config, seed):
    """{name: torch bfloat16 tensor} for every tensor the configuration's model holds."""
    rng = np.random.default_rng(seed)
    W, V = config["width"], config["vocab"]
    t = {}

    def mat(rows, cols, gain=1.0):
        return rng.normal(0.0, gain / np.sqrt(cols), size=(rows, cols))

    t["embed"] = rng.normal(0.0, 1.0, size=(V, W))
    t["head"] = mat(V, W)
    t["final.norm"] = np.asarray(rng.uniform(0.7, 1.4))
    loop = config.get("loop")
    if loop:
        t["loop.step"] = rng.normal(0.0, 0.5, size=(loop["times"], W))
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}", layer["mixer"]
        t[p + ".norm1"] = np.asarray(rng.uniform(0.7, 1.4))
        t[p + ".ls1"] = rng.uniform(0.4, 1.2, size=W) * rng.choice([-1.0, 1.0], size=W)
        if layer["type"] == "attention":
            t[p + ".mix.q"] = mat(m["heads"] * m["dim"], W, 3.0)
            t[p + ".mix.k"] = mat(m["kv_heads"] * m["dim"], W, 3.0)
            t[p + ".mix.v"] = mat(m["kv_heads"] * m["vdim"], W)
            t[p + ".mix.o"] = mat(W, m["heads"] * m["vdim"])
        else:
            H = m["heads"]
            t[p + ".mix.q"] = mat(H * m["dim"], W, 2.0)
            t[p + ".mix.k"] = mat(H * m["dim"], W, 2.0)
            t[p + ".mix.v"] = mat(H * m["vdim"], W)
            t[p + ".mix.g"] = mat(H * m["vdim"], W, 2.0)
            t[p + ".mix.o"] = mat(W, H * m["vdim"])
            t[p + ".mix.norm"] = 1.0 + rng.normal(0.0, 0.2, size=H * m["vdim"])
            t[p + ".mix.i"] = mat(H, W, 3.0)
            t[p + ".mix.i.b"] = rng.normal(0.0, 1.0, size=H)
            t[p + ".mix.f"] = mat(H, W, 3.0)
            t[p + ".mix.f.b"] = rng.normal(2.0, 1.0, size=H)
        if layer.get("mlp"):
            F = layer["mlp"]["ff"]
            t[p + ".mlp.up"] = mat(F, W)
            t[p + ".mlp.down"] = mat(W, F)
            t[p + ".mlp.act"] = rng.normal(0.0, 1.0, size=2)
            t[p + ".ls2"] = rng.uniform(0.4, 1.2, size=W) * rng.choice([-1.0, 1.0], size=W)
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

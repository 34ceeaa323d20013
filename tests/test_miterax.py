"""Miterax without a GPU: the configuration reader, the model as data (run order, tensors, cache needs), and the
plain implementation's mechanisms against other ways of writing the same formulas."""
import copy
import json
import math

import numpy as np
import pytest

import miterax_models as mm
from plain import miterax_plain as plain


def spec_of(config):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import config_and_spec
    return config_and_spec(config)


def test_architecture_is_registered():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import registered_architectures
    assert "Miterax" in registered_architectures()


@pytest.mark.parametrize("name", sorted(mm.CONFIGS))
def test_spec_asks_for_the_tensors_of_the_configuration(name):
    from tinyinfer_amd.models.model import Model
    config = mm.CONFIGS[name]
    typed, spec = spec_of(config)
    model = Model(spec)
    want = {k: tuple(v.shape) for k, v in mm.draw_weights(config, 1).items()}
    got = {k: tuple(v.shape) for k, v in model.tensors().items() if not v.optional}
    assert got == want
    assert typed["width"] == config["width"]


def test_run_order_and_caches_of_a_loop():
    from tinyinfer_amd.models.model import Model
    config = mm.CONFIGS["loop3"]
    _, spec = spec_of(config)
    # three real layers, then one adding layer per pass; each pass: its vector, then layers 0 and 1
    assert spec.run_order() == [3, 0, 1, 4, 0, 1, 5, 0, 1, 2]
    model = Model(spec)
    needs = {type(n).__name__: (n, layers) for n, layers in model.cache_groups}
    # a cache layer per run: layer 0 (attention) runs three times, layer 2 once, but they need different pages
    kv = [(n, c) for n, c in model.cache_groups if type(n).__name__ == "PagedKVNeed"]
    assert sorted((n.head_dim, n.v_dim, c) for n, c in kv) == [(16, 24, 3), (20, 12, 1)]
    state, count = needs["StateNeed"]
    assert state.shape == (2, 16 * 24 + 16 + 1) and count == 3


def test_no_loop_runs_the_layers_in_order():
    _, spec = spec_of(mm.CONFIGS["noloop"])
    assert spec.run_order() == [0, 1, 2]
    assert plain.run_order(mm.CONFIGS["noloop"]) == [(0, None), (1, None), (2, None)]


def test_plain_run_order_of_a_loop():
    order = plain.run_order(mm.CONFIGS["odd"])
    assert [i for i, _ in order] == [0, 1, 2, 3, 1, 2, 3]
    assert [t for _, t in order] == [None, 0, None, None, 1, None, None]


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "conv"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"].pop("gate_cap"), "gate_cap"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "moe"), "moe"),
    (lambda c: c["loop"].__setitem__("stop", 9), "stop"),
    (lambda c: c["loop"].__setitem__("times", 0), "times"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("dim", 300), "256"),
])
def test_bad_configurations_are_refused_by_name(change, word):
    from tinyinfer_amd.config.base import ConfigError
    from tinyinfer_amd.models.model import Model
    config = copy.deepcopy(mm.CONFIGS["loop3"])
    change(config)
    with pytest.raises((ConfigError, ValueError)) as e:
        _, spec = spec_of(config)
        Model(spec)
    assert word in str(e.value)


# ------------------------------------------------------------------ the plain implementation's mechanisms
def test_sinusoid_entries():
    s = plain.sinusoid([0, 3, 1000], 6)
    assert np.allclose(s[0], [0, 1, 0, 1, 0, 1])
    f1 = 10000.0 ** (-2.0 / 6)
    assert math.isclose(s[1, 2], math.sin(3 * f1)) and math.isclose(s[1, 3], math.cos(3 * f1))
    assert math.isclose(s[2, 0], math.sin(1000.0)) and math.isclose(s[2, 5], math.cos(1000.0 * 10000.0 ** (-4.0 / 6)))


def test_xielu_pieces_meet_and_grow_as_written():
    p, q = 0.3, -0.7
    ap, an = math.log1p(math.exp(p)), 0.5 + math.log1p(math.exp(q))
    z = np.array([-3.0, -1e-9, 0.0, 1e-9, 2.0])
    y = plain.xielu(z, p, q)
    assert math.isclose(y[4], ap * 4 + 1.0)
    assert math.isclose(y[0], an * (math.exp(-3.0) - 1 + 3.0) - 1.5)
    assert abs(y[1]) < 1e-8 and y[2] == 0.0 and abs(y[3]) < 1e-8


def test_query_temperature_steps():
    assert plain.query_temperature(0, 0.3, 4) == 1.0
    assert plain.query_temperature(2, 0.3, 4) == 1.0            # floor(3 / 4) = 0
    assert math.isclose(plain.query_temperature(3, 0.3, 4), 1 + 0.3 * math.log(2))
    assert math.isclose(plain.query_temperature(11, 0.3, 4), 1 + 0.3 * math.log(4))


def test_attention_against_a_loop_over_positions():
    rng = np.random.default_rng(3)
    m = dict(heads=4, kv_heads=2, dim=6, vdim=5, scale=0.4, softcap=3.0, q_temp=dict(coef=0.5, every=2))
    W, T = 10, 9
    w = {"a.q": rng.normal(size=(24, W)), "a.k": rng.normal(size=(12, W)), "a.v": rng.normal(size=(10, W)),
         "a.o": rng.normal(size=(W, 20))}
    h = rng.normal(size=(T, W))
    got = plain.attention(h, w, "a", m)
    q = (h @ w["a.q"].T).reshape(T, 4, 6)
    k = (h @ w["a.k"].T).reshape(T, 2, 6)
    v = (h @ w["a.v"].T).reshape(T, 2, 5)
    rows = []
    for i in range(T):
        heads = []
        for hd in range(4):
            g = hd // 2
            qi = q[i, hd] * (1 + 0.5 * math.log((i + 1) // 2 + 1))
            s = np.array([3.0 * math.tanh(0.4 * float(qi @ k[j, g]) / 3.0) for j in range(i + 1)])
            p = np.exp(s - s.max())
            p /= p.sum()
            heads.append(p @ v[: i + 1, g])
        rows.append(np.concatenate(heads) @ w["a.o"].T)
    assert np.allclose(got, np.stack(rows), atol=1e-12)


def test_mlstm_against_its_unstabilised_sum():
    """Without the running maximum the memory is a plain weighted sum: S_t = sum_j exp(i_j + sum_(l > j) f_l) k_j v_j^T, and the
    output divides by max(|n . q|, 1) (the floor exp(-m) e^m = 1 in these terms, up to the 1e-6)."""
    rng = np.random.default_rng(5)
    H, d, dv, W, T, cap = 2, 3, 4, 7, 6, 4.0
    m = dict(heads=H, dim=d, vdim=dv, gate_cap=cap)
    w = {"m.q": rng.normal(size=(H * d, W)), "m.k": rng.normal(size=(H * d, W)), "m.v": rng.normal(size=(H * dv, W)),
         "m.g": rng.normal(size=(H * dv, W)), "m.o": rng.normal(size=(W, H * dv)), "m.norm": rng.normal(size=H * dv),
         "m.i": rng.normal(size=(H, W)) * 0.3, "m.i.b": rng.normal(size=H), "m.f": rng.normal(size=(H, W)), "m.f.b": rng.normal(size=H)}
    h = rng.normal(size=(T, W))
    got = plain.mlstm(h, w, "m", m, 1e-6)
    q = (h @ w["m.q"].T).reshape(T, H, d) / math.sqrt(d)
    k = (h @ w["m.k"].T).reshape(T, H, d)
    v = (h @ w["m.v"].T).reshape(T, H, dv)
    ig = cap * np.tanh((h @ w["m.i"].T + w["m.i.b"]) / cap)
    fg = plain.logsigmoid(cap * np.tanh((h @ w["m.f"].T + w["m.f.b"]) / cap))
    o = np.zeros((T, H, dv))
    for hd in range(H):
        for t in range(T):
            S, n = np.zeros((d, dv)), np.zeros(d)
            mmax = 0.0          # the stabiliser's value, to scale the 1e-6 as the cell does
            for j in range(t + 1):
                wj = math.exp(ig[j, hd] + fg[j + 1: t + 1, hd].sum())
                S += wj * np.outer(k[j, hd], v[j, hd])
                n += wj * k[j, hd]
            run = 0.0
            for j in range(t + 1):
                run = max(fg[j, hd] + run, ig[j, hd])
            mmax = run
            o[t, hd] = (S.T @ q[t, hd]) / (max(abs(float(n @ q[t, hd])), 1.0) + 1e-6 * math.exp(mmax))
    o = plain.rms_unit(o, 1e-6).reshape(T, H * dv) * w["m.norm"]
    want = (o * plain.sigmoid(h @ w["m.g"].T)) @ w["m.o"].T
    assert np.allclose(got, want, rtol=1e-9, atol=1e-9)


def test_a_layer_scale_or_a_step_vector_left_out_changes_the_logits():
    config = mm.CONFIGS["loop3"]
    w = mm.as_float64(mm.draw_weights(config, 11))
    toks = [5, 9, 100, 3, 77, 1, 2]
    base = plain.forward(config, w, toks)
    for name in ("l0.ls1", "l1.ls2", "loop.step", "l2.norm1"):
        w2 = dict(w)
        w2[name] = np.ones_like(w[name]) if name != "loop.step" else np.zeros_like(w[name])
        assert np.abs(plain.forward(config, w2, toks) - base).max() > 1e-3, name

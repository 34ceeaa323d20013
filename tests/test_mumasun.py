"""Mumasun without a GPU: the configuration reader, the model as data (tensors, cache needs), the cache manager's
handling of keys that are read per block, and the plain implementation's mechanisms against other ways of writing
the same formulas."""
import copy
import math

import numpy as np
import pytest

import mumasun_models as mm
from plain import mumasun_plain as plain


def spec_of(config):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import config_and_spec
    return config_and_spec(config)


def test_architecture_is_registered():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import registered_architectures
    assert "Mumasun" in registered_architectures()


@pytest.mark.parametrize("name", sorted(mm.CONFIGS))
def test_spec_asks_for_the_tensors_of_the_configuration(name):
    from tinyinfer_amd.models.model import Model
    config = mm.CONFIGS[name]
    typed, spec = spec_of(config)
    model = Model(spec)
    want = {k: tuple(v.shape) for k, v in mm.draw_weights(config, 1).items()}
    got = {k: tuple(v.shape) for k, v in model.tensors().items() if not v.optional}
    assert got == want
    assert typed["width"] == config["width"] and typed["logit_scale"] == config["logit_scale"]


def test_cache_needs_pages_per_block_and_a_state_per_convolution():
    from tinyinfer_amd.models.model import Model
    _, spec = spec_of(mm.CONFIGS["mixed"])
    model = Model(spec)
    kv = sorted((n.kv_heads, n.head_dim, n.v_dim, n.block, c) for n, c in model.cache_groups if type(n).__name__ == "PagedKVNeed")
    # a row's two maps lie side by side: keys of 2 x dim; layers 0 and 2 differ in sizes, so three groups of one layer
    assert kv == [(1, 32, 24, 24, 1), (2, 16, 8, 24, 1), (2, 24, 8, 50, 1)]
    states = sorted((n.shape, c) for n, c in model.cache_groups if type(n).__name__ == "StateNeed")
    # taps - 1 rows of all channels of q, k and v
    assert states == [((1, 2 * 2 * 12 + 2 * 2 * 12 + 2 * 8), 1), ((2, 4 * 2 * 8 + 2 * 2 * 8 + 2 * 8), 1), ((3, 3 * 2 * 16 + 2 * 16 + 24), 1)]
    # one tap: no state at all
    _, spec = spec_of(mm.CONFIGS["odd"])
    shapes = [n.shape for n, _ in Model(spec).cache_groups if type(n).__name__ == "StateNeed"]
    assert sorted(shapes) == [(1, 5 * 2 * 6 + 5 * 2 * 6 + 5 * 10), (4, 2 * 18 + 2 * 18 + 33)]


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].__setitem__("type", "mlstm"), "mlstm"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 2), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"].pop("diff"), "diff"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "size"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"), "dense"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 6), "top"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("ff"), "ff"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("dim", 300), "256"),
])
def test_bad_configurations_are_refused_by_name(change, word):
    from tinyinfer_amd.config.base import ConfigError
    from tinyinfer_amd.models.model import Model
    config = copy.deepcopy(mm.CONFIGS["mixed"])
    change(config)
    with pytest.raises((ConfigError, ValueError)) as e:
        _, spec = spec_of(config)
        Model(spec)
    assert word in str(e.value)


def test_defaults_are_filled_in():
    config = copy.deepcopy(mm.CONFIGS["mixed"])
    m = config["layers"][1]["mixer"]
    for key in ("kv_heads", "vdim", "scale", "conv", "mask", "rot"):
        m.pop(key)
    config.pop("logit_scale")
    typed, spec = spec_of(config)
    from tinyinfer_amd.models.model import Model
    assert not any(".conv" in name for name in Model(spec).tensors() if name.startswith("l1."))
    t = typed["layers"][1]["mixer"]
    assert t["kv_heads"] == 2 and t["vdim"] == 12 and t["conv"] is None and t["mask"] is None and t["rot"] is None
    assert abs(t["scale"] - 12 ** -0.5) < 1e-12 and typed["logit_scale"] == 1.0


# ------------------------------------------------------------------------------ the cache manager
def test_pages_before_the_block_of_the_next_token_go_back():
    from tinyinfer_amd.cache import CacheManager
    from tinyinfer_amd.spec import PagedKVNeed
    P, block = 4, 10
    cache = CacheManager([(PagedKVNeed(1, 8, None, None, block), 1)], page_size=P, num_pages=8, max_requests=2, max_seq=64)
    cache.admit("a")
    length = 0
    for n in (3, 6, 1, 1, 9, 1, 12):          # portions that end inside, at and beyond a block's edge
        cache.reserve("a", n)
        cache.commit("a", n)
        length += n
        first_pos = length // block * block      # what the next token still reads
        table = cache.table(0, "a")
        for i, page in enumerate(table):
            wholly_before = (i + 1) * P <= first_pos
            assert (page < 0) == wholly_before, (length, i, table)
        cache.check()
    # one token at a time over an edge: the page goes back at the step that completes the block
    cache.release("a")
    cache.admit("b")
    free0 = cache.num_free_pages()
    for t in range(25):
        cache.reserve_one_each(["b"])
        cache.commit_one_each(["b"])
        held = sum(1 for p in cache.table(0, "b") if p >= 0)
        first_pos = (t + 1) // block * block
        assert held == -(-(t + 1) // P) - first_pos // P, (t, cache.table(0, "b"))
        assert cache.num_free_pages() == free0 - held
    cache.check()


# ------------------------------------------------------------------------------ the plain implementation
def test_short_conv_is_a_causal_correlation():
    rng = np.random.default_rng(0)
    u, taps = rng.normal(size=(9, 3)), rng.normal(size=(3, 4))
    y = plain.short_conv(u, taps)
    for c in range(3):
        full = np.convolve(u[:, c], taps[c, ::-1])[:9]          # the last tap weighs the token itself
        assert np.allclose(y[:, c], full)
    assert np.allclose(y[0], u[0] * taps[:, -1])                 # nothing before the first token
    assert np.allclose(plain.short_conv(u, taps[:, -1:]), u * taps[:, -1])


def test_yarn_frequencies_at_their_ends():
    rot = dict(base=10000.0, dims=32, scaling=dict(factor=4.0, original=256, fast=32.0, slow=1.0))
    f, mag = plain.yarn_frequencies(rot)
    plain_f = np.array([10000.0 ** (-2 * i / 32) for i in range(16)])
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    assert np.allclose(f[0], plain_f[0])                         # the fastest pair keeps its frequency
    assert np.allclose(f[-1], plain_f[-1] / 4.0)                 # the slowest is divided by the factor
    assert (np.diff(f / plain_f) <= 1e-12).all()                 # and the share of the division grows monotonically
    f1, m1 = plain.yarn_frequencies(dict(base=10000.0, dims=32, scaling=None))
    assert np.allclose(f1, plain_f) and m1 == 1.0


def test_partial_rotation_turns_pairs_and_leaves_the_rest():
    rot = dict(base=100.0, dims=4, scaling=None)
    x = np.arange(1.0, 7.0)[None, None, :]                       # one token, one head, six entries
    y = plain.rotate_half_partial(np.repeat(x, 3, axis=0), [0, 1, 5], rot)
    assert np.allclose(y[0], x[0])                               # position 0: no turn
    assert np.allclose(y[:, :, 4:], 5.0 + np.arange(2.0))        # the entries beyond dims pass
    for t, p in enumerate([0, 1, 5]):
        for i, f in enumerate([1.0, 100.0 ** -0.5]):
            z = complex(x[0, 0, i], x[0, 0, i + 2]) * complex(math.cos(p * f), math.sin(p * f))
            assert abs(y[t, 0, i] - z.real) < 1e-12 and abs(y[t, 0, i + 2] - z.imag) < 1e-12


def test_block_mask():
    v = plain.block_mask(7, 3)
    assert v[2].tolist() == [True, True, True, False, False, False, False]
    assert v[3].tolist() == [False, False, False, True, False, False, False]     # the first token of a block sees itself alone
    assert v[5].tolist() == [False, False, False, True, True, True, False]
    assert plain.block_mask(5, 100).tolist() == np.tril(np.ones((5, 5), dtype=bool)).tolist()


def test_router_takes_the_largest_scores_and_keeps_them_unnormalised():
    h = np.array([[1.0, 0.0], [0.0, -2.0]])
    router = np.array([[3.0, 0.0], [1.0, 1.0], [2.0, -1.0], [3.0, 0.5]])
    idx, score = plain.router_choice(h, router, 2)
    assert idx.tolist() == [[0, 3], [2, 0]]                      # equal scores: the lower index first
    assert np.allclose(score[0], 1 / (1 + math.exp(-3.0))) and np.allclose(score[1], [1 / (1 + math.exp(-2.0)), 0.5])


def test_expert_weight_scales_the_input():
    rng = np.random.default_rng(1)
    W, F = 6, 5
    w = {"m.router": np.array([[10.0] + [0.0] * (W - 1)]), "m.e0.up": rng.normal(size=(F, W)), "m.e0.down": rng.normal(size=(W, F))}
    h = rng.normal(size=(3, W))
    y = plain.moe(h, w, "m", dict(router=dict(experts=1, top=1)))
    s = 1 / (1 + np.exp(-10.0 * h[:, 0]))
    want = (np.maximum((h * s[:, None]) @ w["m.e0.up"].T, 0) ** 2) @ w["m.e0.down"].T
    assert np.allclose(y, want)
    # the square of relu makes that s^2 times the unscaled expert
    assert np.allclose(y, s[:, None] ** 2 * ((np.maximum(h @ w["m.e0.up"].T, 0) ** 2) @ w["m.e0.down"].T))


def test_one_map_alone_is_ordinary_attention():
    """With lambda = 0 (both exponentials equal, diff 0) the second map drops out: softmax attention, head-normed."""
    rng = np.random.default_rng(2)
    T, W, d, dv = 6, 8, 4, 3
    m = dict(heads=1, kv_heads=1, dim=d, vdim=dv, conv=1, diff=0.0, scale=0.5, mask=dict(size=100), rot=dict(base=10.0, dims=0, scaling=None))
    w = {"a.q": rng.normal(size=(2 * d, W)), "a.k": rng.normal(size=(2 * d, W)), "a.v": rng.normal(size=(dv, W)), "a.o": np.eye(dv),
         "a.q.conv": np.ones((2 * d, 1)), "a.k.conv": np.ones((2 * d, 1)), "a.v.conv": np.ones((dv, 1)),
         "a.q.norm": np.ones(d), "a.k.norm": np.ones(d), "a.lq1": np.zeros(d), "a.lk1": np.zeros(d), "a.lq2": np.zeros(d), "a.lk2": np.zeros(d)}
    assert plain.differential_lambda(w, "a", 0.0) == 0.0
    h = rng.normal(size=(T, W))
    y = plain.diff_attention(h, w, "a", m, 1e-6)
    q = plain.rms_unit((h @ w["a.q"].T)[:, :d], 1e-6)
    k = plain.rms_unit((h @ w["a.k"].T)[:, :d], 1e-6)
    s = np.where(np.tril(np.ones((T, T), dtype=bool)), q @ k.T * 0.5, -np.inf)
    p = np.exp(s - s.max(1, keepdims=True))
    a = (p / p.sum(1, keepdims=True)) @ (h @ w["a.v"].T)
    assert np.allclose(y, plain.rms_unit(a, 1e-6))


def test_prefix_of_a_sequence_gives_the_same_logits():
    config = mm.CONFIGS["mixed"]
    w = mm.as_float64(mm.draw_weights(config, 3))
    toks = list(np.random.default_rng(5).integers(0, config["vocab"], size=60))
    full = plain.forward(config, w, toks)
    assert np.allclose(plain.forward(config, w, toks[:31]), full[:31], atol=1e-10)

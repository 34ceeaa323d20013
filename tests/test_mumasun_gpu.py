"""Mumasun on the GPU against the plain implementation: every mechanism alone through the kernels' own object, and the
engine under every way of cutting the work (each request whole; most of it in one step and its last tokens one by
one; portions of changing size down to two tokens; up to four live requests mixed, with so few pages and state
slots that both are used again), in 32-bit and in bfloat16, and greedy generation through the entry point and the
scheduler."""
import math

import numpy as np
import pytest
import torch

import mumasun_models as mm
import traces
from helpers import random_tokens
from plain import mumasun_plain as plain

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# rms of (engine - plain) over rms of the plain logits, per position.  float32: rounding of 32-bit sums against float64.
# bfloat16: operands of every product, cached keys and values and the queries are rounded to 8 bits; the difference of two
# maps and the norm behind it amplify that to a few per cent, while a lost key, a block edge that is one token off, a lost
# convolution state or a wrong expert changes tens of per cent.  Where two experts' scores lie within that rounding of each
# other (a per cent of them: a token in twenty or so per routed layer), bfloat16 may pick the other one, and that token's
# logits then differ by tens of per cent with nothing wrong: in bfloat16 the bound holds for all but 8 % of the positions
# and the median error stays under 2 %; 32-bit holds everywhere.
TOL = {"float32": 2e-4, "bfloat16": 8e-2}


@pytest.fixture(scope="module")
def ops():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.ops.kernels import get_ops
    return get_ops()


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a)).to(dtype).to("cuda")


def f64(t):
    return t.detach().to("cpu", torch.float64).numpy()


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float64).numpy()


# ---------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("H", [50, 192, 1030])
def test_norm_into_the_residual(ops, H):
    rng = np.random.default_rng(H)
    x0, y, g = rng.normal(size=(5, H)), rng.normal(size=(5, H)) * 3, 1.0 + rng.normal(size=H) * 0.2
    normed = plain.rms_unit(y, 1e-5) * g
    x = dev(x0)
    ops.norm_residual(x, dev(y), dev(g), 1e-5, True)
    assert np.abs(f64(x) - (x0 + normed)).max() < 3e-6
    x = dev(y)
    ops.norm_residual(x, x, dev(g), 1e-5, False)           # in place: what the embedding's norm does
    assert np.abs(f64(x) - normed).max() < 3e-6
    # rows gathered and summed first (what the experts of a token left), in the order given
    src = rng.normal(size=(11, H))
    gather = np.array([[3, 0], [10, 10], [1, 7], [2, 9], [5, 4]], dtype=np.int32)
    x = dev(x0)
    ops.norm_residual(x, dev(src), dev(g), 1e-5, True, dev(gather, torch.int32))
    want = x0 + plain.rms_unit(src[gather[:, 0]] + src[gather[:, 1]], 1e-5) * g
    assert np.abs(f64(x) - want).max() < 3e-6
    # a rounded copy of the new residual beside it
    x, copy = dev(x0), torch.empty(5, H, device="cuda", dtype=torch.bfloat16)
    ops.norm_residual(x, dev(y), dev(g), 1e-5, True, None, copy)
    assert np.abs(f64(x) - (x0 + normed)).max() < 3e-6
    assert torch.equal(copy, x.to(torch.bfloat16))


def test_round_rows_and_scale(ops):
    x0 = np.random.default_rng(1).normal(size=(7, 19)).astype(np.float32)
    for src in (x0, x0[:, :16]):                            # a count that is no multiple of eight, and one that is
        src = np.ascontiguousarray(src)
        out = torch.empty(src.shape, device="cuda", dtype=torch.bfloat16)
        ops.round_rows(dev(src), out)
        assert np.array_equal(f64(out), bf16_round(src))
    x = dev(x0)
    ops.scale(x, 0.3)
    assert np.abs(f64(x) - x0 * np.float32(0.3)).max() < 1e-7


def conv_steps(ops, u, taps, cuts, n_slots=3):
    """Two sequences (slots 2 and 0) fed side by side in the given cuts; returns their outputs."""
    T, C = u[0].shape
    K = taps.shape[1]
    state = torch.zeros(n_slots, K - 1, C, device="cuda") if K > 1 else None
    outs = [[], []]
    at = 0
    for n in cuts:
        n = min(n, T - at)
        if n == 0:
            break
        rows = np.concatenate([u[0][at:at + n], u[1][at:at + n]])
        entries = np.array([[0, n, at, 2], [n, n, at, 0]], dtype=np.int32)
        entry_of = np.array([0] * n + [1] * n, dtype=np.int32)
        pos = np.concatenate([np.arange(at, at + n)] * 2).astype(np.int32)
        out = torch.full((2 * n, C), 7.0, device="cuda")
        ops.short_conv(dev(rows), dev(taps), state, dev(entries, torch.int32), dev(entry_of, torch.int32), dev(pos, torch.int32), out)
        o = f64(out)
        outs[0].append(o[:n])
        outs[1].append(o[n:])
        at += n
    return np.concatenate(outs[0]), np.concatenate(outs[1])


@pytest.mark.parametrize("K,C", [(4, 37), (2, 300), (1, 8), (6, 5)])
def test_short_conv_carries_its_state_through_any_cut(ops, K, C):
    rng = np.random.default_rng(K * 100 + C)
    T = 41
    u = [rng.normal(size=(T, C)), rng.normal(size=(T, C))]
    taps = rng.normal(size=(C, K))
    want = [plain.short_conv(x, taps) for x in u]
    results = []
    for cuts in ([T], [1] * T, [3, 1, 1, 2, 7, 1, 2, 2, 30], [2] * 21, [K - 1 or 1, 1, K, 40]):
        a, b = conv_steps(ops, u, taps, cuts)
        assert np.abs(a - want[0]).max() < 5e-6 and np.abs(b - want[1]).max() < 5e-6, cuts
        results.append((a, b))
    for a, b in results[1:]:                                # the same bits however the rows were cut
        assert np.array_equal(a, results[0][0]) and np.array_equal(b, results[0][1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_convolution_inside_the_preparation_gives_the_same_bits(ops, dtype):
    """The projections of two requests in several cuts: convolution, then preparation, against the preparation that takes the
    convolution in.  Queries and pages hold the same bits, and so does the state that is left."""
    rng = np.random.default_rng(5)
    heads, kv, dk, dv, P, K, T = 3, 1, 12, 20, 8, 4, 37
    C = heads * 2 * dk + kv * (2 * dk + dv)
    u = [rng.normal(size=(T, C)), rng.normal(size=(T, C))]
    taps = dev(rng.normal(size=(C, K)))
    qw, kw = dev(1.0 + rng.normal(size=dk) * 0.2), dev(1.0 + rng.normal(size=dk) * 0.2)
    inv = dev(np.array([50.0 ** (-2.0 * i / 8) for i in range(4)]))
    table = dev(np.array([[4, 1, 7, 0, 9], [2, 8, 3, 6, 5]]), torch.int32)
    results = []
    for inside in (False, True):
        state = torch.zeros(3, K - 1, C, device="cuda")
        pool = torch.zeros(10, kv, P, 2 * dk + dv, device="cuda", dtype=DT[dtype])
        qs, at = [], 0
        for n in (5, 1, 2, 1, 20, 3, 5):
            rows = dev(np.concatenate([u[0][at:at + n], u[1][at:at + n]]))
            entries = dev([[0, n, at, 2], [n, n, at, 0]], torch.int32)
            entry_of = dev([0] * n + [1] * n, torch.int32)
            pos = dev(list(range(at, at + n)) * 2, torch.int32)
            q_out = torch.empty(2 * n, heads * 2 * dk, device="cuda", dtype=DT[dtype])
            if inside:
                ops.diff_qk_prep(rows, qw, kw, inv, None, pos, entry_of, table, pool, q_out, 1e-5, heads, kv, dk, dv, 8, 1.1,
                                 taps=taps, state=state, entries=entries)
            else:
                mixed = torch.empty_like(rows)
                ops.short_conv(rows, taps, state, entries, entry_of, pos, mixed)
                ops.diff_qk_prep(mixed, qw, kw, inv, None, pos, entry_of, table, pool, q_out, 1e-5, heads, kv, dk, dv, 8, 1.1)
            qs.append(q_out)
            at += n
        results.append((torch.cat(qs), pool, state))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    assert results[0][2].abs().sum() > 0


def paged(rng, n_tokens, P, extra_pages=3):
    n_pages = -(-n_tokens // P)
    ids = rng.permutation(n_pages + extra_pages)[:n_pages]
    return np.asarray(ids, dtype=np.int32)[None, :], n_pages + extra_pages


def plain_maps(q, k, v, scale, block, lam, eps, out_scale, per):
    """o [T, heads, dv] of prepared q [T, heads, 2, d], k [T, kv, 2, d], v [T, kv, dv]."""
    T, H = q.shape[:2]
    visible = plain.block_mask(T, block) if block else np.tril(np.ones((T, T), dtype=bool))
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        a = [plain.softmax_rows(q[:, h, mp] @ k[:, h // per, mp].T * scale, visible) @ v[:, h // per] for mp in range(2)]
        out[:, h] = plain.rms_unit(a[0] - lam * a[1], eps) * out_scale
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv,dk,dv,P,block,rot_dims", [(4, 2, 16, 24, 16, 40, 8), (3, 3, 7, 9, 4, 13, 6), (6, 1, 40, 33, 64, 150, 40),
                                                              (2, 2, 32, 64, 16, 64, 32), (2, 1, 64, 32, 16, 100, 0), (1, 1, 130, 256, 8, 50, 2),
                                                              (2, 1, 24, 16, 16, 1000, 12), (16, 2, 128, 128, 32, 40, 64), (4, 4, 64, 128, 16, 70, 20),
                                                              (3, 1, 32, 32, 16, 33, 32)])
def test_prepared_keys_and_differential_attention(ops, dtype, heads, kv, dk, dv, P, block, rot_dims):
    """q/k/v of a whole request normed, rotated and written in two portions, then the attention of every row.  On the
    entries that are not rotated, the last row's first map points at the second key of its block (far back), and its
    second map at the key just before the block: losing the first or seeing the second shows."""
    rng = np.random.default_rng(dk * 1000 + dv)
    T, eps, lam, out_scale = 150, 1e-5, 0.8, 0.6
    scale = 1.0 / math.sqrt(dk)
    per = heads // kv
    q = rng.normal(size=(T, heads, 2, dk))
    k = rng.normal(size=(T, kv, 2, dk))
    v = rng.normal(size=(T, kv, dv))
    qw, kw = 1.0 + rng.normal(size=dk) * 0.2, 1.0 + rng.normal(size=dk) * 0.2
    rot = dict(base=300.0, dims=rot_dims, scaling=dict(factor=3.0, original=40, fast=8.0, slow=1.0) if rot_dims > 4 else None)
    freq, mag = plain.yarn_frequencies(rot) if rot_dims else (np.zeros(0), 1.0)
    first_of_block = (T - 1) // block * block
    if rot_dims < dk and first_of_block > 0:
        group = np.arange(heads) // per
        k[first_of_block + 1, :, 0, rot_dims:] *= 4
        k[first_of_block - 1, :, 1, rot_dims:] *= 4
        q[T - 1, :, 0, rot_dims:] = k[first_of_block + 1][group, 0, rot_dims:]
        q[T - 1, :, 1, rot_dims:] = k[first_of_block - 1][group, 1, rot_dims:]
    qkv = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], axis=1)
    table, n_pages = paged(rng, T, P)
    pool = torch.zeros(n_pages, kv, P, 2 * dk + dv, device="cuda", dtype=DT[dtype])
    q_out = torch.empty(T, heads * 2 * dk, device="cuda", dtype=DT[dtype])
    pos = np.arange(T, dtype=np.int32)
    slots = np.zeros(T, dtype=np.int32)
    inv = dev(freq) if rot_dims else None
    # a table for the first 100 positions only: the rest take the angle in 32-bit on the device
    tab = None
    if rot_dims:
        ang = np.arange(100)[:, None] * freq[None, :]
        tab = dev(np.stack([np.cos(ang) * mag, np.sin(ang) * mag], axis=-1))
    cut = 37
    for lo, hi in ((0, cut), (cut, T)):
        ops.diff_qk_prep(dev(qkv[lo:hi]), dev(qw), dev(kw), inv, tab, dev(pos[lo:hi], torch.int32), dev(slots[lo:hi], torch.int32),
                         dev(table, torch.int32), pool, q_out[lo:hi], eps, heads, kv, dk, dv, rot_dims, mag)
    qn = plain.rms_unit(q, eps) * qw
    kn = plain.rms_unit(k, eps) * kw
    if rot_dims:
        qn, kn = plain.rotate_half_partial(qn, pos, rot), plain.rotate_half_partial(kn, pos, rot)
    tol = 3e-5 if dtype == "float32" else 2.0 ** -7
    assert np.abs(f64(q_out).reshape(T, heads, 2, dk) - qn).max() < tol * max(1.0, np.abs(qn).max())
    # what the pages hold
    pages = f64(pool)
    flat = pages.reshape(n_pages, -1)
    for t in (0, 1, P - 1, P, cut - 1, cut, T - 1):
        pg = flat[table[0, t // P]]
        keys = pg[:kv * P * 2 * dk].reshape(kv, P, 2, dk)[:, t % P]
        vals = pg[kv * P * 2 * dk:].reshape(kv, dv, P)[:, :, t % P]
        assert np.abs(keys - kn[t]).max() < tol * max(1.0, np.abs(kn).max()), t
        assert np.abs(vals - v[t]).max() < tol * max(1.0, np.abs(v).max()), t
    out = torch.empty(T, heads * dv, device="cuda", dtype=DT[dtype])
    ops.diff_attention(q_out, pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32), out, heads, kv, dk, dv, scale,
                       lam, eps, out_scale, block=block)
    if dtype == "bfloat16":
        qn, kn, v = bf16_round(qn), bf16_round(kn), bf16_round(v)
    want = plain_maps(qn, kn, v, scale, block, lam, eps, out_scale, per).reshape(T, -1)
    err = np.abs(f64(out) - want)
    bound = 2e-4 if dtype == "float32" else 3e-2           # the output is normed: entries of order one
    assert err.max() < bound, (np.unravel_index(err.argmax(), err.shape), err.max())
    if dtype == "bfloat16" and dk in (32, 64, 128) and dv in (32, 64, 128) and P % 16 == 0:
        # the matrix-core kernels: the request as one portion in tiles of 64 rows (the last one short), then every row as a
        # single token (a step of decoded tokens), then some rows as tiles beside others as single tokens
        entries = dev([[0, T, 0, 0]], torch.int32)
        tiles = dev([[0, r, min(64, T - r)] for r in range(0, T, 64)], torch.int32)
        args = (q_out, pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32))
        calls = ops.timing_report() and None
        ops.count_calls(True)
        for shared in (True, False):       # a tile's wavefronts share keys and values through LDS, or each fetches its own
            ops.use_shared_tiles = shared
            for lists in (dict(tiles=tiles, entries=entries), dict(all_rows=True),
                          dict(tiles=tiles[:1], entries=entries, rows=dev(list(range(64, T)), torch.int32))):
                fast = torch.zeros(T, heads * dv, device="cuda", dtype=DT[dtype])
                ops.diff_attention(*args, fast, heads, kv, dk, dv, scale, lam, eps, out_scale, block=block, **lists)
                err = np.abs(f64(fast) - want)
                assert err.max() < bound, (shared, list(lists), np.unravel_index(err.argmax(), err.shape), err.max())
        ops.use_shared_tiles = True
        # single tokens with a row's keys split over three workgroups, their shares merged by a kernel of its own
        ops.force_decode_splits = 3
        fast = torch.zeros(T, heads * dv, device="cuda", dtype=DT[dtype])
        ops.diff_attention(*args, fast, heads, kv, dk, dv, scale, lam, eps, out_scale, block=block, all_rows=True, context=T)
        ops.force_decode_splits = 0
        err = np.abs(f64(fast) - want)
        assert err.max() < bound, ("split", np.unravel_index(err.argmax(), err.shape), err.max())
        took = [c["name"] for c in ops.timing_report()]
        ops.count_calls(False)
        assert took and all("[mfma]" in n for n in took), took
    # no blocks: every earlier key is visible
    ops.diff_attention(q_out, pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32), out, heads, kv, dk, dv, scale,
                       lam, eps, out_scale, block=0)
    want = plain_maps(qn, kn, v, scale, 0, lam, eps, out_scale, per).reshape(T, -1)
    assert np.abs(f64(out) - want).max() < bound


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_router_and_experts(ops, dtype):
    rng = np.random.default_rng(11)
    # the last two: enough pairs for the grouped matrix-core path in bfloat16 (experts with no token, with one, with hundreds)
    for M, W, E, top, F in [(9, 48, 5, 2, 40), (3, 50, 1, 1, 9), (17, 130, 70, 8, 33), (4, 64, 8, 8, 64), (300, 96, 11, 3, 160),
                            (200, 64, 40, 1, 32)]:
        h = bf16_round(rng.normal(size=(M, W)))
        router = rng.normal(size=(E, W)) * 2 / math.sqrt(W)
        up = bf16_round(rng.normal(size=(E, F, W)) / math.sqrt(W))
        down = bf16_round(rng.normal(size=(E, W, F)) / math.sqrt(F))
        ids = torch.empty(M, top, device="cuda", dtype=torch.int32)
        wts = torch.empty(M, top, device="cuda")
        ops.moe_route(dev(h, DT[dtype]), dev(router), ids, wts, top)
        idx, score = plain.router_choice(h, router.astype(np.float32).astype(np.float64), top)
        assert np.array_equal(ids.cpu().numpy(), idx)
        assert np.abs(f64(wts) - score).max() < 2e-6
        w = {"m.router": router.astype(np.float32).astype(np.float64)}
        for e in range(E):
            w[f"m.e{e}.up"], w[f"m.e{e}.down"] = up[e], down[e]
        y = torch.full((M, W), 5.0, device="cuda")
        ops.moe_experts(dev(h, DT[dtype]), ids, wts, dev(up.reshape(E * F, W), DT[dtype]), dev(down.reshape(E * W, F), DT[dtype]), y, E)
        want = plain.moe(h, w, "m", dict(router=dict(experts=E, top=top)))
        tol = 2e-5 if dtype == "float32" else 2e-2
        assert np.abs(f64(y) - want).max() < tol * max(1.0, np.abs(want).max())
        # the score on the expert's output instead, softmax scores renormalised over the chosen
        ops.moe_route(dev(h, DT[dtype]), dev(router), ids, wts, top, "softmax", True)
        z = h @ router.astype(np.float32).astype(np.float64).T
        p = np.exp(z - z.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        order = np.argsort(-p, axis=1, kind="stable")[:, :top]
        chosen = np.take_along_axis(p, order, 1)
        assert np.array_equal(ids.cpu().numpy(), order)
        assert np.abs(f64(wts) - chosen / chosen.sum(1, keepdims=True)).max() < 2e-6
        ops.moe_experts(dev(h, DT[dtype]), ids, wts, dev(up.reshape(E * F, W), DT[dtype]), dev(down.reshape(E * W, F), DT[dtype]), y, E, False)
        want = np.zeros((M, W))
        for m in range(M):
            for e, s in zip(order[m], f64(wts)[m]):
                want[m] += s * (plain.relu_squared(h[m] @ up[e].T) @ down[e].T)
        assert np.abs(f64(y) - want).max() < tol * max(1.0, np.abs(want).max())


def test_equal_scores_go_to_the_lower_index(ops):
    h = np.zeros((2, 8))
    h[1, 0] = 1.0
    router = np.zeros((70, 8))
    router[[5, 66, 69], 0] = 2.0
    ids = torch.empty(2, 3, device="cuda", dtype=torch.int32)
    wts = torch.empty(2, 3, device="cuda")
    ops.moe_route(dev(h), dev(router), ids, wts, 3)
    assert ids.cpu().numpy().tolist() == [[0, 1, 2], [5, 66, 69]]
    assert np.allclose(f64(wts)[0], 0.5)


# --------------------------------------------------------------------------------------- the engine
REQUEST_LENGTHS = {"a": 97, "b": 45, "c": 130, "d": 33, "e": 71, "f": 58}
PROMPT_LENGTHS = {"a": 60, "b": 12, "c": 101, "d": 30, "e": 2, "f": 41}
_made = {}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    def get(name):
        if name not in _made:
            config = mm.CONFIGS[name]
            weights = mm.draw_weights(config, seed=len(name) * 13 + 2)
            path = mm.write_folder(str(tmp_path_factory.mktemp("mumasun_" + name)), config, 0, weights)
            requests = {r: random_tokens(n, config["vocab"], 17 + i) for i, (r, n) in enumerate(REQUEST_LENGTHS.items())}
            w = mm.as_float64(weights)
            want = {r: plain.forward(config, w, t) for r, t in requests.items()}
            _made[name] = (path, requests, want, w)
        return _made[name]
    return get


def build_engine(folder, dtype, max_tokens, page_size=16, max_requests=4):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.engine import Engine
    return Engine.from_folder(folder, dtype, page_size=page_size, max_tokens=max_tokens, max_requests=max_requests, max_seq=max_tokens)


def replay(engine, trace):
    from tinyinfer_amd.engine import StepEntry
    got = {}
    for step in trace:
        logits = engine.step([StepEntry(r, t, w) for r, t, w in step["entries"]])
        rows = None if logits is None else logits.cpu().numpy().astype(np.float64)
        i = 0
        for r, _, w in step["entries"]:
            for _ in w:
                got.setdefault(r, []).append(rows[i])
                i += 1
        for r in step["end"]:
            engine.release(r)
        engine.cache.check()
    return {r: np.stack(v) for r, v in got.items()}


def errors(got, want):
    assert got.shape == want.shape, (got.shape, want.shape)
    d = got - want
    d = d - d.mean(axis=1, keepdims=True)
    ref = want - want.mean(axis=1, keepdims=True)
    return np.sqrt((d ** 2).mean(axis=1)) / np.sqrt((ref ** 2).mean(axis=1))


def worst(got, want):
    w, where = 0.0, None
    for r in want:
        e = errors(got[r], want[r])
        if e.max() > w:
            w, where = float(e.max()), (r, int(e.argmax()))
    return w, where


def within(got, want, dtype):
    """32-bit: every position within the bound.  bfloat16: all but 8 % of them, and the median far below it."""
    if dtype == "float32":
        w, where = worst(got, want)
        return w < TOL[dtype], (w, where)
    e = np.concatenate([errors(got[r], want[r]) for r in want])
    over = float((e > TOL[dtype]).mean())
    return over <= 0.08 and float(np.median(e)) < 2e-2, (over, float(np.median(e)), float(e.max()))


def make_trace(mode, requests):
    if mode == "whole":
        return traces.whole(requests)
    if mode == "tail":
        return traces.tail_one_by_one(requests, 32)
    if mode == "portions":
        return traces.portions(requests)
    return traces.mixed(requests, PROMPT_LENGTHS, live=4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page_size", [("mixed", 8), ("odd", 4), ("wide", 16)])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_engine_matches_plain(folders, name, page_size, dtype, mode):
    folder, requests, want, _ = folders(name)
    trace = make_trace(mode, requests)
    n_tok = traces.max_pages(trace, page_size) * page_size      # the tightest pool: pages are handed out again
    engine = build_engine(folder, dtype, n_tok, page_size)
    got = replay(engine, trace)
    assert not engine.cache.live_requests()
    ok, seen = within(got, want, dtype)
    assert ok, (name, mode, dtype, seen)


@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_cuts_agree_bit_for_bit_in_float32(folders, name):
    """Token by token from the first token on, in portions, and whole: in 32-bit every sum is taken in an order that does
    not depend on the step, so the logits are the same bits."""
    folder, requests, _, _ = folders(name)
    some = {r: requests[r][:40] for r in ("b", "d")}
    results = []
    for trace in (traces.whole(some), traces.tail_one_by_one(some, 39), traces.portions(some), traces.mixed(some, {"b": 20, "d": 3}, live=2)):
        engine = build_engine(folder, "float32", 256)
        results.append(replay(engine, trace))
    for other in results[1:]:
        for r in some:
            assert np.array_equal(results[0][r], other[r]), r


def test_a_state_slot_used_again_starts_from_zero(folders):
    """One slot only: the second request gets the slot (and the pages) the first one gave back; what the first left in the
    convolution's state must not reach the second's first tokens."""
    folder, requests, want, _ = folders("mixed")
    engine = build_engine(folder, "float32", 192, page_size=8, max_requests=1)
    for r in ("c", "b", "c"):
        got = replay(engine, traces.portions({r: requests[r]}))
        w, where = worst(got, {r: want[r]})
        assert w < TOL["float32"], (r, w, where)


def test_long_decoding_over_many_blocks(folders):
    """A prompt of 70 tokens in portions of 32, then 230 tokens one by one: the decoded tokens pass a dozen block edges of
    the layers with blocks of 24 and several of the one with 50, pages of 8 go back behind them, the rotation's table ends
    before the sequence does (max_seq below it would refuse; here the pool is large enough)."""
    from tinyinfer_amd.engine import StepEntry
    folder, _, _, w = folders("mixed")
    config = mm.CONFIGS["mixed"]
    toks = random_tokens(300, config["vocab"], 99)
    want = plain.forward(config, w, toks)
    for dtype in ("float32", "bfloat16"):
        engine = build_engine(folder, dtype, 320, page_size=8)
        rows, at = [], 0
        while at < 70:
            n = min(32, 70 - at)
            rows.append(engine.step([StepEntry("x", toks[at:at + n], list(range(n)))]).cpu().numpy())
            at += n
        for t in toks[70:]:
            rows.append(engine.step([StepEntry("x", [t], [0])]).cpu().numpy())
            engine.cache.check()
        got = np.concatenate(rows).astype(np.float64)
        # pages before the current block have gone back: at most a block of 50 and the page under way are held
        assert engine.cache.num_free_pages() >= 320 // 8 - (50 // 8 + 2)
        ok, seen = within({"x": got}, {"x": want}, dtype)
        assert ok, (dtype, seen)


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generation_through_the_entry_point(folders, use_graph):
    """Several prompts of unequal length at once through LLM.generate: the scheduler cuts the prompts into portions of 16
    and batches decoding requests; every generated token is the plain model's argmax."""
    import tinyinfer_amd as ti
    folder, requests, _, w = folders("mixed")
    config = mm.CONFIGS["mixed"]
    prompts = [requests["b"][:37], requests["d"][:5], requests["e"][:50], requests["f"][:1]]
    n_new = 12
    llm = ti.LLM(folder, dtype="float32", max_seq=128, max_requests=3, chunk_size=16, max_batched_tokens=40, use_graph=use_graph)
    got = llm.generate(prompts, max_new_tokens=n_new, temperature=0.0)
    for p, g in zip(prompts, got):
        toks = list(p)
        for _ in range(n_new):
            logits = plain.forward(config, w, toks)[-1]
            best = int(np.argmax(logits))
            margin = logits[best] - np.partition(logits, -2)[-2]
            toks.append(best)
            if margin < 1e-3:          # a tie within rounding: what follows may differ legitimately
                break
        n = len(toks) - len(p)
        assert g[:n] == toks[len(p):], (p[:3], g, toks[len(p):])


def plain_greedy(config, w, prompt, n_new):
    """(generated ids, how many of them stand clear of a tie within rounding)."""
    toks, sure = list(prompt), 0
    for k in range(n_new):
        logits = plain.forward(config, w, toks)[-1]
        best = int(np.argmax(logits))
        if sure == k and logits[best] - np.partition(logits, -2)[-2] > 1e-3:
            sure = k + 1
        toks.append(best)
    return toks[len(prompt):], sure


def test_command_line_generates_from_a_mumasun_folder(folders):
    """bin/tinyinfer picks the model by config.json: token ids in, the plain model's greedy tokens out; with --cuda-graph too."""
    import os
    import subprocess
    import sys
    folder, requests, _, w = folders("odd")
    config = mm.CONFIGS["odd"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p1, p2 = requests["b"][:11], requests["d"][:4]
    for extra in ([], ["--cuda-graph"]):
        run = subprocess.run([sys.executable, os.path.join(root, "bin", "tinyinfer"), "-m", folder, "-n", "6", "-p", ",".join(map(str, p1)),
                              "-p", " ".join(map(str, p2)), "--dtype", "float32", "--max-seq", "64"] + extra,
                             capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr[-2000:]
        outputs = [l[len("[output] "):].split() for l in run.stdout.split("\n") if l.startswith("[output] ")]
        assert len(outputs) == 2
        for p, got in zip((p1, p2), outputs):
            want, sure = plain_greedy(config, w, p, 6)
            assert [int(t) for t in got][:sure] == want[:sure], (got, want)


def test_random_weights_drawn_on_the_device_run():
    """A config.json alone: the parts' declared distributions give a model that steps (what the bench tool measures)."""
    from tinyinfer_amd.engine import Engine, StepEntry
    for name in ("mixed", "wide"):
        engine = Engine.from_config(mm.CONFIGS[name], seed=3, dtype="bfloat16", page_size=16, max_tokens=256, max_requests=2, max_seq=256)
        toks = random_tokens(70, mm.CONFIGS[name]["vocab"], 1)
        a = engine.step([StepEntry("x", toks, [69])]).cpu().numpy()
        engine.release("x")
        assert engine.step([StepEntry("y", toks[:69], [])]) is None
        b = engine.step([StepEntry("y", toks[69:], [0])]).cpu().numpy()
        assert np.isfinite(a).all() and a.std() > 0
        assert np.abs(a - b).max() < 0.08 * max(1e-6, np.abs(a).max())


def test_trace_replay_program(folders, tmp_path):
    """The replay program on a Mumasun folder: it picks the model by config.json and writes the logits the engine gives."""
    import os
    import subprocess
    import sys
    folder, requests, want, _ = folders("odd")
    some = {r: requests[r] for r in ("b", "d", "f")}
    trace = traces.mixed(some, PROMPT_LENGTHS, live=2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", str(traces.max_tokens(trace))], input=traces.to_jsonl(trace), text=True,
                          capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    V = mm.CONFIGS["odd"]["vocab"]
    got = {}
    for i, step in enumerate(trace):
        assert f"done {i}" in proc.stdout
        rows = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V).astype(np.float64)
        k = 0
        for r, _, wnt in step["entries"]:
            for _ in wnt:
                got.setdefault(r, []).append(rows[k])
                k += 1
    w, where = worst({r: np.stack(v) for r, v in got.items()}, {r: want[r] for r in some})
    assert w < TOL["float32"], (w, where)

"""Seeded random sweeps: shapes, views, dtypes and parameters drawn at random, the device result checked against the
CPU checker (numpy where the checker restates a quirk of the reference that the device does not share).

Every case prints what it is before it runs, so a failure (or a crash) names its case in the captured output.
The tolerances are those of the per-operator tests."""
import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import ops

pytestmark = pytest.mark.gpu
INTS = [ta.int8, ta.int16, ta.int32, ta.int64]
FLOATS = [ta.float16, ta.bfloat16, ta.float32, ta.float64]
EXTENTS = [1, 2, 3, 5, 8, 16, 17, 31, 64, 100, 128, 257, 513]


def rand_shape(rng, limit, min_rank=1, max_rank=4):
    rank = int(rng.integers(min_rank, max_rank + 1))
    while True:
        shape = [int(rng.choice(EXTENTS)) for _ in range(rank)]
        if np.prod(shape) <= limit:
            return shape


def random_view(rng, h, d):
    """The same random view (none, a transposition, a strided slice or a permutation) of a host and a device tensor."""
    r = rng.random()
    if r < 0.5 or h.rank < 2:
        return h, d
    if r < 0.7:
        i, j = sorted(rng.choice(h.rank, 2, replace=False).tolist())
        return h.transpose(i, j), d.transpose(i, j)
    if r < 0.9:
        axis = int(rng.integers(0, h.rank))
        n = h.shape[axis]
        if n < 3:
            return h, d
        first = int(rng.integers(0, n // 2))
        last = int(rng.integers(first + 1, n + 1))
        step = int(rng.choice([1, 1, 2]))
        index = tuple(slice(first, last, step) if k == axis else slice(None) for k in range(h.rank))
        return h[index], d[index]
    order = rng.permutation(h.rank).tolist()
    return h.permute(*order), d.permute(*order)


def same_bits(got, want):
    return got.dtype is want.dtype and got.shape == want.shape and bool((got.storage() == want.storage()).all())


def within(got, want, rtol, atol):
    g, w = got.astype(np.float64), want.astype(np.float64)
    with np.errstate(invalid="ignore"):   # inf - inf where both sides agree on an infinity
        return got.shape == want.shape and bool(((np.abs(g - w) <= atol + rtol * np.abs(w)) | (g == w)).all())


def test_random_convolutions(device, oracle):
    rng = np.random.default_rng(101)
    done = 0
    while done < 120:
        n = int(rng.integers(1, 4))
        c = int(rng.choice([1, 2, 3, 4, 8, 16, 32, 48, 64, 96, 128, 160, 192, 256]))
        h, w = int(rng.integers(3, 41)), int(rng.integers(3, 41))
        if rng.random() < 0.6:
            w = max(8, w // 8 * 8)
        o = int(rng.choice([1, 5, 16, 32, 40, 64, 70, 128, 200, 256, 512]))
        kh = int(rng.integers(1, 8))
        kw = kh if rng.random() < 0.7 else int(rng.integers(1, 8))
        if rng.random() < 0.3:
            kh = kw = 3
        if rng.random() < 0.2:
            kh = kw = 1
        sh = int(rng.integers(1, 4))
        sw = sh if rng.random() < 0.8 else int(rng.integers(1, 4))
        ph = int(rng.integers(0, 4))
        pw = ph if rng.random() < 0.8 else int(rng.integers(0, 4))
        if done % 2:   # the shapes the 3x3 and 1x1 kernels take: many channels, rows of whole 16-byte vectors
            n, c, w, h = int(rng.integers(1, 6)), int(rng.choice([32, 64, 96, 128, 160, 192, 256])), int(rng.choice([8, 16, 24, 32, 40, 56])), int(rng.integers(3, 61))
            o = int(rng.choice([32, 64, 70, 128, 256, 512]))
            kh = kw = int(rng.choice([1, 3]))
            sh = sw = int(rng.choice([1, 2]))
            ph = pw = int(rng.choice([0, 1])) if kh == 3 else 0
        if h + 2 * ph < kh or w + 2 * pw < kw:
            continue
        ho, wo = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
        if n * o * ho * wo * c * kh * kw > 1.5e8:
            continue
        dtype = [ta.float16, ta.bfloat16, ta.float32][int(rng.integers(0, 3))]
        bias = bool(rng.random() < 0.5)
        what = f"conv {done}: N={n} C={c} H={h} W={w} O={o} K=({kh},{kw}) s=({sh},{sw}) p=({ph},{pw}) {dtype} bias={bias}"
        print(what, flush=True)
        fan_in = c * kh * kw
        lim = 2 * (2.0 / fan_in) ** 0.5
        hx, dx = support.both(support.values_for(dtype, 7, 1 + done, (n, c, h, w), -2, 2), dtype, device)
        hw, dw = support.both(support.values_for(dtype, 7, 1000 + done, (o, c, kh, kw), -lim, lim), dtype, device)
        hb, db = support.both(support.values_for(dtype, 7, 2000 + done, (o,), -2, 2), dtype, device) if bias else (None, None)
        want = ops.convolve2d(hx, hw, hb, (sh, sw), (ph, pw)).numpy()
        got = ops.convolve2d(dx, dw, db, (sh, sw), (ph, pw)).numpy()
        if dtype is ta.float32:
            rtol, atol = 1e-5, fan_in * 2.0 ** -24 * 4
        else:
            rtol, atol = (2e-3 if dtype is ta.float16 else 2.0 ** -7), 1e-3
        assert np.isfinite(got.astype(np.float64)).all() and within(got, want, rtol, atol), what
        done += 1


def test_random_matrix_products(device, oracle):
    rng = np.random.default_rng(102)

    def extent(limit):
        r = rng.random()
        if r < 0.15:
            return int(rng.integers(1, 9))
        if r < 0.55:
            return int(rng.integers(1, limit // 8 + 1)) * 8
        return int(rng.integers(1, limit + 1))

    for done in range(160):
        m, n, k = extent(520), extent(520), extent(1200)
        if rng.random() < 0.1:
            k = int(rng.integers(1, 5)) * 1024
        while m * n * k > 6e7:
            m = max(1, m // 2)
        r = rng.random()
        if r < 0.6:
            ba, bb = (), ()
        elif r < 0.75:
            ba, bb = (int(rng.integers(1, 4)),), ()
        elif r < 0.9:
            ba = bb = (int(rng.integers(1, 3)), int(rng.integers(1, 4)))
        else:
            ba, bb = (2, 1), (1, 3)
        first_t, second_t = bool(rng.random() < 0.35), bool(rng.random() < 0.6)
        sa = ba + ((k, m) if first_t else (m, k))
        sb = bb + ((n, k) if second_t else (k, n))
        va = [("transpose", (-1, -2))] if first_t else []
        vb = [("transpose", (-1, -2))] if second_t else []
        dtype = [ta.float16, ta.bfloat16, ta.float32, ta.float16, ta.bfloat16, ta.float64, ta.int32][int(rng.integers(0, 7))]
        what = f"gemm {done}: M={m} N={n} K={k} batch={ba}x{bb} tA={first_t} tB={second_t} {dtype}"
        print(what, flush=True)
        lo, hi = (-3, 3) if dtype.is_integral else (-1, 1)
        ha, da = support.both(support.values_for(dtype, 11, 1 + done, sa, lo, hi), dtype, device)
        hb, db = support.both(support.values_for(dtype, 11, 5000 + done, sb, lo, hi), dtype, device)
        want = ops.matmul(support.apply_view(ha, va), support.apply_view(hb, vb)).numpy()
        got = ops.matmul(support.apply_view(da, va), support.apply_view(db, vb)).numpy()
        if dtype.is_integral:
            rtol, atol = 0, 0
        elif dtype is ta.float32:
            rtol, atol = 1e-5, k * 2.0 ** -24
        elif dtype is ta.float64:
            rtol, atol = 1e-13, k * 2.0 ** -53
        else:
            rtol, atol = (2e-3 if dtype is ta.float16 else 2.0 ** -7), 1e-3
        assert within(got, want, rtol, atol), what


PAIRS = ([(d, d) for d in INTS + FLOATS] +
         [(ta.int8, ta.int32), (ta.int64, ta.int16), (ta.int32, ta.float32), (ta.float64, ta.int32), (ta.float32, ta.float64),
          (ta.float16, ta.float32), (ta.float32, ta.bfloat16), (ta.bfloat16, ta.float64)])


def test_random_elementwise_compare_reduce(device, oracle):
    rng = np.random.default_rng(103)
    for done in range(400):
        kind = str(rng.choice(["binary", "unary", "reduce", "compare"]))
        if kind == "binary":
            pair = PAIRS[int(rng.integers(0, len(PAIRS)))]
            out = rand_shape(rng, 300000)
            sa = [1 if rng.random() < 0.25 else n for n in out]
            sb = [1 if rng.random() < 0.25 else n for n in out]
            if rng.random() < 0.3:
                sb = sb[int(rng.integers(0, len(sb))):]
            op = str(rng.choice(["add", "sub", "mul"]))
            what = f"{done}: {op} {pair[0]} {sa} x {pair[1]} {sb}"
            print(what, flush=True)
            ha, da = support.both(support.values_for(pair[0], 13, 1 + done, sa, -100, 100), pair[0], device)
            hb, db = support.both(support.values_for(pair[1], 13, 7000 + done, sb, -100, 100), pair[1], device)
            assert same_bits(getattr(ops, op)(da, db), getattr(ops, op)(ha, hb)), what
        elif kind == "unary":
            dtype = FLOATS[int(rng.integers(0, 4))]
            shape = rand_shape(rng, 300000)
            op = str(rng.choice(["neg", "abs", "exp", "log", "sqrt", "sin", "cos", "tanh"]))
            what = f"{done}: {op} {dtype} {shape}"
            print(what, flush=True)
            lo, hi = (0.1, 4) if op in ("log", "sqrt") else (-4, 4)
            h, d = support.both(support.values_for(dtype, 13, 1 + done, shape, lo, hi), dtype, device)
            h, d = random_view(rng, h, d)
            rtol = {ta.float16: 2.0 ** -9, ta.bfloat16: 2.0 ** -6, ta.float32: 1e-5, ta.float64: 1e-12}[dtype]
            assert within(getattr(ops, op)(d).numpy(), getattr(ops, op)(h).numpy(), rtol, 0.0 if dtype is ta.float64 else 1e-6), what
        elif kind == "compare":
            dtype = (INTS + FLOATS)[int(rng.integers(0, 8))]
            shape = rand_shape(rng, 300000)
            op = str(rng.choice(["eq", "ne", "gt", "ge", "lt", "le"]))
            what = f"{done}: {op} {dtype} {shape}"
            print(what, flush=True)
            ha, da = support.both(np.round(support.values_for(dtype, 13, 1 + done, shape, -3, 3).astype(np.float64)), dtype, device)
            hb, db = support.both(np.round(support.values_for(dtype, 13, 9000 + done, shape, -3, 3).astype(np.float64)), dtype, device)
            want, got = getattr(ops, op)(ha, hb), getattr(ops, op)(da, db)
            assert got.shape == want.shape and (got.numpy() == want.numpy()).all(), what
        else:
            dtype = [ta.float32, ta.float16, ta.bfloat16, ta.float64, ta.int32, ta.int8, ta.int64][int(rng.integers(0, 7))]
            shape = rand_shape(rng, 600000)
            axis, keep = int(rng.integers(0, len(shape))), bool(rng.random() < 0.3)
            op = str(rng.choice(["argmax", "argmin", "max", "min", "sum", "mean"]))
            if op == "mean" and dtype.is_integral:
                op = "sum"
            what = f"{done}: {op} {dtype} {shape} axis={axis} keep={keep}"
            print(what, flush=True)
            # small integers (with both zeros among them): ties everywhere, and sums are exact in every type
            x = np.round(support.values_for(dtype, 13, 1 + done, shape, -3, 3).astype(np.float64))
            h, d = support.both(x, dtype, device)
            if rng.random() < 0.4:
                h2, d2 = random_view(rng, h, d)
                if h2.rank == h.rank:
                    h, d = h2, d2
            want, got = getattr(ops, op)(h, axis, keep), getattr(ops, op)(d, axis, keep)
            if op in ("sum", "mean") and not dtype.is_integral:
                rtol = {ta.float16: 2.0 ** -10, ta.bfloat16: 2.0 ** -7, ta.float32: 1e-6, ta.float64: 1e-14}[dtype]
                assert within(got.numpy(), want.numpy(), rtol, rtol), what
            else:
                assert same_bits(got, want), what


def test_random_moves_and_the_rest(device, oracle):
    rng = np.random.default_rng(104)
    every = INTS + FLOATS
    for done in range(300):
        kind = str(rng.choice(["repeat", "concat", "outer", "tri", "scale", "repack", "cpy", "pow", "allclose", "polar"]))
        dtype = every[int(rng.integers(0, 8))]
        if kind == "repeat":
            shape = rand_shape(rng, 60000)
            times = int(rng.integers(1, 5))
            h, d = support.both(support.values_for(dtype, 17, 1 + done, shape, -100, 100), dtype, device)
            h, d = random_view(rng, h, d)
            axis = int(rng.integers(0, h.rank))
            what = f"{done}: repeat {dtype} {h} axis={axis} x{times}"
            print(what, flush=True)
            assert same_bits(ops.repeat(d, times, axis), ops.repeat(h, times, axis)), what
        elif kind == "concat":
            shape = rand_shape(rng, 60000)
            axis = int(rng.integers(0, len(shape)))
            other = list(shape)
            other[axis] = int(rng.integers(1, 40))
            h1, d1 = support.both(support.values_for(dtype, 17, 1 + done, shape, -100, 100), dtype, device)
            h2, d2 = support.both(support.values_for(dtype, 17, 9000 + done, other, -100, 100), dtype, device)
            x1, x2 = h1.numpy(), h2.numpy()
            if rng.random() < 0.3 and len(shape) >= 2:
                i, j = sorted(rng.choice(len(shape), 2, replace=False).tolist())
                d1, d2 = d1.transpose(i, j), d2.transpose(i, j)
                x1, x2 = np.swapaxes(x1, i, j), np.swapaxes(x2, i, j)
                axis = j if axis == i else i if axis == j else axis
            what = f"{done}: concat {dtype} {d1} + {d2} axis={axis}"
            print(what, flush=True)
            # against numpy: the reference's CPU kernel addresses what follows the axis with one stride
            # (src/cpu/concat.cpp:66,76) and is only right with at most one dimension behind it
            got = ops.concatenate(d1, d2, axis).numpy()
            want = np.concatenate([x1, x2], axis=axis)
            assert got.shape == want.shape and (got == want).all(), what
        elif kind == "outer":
            n, m = int(rng.integers(1, 700)), int(rng.integers(1, 700))
            second = every[int(rng.integers(0, 8))] if rng.random() < 0.3 else dtype
            what = f"{done}: outer {dtype}[{n}] x {second}[{m}]"
            print(what, flush=True)
            h1, d1 = support.both(support.values_for(dtype, 17, 1 + done, (n,), -10, 10), dtype, device)
            h2, d2 = support.both(support.values_for(second, 17, 9000 + done, (m,), -10, 10), second, device)
            try:
                want = ops.outer(h1, h2)
            except ta.TannicError:
                with pytest.raises(ta.TannicError):   # a pair the reference's table gets wrong: refused on both sides
                    ops.outer(d1, d2)
                continue
            assert same_bits(ops.outer(d1, d2), want), what
        elif kind == "tri":
            shape = rand_shape(rng, 60000, 2, 4)
            k = int(rng.integers(-5, 6))
            name = str(rng.choice(["triu", "tril"]))
            what = f"{done}: {name} {dtype} {shape} k={k}"
            print(what, flush=True)
            h, d = support.both(support.values_for(dtype, 17, 1 + done, shape, -100, 100), dtype, device)
            try:
                want = getattr(ops, name)(h, k)
            except ta.TannicError:
                with pytest.raises(ta.TannicError):
                    getattr(ops, name)(d, k)
                continue
            assert same_bits(getattr(ops, name)(d, k), want), what
        elif kind == "scale":
            shape = rand_shape(rng, 200000)
            value = float(rng.integers(-5, 6)) if dtype.is_integral else float(rng.uniform(-3, 3))
            what = f"{done}: scale {dtype} {shape} by {value}"
            print(what, flush=True)
            h, d = support.both(support.values_for(dtype, 17, 1 + done, shape, -20, 20), dtype, device)
            h, d = random_view(rng, h, d)
            assert same_bits(ops.scale(d, value), ops.scale(h, value)), what
        elif kind == "repack":
            shape = rand_shape(rng, 200000)
            h, d = support.both(support.values_for(dtype, 17, 1 + done, shape, -100, 100), dtype, device)
            h, d = random_view(rng, h, d)
            what = f"{done}: repack {dtype} {h}"
            print(what, flush=True)
            assert same_bits(ops.repack(d), ops.repack(h)), what
        elif kind == "cpy":
            shape = rand_shape(rng, 100000, 2, 4)
            what = f"{done}: copy into a window, {dtype} {shape}"
            print(what, flush=True)
            hs, ds = support.both(support.values_for(dtype, 17, 1 + done, shape, -100, 100), dtype, device)
            whole = [n + int(rng.integers(0, 4)) for n in shape]
            hd, dd = support.both(support.values_for(dtype, 17, 9000 + done, whole, -100, 100), dtype, device)
            window = tuple(slice(b - n, b) for n, b in zip(shape, whole))
            ops.copy_into(hd[window], hs)
            ops.copy_into(dd[window], ds)
            assert (hd.storage() == dd.to(ta.Host()).storage()).all(), what
        elif kind == "pow":
            pair = [(ta.float32, ta.float32), (ta.float64, ta.float64), (ta.int32, ta.float32), (ta.float32, ta.float64),
                    (ta.float16, ta.float32)][int(rng.integers(0, 5))]
            shape = rand_shape(rng, 100000)
            what = f"{done}: pow {pair} {shape}"
            print(what, flush=True)
            h1, d1 = support.both(support.values_for(pair[0], 17, 1 + done, shape, 0.5, 3), pair[0], device)
            h2, d2 = support.both(support.values_for(pair[1], 17, 9000 + done, shape, -2, 2), pair[1], device)
            want, got = ops.pow(h1, h2), ops.pow(d1, d2)
            assert got.dtype is want.dtype and within(got.numpy(), want.numpy(), 1e-12 if want.dtype is ta.float64 else 4e-6, 0.0), what
        elif kind == "allclose":
            kind_of_float = FLOATS[int(rng.integers(0, 4))]
            shape = rand_shape(rng, 300000)
            what = f"{done}: allclose {kind_of_float} {shape}"
            print(what, flush=True)
            x = support.values_for(kind_of_float, 17, 1 + done, shape, -4, 4)
            y = x.copy()
            if rng.random() < 0.5:
                y.flat[int(rng.integers(0, y.size))] += 1.0
            h1, d1 = support.both(x, kind_of_float, device)
            h2, d2 = support.both(y, kind_of_float, device)
            assert ops.allclose(d1, d2) == ops.allclose(h1, h2), what
        else:
            kind_of_float = [ta.float32, ta.float64][int(rng.integers(0, 2))]
            shape = rand_shape(rng, 100000)
            what = f"{done}: polar {kind_of_float} {shape}"
            print(what, flush=True)
            h1, d1 = support.both(support.values_for(kind_of_float, 17, 1 + done, shape, 0.1, 3), kind_of_float, device)
            h2, d2 = support.both(support.values_for(kind_of_float, 17, 9000 + done, shape, -3, 3), kind_of_float, device)
            want, got = ops.polar(h1, h2).numpy(), ops.polar(d1, d2).numpy()
            tol = 1e-12 if kind_of_float is ta.float64 else 2e-6
            assert got.shape == want.shape and (np.abs(got - want) <= tol * (np.abs(want) + 1)).all(), what


def test_random_matrix_products_of_sliced_views(device):
    """Operands cut out of larger matrices with offsets and steps (so that neither matrix stride need be 1), one of them
    possibly transposed: small integers, every type is exact and numpy decides."""
    rng = np.random.default_rng(105)

    def cut(n):
        first = int(rng.integers(0, max(1, n // 3)))
        last = int(rng.integers(first + 1, n + 1))
        return slice(first, last, int(rng.choice([1, 1, 1, 2])))

    for done in range(150):
        dtype = [ta.float16, ta.bfloat16, ta.float32, ta.int32, ta.float64][int(rng.integers(0, 5))]
        m, k, n = (int(rng.choice([1, 7, 16, 33, 64, 100, 130, 257])) for _ in range(3))
        a = rng.integers(-3, 4, (m + 5, k + 9)).astype(np.float64)
        b = rng.integers(-3, 4, (k + 9, n + 6)).astype(np.float64)
        index_a = (cut(m + 5), cut(k + 9))
        depth = a[index_a].shape[1]
        start = int(rng.integers(0, k + 9 - depth + 1))
        index_b = (slice(start, start + depth), cut(n + 6))
        turned = bool(rng.random() < 0.3)
        what = f"{done}: {dtype} A{a.shape}{index_a} B{b.shape}{index_b} A stored transposed: {turned}"
        print(what, flush=True)
        da = ta.tensor(a.T.copy() if turned else a, dtype, device)
        db = ta.tensor(b, dtype, device)
        va = da[(index_a[1], index_a[0])].transpose(0, 1) if turned else da[index_a]
        got = ops.matmul(va, db[index_b]).numpy().astype(np.float64)
        want = a[index_a] @ b[index_b]
        assert got.shape == want.shape and (got == want).all(), what

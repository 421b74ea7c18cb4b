"""Inputs for the chains of tests/cases/pointwise_chains.h: seeded values with the special cases of each Operation mixed
in (zeros of both signs, NaN, infinities, the extreme integers), and the constants each chain is run with."""
import numpy as np

# constants (four floats, converted by the chain text to the constant's type) and the 3x3 matrix of MxVFloat3
CONSTANTS = {9: (0.25, -3.5, 100.0, 0), 10: (-77, 0, 0, 0), 11: (0.0, -1.5, 2.5, 0), 12: (0.0, -1.5, 2.5, 0), 13: (100, 0, 0, 0),
             14: (-5, 0, 70000, 0), 15: (0x00ffff00, 0, 0, 0), 16: (0x0f0f, 1, -256, 0), 17: (0x7fffff80, 0, 0, 0),
             19: (5, 0, 0, 0), 20: (3, 0, 0, 0)}
MATRIX = (0.299, 0.587, 0.114, -0.168736, -0.331264, 0.5, 0.5, -0.418688, -0.081312)


def inputs(which, cases, h, w, seed):
    in_dtype, cn, _ = cases[which]
    rng = np.random.default_rng(1000 * which + seed)
    shape = (h, w, cn) if cn > 1 else (h, w)
    n = h * w * cn
    if in_dtype == np.float32:
        a = rng.uniform(-8.0, 8.0, n).astype(np.float32)
        if which in (5, 7):                      # Sqrt, Ln: mostly non-negative arguments
            a = np.abs(a) * np.float32(40.0)
        special = [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-38, 3.4e38, -3.4e38, 2.5, 0.25, 88.0, -104.0, 4.0, 1e-45]
        a[: len(special)] = np.array(special, np.float32)[: min(len(special), n)]
        if which == 21:                           # matrix product: finite values only, so NaN payloads do not enter the comparison
            a[: len(special)] = np.float32(1.5)
    elif in_dtype == np.uint8:
        a = rng.integers(0, 256, n, dtype=np.uint8)
        a[:4] = [0, 1, 255, 128]
    elif in_dtype == np.int8:
        a = rng.integers(-128, 128, n).astype(np.int8)
        a[:4] = [-128, 127, 0, -1]
    elif in_dtype == np.int16:
        a = rng.integers(-32768, 32768, n).astype(np.int16)
        a[:4] = [-32768, 32767, 0, -1]
    elif in_dtype == np.int32:
        a = rng.integers(-2**31, 2**31, n, dtype=np.int64).astype(np.int32)
        a[:6] = [-2**31, 2**31 - 1, 0, -1, 1, -77]
    elif in_dtype == np.uint32:
        a = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
        a[:4] = [0, 0xffffffff, 0x80000000, 1]
    else:
        raise TypeError(in_dtype)
    return a.reshape(shape)


def constants(which):
    return CONSTANTS.get(which, (0, 0, 0, 0))


def same(which, got, want, inexact):
    """Bit-exact for every chain but the logarithm and exponential ones (the platform's logf / expf: 1e-5 relative, the
    tolerance this library states for float outputs; NaN and infinities have to match as such)."""
    if which not in inexact:
        return got.tobytes() == want.tobytes()
    g, w = got.astype(np.float64), want.astype(np.float64)
    finite = np.isfinite(w)
    ok = np.array_equal(np.isnan(g), np.isnan(w)) and np.array_equal(g[~finite & ~np.isnan(w)], w[~finite & ~np.isnan(w)])
    tiny = np.abs(w) < 1e-37                         # results in the denormal range: flushing is platform business
    sel = finite & ~tiny
    return bool(ok and np.all(np.abs(g[sel] - w[sel]) <= 1e-5 * np.abs(w[sel])) and np.all(np.abs(g[finite & tiny]) < 2e-37))


def dual_inputs(which, cases, h, w, seed):
    """Two images for the two-image chains: seeded values with zeros, NaN, infinities and the extreme integers mixed in."""
    in_dtype, cn, _ = cases[which]
    rng = np.random.default_rng(7000 + 10 * which + seed)
    shape = (h, w, cn) if cn > 1 else (h, w)
    n = h * w * cn
    out = []
    for k in range(2):
        if in_dtype == np.float32:
            v = rng.uniform(-50.0, 50.0, n).astype(np.float32)
            special = [0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, 3.4e38, 1e-38][k:] + [2.0, -3.0]
            v[: len(special)] = np.array(special, np.float32)
        elif in_dtype == np.uint8:
            v = rng.integers(0, 256, n, dtype=np.uint8)
            v[:4] = [0, 255, 255, 1] if k == 0 else [255, 0, 255, 2]
        elif in_dtype == np.int32:
            v = rng.integers(-2**31, 2**31, n, dtype=np.int64).astype(np.int32)
            v[:2] = [-2**31, 2**31 - 1] if k == 0 else [2**31 - 1, -2**31]
        else:
            v = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
            v[:2] = [0, 0xffffffff]
        out.append(v.reshape(shape))
    return out


def sweep_case(i, cases, dual_cases):
    """Case i of a seeded sweep over the per-channel chains (even i) and the two-image chains (odd i): which chain, image
    size (40 to 900 wide, 1 to 12 rows) and the padding of each pitch in elements of the wider of input and output."""
    rng = np.random.RandomState(110000 + i)
    w, h = int(rng.randint(40, 900)), int(rng.randint(1, 12))
    table = cases if i % 2 == 0 else dual_cases
    keys = sorted(table)
    which = keys[int(rng.randint(0, len(keys)))]
    in_dtype, _, out_dtype = table[which]
    unit = max(np.dtype(in_dtype).itemsize, np.dtype(out_dtype).itemsize)
    return i % 2, which, w, h, [int(rng.randint(0, 4)) * unit for _ in range(2)]

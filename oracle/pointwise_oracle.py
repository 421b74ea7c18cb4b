"""CPU restatement, in numpy, of the per-channel Operations of the reference's basic_ops headers that a fused chain may
hold between its read and its write.  TEST INFRASTRUCTURE: only tests/ may import this file; nothing in the product does.

Every function follows the C++ expression of the reference on one channel, including the type the expression promotes
to (numpy integer arithmetic is done in the promoted type explicitly, then cast like a C conversion):

  Abs, Sqr, Sqrt, Ln, Exp, AbsDiff   FK/algorithms/basic_ops/math.h:26-170
  Max, Min                           FK/algorithms/basic_ops/logical.h:37-88 -> std::max / std::min, (a < b) ? b : a
  BwAnd, BwOr, BwXor, BwNot, shifts  FK/algorithms/basic_ops/bitwise.h:23-157 with the operators of
                                     FK/core/utils/vector_utils.h:565-600
  MxVFloat3<BinaryType>              FK/algorithms/basic_ops/algebraic.h:25-40
  the two-input forms on a pair      FK/algorithms/basic_ops/arithmetic.h:26-124 (Add, Sub, Mul, Div: the channel-wise operators of
                                     vector_utils.h:508-563 on the two halves), and the UnaryType forms in the headers above
  per-channel application            FK/core/constexpr_libs/constexpr_vector_exec.h:24-108

Pinned by: the reference's CPU backend on the same inputs (oracle/_ref, tests/test_oracle_pointwise.py), closed forms
(|x| of known values, x*x, exact square roots, ln(e^k), masks and shifts of known bit patterns, the identity matrix),
and the special values the comparisons fix (NaN, -0, the most negative integer).  Sqrt is correctly rounded and so
bit-exact everywhere; Ln and Exp are the platform's logf / expf: results agree within the tolerance the tests state.
"""
import numpy as np

# which -> (input dtype, input channels, output dtype); the list of tests/cases/pointwise_chains.h
CASES = {
    0: (np.float32, 3, np.float32), 1: (np.int32, 1, np.int32), 2: (np.int8, 3, np.int8), 3: (np.float32, 3, np.float32),
    4: (np.uint8, 3, np.int32), 5: (np.float32, 3, np.float32), 6: (np.uint8, 3, np.float32), 7: (np.float32, 1, np.float32),
    8: (np.float32, 3, np.float32), 9: (np.float32, 3, np.float32), 10: (np.int32, 1, np.int32), 11: (np.float32, 3, np.float32),
    12: (np.float32, 3, np.float32), 13: (np.uint8, 1, np.uint8), 14: (np.int32, 3, np.int32), 15: (np.uint32, 1, np.uint32),
    16: (np.int32, 3, np.int32), 17: (np.uint32, 1, np.uint32), 18: (np.uint32, 1, np.uint32), 19: (np.uint32, 1, np.uint32),
    20: (np.int32, 1, np.int32), 21: (np.float32, 3, np.float32), 22: (np.uint8, 1, np.float32), 23: (np.int16, 2, np.int16),
}
INEXACT = {7, 8, 22}          # logf / expf: the platform's, compared within a tolerance


def _promote(a):
    """The type C++ arithmetic on this channel type is done in: int for everything narrower than int."""
    if a.dtype in (np.uint8, np.int8, np.uint16, np.int16):
        return a.astype(np.int32)
    return a


def op_abs(a):
    if a.dtype.kind == "u":
        return a.copy()
    if a.dtype.kind == "f":
        # s < 0 ? -s : s  -- -0.0 and NaN fail the comparison and come back as they are
        return np.where(a < 0, -a, a).astype(a.dtype)
    wide = _promote(a)
    with np.errstate(over="ignore"):
        return np.where(wide < 0, -wide, wide).astype(a.dtype)      # static_cast<ST>(-s); the most negative value wraps onto itself


def op_sqr(a, out_dtype):
    wide = _promote(a)
    with np.errstate(over="ignore"):
        return (wide * wide).astype(out_dtype)


def op_sqrt(a):
    with np.errstate(invalid="ignore"):
        return np.sqrt(a.astype(np.float32)).astype(np.float32)


def op_ln(a):
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.log(a.astype(np.float32)).astype(np.float32)


def op_exp(a):
    with np.errstate(over="ignore"):
        return np.exp(a.astype(np.float32)).astype(np.float32)


def op_absdiff(a, c, out_dtype):
    wide = _promote(a)
    with np.errstate(over="ignore", invalid="ignore"):
        d = wide - np.asarray(c).astype(wide.dtype)
        if d.dtype.kind == "u":
            return d.astype(out_dtype)                                  # d < 0 never holds
        return np.where(d < 0, -d, d).astype(out_dtype)


def op_max(a, c):
    c = np.broadcast_to(np.asarray(c).astype(a.dtype), a.shape)
    with np.errstate(invalid="ignore"):
        return np.where(a < c, c, a)


def op_min(a, c):
    c = np.broadcast_to(np.asarray(c).astype(a.dtype), a.shape)
    with np.errstate(invalid="ignore"):
        return np.where(c < a, c, a)


def op_bitwise(which, a, c, out_dtype):
    wide = _promote(a)
    c = np.asarray(c).astype(wide.dtype)
    r = {"and": np.bitwise_and, "or": np.bitwise_or, "xor": np.bitwise_xor}[which](wide, c)
    return r.astype(out_dtype)


def op_not(a, out_dtype):
    return np.invert(_promote(a)).astype(out_dtype)


def op_shift(left, a, c, out_dtype):
    wide = _promote(a)
    c = np.asarray(c).astype(wide.dtype)
    with np.errstate(over="ignore"):
        return (np.left_shift(wide, c) if left else np.right_shift(wide, c)).astype(out_dtype)     # >> of a signed value is arithmetic


def op_mxv3(a, m):
    """Row r: (v.x * m[r][0] + v.y * m[r][1]) + v.z * m[r][2], every product and sum rounded to binary32."""
    m = np.asarray(m, np.float32).reshape(3, 3)
    a = a.astype(np.float32)
    out = np.empty_like(a)
    for r in range(3):
        p0 = (a[..., 0] * m[r, 0]).astype(np.float32)
        p1 = (a[..., 1] * m[r, 1]).astype(np.float32)
        p2 = (a[..., 2] * m[r, 2]).astype(np.float32)
        out[..., r] = ((p0 + p1).astype(np.float32) + p2).astype(np.float32)
    return out


def run(which, src, c=(0, 0, 0, 0), m=(1, 0, 0, 0, 1, 0, 0, 0, 1)):
    """Chain number `which` of tests/cases/pointwise_chains.h on src, shaped (H, W) or (H, W, channels)."""
    in_dtype, cn, out_dtype = CASES[which]
    assert src.dtype == in_dtype and (src.ndim == 3 and src.shape[2] == cn or src.ndim == 2 and cn == 1), (which, src.dtype, src.shape)
    cf = np.asarray(c, np.float32)
    const = cf[:cn] if cn > 1 else cf[0]
    as_int = lambda t: np.asarray(const).astype(np.float32).astype(t)      # the chain text converts the float constants like a C cast
    if which in (0, 1, 2, 23): return op_abs(src)
    if which in (3, 4): return op_sqr(src, out_dtype)
    if which in (5, 6): return op_sqrt(src)
    if which == 7: return op_ln(src)
    if which in (8, 22): return op_exp(src)
    if which == 9: return op_absdiff(src, const, out_dtype)
    if which == 10: return op_absdiff(src, as_int(np.int32), out_dtype)
    if which == 11: return op_max(src, const)
    if which == 12: return op_min(src, const)
    if which == 13: return op_max(src, as_int(np.uint8))
    if which == 14: return op_min(src, as_int(np.int32))
    if which == 15: return op_bitwise("and", src, as_int(np.uint32), out_dtype)
    if which == 16: return op_bitwise("or", src, as_int(np.int32), out_dtype)
    if which == 17: return op_bitwise("xor", src, as_int(np.uint32), out_dtype)
    if which == 18: return op_not(src, out_dtype)
    if which == 19: return op_shift(True, src, as_int(np.uint32), out_dtype)
    if which == 20: return op_shift(False, src, as_int(np.int32), out_dtype)
    if which == 21: return op_mxv3(src, m)
    raise KeyError(which)


# two-image chains of tests/cases/pointwise_chains.h (`dual`): which -> (input dtype, channels, output dtype)
DUAL_CASES = {
    0: (np.float32, 3, np.float32), 1: (np.uint8, 3, np.int32), 2: (np.float32, 1, np.float32), 3: (np.float32, 3, np.float32),
    4: (np.float32, 3, np.float32), 5: (np.uint32, 1, np.uint32), 6: (np.float32, 3, np.float32), 7: (np.int32, 1, np.int32),
    8: (np.uint8, 3, np.uint8), 9: (np.uint32, 1, np.uint32), 10: (np.uint32, 1, np.uint32),
}


def saturate_cast_u8(f):
    """cxp::saturate_cast<uchar>(float), FK/core/constexpr_libs/constexpr_saturate.h:91-113: NaN -> 0, round half to even, clamp."""
    f = f.astype(np.float32)
    with np.errstate(invalid="ignore"):
        r = np.rint(f)
        return np.where(np.isnan(f), 0, np.clip(r, 0, 255)).astype(np.uint8)


def run_dual(which, a, b):
    """Two-image chain number `which`: DualSourceRead -> the two-input form of the Operation (-> more) -> write."""
    in_dtype, cn, out_dtype = DUAL_CASES[which]
    assert a.dtype == in_dtype and b.dtype == in_dtype and a.shape == b.shape
    wa, wb = _promote(a), _promote(b)
    with np.errstate(all="ignore"):
        if which == 0: return (a + b).astype(np.float32)
        if which == 1: return np.abs(wa - wb).astype(np.int32)                 # uchar - uchar is an int; d < 0 ? -d : d
        if which == 2: return (a * b).astype(np.float32)
        if which == 3: return (a / b).astype(np.float32)
        if which == 4: return (a - b).astype(np.float32)
        if which == 5: return np.bitwise_xor(a, b)
        if which == 6: return np.where(a < b, b, a)
        if which == 7: return np.where(b < a, b, a)
        if which == 8:
            s = (wa + wb).astype(np.int32)                                      # Add<uchar3, uchar3, int3>
            return saturate_cast_u8(s.astype(np.float32) * np.float32(0.5))
        if which == 9: return np.bitwise_and(a, b)
        if which == 10: return np.bitwise_or(a, b)
    raise KeyError(which)

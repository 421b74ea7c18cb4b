"""ctypes bindings for the test-only CPU oracle (oracle/libfkl_oracle.so) and, when it has been built, the
reference library's own CPU backend behind a C ABI (oracle/_ref/libfkl_ref.so).

Only tests, the smoke check and the CPU-baseline leg of bench.py may import this module.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "libfkl_oracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libfkl_ref.so")

U8, F32, U16 = 0, 1, 2
READ_2D, READ_NV12, READ_NV21, READ_P010, READ_P210, READ_Y210, READ_UYVY, READ_PLANAR = 0, 1, 2, 3, 4, 5, 6, 7
PRESERVE_AR, IGNORE_AR = 0, 1
MUL, ADD, SUB, DIV, REORDER, SATCAST_U8, CAST_F32, YUV2RGB_709_FULL = 1, 2, 3, 4, 5, 6, 7, 8
YUV2RGB, RGB2YUV, RGB2GRAY, ADD_LAST, DISCARD, SATCAST_U16, CLAMP, SATURATE_FLOAT, CAST_TRUNC = 9, 10, 11, 12, 13, 14, 15, 16, 17
WRITE_2D, TENSOR_WRITE, TENSOR_SPLIT, WRITE_YUV, TENSOR_TSPLIT = 0, 1, 2, 3, 4

# fk::PixelFormat / ColorDepth / ColorRange / ColorPrimitives enumerator values, and what the oracle calls each format
PF_NV12, PF_NV21, PF_P010, PF_P210, PF_Y210, PF_UYVY = 0, 1, 3, 6, 8, 10
CD_P8, CD_P10, CD_P12, CD_FN8, CD_FN10, CD_FN12 = 0, 1, 2, 3, 4, 5
CR_LIMITED, CR_FULL = 0, 1
CP_BT601, CP_BT709, CP_BT2020 = 0, 1, 2
PF_READ_KIND = {PF_NV12: READ_NV12, PF_NV21: READ_NV21, PF_P010: READ_P010, PF_P210: READ_P210, PF_Y210: READ_Y210, PF_UYVY: READ_UYVY}
PF_DEPTH = {PF_NV12: CD_P8, PF_NV21: CD_P8, PF_P010: CD_P10, PF_P210: CD_P10, PF_Y210: CD_P10, PF_UYVY: CD_P8}
PF_WIDE = {PF_NV12: False, PF_NV21: False, PF_P010: True, PF_P210: True, PF_Y210: True, PF_UYVY: False}
_NP_ELEM = {np.dtype(np.uint8): U8, np.dtype(np.float32): F32, np.dtype(np.uint16): U16}


def frame_shape(pf: int, width: int, height: int):
    """(rows, samples per row) of the backing array of a width x height frame in pixel format pf."""
    if pf in (PF_NV12, PF_NV21, PF_P010):
        return height + height // 2, width
    if pf == PF_P210:
        return 2 * height, width
    return height, 2 * width       # packed 4:2:2


class Op(C.Structure):
    _fields_ = [("code", C.c_int32), ("p", C.c_float * 4), ("idx", C.c_int32 * 4)]


class Read(C.Structure):
    _fields_ = [
        ("kind", C.c_int32), ("elem", C.c_int32), ("cn", C.c_int32),
        ("width", C.c_int32), ("height", C.c_int32), ("pitch", C.c_int32),
        ("data", C.c_void_p),
        ("has_crop", C.c_int32), ("crop", C.c_int32 * 4),
        ("has_resize", C.c_int32), ("dst_w", C.c_int32), ("dst_h", C.c_int32),
        ("ar", C.c_int32), ("bg", C.c_float * 4),
        ("n_tap_ops", C.c_int32), ("tap_ops", C.POINTER(Op)),
        ("use_default", C.c_int32), ("def_", C.c_float * 4),
        ("warp", C.c_int32), ("warp_m", C.c_float * 9),
        ("deinterlace", C.c_int32),
        ("border", C.c_int32), ("border_value", C.c_float * 4),
        ("channel_stride", C.c_int64),
    ]


class Write(C.Structure):
    _fields_ = [
        ("kind", C.c_int32), ("elem", C.c_int32), ("cn", C.c_int32), ("data", C.c_void_p),
        ("width", C.c_int32), ("height", C.c_int32), ("planes", C.c_int32), ("color_planes", C.c_int32),
        ("pitch", C.c_int32), ("yuv_format", C.c_int32),
    ]


class ResizeParams(C.Structure):
    _fields_ = [("dst_w", C.c_int32), ("dst_h", C.c_int32), ("fx", C.c_float), ("fy", C.c_float),
                ("x1", C.c_int32), ("y1", C.c_int32), ("x2", C.c_int32), ("y2", C.c_int32)]


class MT(C.Structure):
    _fields_ = [("mt", C.c_uint32 * 624), ("idx", C.c_int32)]


_oracle = None
_ref = None


def oracle():
    global _oracle
    if _oracle is None:
        lib = C.CDLL(ORACLE_SO)
        lib.fklo_execute.restype = C.c_int
        lib.fklo_execute.argtypes = [C.c_int32, C.POINTER(Read), C.c_int32, C.POINTER(Op), C.c_int32, C.POINTER(Write)]
        lib.fklo_compute_resize_params.restype = None
        lib.fklo_compute_resize_params.argtypes = [C.c_int32] * 5 + [C.POINTER(ResizeParams)]
        lib.fklo_saturate_cast_u8.restype = C.c_uint8
        lib.fklo_saturate_cast_u8.argtypes = [C.c_float]
        lib.fklo_banker_round.restype = C.c_float
        lib.fklo_banker_round.argtypes = [C.c_float]
        lib.fklo_round_half_away.restype = C.c_float
        lib.fklo_round_half_away.argtypes = [C.c_float]
        lib.fklo_yuv2rgb_709_full_matrix.restype = None
        lib.fklo_yuv2rgb_709_full_matrix.argtypes = [C.POINTER(C.c_float)]
        lib.fklo_yuv2rgb_709_full.restype = None
        lib.fklo_yuv2rgb_709_full.argtypes = [C.POINTER(C.c_uint8), C.POINTER(C.c_float)]
        lib.fklo_color_matrix.restype = C.c_int
        lib.fklo_color_matrix.argtypes = [C.c_int32] * 4 + [C.POINTER(C.c_float)]
        lib.fklo_depth_constants.restype = C.c_int
        lib.fklo_depth_constants.argtypes = [C.c_int32] + [C.POINTER(C.c_float)] * 3
        lib.fklo_saturate_cast_u16.restype = C.c_uint16
        lib.fklo_saturate_cast_u16.argtypes = [C.c_float]
        lib.fklo_bilinear.restype = C.c_float
        lib.fklo_bilinear.argtypes = [C.c_float] * 6
        lib.fklo_mt_seed.restype = None
        lib.fklo_mt_seed.argtypes = [C.POINTER(MT), C.c_uint32]
        lib.fklo_mt_next.restype = C.c_uint32
        lib.fklo_mt_next.argtypes = [C.POINTER(MT)]
        lib.fklo_mt_fill_bytes.restype = None
        lib.fklo_mt_fill_bytes.argtypes = [C.POINTER(MT), C.c_void_p, C.c_uint64]
        lib.fklo_mt_fill_unit_floats.restype = None
        lib.fklo_mt_fill_unit_floats.argtypes = [C.POINTER(MT), C.c_void_p, C.c_uint64]
        lib.fklo_mt_fill_range_floats.restype = None
        lib.fklo_mt_fill_range_floats.argtypes = [C.POINTER(MT), C.c_void_p, C.c_uint64, C.c_float, C.c_float]
        lib.fklo_mt_fill_u32.restype = None
        lib.fklo_mt_fill_u32.argtypes = [C.POINTER(MT), C.c_void_p, C.c_uint64]
        _oracle = lib
    return _oracle


def have_ref() -> bool:
    return os.path.exists(REF_SO)


def ref():
    global _ref
    if _ref is None:
        lib = C.CDLL(REF_SO)
        for name in dir(lib):
            pass
        _ref = lib
    return _ref


# The same harness compiled against THIS repository's headers (oracle/Makefile, target hostexec): the chains then run on
# this repository's TransformDPP<ParArch::CPU> executor.  `with host_executor():` makes the ref_* wrappers below call it.
HOSTEXEC_SO = os.path.join(ROOT, "oracle", "libfkl_hostexec.so")


def have_hostexec() -> bool:
    return os.path.exists(HOSTEXEC_SO)


class host_executor:
    def __enter__(self):
        global _ref
        self.saved = _ref
        _ref = C.CDLL(HOSTEXEC_SO)
        return _ref

    def __exit__(self, *exc):
        global _ref
        _ref = self.saved
        return False


# ---- helpers to describe chains to the oracle -----------------------------------------------------------

def op(code, p=(0, 0, 0, 0), idx=(0, 0, 0, 0)) -> Op:
    o = Op()
    o.code = code
    pv = list(np.asarray(p, dtype=np.float32).reshape(-1))
    pv = (pv + [pv[-1]] * 4)[:4] if len(pv) == 1 else (pv + [0.0] * 4)[:4]
    for i in range(4):
        o.p[i] = float(pv[i])
        o.idx[i] = int(idx[i])
    return o


def ops_array(ops):
    arr = (Op * max(1, len(ops)))()
    for i, o in enumerate(ops):
        arr[i] = o
    return arr


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


def read_2d(a: np.ndarray, cn: int, crop=None, resize=None, ar=IGNORE_AR, bg=(0, 0, 0, 0), tap_ops=None,
            pitch=None, width=None) -> Read:
    """`a` is (H, W, cn) uint8/float32 or (H, W) for cn == 1 (possibly a padded row buffer if pitch given)."""
    r = Read()
    r.kind = READ_2D
    r.elem = _NP_ELEM[a.dtype]
    r.cn = cn
    r.height = a.shape[0]
    r.width = int(width) if width is not None else a.shape[1]
    r.pitch = int(pitch) if pitch is not None else a.strides[0]
    r.data = _ptr(a)
    _fill_common(r, crop, resize, ar, bg, tap_ops)
    return r


def read_nv12(buf: np.ndarray, width: int, height: int, resize=None, ar=IGNORE_AR, tap_ops=None) -> Read:
    r = Read()
    r.kind = READ_NV12
    r.elem = U8
    r.cn = 3
    r.width, r.height = width, height
    r.pitch = buf.strides[0]
    r.data = _ptr(buf)
    _fill_common(r, None, resize, ar, (0, 0, 0, 0), tap_ops)
    return r


def read_yuv(pf: int, buf: np.ndarray, width: int, height: int, resize=None, ar=IGNORE_AR, tap_ops=None) -> Read:
    """A frame in pixel format pf (see frame_shape) of uint8 or uint16 samples."""
    r = Read()
    r.kind = PF_READ_KIND[pf]
    r.elem = U16 if PF_WIDE[pf] else U8
    r.cn = 3
    r.width, r.height = width, height
    r.pitch = buf.strides[0]
    r.data = _ptr(buf)
    _fill_common(r, None, resize, ar, (0, 0, 0, 0), tap_ops)
    return r


def write_yuv(pf: int, buf: np.ndarray, width: int, height: int) -> Write:
    w = Write()
    w.kind = WRITE_YUV
    w.elem = U16 if PF_WIDE[pf] else U8
    w.cn = 3
    w.data = _ptr(buf)
    w.width, w.height, w.planes, w.color_planes = width, height, 1, 1
    w.pitch = buf.strides[0]
    w.yuv_format = PF_READ_KIND[pf]
    return w


def _fill_common(r, crop, resize, ar, bg, tap_ops):
    if crop is not None:
        r.has_crop = 1
        for i in range(4):
            r.crop[i] = int(crop[i])
    if resize is not None:
        r.has_resize = 1
        r.dst_w, r.dst_h = int(resize[0]), int(resize[1])
        r.ar = ar
    for i in range(min(4, len(bg))):
        r.bg[i] = float(bg[i])
    if tap_ops:
        arr = ops_array(tap_ops)
        r._keep = arr  # keep alive
        r.n_tap_ops = len(tap_ops)
        r.tap_ops = C.cast(arr, C.POINTER(Op))


def write(kind, a: np.ndarray, cn: int, width: int, height: int, planes: int = 1, color_planes: int = 1,
          pitch=None) -> Write:
    w = Write()
    w.kind = kind
    w.elem = _NP_ELEM[a.dtype]
    w.cn = cn
    w.data = _ptr(a)
    w.width, w.height, w.planes, w.color_planes = width, height, planes, color_planes
    esz = a.dtype.itemsize
    if pitch is None:
        pitch = width * esz * (1 if kind in (TENSOR_SPLIT, TENSOR_TSPLIT) else cn)
    w.pitch = int(pitch)
    return w


def execute(reads, ops, writes) -> None:
    ra = (Read * len(reads))(*reads)
    wa = (Write * len(writes))(*writes)
    oa = ops_array(ops)
    rc = oracle().fklo_execute(len(reads), ra, len(ops), oa, len(writes), wa)
    if rc != 0:
        raise RuntimeError(f"fklo_execute failed with code {rc}")


# ---- the five benchmark chains, through the oracle ------------------------------------------------------

def oracle_crop_resize_par_u8(src, rects, dst, bg, mul, sub):
    dw, dh = dst
    b = len(rects)
    out = np.zeros((b, dh, dw, 3), np.uint8)
    reads = [read_2d(src, 3, crop=rects[i], resize=dst, ar=PRESERVE_AR, bg=bg) for i in range(b)]
    execute(reads, [op(MUL, mul), op(SUB, sub), op(SATCAST_U8)], [write(TENSOR_WRITE, out, 3, dw, dh, b, 1)])
    return out


PRESERVE_AR_RN_EVEN, PRESERVE_AR_LEFT = 2, 3


def oracle_letterbox_ar(ar, src, rect, dst, bg):
    """src (H,W,3) u8 -> crop -> letterboxed bilinear resize in aspect-ratio mode `ar` -> (dh,dw,3) f32."""
    dw, dh = dst
    out = np.zeros((dh, dw, 3), np.float32)
    execute([read_2d(src, 3, crop=rect, resize=dst, ar=ar, bg=bg)], [], [write(WRITE_2D, out, 3, dw, dh)])
    return out


def oracle_crop_resize_norm_split(src, rects, dst, sub, div):
    dw, dh = dst
    b = len(rects)
    out = np.zeros((b, 3, dh, dw), np.float32)
    reads = [read_2d(src, 3, crop=rects[i], resize=dst, ar=IGNORE_AR) for i in range(b)]
    execute(reads, [op(REORDER, idx=(2, 1, 0, 0)), op(SUB, sub), op(DIV, div)],
            [write(TENSOR_SPLIT, out, 3, dw, dh, b, 3)])
    return out


def _defaulted(r: Read, default) -> Read:
    r.use_default = 1
    for i, v in enumerate(default):
        r.def_[i] = float(v)
    return r


def oracle_crop_resize_default_norm_split(src, rects, dst, used, default, sub, div):
    """Configuration-3 chain with BatchRead<CONDITIONAL_WITH_DEFAULT>: planes >= used yield `default` (float3)."""
    dw, dh = dst
    b = len(rects)
    out = np.zeros((b, 3, dh, dw), np.float32)
    reads = [read_2d(src, 3, crop=rects[i], resize=dst, ar=IGNORE_AR) for i in range(b)]
    for i in range(used, b):
        _defaulted(reads[i], default)
    execute(reads, [op(REORDER, idx=(2, 1, 0, 0)), op(SUB, sub), op(DIV, div)],
            [write(TENSOR_SPLIT, out, 3, dw, dh, b, 3)])
    return out


def oracle_batch_default_cast_mul(srcs, active, default, mul):
    """B uchar3 images, planes >= active yield `default` (uchar3); Cast to float3, Mul; Tensor<float3> B x H x W x 3."""
    b = len(srcs)
    h, w = srcs[0].shape[:2]
    out = np.zeros((b, h, w, 3), np.float32)
    reads = [read_2d(srcs[i], 3) for i in range(b)]
    for i in range(active, b):
        _defaulted(reads[i], default)
    execute(reads, [op(CAST_F32), op(MUL, mul)], [write(TENSOR_WRITE, out, 3, w, h, b, 1)])
    return out


def oracle_warp(src, cn, matrix, dst, perspective):
    """Warping<Affine|Perspective> of an (H,W[,cn]) u8/f32 image into a (dh,dw[,cn]) float image."""
    dw, dh = dst
    out = np.zeros((dh, dw, cn) if cn > 1 else (dh, dw), np.float32)
    r = read_2d(src, cn)
    r.warp = 2 if perspective else 1
    r.dst_w, r.dst_h = dw, dh
    m = np.zeros(9, np.float32)
    m[: (9 if perspective else 6)] = np.asarray(matrix, np.float32).ravel()
    for i in range(9):
        r.warp_m[i] = float(m[i])
    execute([r], [], [write(WRITE_2D, out, cn, dw, dh)])
    return out


def ref_warp_u8x3(src, matrix, dst, perspective):
    dw, dh = dst
    out = np.zeros((dh, dw, 3), np.float32)
    m = np.zeros(9, np.float32)
    m[: (9 if perspective else 6)] = np.asarray(matrix, np.float32).ravel()
    rc = ref().fklref_warp_u8x3(C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0], _f32p(m), int(bool(perspective)),
                                dw, dh, C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def warp_kind(dtype, cn):
    """The pixel-type number of fklref_warp_kind / fklcase_warp_kind."""
    return {("uint8", 4): 2, ("uint16", 3): 3, ("uint8", 1): 4}[(np.dtype(dtype).name, cn)]


def ref_warp(src, matrix, dst, perspective):
    """As ref_warp_u8x3 for (H,W,4) uint8, (H,W,3) uint16 and (H,W) uint8 images."""
    cn = src.shape[2] if src.ndim == 3 else 1
    dw, dh = dst
    out = np.zeros((dh, dw, cn) if cn > 1 else (dh, dw), np.float32)
    m = np.zeros(9, np.float32)
    m[: (9 if perspective else 6)] = np.asarray(matrix, np.float32).ravel()
    rc = ref().fklref_warp_kind(warp_kind(src.dtype, cn), C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0], _f32p(m),
                                int(bool(perspective)), dw, dh, C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


DEINTERLACE_BLEND, DEINTERLACE_LINEAR_EVEN, DEINTERLACE_LINEAR_ODD = 1, 2, 3


def oracle_deinterlace(src, cn, mode):
    """Deinterlace of an (H,W[,cn]) u8/f32 image into a float image of the same shape."""
    h, w = src.shape[:2]
    out = np.zeros((h, w, cn) if cn > 1 else (h, w), np.float32)
    r = read_2d(src, cn)
    r.deinterlace = mode
    execute([r], [], [write(WRITE_2D, out, cn, w, h)])
    return out


def ref_deinterlace_u8x3(src, mode):
    h, w = src.shape[:2]
    out = np.zeros((h, w, 3), np.float32)
    rc = ref().fklref_deinterlace_u8x3(C.c_void_p(_ptr(src)), w, h, src.strides[0], int(mode), C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def oracle_batch_muladd_sat(srcs, mul, add):
    b = len(srcs)
    h, w = srcs[0].shape[:2]
    outs = [np.zeros((h, w, 3), np.uint8) for _ in range(b)]
    reads = [read_2d(srcs[i], 3, tap_ops=[op(MUL, mul[i]), op(ADD, add[i])]) for i in range(b)]
    execute(reads, [op(SATCAST_U8)], [write(WRITE_2D, outs[i], 3, w, h) for i in range(b)])
    return outs


def oracle_add_mul_chain(src, n_ops, addv, mulv):
    h, w = src.shape
    out = np.zeros((h, w), np.float32)
    ops = [op(ADD, [addv]) if i % 2 == 0 else op(MUL, [mulv]) for i in range(n_ops)]
    execute([read_2d(src, 1)], ops, [write(WRITE_2D, out, 1, w, h)])
    return out


def oracle_nv12_rgb_resize_split(nv12, width, height, dst, scale):
    dw, dh = dst
    out = np.zeros((3, dh, dw), np.float32)
    execute([read_nv12(nv12, width, height, resize=dst, tap_ops=[op(YUV2RGB_709_FULL)])],
            [op(MUL, [scale])], [write(TENSOR_SPLIT, out, 3, dw, dh, 1, 3)])
    return out


def oracle_crop_swap_u8(src, rects):
    b = len(rects)
    cw, ch = int(rects[0][2]), int(rects[0][3])
    out = np.zeros((b, ch, cw, 3), np.uint8)
    reads = [read_2d(src, 3, crop=rects[i]) for i in range(b)]
    execute(reads, [op(REORDER, idx=(2, 1, 0, 0))], [write(TENSOR_WRITE, out, 3, cw, ch, b, 1)])
    return out


# ---- the same chains through the reference's CPU backend ------------------------------------------------

def _f32p(a):
    return np.ascontiguousarray(a, dtype=np.float32).ctypes.data_as(C.POINTER(C.c_float))


def _i32p(a):
    return np.ascontiguousarray(a, dtype=np.int32).ctypes.data_as(C.POINTER(C.c_int32))


def ref_crop_resize_par_u8(src, rects, dst, bg, mul, sub):
    assert len(rects) == 5
    dw, dh = dst
    out = np.zeros((5, dh, dw, 3), np.uint8)
    rc = ref().fklref_crop_resize_par_u8_b5(C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0],
                                            _i32p(rects), dw, dh, _f32p(bg), _f32p(mul), _f32p(sub),
                                            C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def ref_crop_resize_norm_split(src, rects, dst, sub, div):
    b = len(rects)
    fn = {8: "fklref_crop_resize_norm_split_b8", 64: "fklref_crop_resize_norm_split_b64"}[b]
    dw, dh = dst
    out = np.zeros((b, 3, dh, dw), np.float32)
    rc = getattr(ref(), fn)(C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0], _i32p(rects), dw, dh,
                            _f32p(sub), _f32p(div), C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def ref_crop_resize_default_norm_split(src, rects, dst, used, default, sub, div):
    assert len(rects) == 8
    dw, dh = dst
    out = np.zeros((8, 3, dh, dw), np.float32)
    rc = ref().fklref_crop_resize_default_norm_split_b8(
        C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0], _i32p(rects), dw, dh, int(used),
        _f32p(default), _f32p(sub), _f32p(div), C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def ref_batch_default_cast_mul(srcs, active, default, mul):
    assert len(srcs) == 4
    h, w = srcs[0].shape[:2]
    out = np.zeros((4, h, w, 3), np.float32)
    sp = (C.c_void_p * 4)(*[_ptr(s) for s in srcs])
    d = np.ascontiguousarray(default, np.uint8)
    rc = ref().fklref_batch_default_cast_mul_b4(sp, w, h, srcs[0].strides[0], int(active), C.c_void_p(_ptr(d)), _f32p(mul),
                                                C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def ref_batch_muladd_sat(srcs, mul, add):
    b = len(srcs)
    fn = {4: "fklref_batch_muladd_sat_b4", 100: "fklref_batch_muladd_sat_b100"}[b]
    h, w = srcs[0].shape[:2]
    outs = [np.zeros((h, w, 3), np.uint8) for _ in range(b)]
    sp = (C.c_void_p * b)(*[_ptr(s) for s in srcs])
    op_ = (C.c_void_p * b)(*[_ptr(o) for o in outs])
    rc = getattr(ref(), fn)(sp, w, h, srcs[0].strides[0], _f32p(mul), _f32p(add), op_, outs[0].strides[0])
    assert rc == 0
    return outs


def ref_add_mul_chain(src, n_ops, addv, mulv, tf=0):
    h, w = src.shape
    out = np.zeros((h, w), np.float32)
    rc = ref().fklref_add_mul_chain(C.c_void_p(_ptr(src)), w, h, src.strides[0], n_ops, C.c_float(addv),
                                    C.c_float(mulv), C.c_void_p(_ptr(out)), out.strides[0], tf)
    assert rc == 0
    return out


def ref_nv12_rgb_resize_split(nv12, width, height, dst, scale):
    dw, dh = dst
    out = np.zeros((3, dh, dw), np.float32)
    rc = ref().fklref_nv12_rgb_resize_split(C.c_void_p(_ptr(nv12)), width, height, nv12.strides[0], dw, dh,
                                            C.c_float(scale), C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


def ref_crop_swap_u8(src, rects):
    assert len(rects) == 4
    cw, ch = int(rects[0][2]), int(rects[0][3])
    out = np.zeros((4, ch, cw, 3), np.uint8)
    rc = ref().fklref_crop_swap_u8_b4(C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0],
                                      _i32p(rects), C.c_void_p(_ptr(out)))
    assert rc == 0
    return out


# ---- pixel formats and colour conversions ----------------------------------------------------------------

def oracle_color_matrix(cd, cr, cp, to_rgb):
    m = (C.c_float * 9)()
    assert oracle().fklo_color_matrix(cd, cr, cp, int(bool(to_rgb)), m) == 0
    return np.array(list(m), np.float32)


def ref_color_matrix(cd, cr, cp, to_rgb):
    m = np.zeros(9, np.float32)
    assert ref().fklref_color_matrix(cd, cr, cp, int(bool(to_rgb)), _f32p(m)) == 0
    return m


def oracle_yuv_to_rgb(pf, cr, cp, frame, width, height):
    out = np.zeros((height, width, 3), np.float32)
    execute([read_yuv(pf, frame, width, height)], [op(YUV2RGB, idx=(PF_DEPTH[pf], cr, cp, 0))], [write(WRITE_2D, out, 3, width, height)])
    return out


def ref_yuv_to_rgb(pf, cr, cp, frame, width, height):
    out = np.zeros((height, width, 3), np.float32)
    rc = ref().fklref_yuv_to_rgb(pf, cr, cp, C.c_void_p(_ptr(frame)), width, height, frame.strides[0], C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


def _satcast(pf):
    return SATCAST_U16 if PF_WIDE[pf] else SATCAST_U8


def oracle_rgb_to_yuv(pf, cr, cp, rgb, frame):
    """rgb (H,W,3) uint8/uint16; `frame` is the pre-filled backing array the chain stores into (returned)."""
    h, w = rgb.shape[:2]
    execute([read_2d(rgb, 3)], [op(RGB2YUV, idx=(PF_DEPTH[pf], cr, cp, 0)), op(_satcast(pf))], [write_yuv(pf, frame, w, h)])
    return frame


def ref_rgb_to_yuv(pf, cr, cp, rgb, frame):
    h, w = rgb.shape[:2]
    rc = ref().fklref_rgb_to_yuv(pf, cr, cp, C.c_void_p(_ptr(rgb)), w, h, rgb.strides[0], C.c_void_p(_ptr(frame)), frame.strides[0])
    assert rc == 0, rc
    return frame


YUV_RESIZE_COMBO = {PF_NV21: (CR_FULL, CP_BT601), PF_UYVY: (CR_LIMITED, CP_BT709), PF_P010: (CR_LIMITED, CP_BT2020)}


def oracle_yuv_resize(pf, frame, width, height, dst, scale):
    dw, dh = dst
    cr, cp = YUV_RESIZE_COMBO[pf]
    out = np.zeros((dh, dw, 3), np.float32)
    execute([read_yuv(pf, frame, width, height, resize=dst, tap_ops=[op(YUV2RGB, idx=(PF_DEPTH[pf], cr, cp, 0))])],
            [op(MUL, [scale])], [write(WRITE_2D, out, 3, dw, dh)])
    return out


def ref_yuv_resize(pf, frame, width, height, dst, scale):
    dw, dh = dst
    out = np.zeros((dh, dw, 3), np.float32)
    rc = ref().fklref_yuv_resize(pf, C.c_void_p(_ptr(frame)), width, height, frame.strides[0], dw, dh, C.c_float(scale),
                                 C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


def oracle_convert_depth(cd, cr, cp, to_rgb, src):
    h, w = src.shape[:2]
    out = np.zeros((h, w, 3), np.float32)
    execute([read_2d(src, 3)], [op(YUV2RGB if to_rgb else RGB2YUV, idx=(cd, cr, cp, 0))], [write(WRITE_2D, out, 3, w, h)])
    return out


def ref_convert_depth(cd, cr, cp, to_rgb, src):
    h, w = src.shape[:2]
    out = np.zeros((h, w, 3), np.float32)
    rc = ref().fklref_convert_depth(cd, cr, cp, int(bool(to_rgb)), C.c_void_p(_ptr(src)), w, h, src.strides[0], C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


# ColorConversion codes exercised by the case drivers: which -> (input dtype, cn in, output dtype, cn out, oracle ops)
_SWAP3, _SWAP4 = (2, 1, 0, 0), (2, 1, 0, 3)
COLOR_CODES = {
    0: (np.uint8, 3, np.uint8, 4, lambda: [op(ADD_LAST, [255.0])]),                                    # BGR2BGRA
    1: (np.uint8, 4, np.uint8, 3, lambda: [op(DISCARD, idx=(3, 0, 0, 0))]),                              # BGRA2BGR
    2: (np.uint8, 3, np.uint8, 4, lambda: [op(REORDER, idx=_SWAP3), op(ADD_LAST, [255.0])]),            # BGR2RGBA
    3: (np.uint8, 4, np.uint8, 3, lambda: [op(REORDER, idx=_SWAP4), op(DISCARD, idx=(3, 0, 0, 0))]),     # BGRA2RGB
    4: (np.uint8, 4, np.uint8, 4, lambda: [op(REORDER, idx=_SWAP4)]),                                   # BGRA2RGBA
    5: (np.uint8, 3, np.uint8, 1, lambda: [op(RGB2GRAY, idx=(U8, 0, 0, 0))]),                            # RGB2GRAY
    6: (np.uint8, 3, np.uint8, 1, lambda: [op(REORDER, idx=_SWAP3), op(RGB2GRAY, idx=(U8, 0, 0, 0))]),   # BGR2GRAY
    7: (np.uint8, 4, np.uint8, 1, lambda: [op(RGB2GRAY, idx=(U8, 0, 0, 0))]),                            # RGBA2GRAY
    8: (np.uint8, 4, np.uint8, 1, lambda: [op(REORDER, idx=_SWAP4), op(RGB2GRAY, idx=(U8, 0, 0, 0))]),   # BGRA2GRAY
    9: (np.float32, 3, np.float32, 1, lambda: [op(RGB2GRAY, idx=(F32, 0, 0, 0))]),                       # RGB2GRAY, float
    10: (np.uint16, 3, np.uint16, 4, lambda: [op(ADD_LAST, [1023.0])]),                                 # BGR2BGRA, 10 bit
}


def _image(shape_hw, cn, dtype):
    h, w = shape_hw
    return np.zeros((h, w, cn) if cn > 1 else (h, w), dtype)


def oracle_convert_code(which, src):
    _, cin, odt, cout, ops = COLOR_CODES[which]
    h, w = src.shape[:2]
    out = _image((h, w), cout, odt)
    execute([read_2d(src, cin)], ops(), [write(WRITE_2D, out, cout, w, h)])
    return out


def ref_convert_code(which, src):
    _, cin, odt, cout, _ = COLOR_CODES[which]
    h, w = src.shape[:2]
    out = _image((h, w), cout, odt)
    rc = ref().fklref_convert_code(which, C.c_void_p(_ptr(src)), w, h, src.strides[0], C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


NORMALIZE = {0: (np.uint8, 255.0), 1: (np.uint16, 1023.0)}


def oracle_normalize(which, src):
    h, w = src.shape[:2]
    out = np.zeros((h, w, 3), np.float32)
    execute([read_2d(src, 3)], [op(DIV, [NORMALIZE[which][1]])], [write(WRITE_2D, out, 3, w, h)])
    return out


def ref_normalize(which, src):
    h, w = src.shape[:2]
    out = np.zeros((h, w, 3), np.float32)
    rc = ref().fklref_normalize(which, C.c_void_p(_ptr(src)), w, h, src.strides[0], C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


# ---- SaturateDepth / DenormalizePixel / SaturateDenormalizePixel / SaturateFloat / Saturate -----------------------------
# which -> (input channels, output dtype, oracle operations given (lo, hi)); the list of tests/cases/color_chains.h
DEPTH_OPS = {
    0: (1, np.float32, lambda lo, hi: [op(CLAMP, [0.0, 255.0])]),
    1: (1, np.float32, lambda lo, hi: [op(CLAMP, [0.0, 1023.0])]),
    2: (3, np.uint8, lambda lo, hi: [op(MUL, [255.0]), op(CAST_TRUNC, idx=(U8, 0, 0, 0))]),
    3: (3, np.float32, lambda lo, hi: [op(MUL, [255.0]), op(CAST_TRUNC, idx=(F32, 0, 0, 0))]),
    4: (3, np.uint8, lambda lo, hi: [op(SATURATE_FLOAT), op(MUL, [255.0]), op(CAST_TRUNC, idx=(U8, 0, 0, 0))]),
    5: (3, np.uint16, lambda lo, hi: [op(SATURATE_FLOAT), op(MUL, [1023.0]), op(CAST_TRUNC, idx=(U16, 0, 0, 0))]),
    6: (4, np.float32, lambda lo, hi: [op(SATURATE_FLOAT)]),
    7: (3, np.float32, lambda lo, hi: [op(CLAMP, [lo, hi])]),
    8: (3, np.uint16, lambda lo, hi: [op(MUL, [4095.0]), op(CAST_TRUNC, idx=(U16, 0, 0, 0))]),
    9: (4, np.uint8, lambda lo, hi: [op(SATURATE_FLOAT), op(MUL, [255.0]), op(CAST_TRUNC, idx=(U8, 0, 0, 0))]),
}


def _depth_out(which, src):
    cn, dt, _ = DEPTH_OPS[which]
    h, w = src.shape[:2]
    return np.zeros((h, w, cn) if cn > 1 else (h, w), dt)


def oracle_depth_ops(which, src, lo=0.0, hi=1.0):
    """src (H,W,cn) or (H,W) float32."""
    cn, _, make = DEPTH_OPS[which]
    out = _depth_out(which, src)
    execute([read_2d(src, cn)], make(lo, hi), [write(WRITE_2D, out, cn, src.shape[1], src.shape[0])])
    return out


def ref_depth_ops(which, src, lo=0.0, hi=1.0):
    out = _depth_out(which, src)
    rc = ref().fklref_depth_ops(which, C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0], C.c_void_p(_ptr(out)), out.strides[0],
                                C.c_float(lo), C.c_float(hi))
    assert rc == 0, rc
    return out


# ---- per-channel Operations (tests/cases/pointwise_chains.h; numpy restatement: oracle/pointwise_oracle.py) ----------

def pointwise_oracle():
    import importlib.util
    spec = importlib.util.spec_from_file_location("pointwise_oracle", os.path.join(ROOT, "oracle", "pointwise_oracle.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def ref_pointwise(which, src, c=(0, 0, 0, 0), m=(1, 0, 0, 0, 1, 0, 0, 0, 1)):
    """Chain `which` of tests/cases/pointwise_chains.h on the reference's CPU backend (or, under host_executor, on this
    repository's own CPU executor)."""
    in_dtype, cn, out_dtype = pointwise_oracle().CASES[which]
    src = np.ascontiguousarray(src, dtype=in_dtype)
    out = np.zeros(src.shape, out_dtype)
    rc = ref().fklref_pointwise(int(which), C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0], C.c_void_p(_ptr(out)),
                                out.strides[0], _f32p(np.asarray(c, np.float32)), _f32p(np.asarray(m, np.float32)))
    assert rc == 0, rc
    return out


def ref_dual(which, a, b, pad=(0, 0)):
    """Two-image chain `which` of tests/cases/pointwise_chains.h on the reference's CPU backend; `pad`: extra bytes at the end
    of the rows of the first and of the second image (the two sources have pitches of their own)."""
    in_dtype, cn, out_dtype = pointwise_oracle().DUAL_CASES[which]
    h, w = a.shape[:2]
    row = w * cn * np.dtype(in_dtype).itemsize
    bufs = []
    for img, extra in ((a, pad[0]), (b, pad[1])):
        buf = np.zeros((h, row + extra), np.uint8)
        buf[:, :row] = np.ascontiguousarray(img, dtype=in_dtype).view(np.uint8).reshape(h, row)
        bufs.append(buf)
    out = np.zeros(a.shape, out_dtype)
    rc = ref().fklref_dual(int(which), C.c_void_p(_ptr(bufs[0])), C.c_void_p(_ptr(bufs[1])), w, h, bufs[0].strides[0], bufs[1].strides[0],
                           C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


# SplitWrite chains of tests/cases/pointwise_chains.h: which -> (input dtype, channels, output dtype)
SPLIT_WRITE_CASES = {0: (np.uint8, 3, np.uint8), 1: (np.uint8, 3, np.float32), 2: (np.float32, 4, np.float32),
                     3: (np.uint8, 3, np.float32), 4: (np.float32, 2, np.float32)}


def oracle_split_write(which, src, dst=None, c=(1, 1, 1, 1)):
    """The planes SplitWrite<_2D, T> leaves: channel k of every value in image k (FK/algorithms/basic_ops/
    memory_operations.h:361-377).  Chain 1 multiplies by c first, chain 3 crops and resizes to dst = (dw, dh) first."""
    _, cn, out_dtype = SPLIT_WRITE_CASES[which]
    h, w = src.shape[:2]
    if which == 1:
        val = (src.astype(np.float32) * np.asarray(c[:3], np.float32)).astype(np.float32)
    elif which == 3:
        dw, dh = dst
        val = np.zeros((dh, dw, 3), np.float32)
        execute([read_2d(src, 3, crop=np.array([8, 4, w - 16, h - 8], np.int32), resize=(dw, dh), ar=IGNORE_AR)], [],
                [write(WRITE_2D, val, 3, dw, dh)])
    else:
        val = src
    return [np.ascontiguousarray(val[..., k]).astype(out_dtype) for k in range(cn)]


def ref_split_write(which, src, dst=None, c=(1, 1, 1, 1), pad=(0, 0, 0, 0)):
    """The same chains on the reference's CPU backend; `pad` = extra elements at the end of each output image's rows."""
    in_dtype, cn, out_dtype = SPLIT_WRITE_CASES[which]
    src = np.ascontiguousarray(src, dtype=in_dtype)
    h, w = src.shape[:2]
    dw, dh = dst if dst is not None else (w, h)
    bufs = [np.full((dh, dw + pad[k]), 0, out_dtype) for k in range(cn)]
    outs = (C.c_void_p * 4)(*[C.c_void_p(_ptr(b)) for b in bufs])
    pitches = (C.c_int * 4)(*[b.strides[0] for b in bufs])
    rc = ref().fklref_split_write(int(which), C.c_void_p(_ptr(src)), w, h, src.strides[0], dw, dh, outs, pitches,
                                  _f32p(np.asarray(c, np.float32)))
    assert rc == 0, rc
    return [np.ascontiguousarray(b[:, :dw]) for b in bufs]


# ---- transposed tensors: TensorTSplit / TensorTPack --------------------------------------------------------------------

def oracle_transposed_round_trip(images, mul, mul2):
    """images: list of (H,W,3) u8.  Returns (tensor_t (3, planes, H, W) f32, packed (planes, H, W, 3) f32): image z -> Cast ->
    Mul -> TensorTSplit into plane z, then TensorTPack -> Mul -> TensorWrite."""
    planes = len(images)
    h, w = images[0].shape[:2]
    tensor_t = np.zeros((3, planes, h, w), np.float32)
    for z, img in enumerate(images):
        view = tensor_t[:, z:]                       # plane z first; channel planes stay planes * h * w elements apart
        wr = write(TENSOR_TSPLIT, view, 3, w, h, planes, 3)
        execute([read_2d(img, 3)], [op(CAST_F32), op(MUL, [mul])], [wr])
    packed = np.zeros((planes, h, w, 3), np.float32)
    reads = []
    for z in range(planes):
        r = Read()
        r.kind, r.elem, r.cn, r.width, r.height, r.pitch = READ_PLANAR, F32, 3, w, h, w * 4
        r.data = _ptr(tensor_t[0, z])
        r.channel_stride = tensor_t.strides[0]
        reads.append(r)
    execute(reads, [op(MUL, [mul2])], [write(TENSOR_WRITE, packed, 3, w, h, planes, 1)])
    return tensor_t, packed


def ref_transposed_round_trip(images, mul, mul2):
    planes = len(images)
    h, w = images[0].shape[:2]
    tensor_t = np.zeros((3, planes, h, w), np.float32)
    packed = np.zeros((planes, h, w, 3), np.float32)
    ptrs = (C.c_void_p * planes)(*[_ptr(i) for i in images])
    rc = ref().fklref_transposed_round_trip(ptrs, planes, w, h, images[0].strides[0], C.c_float(mul), C.c_void_p(_ptr(tensor_t)), C.c_float(mul2),
                                            C.c_void_p(_ptr(packed)))
    assert rc == 0, rc
    return tensor_t, packed


def ref_circular_transposed(batch, oldest_first, images, fill):
    h, w = images[0].shape[:2]
    states = np.zeros((len(images), batch, 3, h, w), np.float32)
    ptrs = (C.c_void_p * len(images))(*[_ptr(i) for i in images])
    rc = ref().fklref_circular_transposed(batch, int(bool(oldest_first)), ptrs, len(images), w, h, images[0].strides[0], C.c_float(fill),
                                          C.c_void_p(_ptr(states)))
    assert rc == 0, rc
    return states


# ---- padding through BorderReader ---------------------------------------------------------------------------
BORDER_CONSTANT, BORDER_REPLICATE, BORDER_REFLECT, BORDER_WRAP, BORDER_REFLECT_101 = 0, 1, 2, 3, 4


def pad_kind(dtype, cn):
    """The element number of tests/cases/border_chains.h for images of `cn` channels of `dtype`."""
    return {("uint8", 3): 0, ("float32", 1): 1, ("uint8", 4): 2, ("uint16", 3): 3, ("uint8", 1): 4, ("float32", 3): 5}[(np.dtype(dtype).name, cn)]


def oracle_pad(src, border_type, left, top, out_w, out_h, value=(0, 0, 0)):
    """src (H,W,cn) or (H,W) of uint8, uint16 or float32; the output grid starts `left`/`top` pixels before the image origin."""
    cn = src.shape[2] if src.ndim == 3 else 1
    out = np.zeros((out_h, out_w, cn) if cn > 1 else (out_h, out_w), src.dtype)
    r = read_2d(src, cn, crop=(-left, -top, out_w, out_h))
    r.border = 1 + border_type
    for i, v in enumerate(value[:4]):
        r.border_value[i] = float(v)
    execute([r], [], [write(WRITE_2D, out, cn, out_w, out_h)])
    return out


def ref_pad(src, border_type, left, top, out_w, out_h, value=(0, 0, 0)):
    cn = src.shape[2] if src.ndim == 3 else 1
    out = np.zeros((out_h, out_w, cn) if cn > 1 else (out_h, out_w), src.dtype)
    v = np.zeros(4, np.float32)
    v[: len(value)] = value
    rc = ref().fklref_pad(pad_kind(src.dtype, cn), int(border_type), C.c_void_p(_ptr(src)), src.shape[1], src.shape[0], src.strides[0],
                          int(left), int(top), int(out_w), int(out_h), _f32p(v), C.c_void_p(_ptr(out)), out.strides[0])
    assert rc == 0, rc
    return out


# ---- divergent launches and the CircularTensor window -----------------------------------------------------------
# A DivergentBatchTransformDPP launch is, plane by plane, an ordinary chain (data_parallel_patterns.h:322-331): the
# helpers below pick the sequence of each plane and let the C oracle run that plane's chain.

def oracle_divergent_mixed(tensor4, mul, img):
    """tensor4 (4,h,w,3) f32; planes 0 and 3: tensor plane * mul; planes 1 and 2: img (ih,iw,3) u8 resized to (w,h)."""
    _, h, w, _ = tensor4.shape
    out = np.zeros((4, h, w, 3), np.float32)
    for z in range(4):
        if z in (0, 3):
            execute([read_2d(tensor4[z], 3)], [op(MUL, [mul])], [write(WRITE_2D, out[z], 3, w, h)])
        else:
            execute([read_2d(img, 3, resize=(w, h))], [], [write(WRITE_2D, out[z], 3, w, h)])
    return out


def ref_divergent_two(a, b, add):
    h, w = a.shape
    out = np.zeros((2, h, w), np.uint32)
    assert ref().fklref_divergent_two(C.c_void_p(_ptr(a)), C.c_void_p(_ptr(b)), w, h, a.strides[0], C.c_uint32(add), C.c_void_p(_ptr(out))) == 0
    return out


def ref_divergent_mixed(tensor4, mul, img):
    _, h, w, _ = tensor4.shape
    out = np.zeros((4, h, w, 3), np.float32)
    assert ref().fklref_divergent_mixed(C.c_void_p(_ptr(tensor4)), w, h, C.c_float(mul), C.c_void_p(_ptr(img)), img.shape[1], img.shape[0],
                                        img.strides[0], C.c_void_p(_ptr(out))) == 0
    return out


class OracleWindow:
    """CircularTensor<float, 3, batch, order, Standard> restated (circular_tensor.h:111-161): `out` is the tensor the
    caller sees (batch, 3, h, w), `temp` the hidden circular copy, whose planes hold nothing defined (NaN here)
    until an update has stored into them."""

    def __init__(self, batch, oldest_first, w, h, fill):
        self.batch, self.order, self.w, self.h = batch, int(bool(oldest_first)), w, h
        self.out = np.full((batch, 3, h, w), fill, np.float32)
        self.temp = np.full((batch, 3, h, w), np.nan, np.float32)
        self.next = 0
        lib = oracle()
        lib.fklo_circular_plane.restype = C.c_int32
        lib.fklo_circular_plane.argtypes = [C.c_int32] * 4
        lib.fklo_window_sequence.restype = C.c_int32
        lib.fklo_window_sequence.argtypes = [C.c_int32] * 3

    def update(self, img):
        """img (h,w,3) u8 -> SaturateCast<uchar3, float3> -> TensorSplit."""
        lib = oracle()
        value = np.zeros((1, 3, self.h, self.w), np.float32)
        execute([read_2d(img, 3)], [op(CAST_F32)], [write(TENSOR_SPLIT, value, 3, self.w, self.h, 1, 3)])
        read_dir = 0 if self.order == 1 else 1            # OldestFirst reads Ascendent, NewestFirst Descendent
        new = self.out.copy()
        for z in range(self.batch):
            if lib.fklo_window_sequence(self.order, self.batch, z) == 0:
                self.temp[lib.fklo_circular_plane(0, self.batch, z, self.next)] = value[0]      # MidWrite, Ascendent
                new[z] = value[0]
        for z in range(self.batch):
            if lib.fklo_window_sequence(self.order, self.batch, z) == 1:
                new[z] = self.temp[lib.fklo_circular_plane(read_dir, self.batch, z, self.next)]
        self.out = new
        self.next = (self.next + 1) % self.batch
        return self.out


def oracle_circular(batch, oldest_first, images, fill):
    """States after each update, (iters, batch, 3, h, w); planes copied from never-written hidden planes are NaN."""
    h, w = images[0].shape[:2]
    win = OracleWindow(batch, oldest_first, w, h, fill)
    return np.stack([win.update(img).copy() for img in images])


def ref_circular(batch, oldest_first, images, fill):
    h, w = images[0].shape[:2]
    states = np.zeros((len(images), batch, 3, h, w), np.float32)
    ptrs = (C.c_void_p * len(images))(*[_ptr(i) for i in images])
    rc = ref().fklref_circular(batch, int(bool(oldest_first)), ptrs, len(images), w, h, images[0].strides[0], C.c_float(fill), C.c_void_p(_ptr(states)))
    assert rc == 0, rc
    return states

"""Python handle on the benchmark chains spelled with the C++ host API (tests/cases/fkl_cases.cpp).

Each function takes torch CUDA tensors (device memory only -- torch is plumbing here), enqueues ONE fused kernel
through executeOperations<TransformDPP<>> on torch's current stream and returns without synchronising.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from fusedkernellibrary_amd import ROOT_DIR, lib

CASES_SO = os.path.join(ROOT_DIR, "tests", "cases", "libfkl_cases.so")
_cases = None


def cases() -> C.CDLL:
    global _cases
    if _cases is None:
        lib()  # the C-ABI library first, so its symbols resolve
        if not os.path.exists(CASES_SO):
            raise RuntimeError(f"{CASES_SO} is missing: run __graft_entry__.build()")
        c = C.CDLL(CASES_SO)
        c.fklcase_last_error.restype = C.c_char_p
        c.fklcase_timed_start_ns.restype = C.c_longlong
        c.fklcase_time_next.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        _cases = c
    return _cases


def _ok(rc: int) -> None:
    if rc == 2:
        raise RuntimeError("the case driver has no chain for this combination of arguments (see tests/cases/*_chains.h)")
    if rc != 0:
        raise RuntimeError(cases().fklcase_last_error().decode())


def set_reps(reps: int) -> None:
    """The next chain call enqueues its kernel `reps` times back to back through the C++ host API."""
    cases().fklcase_set_reps(int(reps))


def time_next(stream, first_event, last_event) -> None:
    """The next chain call records `first_event` on `stream` before its first launch and `last_event` after its last."""
    cases().fklcase_time_next(stream, first_event, last_event)


def timed_start_ns() -> int:
    """CLOCK_MONOTONIC (nanoseconds) at the start of the last chain call that was timed with time_next."""
    return int(cases().fklcase_timed_start_ns())


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(t.data_ptr())


def _host(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def crop_resize_par_u8(src, rects, dst, bg, mul, sub, out):
    """src (H,W,3) u8 cuda; rects (5,4) int32 host; out (5,dh,dw,3) u8 cuda."""
    assert len(rects) == 5
    r, b, m, s = _host(rects, np.int32), _host(bg, np.float32), _host(mul, np.float32), _host(sub, np.float32)
    _ok(cases().fklcase_crop_resize_par_u8_b5(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0),
                                              r.ctypes.data_as(C.c_void_p), int(dst[0]), int(dst[1]),
                                              b.ctypes.data_as(C.c_void_p), m.ctypes.data_as(C.c_void_p),
                                              s.ctypes.data_as(C.c_void_p), _p(out)))


def crop_resize_norm_split(src, rects, dst, sub, div, out):
    """src (H,W,3) u8 cuda; rects (B,4) int32 host, B in {8,64}; out (B,3,dh,dw) f32 cuda."""
    fn = {8: "fklcase_crop_resize_norm_split_b8", 64: "fklcase_crop_resize_norm_split_b64"}[len(rects)]
    r, s, d = _host(rects, np.int32), _host(sub, np.float32), _host(div, np.float32)
    _ok(getattr(cases(), fn)(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0), r.ctypes.data_as(C.c_void_p),
                             int(dst[0]), int(dst[1]), s.ctypes.data_as(C.c_void_p), d.ctypes.data_as(C.c_void_p), _p(out)))


def batch_muladd_sat(srcs, mul, add, outs):
    """srcs/outs: lists of B (H,W,3) u8 cuda tensors, B in {4,100}; mul/add (B,3) f32 host."""
    b = len(srcs)
    fn = {4: "fklcase_batch_muladd_sat_b4", 100: "fklcase_batch_muladd_sat_b100"}[b]
    m, a = _host(mul, np.float32), _host(add, np.float32)
    sp = (C.c_void_p * b)(*[s.data_ptr() for s in srcs])
    op = (C.c_void_p * b)(*[o.data_ptr() for o in outs])
    _ok(getattr(cases(), fn)(_stream(), sp, srcs[0].shape[1], srcs[0].shape[0], srcs[0].stride(0),
                             m.ctypes.data_as(C.c_void_p), a.ctypes.data_as(C.c_void_p), op, outs[0].stride(0)))


def add_mul_chain(src, n_ops, addv, mulv, out, tf=0):
    """src/out (H,W) f32 cuda."""
    _ok(cases().fklcase_add_mul_chain(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4, int(n_ops),
                                      C.c_float(float(addv)), C.c_float(float(mulv)), _p(out), out.stride(0) * 4, int(tf)))


def nv12_rgb_resize_split(nv12, width, height, dst, scale, out):
    """nv12 (H*3/2, W) u8 cuda; out (3,dh,dw) f32 cuda."""
    _ok(cases().fklcase_nv12_rgb_resize_split(_stream(), _p(nv12), int(width), int(height), nv12.stride(0), int(dst[0]),
                                              int(dst[1]), C.c_float(float(scale)), _p(out)))


def crop_swap_u8(src, rects, out):
    assert len(rects) == 4
    r = _host(rects, np.int32)
    _ok(cases().fklcase_crop_swap_u8_b4(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0),
                                        r.ctypes.data_as(C.c_void_p), _p(out)))


def copy_f32(src, out):
    """src/out (H,W) f32 cuda: read -> write with no compute operation."""
    _ok(cases().fklcase_copy_f32(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4, _p(out), out.stride(0) * 4))


def div_f32(src, d, out):
    """src/out (H,W) f32 cuda: out = src / d through Read -> Div -> Write."""
    _ok(cases().fklcase_div_f32(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4, C.c_float(float(d)),
                                _p(out), out.stride(0) * 4))


def normalise_mode(kind, sub, div) -> int:
    """fkd::Div's mode word for (x - sub) / div behind a bounded read (kind 0), a float image (1), a letterboxed resize (2):
    low two bits as div_mode, bit 2 set when the chain proves the range and the device skips its per-element test."""
    return int(cases().fklcase_normalise_mode(int(kind), _host(sub, np.float32).ctypes.data_as(C.POINTER(C.c_float)),
                                              _host(div, np.float32).ctypes.data_as(C.POINTER(C.c_float))))


def div_mode(d) -> int:
    """0 generic division, 1 five-instruction sequence, 2 two-instruction sequence proven exact for this divisor."""
    l = cases()
    l.fklcase_div_mode.argtypes = [C.c_float]
    return int(l.fklcase_div_mode(C.c_float(d)))


def div_f32_forced(src, d, mode, out):
    """Read2D<float> -> Div(d) -> Write2D<float> with the division sequence given by the caller (see div_mode)."""
    h, w = src.shape
    _ok(cases().fklcase_div_f32_forced(_stream(), _p(src), w, h, src.stride(0) * 4, C.c_float(float(d)), int(mode), _p(out),
                                       out.stride(0) * 4))


def div_f32x3(src, d, out):
    """src/out (H,W,3) f32 cuda, d three divisors (one per channel)."""
    dd = _host(d, np.float32)
    _ok(cases().fklcase_div_f32x3(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4,
                                  dd.ctypes.data_as(C.c_void_p), _p(out), out.stride(0) * 4))


def saturate_f32_u8(src, out):
    """src (H,W) f32 cuda, out (H,W) u8 cuda: SaturateCast<float, uchar>."""
    _ok(cases().fklcase_saturate_f32_u8(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4, _p(out), out.stride(0)))


def crop_resize_default_norm_split(src, rects, dst, used, default, sub, div, out):
    """Configuration-3 chain on 8 crops with BatchRead<CONDITIONAL_WITH_DEFAULT>: planes >= used yield `default`."""
    assert len(rects) == 8
    r, d, s, v = _host(rects, np.int32), _host(default, np.float32), _host(sub, np.float32), _host(div, np.float32)
    _ok(cases().fklcase_crop_resize_default_norm_split_b8(
        _stream(), _p(src), src.shape[1], src.shape[0], src.stride(0), r.ctypes.data_as(C.c_void_p), int(dst[0]), int(dst[1]),
        int(used), d.ctypes.data_as(C.c_void_p), s.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p), _p(out)))


def batch_default_cast_mul(srcs, active, default, mul, out):
    """4 (H,W,3) u8 cuda images, planes >= active yield `default` (3 bytes); out (4,H,W,3) f32 cuda."""
    assert len(srcs) == 4
    sp = (C.c_void_p * 4)(*[s.data_ptr() for s in srcs])
    d, m = _host(default, np.uint8), _host(mul, np.float32)
    _ok(cases().fklcase_batch_default_cast_mul_b4(_stream(), sp, srcs[0].shape[1], srcs[0].shape[0], srcs[0].stride(0), int(active),
                                                  d.ctypes.data_as(C.c_void_p), m.ctypes.data_as(C.c_void_p), _p(out)))


def set_and_loop_f32(n, init, add, iterations):
    """setTo(init) on a library-owned 1-D float array, StaticLoop<Add<float>, iterations>(add), download: (n,) f32."""
    out = np.empty(n, np.float32)
    _ok(cases().fklcase_set_and_loop_f32(_stream(), int(n), C.c_float(float(init)), C.c_float(float(add)), int(iterations),
                                         out.ctypes.data_as(C.c_void_p)))
    return out


def set_to_transposed(w, h, planes, color_planes, sentinel, value):
    """setTo on a TensorT<float> that held `sentinel` everywhere; returns the device copy, (color_planes * planes, h, w) f32."""
    out = np.zeros((color_planes * planes, h, w), np.float32)
    _ok(cases().fklcase_set_to_transposed(_stream(), int(w), int(h), int(planes), int(color_planes), C.c_float(float(sentinel)),
                                          C.c_float(float(value)), out.ctypes.data_as(C.c_void_p)))
    return out


def set_to_shapes(w, h, planes, v3, vf):
    """setTo on a pitched (h,w) uchar3 image and a (planes,h,w) float tensor; returns (image rows incl. pitch, pitch, tensor)."""
    img = np.zeros(h * (w * 3 + 1024), np.uint8)
    pitch = C.c_int(0)
    ten = np.empty((planes, h, w), np.float32)
    v = _host(v3, np.uint8)
    _ok(cases().fklcase_set_to_shapes(_stream(), int(w), int(h), int(planes), v.ctypes.data_as(C.c_void_p), C.c_float(float(vf)),
                                      img.ctypes.data_as(C.c_void_p), C.byref(pitch), ten.ctypes.data_as(C.c_void_p)))
    return img[: pitch.value * h].reshape(h, pitch.value), pitch.value, ten


def uncompiled_pointwise_f32(src, out):
    """(H,W) f32 cuda: ((x*1.5 - 0.25) / 3) + 7 -- a chain that is not in the ahead-of-time list."""
    _ok(cases().fklcase_uncompiled_pointwise_f32(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4, _p(out), out.stride(0) * 4))


def uncompiled_gray_resize(src, rect, dst, mul, out):
    """(H,W) u8 cuda -> crop -> bilinear (dst = (w,h)) -> * mul -> out (dh,dw) f32 cuda."""
    r = _host(rect, np.int32)
    _ok(cases().fklcase_uncompiled_gray_resize(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0), r.ctypes.data_as(C.c_void_p),
                                               int(dst[0]), int(dst[1]), C.c_float(float(mul)), _p(out), out.stride(0) * 4))


def uncompiled_letterbox_split_b3(src, rects, dst, bg, mul, out):
    """(H,W,3) u8 cuda, 3 crops -> letterboxed bilinear (dst = (w,h)) -> * mul -> out (3,3,dh,dw) f32 cuda."""
    r, b, m = _host(rects, np.int32), _host(bg, np.float32), _host(mul, np.float32)
    _ok(cases().fklcase_uncompiled_letterbox_split_b3(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0),
                                                      r.ctypes.data_as(C.c_void_p), int(dst[0]), int(dst[1]),
                                                      b.ctypes.data_as(C.c_void_p), m.ctypes.data_as(C.c_void_p), _p(out)))


def uncompiled_resize_split(kind, src, rect, dst, mul, out):
    """kind 0: (H,W,2) u8, 1: (H,W,4) u8, 2: (H,W,3) u16 cuda -> crop -> bilinear (dst = (w,h)) -> * mul -> out (cn,dh,dw) f32 cuda."""
    r = _host(rect, np.int32)
    _ok(cases().fklcase_uncompiled_resize_split(_stream(), int(kind), _p(src), src.shape[1], src.shape[0], src.stride(0) * src.element_size(),
                                                r.ctypes.data_as(C.c_void_p), int(dst[0]), int(dst[1]), C.c_float(float(mul)), _p(out)))


def uncompiled_float4_resize(src, dst, out):
    """(H,W,4) f32 cuda -> bilinear -> out (dh,dw,4) f32 cuda."""
    _ok(cases().fklcase_uncompiled_float4_resize(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * 4, int(dst[0]), int(dst[1]),
                                                 _p(out), out.stride(0) * 4))


def warp(src, matrix, perspective, dst, out, kind=None):
    """src (H,W,3) u8 or (H,W) f32 cuda; matrix 2x3 (affine) or 3x3 (perspective); out (dh,dw,3) / (dh,dw) f32 cuda.
    `kind`: 2 (H,W,4) u8, 3 (H,W,3) u16 travelling as int16, 4 (H,W) u8 -- chains compiled on first use."""
    m = np.zeros(9, np.float32)
    m[: (9 if perspective else 6)] = np.asarray(matrix, np.float32).ravel()
    if kind is not None:
        _ok(cases().fklcase_warp_kind(_stream(), int(kind), _p(src), src.shape[1], src.shape[0], src.stride(0) * src.element_size(),
                                      m.ctypes.data_as(C.c_void_p), int(bool(perspective)), int(dst[0]), int(dst[1]), _p(out), out.stride(0) * 4))
        return
    is_u8 = src.element_size() == 1
    fn = cases().fklcase_warp_u8x3 if is_u8 else cases().fklcase_warp_f32
    esz = 1 if is_u8 else 4
    _ok(fn(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * esz, m.ctypes.data_as(C.c_void_p), int(bool(perspective)),
           int(dst[0]), int(dst[1]), _p(out), out.stride(0) * 4))


def deinterlace(src, mode, out):
    """src (H,W,3) u8 or (H,W) f32 cuda; mode 1 BLEND, 2 INTER_LINEAR keeping even lines, 3 keeping odd; out f32 same shape."""
    is_u8 = src.element_size() == 1
    fn = cases().fklcase_deinterlace_u8x3 if is_u8 else cases().fklcase_deinterlace_f32
    _ok(fn(_stream(), _p(src), src.shape[1], src.shape[0], src.stride(0) * (1 if is_u8 else 4), int(mode), _p(out), out.stride(0) * 4))


# ---- pixel formats and colour conversions (tests/cases/color_chains.h) ------------------------------------
# pf / cd / cr / cp are the enumerator values of fk::PixelFormat, ColorDepth, ColorRange and ColorPrimitives.

def _pitch(t):
    return t.stride(0) * t.element_size()


def yuv_to_rgb(pf, cr, cp, frame, width, height, out):
    """frame: 2-D u8/i16 cuda tensor holding a width x height frame in pixel format pf; out (H,W,3) f32 cuda."""
    _ok(cases().fklcase_yuv_to_rgb(_stream(), int(pf), int(cr), int(cp), _p(frame), int(width), int(height), _pitch(frame), _p(out), _pitch(out)))


def rgb_to_yuv(pf, cr, cp, rgb, frame):
    """rgb (H,W,3) u8/i16 cuda; frame: 2-D cuda tensor the chain stores the pixel-format frame into."""
    _ok(cases().fklcase_rgb_to_yuv(_stream(), int(pf), int(cr), int(cp), _p(rgb), rgb.shape[1], rgb.shape[0], _pitch(rgb), _p(frame), _pitch(frame)))


def yuv_resize(pf, frame, width, height, dst, scale, out):
    """ReadYUV -> ConvertYUVToRGB -> bilinear resize to dst = (w, h) -> * scale; out (dh,dw,3) f32 cuda."""
    _ok(cases().fklcase_yuv_resize(_stream(), int(pf), _p(frame), int(width), int(height), _pitch(frame), int(dst[0]), int(dst[1]),
                                   C.c_float(float(scale)), _p(out), _pitch(out)))


def convert_depth(cd, cr, cp, to_rgb, src, out):
    """src (H,W,3) u8/i16/f32 cuda pixels of depth cd -> ConvertYUVToRGB or ConvertRGBToYUV -> out (H,W,3) f32 cuda."""
    _ok(cases().fklcase_convert_depth(_stream(), int(cd), int(cr), int(cp), int(bool(to_rgb)), _p(src), src.shape[1], src.shape[0], _pitch(src),
                                      _p(out), _pitch(out)))


def convert_code(which, src, out):
    """ColorConversion<code> number `which` of the list in tests/cases/color_chains.h."""
    _ok(cases().fklcase_convert_code(_stream(), int(which), _p(src), src.shape[1], src.shape[0], _pitch(src), _p(out), _pitch(out)))


def normalize(which, src, out):
    """NormalizePixel<uchar3, p8bit> (which = 0) or <ushort3, p10bit> (which = 1); out (H,W,3) f32 cuda."""
    _ok(cases().fklcase_normalize(_stream(), int(which), _p(src), src.shape[1], src.shape[0], _pitch(src), _p(out), _pitch(out)))


def depth_ops(which, src, out, lo=0.0, hi=1.0):
    """Operation number `which` of depth_ops in tests/cases/color_chains.h on src (H,W[,cn]) f32 cuda -> out cuda."""
    _ok(cases().fklcase_depth_ops(_stream(), int(which), _p(src), src.shape[1], src.shape[0], _pitch(src), _p(out), _pitch(out),
                                  C.c_float(float(lo)), C.c_float(float(hi))))


def letterbox_ar(ar, src, rect, bg, out):
    """src (H,W,3) u8 cuda -> Crop(rect = x, y, w, h) -> Resize<INTER_LINEAR, ar>(out's size, bg) -> out (dh,dw,3) f32 cuda;
    ar: 0 PRESERVE_AR, 2 PRESERVE_AR_RN_EVEN, 3 PRESERVE_AR_LEFT."""
    r = _host(rect, np.int32)
    b = _host(bg, np.float32)
    _ok(cases().fklcase_letterbox_ar(_stream(), int(ar), _p(src), src.shape[1], src.shape[0], _pitch(src), r.ctypes.data_as(C.c_void_p),
                                     out.shape[1], out.shape[0], b.ctypes.data_as(C.c_void_p), _p(out), _pitch(out)))


def pointwise(which, src_bytes, width, height, out_bytes, c=(0, 0, 0, 0), m=(1, 0, 0, 0, 1, 0, 0, 0, 1)):
    """Chain number `which` of tests/cases/pointwise_chains.h.  src_bytes / out_bytes: 2-D u8 cuda tensors holding `height`
    rows of `width` elements of the chain's input / output type (a row may be longer than its elements: the pitch)."""
    cv = np.ascontiguousarray(c, dtype=np.float32)
    mv = np.ascontiguousarray(m, dtype=np.float32)
    _ok(cases().fklcase_pointwise(_stream(), int(which), _p(src_bytes), int(width), int(height), _pitch(src_bytes), _p(out_bytes),
                                  _pitch(out_bytes), cv.ctypes.data_as(C.c_void_p), mv.ctypes.data_as(C.c_void_p)))


def split_write(which, src_bytes, width, height, outs, dst=None, c=(1, 1, 1, 1)):
    """SplitWrite chain number `which` of tests/cases/pointwise_chains.h.  src_bytes: 2-D u8 cuda tensor holding the input
    image's rows; outs: one 2-D cuda tensor per channel (each may have a pitch of its own); dst = (dw, dh) for chain 3."""
    dw, dh = dst if dst is not None else (width, height)
    ptrs = (C.c_void_p * 4)(*[C.c_void_p(o.data_ptr()) for o in outs])
    pitches = (C.c_int * 4)(*[_pitch(o) for o in outs])
    cv = np.ascontiguousarray(c, dtype=np.float32)
    _ok(cases().fklcase_split_write(_stream(), int(which), _p(src_bytes), int(width), int(height), _pitch(src_bytes), int(dw), int(dh),
                                    ptrs, pitches, cv.ctypes.data_as(C.c_void_p)))


def dual(which, a_bytes, b_bytes, width, height, out_bytes):
    """Two-image chain number `which` of tests/cases/pointwise_chains.h; the three arguments are 2-D u8 cuda tensors holding
    the rows of the two inputs and of the output (each with a pitch of its own)."""
    _ok(cases().fklcase_dual(_stream(), int(which), _p(a_bytes), _p(b_bytes), int(width), int(height), _pitch(a_bytes), _pitch(b_bytes),
                             _p(out_bytes), _pitch(out_bytes)))


def pad(src, border_type, left, top, out, value=(0, 0, 0), kind=None):
    """src (H,W,3) u8 or (H,W) f32 cuda -> BorderReader<border_type> -> Crop starting `left`/`top` pixels before the origin -> out.
    `kind`: the element number of border_chains.h for other pixel types (uint16 images travel as int16 tensors)."""
    v = np.zeros(4, np.float32)
    v[: len(value)] = value
    if kind is None:
        kind = 0 if src.element_size() == 1 else 1
    _ok(cases().fklcase_pad(_stream(), int(kind), int(border_type), _p(src), src.shape[1], src.shape[0], _pitch(src),
                            int(left), int(top), out.shape[1], out.shape[0], v.ctypes.data_as(C.c_void_p), _p(out), _pitch(out)))


# ---- divergent launches and the CircularTensor window (tests/cases/circular_chains.h) -------------------------------

def divergent_two(a, b, add, out):
    """a, b (H,W) i32-typed cuda tensors holding uint32; out (2,H,W): plane 0 = a + add, plane 1 = b, in ONE launch."""
    _ok(cases().fklcase_divergent_two(_stream(), _p(a), _p(b), a.shape[1], a.shape[0], _pitch(a), C.c_uint32(int(add)), _p(out)))


def divergent_mixed(tensor4, mul, img, out):
    """tensor4 (4,H,W,3) f32 cuda, img (ih,iw,3) u8 cuda, out (4,H,W,3) f32 cuda: planes 0,3 = tensor4 * mul, planes 1,2 = img resized."""
    _ok(cases().fklcase_divergent_mixed(_stream(), _p(tensor4), tensor4.shape[2], tensor4.shape[1], C.c_float(float(mul)), _p(img), img.shape[1],
                                        img.shape[0], _pitch(img), _p(out)))


def circular(batch, oldest_first, images, fill):
    """images: list of (H,W,3) u8 cuda tensors fed one by one to CircularTensor::update; returns the tensor after each update,
    (iters, batch, 3, H, W) float32 on the host."""
    h, w = images[0].shape[:2]
    states = np.zeros((len(images), batch, 3, h, w), np.float32)
    ptrs = (C.c_void_p * len(images))(*[i.data_ptr() for i in images])
    _ok(cases().fklcase_circular(_stream(), int(batch), int(bool(oldest_first)), ptrs, len(images), w, h, _pitch(images[0]), C.c_float(float(fill)),
                                 states.ctypes.data_as(C.c_void_p)))
    return states


def transposed_round_trip(images, mul, tensor_t, mul2, packed):
    """images: list of (H,W,3) u8 cuda; tensor_t (3, planes, H, W) f32 cuda; packed (planes, H, W, 3) f32 cuda."""
    h, w = images[0].shape[:2]
    ptrs = (C.c_void_p * len(images))(*[i.data_ptr() for i in images])
    _ok(cases().fklcase_transposed_round_trip(_stream(), ptrs, len(images), w, h, _pitch(images[0]), C.c_float(float(mul)), _p(tensor_t),
                                              C.c_float(float(mul2)), _p(packed)))


def circular_transposed(batch, oldest_first, images, fill):
    """circular() with ColorPlanes::Transposed and TensorTSplit; same result layout."""
    h, w = images[0].shape[:2]
    states = np.zeros((len(images), batch, 3, h, w), np.float32)
    ptrs = (C.c_void_p * len(images))(*[i.data_ptr() for i in images])
    _ok(cases().fklcase_circular_transposed(_stream(), int(batch), int(bool(oldest_first)), ptrs, len(images), w, h, _pitch(images[0]),
                                            C.c_float(float(fill)), states.ctypes.data_as(C.c_void_p)))
    return states


def circular_update_b8(images, release=False):
    """One CircularTensor<float,3,8,NewestFirst>::update per repetition (set_reps), cycling through `images` ((H,W,3) u8 cuda)."""
    h, w = images[0].shape[:2]
    ptrs = (C.c_void_p * len(images))(*[i.data_ptr() for i in images])
    _ok(cases().fklcase_circular_update_b8(_stream(), ptrs, len(images), w, h, _pitch(images[0]), int(bool(release))))

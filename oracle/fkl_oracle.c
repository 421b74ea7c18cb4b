/*
 * fkl_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE (see fkl_oracle.h).
 *
 * Plain-C restatement of FKL's fused data-parallel path on its CPU backend.
 * Reference paths are relative to the reference root; FK/ = include/fused_kernel/.
 */
#include "fkl_oracle.h"

#include <math.h>
#include <string.h>

/* One value travelling through the chain: uchar, ushort or float channels. */
typedef struct {
    int elem; /* FKLO_U8 / FKLO_F32 / FKLO_U16 */
    int cn;
    float f[4];
    uint8_t u[4];
    uint16_t h[4];
} fklo_val;

/* ---- scalar helpers ---------------------------------------------------- */

/* cxp::round, FK/core/constexpr_libs/constexpr_cmath.h:354-385: half away from
 * zero (std::round at run time). Used on the host for letterbox sizes. */
float fklo_round_half_away(float s) {
    if (s != s || isinf(s) || s == 0.0f) return s;
    const float a = s < 0.0f ? -s : s;
    if (a >= 8388608.0f) return s;
    const float t = (float)(int)a;
    const float r = (a - t) >= 0.5f ? t + 1.0f : t;
    return s < 0.0f ? -r : r;
}

/* cxp::banker_round, FK/core/constexpr_libs/constexpr_saturate.h:28-66:
 * truncate |u|, look at the exact remainder, push odd ties up. */
float fklo_banker_round(float u) {
    if (u != u) return u;
    const int neg = u < 0.0f;
    const float a = neg ? -u : u;
    if (a >= 9007199254740992.0f) return u;
    long long i = (long long)a;
    const float diff = a - (float)i;
    if (diff > 0.5f) {
        i += 1;
    } else if (diff >= 0.5f) {
        if (i % 2 != 0) i += 1;
    }
    const float r = (float)i;
    return neg ? -r : r;
}

/* cxp::saturate_cast<uchar>(float), FK/core/constexpr_libs/constexpr_saturate.h:91-113
 * via SaturateCast<I,O>, FK/algorithms/image_processing/saturate.h:25-36. */
uint8_t fklo_saturate_cast_u8(float s) {
    if (s != s) return 0;
    const float r = fklo_banker_round(s);
    if (r >= 255.0f) return 255;
    if (r <= 0.0f) return 0;
    return (uint8_t)r;
}

uint16_t fklo_saturate_cast_u16(float s) {
    if (s != s) return 0;
    const float r = fklo_banker_round(s);
    if (r >= 65535.0f) return 65535;
    if (r <= 0.0f) return 0;
    return (uint16_t)r;
}

/* maxDepthValue, subCoefficients, rangeLimits: FK/algorithms/image_processing/itu_color.h:103-183.  The normalised
 * float depths divide the integer constants by the integer depth's largest value, in binary32. */
typedef struct { float max_v, luma, chroma, limit_y, limit_c; } depth_consts;
static int depth_constants(int depth, depth_consts *d) {
    static const float tab[3][5] = {
        {255.0f, 16.0f, 128.0f, 219.0f, 224.0f},
        {1023.0f, 64.0f, 512.0f, 876.0f, 896.0f},
        {4095.0f, 256.0f, 2048.0f, 3504.0f, 3584.0f}};
    if (depth < 0 || depth > 5) return FKLO_EINVAL;
    const float *t = tab[depth % 3];
    if (depth < 3) {
        d->max_v = t[0]; d->luma = t[1]; d->chroma = t[2]; d->limit_y = t[3]; d->limit_c = t[4];
    } else {
        d->max_v = 1.0f; d->luma = t[1] / t[0]; d->chroma = t[2] / t[0]; d->limit_y = t[3] / t[0]; d->limit_c = t[4] / t[0];
    }
    return FKLO_OK;
}
int fklo_depth_constants(int32_t depth, float *max_value, float *luma_offset, float *chroma_offset) {
    depth_consts d;
    if (depth_constants(depth, &d)) return FKLO_EINVAL;
    *max_value = d.max_v; *luma_offset = d.luma; *chroma_offset = d.chroma;
    return FKLO_OK;
}

/* computeMatrix<CR, CP, direction, CD>, FK/algorithms/image_processing/itu_color.h:185-265, with the luma weights
 * of itu_color.h:150-158.  All arithmetic in binary32, same expression order; limited range scales the luma and
 * chroma columns (to RGB) or rows (to YCbCr). */
int fklo_color_matrix(int32_t depth, int32_t range, int32_t primaries, int32_t to_rgb, float m[9]) {
    static const float kr[3] = {0.299f, 0.2126f, 0.2627f}, kb[3] = {0.114f, 0.0722f, 0.0593f};
    depth_consts d;
    if (depth_constants(depth, &d) || primaries < 0 || primaries > 2 || (range != FKLO_LIMITED && range != FKLO_FULL))
        return FKLO_EINVAL;
    const float Kr = kr[primaries], Kb = kb[primaries];
    const float Kg = 1.0f - Kr - Kb;
    if (to_rgb) {
        m[0] = 1.0f; m[1] = 0.0f;                           m[2] = 2.0f * (1.0f - Kr);
        m[3] = 1.0f; m[4] = -2.0f * Kb * (1.0f - Kb) / Kg;  m[5] = -2.0f * Kr * (1.0f - Kr) / Kg;
        m[6] = 1.0f; m[7] = 2.0f * (1.0f - Kb);             m[8] = 0.0f;
        if (range == FKLO_LIMITED) {
            const float scale_y = d.max_v / d.limit_y, scale_c = d.max_v / d.limit_c;
            for (int r = 0; r < 3; ++r) { m[3 * r] *= scale_y; m[3 * r + 1] *= scale_c; m[3 * r + 2] *= scale_c; }
        }
    } else {
        m[0] = Kr;                          m[1] = Kg;                          m[2] = Kb;
        m[3] = -Kr / (2.0f * (1.0f - Kb));  m[4] = -Kg / (2.0f * (1.0f - Kb));  m[5] = 0.5f;
        m[6] = 0.5f;                        m[7] = -Kg / (2.0f * (1.0f - Kr));  m[8] = -Kb / (2.0f * (1.0f - Kr));
        if (range == FKLO_LIMITED) {
            const float scale_y = d.limit_y / d.max_v, scale_c = d.limit_c / d.max_v;
            for (int i = 0; i < 3; ++i) { m[i] *= scale_y; m[3 + i] *= scale_c; m[6 + i] *= scale_c; }
        }
    }
    return FKLO_OK;
}

/* computeMatrix<Full, bt709, YCbCr2RGB, p8bit>, FK/algorithms/image_processing/itu_color.h:185-265.
 * All arithmetic in binary32, same expression order. */
void fklo_yuv2rgb_709_full_matrix(float m[9]) {
    const float Kr = 0.2126f, Kb = 0.0722f;
    const float Kg = 1.0f - Kr - Kb;
    m[0] = 1.0f; m[1] = 0.0f;                           m[2] = 2.0f * (1.0f - Kr);
    m[3] = 1.0f; m[4] = -2.0f * Kb * (1.0f - Kb) / Kg;  m[5] = -2.0f * Kr * (1.0f - Kr) / Kg;
    m[6] = 1.0f; m[7] = 2.0f * (1.0f - Kb);             m[8] = 0.0f;
}

/* ConvertYUVToRGB<p8bit,Full,bt709>::exec, FK/algorithms/image_processing/color_conversion.h:150-174,
 * MxVFloat3<UnaryType>::exec, FK/algorithms/basic_ops/algebraic.h:50-55: per row three
 * products then (a + b) + c; chroma offset 128 (itu_color.h:120-121); no clamp. */
void fklo_yuv2rgb_709_full(const uint8_t yuv[3], float rgb[3]) {
    float m[9];
    fklo_yuv2rgb_709_full_matrix(m);
    const float v0 = (float)yuv[0];
    const float v1 = (float)yuv[1] - 128.0f;
    const float v2 = (float)yuv[2] - 128.0f;
    for (int r = 0; r < 3; ++r) {
        const float a = v0 * m[3 * r + 0];
        const float b = v1 * m[3 * r + 1];
        const float c = v2 * m[3 * r + 2];
        rgb[r] = (a + b) + c;
    }
}

/* InterpolateComplete<INTER_LINEAR>::exec, FK/algorithms/image_processing/interpolation.h:70-104:
 * weights from the UNCLAMPED x2,y2; each weight one product of two differences;
 * the four terms summed left to right. */
float fklo_bilinear(float p00, float p10, float p01, float p11, float sx, float sy) {
    const int x1 = (int)floorf(sx), y1 = (int)floorf(sy);
    const int x2 = x1 + 1, y2 = y1 + 1;
    const float w00 = ((float)x2 - sx) * ((float)y2 - sy);
    const float w10 = (sx - (float)x1) * ((float)y2 - sy);
    const float w01 = ((float)x2 - sx) * (sy - (float)y1);
    const float w11 = (sx - (float)x1) * (sy - (float)y1);
    return ((p00 * w00 + p10 * w10) + p01 * w01) + p11 * w11;
}

/* Resize<...>::build(backIOp, dstSize, bg) and compute_target_size,
 * FK/algorithms/image_processing/resize.h:164-233 (the three PRESERVE_AR modes) and :266-278 (IGNORE_AR).
 * Factors are computed in double on the host and narrowed once.  PRESERVE_AR_RN_EVEN (:212-221) makes the width the
 * even number at or below the rounded one (or, when that exceeds the destination, the height likewise);
 * PRESERVE_AR_LEFT (:177-191) puts the picture at the left edge instead of centring it. */
void fklo_compute_resize_params(int32_t src_w, int32_t src_h, int32_t dst_w, int32_t dst_h,
                                int32_t ar, fklo_resize_params *out) {
    out->dst_w = dst_w;
    out->dst_h = dst_h;
    if (ar == FKLO_IGNORE_AR) {
        const double cfx = (double)dst_w / (double)src_w;
        const double cfy = (double)dst_h / (double)src_h;
        out->fx = (float)(1.0 / cfx);
        out->fy = (float)(1.0 / cfy);
        out->x1 = 0; out->y1 = 0; out->x2 = dst_w - 1; out->y2 = dst_h - 1;
        return;
    }
    const float scale = (float)dst_h / (float)src_h;
    int tw = (int)fklo_round_half_away(scale * (float)src_w);
    int th = dst_h;
    if (ar == FKLO_PRESERVE_AR_RN_EVEN) tw -= tw % 2;
    if (tw > dst_w) {
        const float scale2 = (float)dst_w / (float)src_w;
        tw = dst_w;
        th = (int)fklo_round_half_away(scale2 * (float)src_h);
        if (ar == FKLO_PRESERVE_AR_RN_EVEN) th -= th % 2;
    }
    const double cfx = (double)tw / (double)src_w;
    const double cfy = (double)th / (double)src_h;
    out->fx = (float)(1.0 / cfx);
    out->fy = (float)(1.0 / cfy);
    out->x1 = ar == FKLO_PRESERVE_AR_LEFT ? 0 : (dst_w - tw) / 2;
    out->y1 = (dst_h - th) / 2;
    out->x2 = out->x1 + tw - 1;
    out->y2 = out->y1 + th - 1;
}

/* ---- ops on values ----------------------------------------------------- */

static float chan_as_float(const fklo_val *v, int c) {
    return v->elem == FKLO_F32 ? v->f[c] : (v->elem == FKLO_U16 ? (float)v->h[c] : (float)v->u[c]);
}

/* MxVFloat3<UnaryType>::exec, FK/algorithms/basic_ops/algebraic.h:42-56: per row three products, (a + b) + c. */
static void mxv3(const float m[9], const float v[3], float out[3]) {
    for (int r = 0; r < 3; ++r) {
        const float a = v[0] * m[3 * r + 0];
        const float b = v[1] * m[3 * r + 1];
        const float c = v[2] * m[3 * r + 2];
        out[r] = (a + b) + c;
    }
}
static int depth_elem(int depth) { return depth == FKLO_P8 ? FKLO_U8 : (depth <= FKLO_P12 ? FKLO_U16 : FKLO_F32); }

/* Add/Sub/Mul/Div<I,P,O,BinaryType>::exec, FK/algorithms/basic_ops/arithmetic.h:26-124 with the
 * channel-wise operators of FK/core/utils/vector_utils.h:508-563 (uchar op float -> float);
 * VectorReorder, FK/algorithms/basic_ops/vector_ops.h:43-56; Cast, FK/algorithms/basic_ops/cast.h:22-33. */
static int apply_op(const fklo_op *op, fklo_val *v) {
    switch (op->code) {
    case FKLO_MUL: case FKLO_ADD: case FKLO_SUB: case FKLO_DIV: {
        for (int c = 0; c < v->cn; ++c) {
            const float a = chan_as_float(v, c), p = op->p[c];
            float r;
            if (op->code == FKLO_MUL) r = a * p;
            else if (op->code == FKLO_ADD) r = a + p;
            else if (op->code == FKLO_SUB) r = a - p;
            else r = a / p;
            v->f[c] = r;
        }
        v->elem = FKLO_F32;
        return FKLO_OK;
    }
    case FKLO_REORDER: {
        fklo_val t = *v;
        for (int c = 0; c < v->cn; ++c) {
            const int s = op->idx[c];
            if (s < 0 || s >= v->cn) return FKLO_EINVAL;
            v->f[c] = t.f[s];
            v->u[c] = t.u[s];
            v->h[c] = t.h[s];
        }
        return FKLO_OK;
    }
    /* ConvertYUVToRGB / ConvertRGBToYUV<CD, CR, CP>::exec, FK/algorithms/image_processing/color_conversion.h:150-201:
     * offsets subtracted before (to RGB) or added after (to YCbCr) the matrix, luma offset only for limited range. */
    case FKLO_YUV2RGB: case FKLO_RGB2YUV: {
        depth_consts d;
        float m[9];
        const int to_rgb = op->code == FKLO_YUV2RGB;
        if (fklo_color_matrix(op->idx[0], op->idx[1], op->idx[2], to_rgb, m) || depth_constants(op->idx[0], &d)) return FKLO_EINVAL;
        if (v->elem != depth_elem(op->idx[0]) || v->cn != 3) return FKLO_ETYPE;
        float in[3], out[3];
        for (int c = 0; c < 3; ++c) in[c] = chan_as_float(v, c);
        if (to_rgb) {
            if (op->idx[1] == FKLO_LIMITED) in[0] = in[0] - d.luma;
            in[1] = in[1] - d.chroma;
            in[2] = in[2] - d.chroma;
            mxv3(m, in, out);
        } else {
            mxv3(m, in, out);
            if (op->idx[1] == FKLO_LIMITED) out[0] = out[0] + d.luma;
            out[1] = out[1] + d.chroma;
            out[2] = out[2] + d.chroma;
        }
        for (int c = 0; c < 3; ++c) v->f[c] = out[c];
        v->elem = FKLO_F32;
        return FKLO_OK;
    }
    /* RGB2Gray<I, O, CCIR_601>::exec, color_conversion.h:49-80: (R*0.299f + G*0.587f) + B*0.114f through nearbyint
     * (ties to even) and a plain conversion to O.  That includes float outputs: the branch order is is_unsigned,
     * is_signed, is_floating_point, and float is signed. */
    case FKLO_RGB2GRAY: {
        if (v->cn < 3) return FKLO_ETYPE;
        const float l = (chan_as_float(v, 0) * 0.299f + chan_as_float(v, 1) * 0.587f) + chan_as_float(v, 2) * 0.114f;
        v->cn = 1;
        v->elem = op->idx[0];
        if (v->elem == FKLO_F32) v->f[0] = nearbyintf(l);
        else if (v->elem == FKLO_U8) v->u[0] = (uint8_t)(unsigned)nearbyintf(l);
        else if (v->elem == FKLO_U16) v->h[0] = (uint16_t)(unsigned)nearbyintf(l);
        else return FKLO_ETYPE;
        return FKLO_OK;
    }
    /* AddLast<I, O>::exec, FK/algorithms/basic_ops/vector_ops.h:94-118 (AddOpaqueAlpha: color_conversion.h:81-93). */
    case FKLO_ADD_LAST: {
        if (v->cn > 3) return FKLO_ETYPE;
        if (v->elem == FKLO_F32) v->f[v->cn] = op->p[0];
        else if (v->elem == FKLO_U8) v->u[v->cn] = (uint8_t)op->p[0];
        else v->h[v->cn] = (uint16_t)op->p[0];
        v->cn += 1;
        return FKLO_OK;
    }
    /* Discard<I, O>::exec, FK/algorithms/basic_ops/vector_ops.h:22-41. */
    case FKLO_DISCARD: {
        if (op->idx[0] < 1 || op->idx[0] >= v->cn) return FKLO_ETYPE;
        v->cn = op->idx[0];
        return FKLO_OK;
    }
    case FKLO_SATCAST_U16: {
        if (v->elem != FKLO_F32) return FKLO_ETYPE;
        for (int c = 0; c < v->cn; ++c) v->h[c] = fklo_saturate_cast_u16(v->f[c]);
        v->elem = FKLO_U16;
        return FKLO_OK;
    }
    case FKLO_SATCAST_U8: {
        if (v->elem != FKLO_F32) return FKLO_ETYPE;
        for (int c = 0; c < v->cn; ++c) v->u[c] = fklo_saturate_cast_u8(v->f[c]);
        v->elem = FKLO_U8;
        return FKLO_OK;
    }
    /* Saturate<T>::exec, FK/algorithms/image_processing/saturate.h:38-49 -> cxp::clamp, FK/core/constexpr_libs/
     * constexpr_cmath.h:60-62: the two comparisons below, so NaN stays NaN.  SaturateDepth<T, CD>
     * (color_conversion.h:96-107) is this with p = {0, maxDepthValue<CD>}. */
    case FKLO_CLAMP: {
        if (v->elem != FKLO_F32) return FKLO_ETYPE;
        for (int c = 0; c < v->cn; ++c) {
            const float a = v->f[c];
            v->f[c] = (a < op->p[0]) ? op->p[0] : ((op->p[1] < a) ? op->p[1] : a);
        }
        return FKLO_OK;
    }
    /* SaturateFloat<T>::exec, saturate.h:51-64 -> cxp::saturate_float, FK/core/constexpr_libs/constexpr_saturate.h:152-168:
     * fmaxf(0.f, fminf(s, 1.f)) on the host, written out with comparisons so the result does not depend on the C
     * library at hand: fminf(NaN, 1) = 1, and of two zeros fmaxf returns its second operand on x86-64 (glibc's
     * fmaxf ends in maxss), so -0 stays -0 while every other negative value becomes +0. */
    case FKLO_SATURATE_FLOAT: {
        if (v->elem != FKLO_F32) return FKLO_ETYPE;
        for (int c = 0; c < v->cn; ++c) {
            const float s = v->f[c];
            const float t = (s < 1.0f) ? s : 1.0f;
            v->f[c] = (t < 0.0f) ? 0.0f : t;
        }
        return FKLO_OK;
    }
    /* cxp::cast<O>::f, FK/core/constexpr_libs/constexpr_cmath.h:648-662: static_cast per channel; DenormalizePixel<O, CD>
     * (color_conversion.h:109-121) is FKLO_MUL by maxDepthValue<CD> and then this. */
    case FKLO_CAST_TRUNC: {
        if (v->elem != FKLO_F32) return FKLO_ETYPE;
        if (op->idx[0] == FKLO_U8) { for (int c = 0; c < v->cn; ++c) v->u[c] = (uint8_t)v->f[c]; }
        else if (op->idx[0] == FKLO_U16) { for (int c = 0; c < v->cn; ++c) v->h[c] = (uint16_t)v->f[c]; }
        else if (op->idx[0] != FKLO_F32) return FKLO_ETYPE;
        v->elem = op->idx[0];
        return FKLO_OK;
    }
    case FKLO_CAST_F32: {
        if (v->elem != FKLO_F32) {
            for (int c = 0; c < v->cn; ++c) v->f[c] = chan_as_float(v, c);
            v->elem = FKLO_F32;
        }
        return FKLO_OK;
    }
    case FKLO_YUV2RGB_709_FULL: {
        if (v->elem != FKLO_U8 || v->cn != 3) return FKLO_ETYPE;
        fklo_yuv2rgb_709_full(v->u, v->f);
        v->elem = FKLO_F32;
        return FKLO_OK;
    }
    default:
        return FKLO_EINVAL;
    }
}

/* ---- the read stack ---------------------------------------------------- */

/* PerThreadRead<_2D,T>::exec + PtrAccessor<_2D>::cr_point, FK/algorithms/basic_ops/memory_operations.h:26-67,
 * FK/core/data/rawptr.h:202-213: address = data + y*pitch + x*sizeof(T).
 * ReadYUV<NV12>::exec, FK/algorithms/image_processing/color_conversion.h:219-238: Y at (x,y) of the
 * luma plane; (U,V) at element x>>1 of chroma row y>>1, chroma base = data + pitch*height. */
static uint16_t load_u16(const uint8_t *p) { uint16_t v; memcpy(&v, p, 2); return v; }
static int read_is_pixel_format(const fklo_read *r) { return r->kind != FKLO_READ_2D && r->kind != FKLO_READ_PLANAR; }
static int pixel_format_elem(int kind) {
    return (kind == FKLO_READ_P010 || kind == FKLO_READ_P210 || kind == FKLO_READ_Y210) ? FKLO_U16 : FKLO_U8;
}
static void read_source(const fklo_read *r, int x, int y, fklo_val *out) {
    const uint8_t *base = (const uint8_t *)r->data;
    if (r->kind == FKLO_READ_NV12 || r->kind == FKLO_READ_NV21) {
        /* color_conversion.h:219-253; NV21 stores the pair as (V,U) and still yields (Y,U,V) */
        const int vu = r->kind == FKLO_READ_NV21;
        out->elem = FKLO_U8;
        out->cn = 3;
        out->u[0] = base[(int64_t)y * r->pitch + x];
        const uint8_t *chroma = base + (int64_t)r->pitch * r->height + (int64_t)(y >> 1) * r->pitch;
        out->u[1] = chroma[2 * (x >> 1) + (vu ? 1 : 0)];
        out->u[2] = chroma[2 * (x >> 1) + (vu ? 0 : 1)];
        return;
    }
    if (r->kind == FKLO_READ_P010 || r->kind == FKLO_READ_P210) {
        /* color_conversion.h:219-238 with ushort samples; 4:2:0 halves the chroma row index, 4:2:2 does not */
        const int cy = r->kind == FKLO_READ_P010 ? y >> 1 : y;
        out->elem = FKLO_U16;
        out->cn = 3;
        out->h[0] = load_u16(base + (int64_t)y * r->pitch + 2 * (int64_t)x);
        const uint8_t *chroma = base + (int64_t)r->pitch * r->height + (int64_t)cy * r->pitch + 4 * (int64_t)(x >> 1);
        out->h[1] = load_u16(chroma);
        out->h[2] = load_u16(chroma + 2);
        return;
    }
    if (r->kind == FKLO_READ_Y210) {
        /* color_conversion.h:254-266: group x>>1 of row y is Y0 U Y1 V */
        const uint8_t *g = base + (int64_t)y * r->pitch + 8 * (int64_t)(x >> 1);
        out->elem = FKLO_U16;
        out->cn = 3;
        out->h[0] = load_u16(g + ((x & 1) == 0 ? 0 : 4));
        out->h[1] = load_u16(g + 2);
        out->h[2] = load_u16(g + 6);
        return;
    }
    if (r->kind == FKLO_READ_UYVY) {
        /* color_conversion.h:254-266: group x>>1 of row y is U Y0 V Y1 */
        const uint8_t *g = base + (int64_t)y * r->pitch + 4 * (int64_t)(x >> 1);
        out->elem = FKLO_U8;
        out->cn = 3;
        out->u[0] = g[(x & 1) == 0 ? 1 : 3];
        out->u[1] = g[0];
        out->u[2] = g[2];
        return;
    }
    out->elem = r->elem;
    out->cn = r->cn;
    const uint8_t *row = base + (int64_t)y * r->pitch;
    if (r->kind == FKLO_READ_PLANAR) {
        /* TensorPack<T>::exec, FK/algorithms/basic_ops/memory_operations.h:243-290 (channel_stride = width*height elements)
         * and TensorTPack<T>::exec, :292-327 with PtrAccessor<T3D>::cr_point, FK/core/data/rawptr.h:229-235
         * (channel_stride = color_planes_pitch). */
        const int64_t esz = r->elem == FKLO_U8 ? 1 : (r->elem == FKLO_U16 ? 2 : 4);
        for (int c = 0; c < r->cn; ++c) {
            const uint8_t *p = row + (int64_t)x * esz + (int64_t)c * r->channel_stride;
            if (r->elem == FKLO_U8) out->u[c] = *p;
            else if (r->elem == FKLO_U16) out->h[c] = load_u16(p);
            else memcpy(&out->f[c], p, 4);
        }
        return;
    }
    if (r->elem == FKLO_U8) {
        const uint8_t *p = row + (int64_t)x * r->cn;
        for (int c = 0; c < r->cn; ++c) out->u[c] = p[c];
    } else if (r->elem == FKLO_U16) {
        const uint8_t *p = row + 2 * (int64_t)x * r->cn;
        for (int c = 0; c < r->cn; ++c) out->h[c] = load_u16(p + 2 * c);
    } else {
        const float *p = (const float *)row + (int64_t)x * r->cn;
        for (int c = 0; c < r->cn; ++c) out->f[c] = p[c];
    }
}

/* Crop<BackIOp>::exec, FK/algorithms/image_processing/crop.h:36-39: shift by the rect origin, no clipping;
 * then whatever compute ops were fused into the read (FusedOperation, iop_fuser.h:99-106). */
/* BorderReader<BT,...>::exec, FK/algorithms/image_processing/border_reader.h:177-327: idx = low(high(i)) in int
 * arithmetic; n is the extent of the operation behind the border. */
static int iabs(int v) { return v < 0 ? -v : v; }
static int border_fold(int type, int i, int n) {
    const int last = n - 1;
    switch (type) {
    case 1: { const int hi = i < last ? i : last; return hi > 0 ? hi : 0; }                               /* REPLICATE   */
    case 2: { const int hi = last - iabs(last - i) + (i > last); return (iabs(hi) - (hi < 0)) % (last + 1); } /* REFLECT */
    case 3: { const int hi = i < n ? i : i % n; return hi >= 0 ? hi : hi - ((hi - n + 1) / n) * n; }      /* WRAP        */
    default: { const int hi = iabs(last - iabs(last - i)) % (last + 1); return iabs(hi) % (last + 1); }   /* REFLECT_101 */
    }
}

static int read_tap(const fklo_read *r, int x, int y, fklo_val *out) {
    if (r->has_crop) {
        x += r->crop[0];
        y += r->crop[1];
    }
    if (r->border) {
        const int type = r->border - 1;
        if (type < 0 || type > 4) return FKLO_EINVAL;
        if (type == 0) {
            if (!(x >= 0 && x < r->width && y >= 0 && y < r->height)) {
                read_source(r, 0, 0, out);     /* for the type and channel count */
                for (int c = 0; c < out->cn; ++c) {
                    out->f[c] = r->border_value[c];
                    out->u[c] = (uint8_t)r->border_value[c];
                    out->h[c] = (uint16_t)r->border_value[c];
                }
                for (int i = 0; i < r->n_tap_ops; ++i) {
                    const int rc = apply_op(&r->tap_ops[i], out);
                    if (rc) return rc;
                }
                return FKLO_OK;
            }
        } else {
            x = border_fold(type, x, r->width);
            y = border_fold(type, y, r->height);
        }
    }
    read_source(r, x, y, out);
    for (int i = 0; i < r->n_tap_ops; ++i) {
        const int rc = apply_op(&r->tap_ops[i], out);
        if (rc) return rc;
    }
    return FKLO_OK;
}

static void read_extent(const fklo_read *r, int *w, int *h) {
    if (r->has_crop) { *w = r->crop[2]; *h = r->crop[3]; }
    else { *w = r->width; *h = r->height; }
}

/* ResizeComplete<AR,...>::exec / exec_resize, FK/algorithms/image_processing/resize.h:86-98,117-123 and
 * InterpolateComplete<INTER_LINEAR>::exec, interpolation.h:70-104. */
static int read_resized(const fklo_read *r, const fklo_resize_params *rp, int x, int y, fklo_val *out) {
    if (r->ar != FKLO_IGNORE_AR) {
        if (!(x >= rp->x1 && x <= rp->x2 && y >= rp->y1 && y <= rp->y2)) {
            /* params.defaultValue: float_<cn> of the tap type (resize.h:74) */
            out->elem = FKLO_F32;
            out->cn = read_is_pixel_format(r) ? 3 : r->cn;
            for (int c = 0; c < out->cn; ++c) out->f[c] = r->bg[c];
            return FKLO_OK;
        }
        x -= rp->x1;
        y -= rp->y1;
    }
    const float sx = (float)x * rp->fx;
    const float sy = (float)y * rp->fy;
    const int x1 = (int)floorf(sx), y1 = (int)floorf(sy);
    const int x2 = x1 + 1, y2 = y1 + 1;
    int sw, sh;
    read_extent(r, &sw, &sh);
    const int x2r = x2 < sw - 1 ? x2 : sw - 1;
    const int y2r = y2 < sh - 1 ? y2 : sh - 1;
    fklo_val t00, t10, t01, t11;
    int rc;
    if ((rc = read_tap(r, x1, y1, &t00))) return rc;
    if ((rc = read_tap(r, x2r, y1, &t10))) return rc;
    if ((rc = read_tap(r, x1, y2r, &t01))) return rc;
    if ((rc = read_tap(r, x2r, y2r, &t11))) return rc;
    out->elem = FKLO_F32;
    out->cn = t00.cn;
    for (int c = 0; c < t00.cn; ++c) {
        out->f[c] = fklo_bilinear(chan_as_float(&t00, c), chan_as_float(&t10, c),
                                  chan_as_float(&t01, c), chan_as_float(&t11, c), sx, sy);
    }
    return FKLO_OK;
}

/* ---- writers ----------------------------------------------------------- */

/* PerThreadWrite<_2D,T>, TensorWrite<T>, TensorSplit<T>: FK/algorithms/basic_ops/memory_operations.h:84-107,
 * 159-179, 181-212; PtrAccessor<_3D>::point, FK/core/data/rawptr.h:215-226 (plane stride =
 * plane_pitch*color_planes with plane_pitch = pitch*height). */
static const void *val_chan(const fklo_val *v, int c) {
    return v->elem == FKLO_F32 ? (const void *)&v->f[c] : (v->elem == FKLO_U16 ? (const void *)&v->h[c] : (const void *)&v->u[c]);
}
static void store_u16(uint8_t *p, uint16_t s) { memcpy(p, &s, 2); }

/* WriteYUV<PF>::exec, FK/algorithms/image_processing/color_conversion.h:298-389.  The value is (Y,U,V).  Semi-planar
 * formats store Y per pixel and the chroma pair from the pixels the reference lets store it: even x and even y
 * (4:2:0) or even x (4:2:2) for NV12/P010/P210; every pixel for NV21, where the z,y,x loop of the CPU backend leaves
 * the pair of the block's last pixel.  Packed 4:2:2: the even pixel stores U, Y0, V, the odd one Y1. */
static int write_yuv(const fklo_write *w, int x, int y, const fklo_val *v) {
    uint8_t *base = (uint8_t *)w->data;
    const int fmt = w->yuv_format;
    if (v->cn != 3 || v->elem != pixel_format_elem(fmt)) return FKLO_ETYPE;
    if (fmt == FKLO_READ_NV12 || fmt == FKLO_READ_NV21) {
        base[(int64_t)y * w->pitch + x] = v->u[0];
        uint8_t *c = base + (int64_t)w->pitch * w->height + (int64_t)(y >> 1) * w->pitch + 2 * (int64_t)(x >> 1);
        if (fmt == FKLO_READ_NV21) { c[0] = v->u[2]; c[1] = v->u[1]; }
        else if ((x & 1) == 0 && (y & 1) == 0) { c[0] = v->u[1]; c[1] = v->u[2]; }
        return FKLO_OK;
    }
    if (fmt == FKLO_READ_P010 || fmt == FKLO_READ_P210) {
        store_u16(base + (int64_t)y * w->pitch + 2 * (int64_t)x, v->h[0]);
        const int cy = fmt == FKLO_READ_P010 ? y >> 1 : y;
        uint8_t *c = base + (int64_t)w->pitch * w->height + (int64_t)cy * w->pitch + 4 * (int64_t)(x >> 1);
        if ((x & 1) == 0 && (fmt == FKLO_READ_P210 || (y & 1) == 0)) { store_u16(c, v->h[1]); store_u16(c + 2, v->h[2]); }
        return FKLO_OK;
    }
    if (fmt == FKLO_READ_UYVY) {
        uint8_t *g = base + (int64_t)y * w->pitch + 4 * (int64_t)(x >> 1);
        if ((x & 1) == 0) { g[0] = v->u[1]; g[1] = v->u[0]; g[2] = v->u[2]; }
        else g[3] = v->u[0];
        return FKLO_OK;
    }
    if (fmt == FKLO_READ_Y210) {
        uint8_t *g = base + (int64_t)y * w->pitch + 8 * (int64_t)(x >> 1);
        if ((x & 1) == 0) { store_u16(g, v->h[0]); store_u16(g + 2, v->h[1]); store_u16(g + 6, v->h[2]); }
        else store_u16(g + 4, v->h[0]);
        return FKLO_OK;
    }
    return FKLO_EINVAL;
}

static int write_value(const fklo_write *w, int x, int y, int z, const fklo_val *v) {
    if (w->kind == FKLO_WRITE_YUV) return write_yuv(w, x, y, v);
    if (v->elem != w->elem || v->cn != w->cn) return FKLO_ETYPE;
    uint8_t *base = (uint8_t *)w->data;
    const int64_t esz = w->elem == FKLO_U8 ? 1 : (w->elem == FKLO_U16 ? 2 : 4);
    if (w->kind == FKLO_WRITE_2D) {
        uint8_t *p = base + (int64_t)y * w->pitch + (int64_t)x * esz * w->cn;
        for (int c = 0; c < w->cn; ++c) memcpy(p + c * esz, val_chan(v, c), (size_t)esz);
        return FKLO_OK;
    }
    const int64_t plane_pitch = (int64_t)w->pitch * w->height;
    if (w->kind == FKLO_TENSOR_TSPLIT) {
        /* TensorTSplit<T>::exec, FK/algorithms/basic_ops/memory_operations.h:214-241 with PtrAccessor<T3D>::point,
         * FK/core/data/rawptr.h:236-239: data + c*color_planes_pitch + z*plane_pitch + y*pitch, then x elements;
         * color_planes_pitch = plane_pitch * planes (ptr_nd.h:119-125). */
        for (int c = 0; c < w->cn; ++c)
            memcpy(base + (int64_t)c * plane_pitch * w->planes + plane_pitch * z + (int64_t)y * w->pitch + (int64_t)x * esz,
                   val_chan(v, c), (size_t)esz);
        return FKLO_OK;
    }
    uint8_t *row = base + plane_pitch * w->color_planes * z + (int64_t)y * w->pitch;
    if (w->kind == FKLO_TENSOR_WRITE) {
        uint8_t *p = row + (int64_t)x * esz * w->cn;
        for (int c = 0; c < w->cn; ++c) memcpy(p + c * esz, val_chan(v, c), (size_t)esz);
        return FKLO_OK;
    }
    if (w->kind == FKLO_TENSOR_SPLIT) {
        const int64_t plane_px = (int64_t)w->width * w->height;
        for (int c = 0; c < w->cn; ++c) memcpy(row + ((int64_t)x + c * plane_px) * esz, val_chan(v, c), (size_t)esz);
        return FKLO_OK;
    }
    return FKLO_EINVAL;
}

/* ---- the loop ---------------------------------------------------------- */

/* TransformDPP<CPU>::exec, FK/core/execution_model/data_parallel_patterns.h:271-283: for z, y, x over the
 * active threads of the (fused) read; BatchRead picks plane z (batch_operations.h:205-212) and
 * activeThreads = (max W, max H, BATCH) (batch_operations.h:401-424). Planes whose own geometry is smaller
 * than the maximum are rejected here: the reference runs them unchecked, which reads outside the crop. */
/* Warping<WT, BackIOp>::exec and WarpingCoords<WT>::exec, FK/algorithms/image_processing/warping.h:42-96: the
 * destination pixel maps to m * (x, y, 1); inside the source the value is InterpolateComplete<INTER_LINEAR> at
 * that coordinate (interpolation.h:70-104), outside it is 0. */
static int read_warped(const fklo_read *r, int x, int y, fklo_val *out) {
    const float *m = r->warp_m;
    float sx = (m[0] * (float)x + m[1] * (float)y) + m[2];
    float sy = (m[3] * (float)x + m[4] * (float)y) + m[5];
    if (r->warp == 2) {
        const float coeff = 1.0f / ((m[6] * (float)x + m[7] * (float)y) + m[8]);
        sx = coeff * sx;
        sy = coeff * sy;
    }
    int sw, sh;
    read_extent(r, &sw, &sh);
    out->elem = FKLO_F32;
    out->cn = read_is_pixel_format(r) ? 3 : r->cn;
    if (!(sx >= 0.f && sx < (float)sw && sy >= 0.f && sy < (float)sh)) {
        for (int c = 0; c < out->cn; ++c) out->f[c] = 0.f;
        return FKLO_OK;
    }
    const int x1 = (int)floorf(sx), y1 = (int)floorf(sy);
    const int x2 = x1 + 1, y2 = y1 + 1;
    const int x2r = x2 < sw - 1 ? x2 : sw - 1;
    const int y2r = y2 < sh - 1 ? y2 : sh - 1;
    fklo_val t00, t10, t01, t11;
    int rc;
    if ((rc = read_tap(r, x1, y1, &t00))) return rc;
    if ((rc = read_tap(r, x2r, y1, &t10))) return rc;
    if ((rc = read_tap(r, x1, y2r, &t01))) return rc;
    if ((rc = read_tap(r, x2r, y2r, &t11))) return rc;
    out->cn = t00.cn;
    for (int c = 0; c < t00.cn; ++c) {
        out->f[c] = fklo_bilinear(chan_as_float(&t00, c), chan_as_float(&t10, c),
                                  chan_as_float(&t01, c), chan_as_float(&t11, c), sx, sy);
    }
    return FKLO_OK;
}

/* Deinterlace<DType, BackIOp>::exec, FK/algorithms/image_processing/deinterlace.h:44-103.  Sums of uchar channels are
 * ints (C++ promotion), of float channels floats; the result is float_<cn>. */
static int read_deinterlaced(const fklo_read *r, int x, int y, fklo_val *out) {
    int sw, sh;
    read_extent(r, &sw, &sh);
    int average, ya, yb;
    if (r->deinterlace == 1) {
        average = y > 0;
        ya = y; yb = y - 1;                 /* current, above */
    } else {
        const int even = (y & 1) == 0;
        average = r->deinterlace == 2 ? (!even && y != sh - 1) : (even && y != 0);
        ya = y - 1; yb = y + 1;             /* above, below */
        /* the reference assumes an even line count; for an odd one, keeping odd lines, its last line would read
         * past the image: that read is defined here (and in the device code) as the last line */
        if (yb > sh - 1) yb = sh - 1;
    }
    fklo_val a, b;
    int rc;
    if (!average) {
        if ((rc = read_tap(r, x, y, &a))) return rc;
        out->elem = FKLO_F32;
        out->cn = a.cn;
        for (int c = 0; c < a.cn; ++c) out->f[c] = chan_as_float(&a, c) * 1.f;
        return FKLO_OK;
    }
    if ((rc = read_tap(r, x, ya, &a))) return rc;
    if ((rc = read_tap(r, x, yb, &b))) return rc;
    out->elem = FKLO_F32;
    out->cn = a.cn;
    for (int c = 0; c < a.cn; ++c) {
        if (a.elem == FKLO_U8) out->f[c] = (float)((int)a.u[c] + (int)b.u[c] + 1) * 0.5f;
        else if (a.elem == FKLO_U16) out->f[c] = (float)((int)a.h[c] + (int)b.h[c] + 1) * 0.5f;
        else out->f[c] = ((a.f[c] + b.f[c]) + 1.f) * 0.5f;
    }
    return FKLO_OK;
}

/* BatchRead<CONDITIONAL_WITH_DEFAULT>::exec, FK/core/execution_model/operation_model/batch_operations.h:262-273:
 * planes at or beyond usedPlanes return params.default_value, whose type is the plane operation's output type
 * (float_<cn> after a resize, the tap type after fused tap operations, else the element type). */
static void read_default(const fklo_read *r, fklo_val *out) {
    int cn = read_is_pixel_format(r) ? 3 : r->cn;
    int elem = read_is_pixel_format(r) ? pixel_format_elem(r->kind) : r->elem;
    if (r->n_tap_ops > 0 || r->has_resize) {
        /* find the type the read yields by running the tap operations on a dummy element */
        fklo_val probe;
        memset(&probe, 0, sizeof(probe));
        probe.elem = elem;
        probe.cn = cn;
        for (int i = 0; i < r->n_tap_ops; ++i) apply_op(&r->tap_ops[i], &probe);
        elem = r->has_resize ? FKLO_F32 : probe.elem;
        cn = probe.cn;
    }
    memset(out, 0, sizeof(*out));
    out->elem = elem;
    out->cn = cn;
    for (int c = 0; c < cn; ++c) {
        if (elem == FKLO_F32) out->f[c] = r->def[c];
        else if (elem == FKLO_U16) out->h[c] = (uint16_t)r->def[c];
        else out->u[c] = (uint8_t)r->def[c];
    }
}

int fklo_execute(int32_t n_planes, const fklo_read *reads,
                 int32_t n_ops, const fklo_op *ops,
                 int32_t n_writes, const fklo_write *writes) {
    if (n_planes < 1 || !reads || !writes) return FKLO_EINVAL;
    if (n_writes != 1 && n_writes != n_planes) return FKLO_EINVAL;
    int act_w = 0, act_h = 0;
    for (int z = 0; z < n_planes; ++z) {
        int w, h;
        if (reads[z].has_resize && reads[z].warp) return FKLO_EINVAL;
        if (reads[z].has_resize || reads[z].warp) { w = reads[z].dst_w; h = reads[z].dst_h; }
        else read_extent(&reads[z], &w, &h);
        if (z == 0) { act_w = w; act_h = h; }
        else if (w != act_w || h != act_h) return FKLO_EGEOM;
    }
    for (int z = 0; z < n_planes; ++z) {
        const fklo_read *r = &reads[z];
        const fklo_write *w = n_writes == 1 ? &writes[0] : &writes[z];
        const int wz = n_writes == 1 ? z : 0;
        fklo_resize_params rp;
        if (r->has_resize) {
            int sw, sh;
            read_extent(r, &sw, &sh);
            fklo_compute_resize_params(sw, sh, r->dst_w, r->dst_h, r->ar, &rp);
        }
        for (int y = 0; y < act_h; ++y) {
            for (int x = 0; x < act_w; ++x) {
                fklo_val v;
                int rc = FKLO_OK;
                if (r->use_default) read_default(r, &v);
                else if (r->warp) rc = read_warped(r, x, y, &v);
                else if (r->deinterlace) rc = read_deinterlaced(r, x, y, &v);
                else rc = r->has_resize ? read_resized(r, &rp, x, y, &v) : read_tap(r, x, y, &v);
                if (rc) return rc;
                for (int i = 0; i < n_ops; ++i) {
                    if ((rc = apply_op(&ops[i], &v))) return rc;
                }
                if ((rc = write_value(w, x, y, wz, &v))) return rc;
            }
        }
    }
    return FKLO_OK;
}

/* computeCircularThreadIdx<direction, BATCH>, FK/algorithms/basic_ops/memory_operations.h:422-432. */
int32_t fklo_circular_plane(int32_t direction, int32_t batch, int32_t z, int32_t first) {
    if (direction == 0) { const int32_t c = z + first; return c >= batch ? c - batch : c; }
    const int32_t c = first - z;
    return c < 0 ? batch + c : c;
}
/* SequenceSelectorType<CTO, BATCH>::at, FK/core/data/circular_tensor.h:26-35. */
int32_t fklo_window_sequence(int32_t order, int32_t batch, int32_t z) {
    if (order == 0) return z > 0 ? 1 : 0;
    return z != batch - 1 ? 1 : 0;
}

/* ---- synthetic inputs: std::mt19937 ------------------------------------ */

void fklo_mt_seed(fklo_mt19937 *g, uint32_t seed) {
    g->mt[0] = seed;
    for (int i = 1; i < 624; ++i)
        g->mt[i] = 1812433253u * (g->mt[i - 1] ^ (g->mt[i - 1] >> 30)) + (uint32_t)i;
    g->idx = 624;
}

uint32_t fklo_mt_next(fklo_mt19937 *g) {
    if (g->idx >= 624) {
        for (int i = 0; i < 624; ++i) {
            const uint32_t y = (g->mt[i] & 0x80000000u) | (g->mt[(i + 1) % 624] & 0x7fffffffu);
            g->mt[i] = g->mt[(i + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
        }
        g->idx = 0;
    }
    uint32_t y = g->mt[g->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}

void fklo_mt_fill_bytes(fklo_mt19937 *g, uint8_t *dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = (uint8_t)(fklo_mt_next(g) & 0xFFu);
}

void fklo_mt_fill_unit_floats(fklo_mt19937 *g, float *dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = (float)(fklo_mt_next(g) >> 8) * (1.0f / 8388608.0f) - 1.0f;
}

void fklo_mt_fill_range_floats(fklo_mt19937 *g, float *dst, uint64_t n, float a, float b) {
    for (uint64_t i = 0; i < n; ++i)
        dst[i] = a + ((float)(fklo_mt_next(g) >> 8) * (1.0f / 16777216.0f)) * (b - a);
}

void fklo_mt_fill_u32(fklo_mt19937 *g, uint32_t *dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = fklo_mt_next(g);
}

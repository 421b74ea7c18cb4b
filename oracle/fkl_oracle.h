/*
 * fkl_oracle.h -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded CPU restatement of the arithmetic that the Fused
 * Kernel Library (FKL) performs on its fused data-parallel path
 *   executeOperations<TransformDPP<>>(stream, Read, [Crop/Resize], [compute...], Write).
 * It exists so that tests, the smoke check and the CPU-baseline leg of the
 * benchmark have something independent to compare the HIP kernels against.
 * Nothing in the shipped library may include, link or call it.
 *
 * Every function cites the reference file:line whose behaviour it restates
 * (paths relative to the reference root, FK/ = include/fused_kernel/).
 *
 * Pinning status (what each part has been checked against, see tests/):
 *   - saturate cast, BT.709 matrix, BGR swap, round(): known-answer values held
 *     by the reference's own unit tests            -> pinned
 *   - bilinear crop/resize, letterbox geometry, NV12 tap, TensorWrite/Split
 *     addressing, per-plane batch reads            -> pinned against a build of
 *     the reference's CPU backend (oracle/_ref) on all five benchmark
 *     configurations at full size and on randomised reduced cases, plus the
 *     committed golden fixtures derived from that build, plus closed forms
 *     (ramp image, identity resize, exact 2x, constant chroma).
 *   No function of this file is "parity unpinned".
 *
 * Build: gcc -std=c99 -O2 -ffp-contract=off (no -ffast-math).  With
 * contraction off every + - * / below is one IEEE-754 binary32 rounding,
 * which is what makes the result compiler independent.
 */
#ifndef FKL_ORACLE_H
#define FKL_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { FKLO_U8 = 0, FKLO_F32 = 1, FKLO_U16 = 2 };

enum fklo_read_kind {
    FKLO_READ_2D = 0,   /* PerThreadRead<_2D,T>: pitched array of cn-channel elements */
    FKLO_READ_NV12 = 1, /* ReadYUV<NV12>: luma plane + interleaved half-res chroma    */
    FKLO_READ_NV21 = 2, /* ReadYUV<NV21>: as NV12 with the chroma pair stored (V,U)   */
    FKLO_READ_P010 = 3, /* ReadYUV<P010>: NV12 layout with 16-bit samples             */
    FKLO_READ_P210 = 4, /* ReadYUV<P210>: 16-bit samples, chroma rows at full height  */
    FKLO_READ_Y210 = 5, /* ReadYUV<Y210>: packed 16-bit Y0 U Y1 V                     */
    FKLO_READ_UYVY = 6, /* ReadYUV<UYVY>: packed 8-bit U Y0 V Y1                      */
    FKLO_READ_PLANAR = 7 /* TensorPack<T> / TensorTPack<T>: cn channel planes of elem, channel_stride bytes apart;
                            data = channel 0 of this image plane                        */
};

enum fklo_aspect { FKLO_PRESERVE_AR = 0, FKLO_IGNORE_AR = 1, FKLO_PRESERVE_AR_RN_EVEN = 2, FKLO_PRESERVE_AR_LEFT = 3 };

enum fklo_opcode {
    FKLO_MUL = 1,              /* out = in * p   (per channel, result float)           */
    FKLO_ADD = 2,              /* out = in + p                                         */
    FKLO_SUB = 3,              /* out = in - p                                         */
    FKLO_DIV = 4,              /* out = in / p   (IEEE division)                       */
    FKLO_REORDER = 5,          /* out[c] = in[idx[c]]  (BGR<->RGB is idx = 2,1,0)      */
    FKLO_SATCAST_U8 = 6,       /* float -> uchar: NaN->0, round-half-even, clamp       */
    FKLO_CAST_F32 = 7,         /* uchar -> float static_cast (no-op on float)          */
    FKLO_YUV2RGB_709_FULL = 8, /* uchar3 (Y,U,V) -> float3 RGB, BT.709 full range 8bit */
    FKLO_YUV2RGB = 9,          /* ConvertYUVToRGB<depth, range, primaries>: idx[0..2]  */
    FKLO_RGB2YUV = 10,         /* ConvertRGBToYUV<depth, range, primaries>: idx[0..2]  */
    FKLO_RGB2GRAY = 11,        /* RGB2Gray<I, O>: idx[0] = element type of O           */
    FKLO_ADD_LAST = 12,        /* one more channel holding p[0] (AddOpaqueAlpha)       */
    FKLO_DISCARD = 13,         /* keep the first idx[0] channels                       */
    FKLO_SATCAST_U16 = 14,     /* float -> ushort: NaN->0, round-half-even, clamp      */
    FKLO_CLAMP = 15,           /* Saturate<T> / SaturateDepth: (v<p[0]) ? p[0] : ((p[1]<v) ? p[1] : v)       */
    FKLO_SATURATE_FLOAT = 16,  /* SaturateFloat<T>: fmaxf(0, fminf(v, 1)); NaN -> 1, -0 stays -0            */
    FKLO_CAST_TRUNC = 17       /* float -> element type idx[0] like a C cast (DenormalizePixel after FKLO_MUL) */
};

enum fklo_write_kind {
    FKLO_WRITE_2D = 0,      /* PerThreadWrite<_2D,T>; one fklo_write per plane when batched */
    FKLO_TENSOR_WRITE = 1,  /* TensorWrite<T>: AoS, plane z at z*plane_pitch*color_planes   */
    FKLO_TENSOR_SPLIT = 2,  /* TensorSplit<T>: planar, channel c at +c*width*height elems   */
    FKLO_WRITE_YUV = 3,     /* WriteYUV<PF>: yuv_format names the layout (a fklo_read_kind) */
    FKLO_TENSOR_TSPLIT = 4  /* TensorTSplit<T>: channel c at +c*pitch*height*planes bytes, plane z at +z*pitch*height */
};

/* Values of fk::ColorDepth, fk::ColorRange, fk::ColorPrimitives (FK/algorithms/image_processing/itu_color.h:26-29). */
enum { FKLO_P8 = 0, FKLO_P10 = 1, FKLO_P12 = 2, FKLO_FN8 = 3, FKLO_FN10 = 4, FKLO_FN12 = 5 };
enum { FKLO_LIMITED = 0, FKLO_FULL = 1 };
enum { FKLO_BT601 = 0, FKLO_BT709 = 1, FKLO_BT2020 = 2 };

typedef struct {
    int32_t code;
    float p[4];
    int32_t idx[4];
} fklo_op;

typedef struct {
    int32_t kind;            /* fklo_read_kind */
    int32_t elem;            /* FKLO_U8 / FKLO_F32 / FKLO_U16 (READ_2D); pixel formats fix their own */
    int32_t cn;              /* channels of one element (READ_2D); pixel formats yield 3 */
    int32_t width, height;   /* READ_2D: element grid; pixel formats: image size in pixels */
    int32_t pitch;           /* bytes per row */
    const void *data;
    int32_t has_crop;
    int32_t crop[4];         /* x, y, w, h */
    int32_t has_resize;
    int32_t dst_w, dst_h;
    int32_t ar;              /* fklo_aspect */
    float bg[4];             /* letterbox background (PRESERVE_AR) */
    int32_t n_tap_ops;       /* ops fused INTO the read: run on every source tap */
    const fklo_op *tap_ops;
    int32_t use_default;     /* BatchRead<CONDITIONAL_WITH_DEFAULT>, plane index >= usedPlanes: every element of */
    float def[4];            /* this plane is def, typed like the read's output, and nothing is read             */
    int32_t warp;            /* 0 none, 1 Warping<Affine>, 2 Warping<Perspective>; output grid dst_w x dst_h,     */
    float warp_m[9];         /* row-major transform (affine uses the first two rows); excludes has_resize         */
    int32_t deinterlace;     /* 0 none, 1 Deinterlace<BLEND>, 2 <INTER_LINEAR> keeping even lines, 3 keeping odd   */
    int32_t border;          /* BorderReader between the source and the crop: 0 none, else 1 + fk::BorderType       */
    float border_value[4];   /* (1 CONSTANT, 2 REPLICATE, 3 REFLECT, 4 WRAP, 5 REFLECT_101); CONSTANT's value, typed  */
                             /* like the source element                                                             */
    int64_t channel_stride;  /* FKLO_READ_PLANAR: bytes from one channel plane to the next                                  */
} fklo_read;

typedef struct {
    int32_t kind;            /* fklo_write_kind */
    int32_t elem;            /* element base type of the stored value */
    int32_t cn;              /* channels of the stored value */
    void *data;
    int32_t width, height, planes, color_planes;
    int32_t pitch;           /* bytes per row */
    int32_t yuv_format;      /* FKLO_WRITE_YUV: fklo_read_kind of the layout; width, height = image size in pixels */
} fklo_write;

typedef struct {
    int32_t dst_w, dst_h;
    float fx, fy;            /* source step per output pixel */
    int32_t x1, y1, x2, y2;  /* letterbox rectangle (inclusive) */
} fklo_resize_params;

/* Errors */
enum { FKLO_OK = 0, FKLO_EINVAL = 1, FKLO_ETYPE = 2, FKLO_EGEOM = 3 };

/* Run one fused chain: for z, for y, for x (FK/core/execution_model/data_parallel_patterns.h:271-283).
 * n_writes is 1 (single target) or n_planes (BatchWrite of 2-D targets). */
int fklo_execute(int32_t n_planes, const fklo_read *reads,
                 int32_t n_ops, const fklo_op *ops,
                 int32_t n_writes, const fklo_write *writes);

/* Building blocks, exported so tests can pin them one by one. */
void fklo_compute_resize_params(int32_t src_w, int32_t src_h, int32_t dst_w, int32_t dst_h,
                                int32_t ar, fklo_resize_params *out);
uint8_t fklo_saturate_cast_u8(float v);
float fklo_banker_round(float v);
float fklo_round_half_away(float v);
void fklo_yuv2rgb_709_full_matrix(float m[9]);
/* ccMatrix<range, primaries, direction, depth> (row major) and the offsets of the depth. */
int fklo_color_matrix(int32_t depth, int32_t range, int32_t primaries, int32_t to_rgb, float m[9]);
int fklo_depth_constants(int32_t depth, float *max_value, float *luma_offset, float *chroma_offset);
uint16_t fklo_saturate_cast_u16(float v);
void fklo_yuv2rgb_709_full(const uint8_t yuv[3], float rgb[3]);
/* 4-tap bilinear of one channel given the four tap values already converted
 * to float; (sx, sy) is the source coordinate. */
float fklo_bilinear(float p00, float p10, float p01, float p11, float sx, float sy);

/* Circular-buffer plane of logical plane z (computeCircularThreadIdx, FK/algorithms/basic_ops/memory_operations.h:422-432):
 * direction 0 Ascendent, 1 Descendent.  Sequence of CircularTensor::update that owns plane z (the selector of CircularTensor::update,
 * FK/core/data/circular_tensor.h:26-35): 0 the caller's chain, 1 the copy; order 0 NewestFirst, 1 OldestFirst. */
int32_t fklo_circular_plane(int32_t direction, int32_t batch, int32_t z, int32_t first);
int32_t fklo_window_sequence(int32_t order, int32_t batch, int32_t z);

/* Deterministic synthetic inputs: raw std::mt19937 outputs. */
typedef struct { uint32_t mt[624]; int32_t idx; } fklo_mt19937;
void fklo_mt_seed(fklo_mt19937 *g, uint32_t seed);
uint32_t fklo_mt_next(fklo_mt19937 *g);
void fklo_mt_fill_bytes(fklo_mt19937 *g, uint8_t *dst, uint64_t n);            /* gen() & 0xFF          */
void fklo_mt_fill_unit_floats(fklo_mt19937 *g, float *dst, uint64_t n);        /* (gen()>>8)*2^-23 - 1  */
void fklo_mt_fill_range_floats(fklo_mt19937 *g, float *dst, uint64_t n, float a, float b); /* a + (gen()>>8)*2^-24*(b-a) */
void fklo_mt_fill_u32(fklo_mt19937 *g, uint32_t *dst, uint64_t n);

#ifdef __cplusplus
}
#endif
#endif

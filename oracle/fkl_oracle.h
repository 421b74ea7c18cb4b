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

enum { FKLO_U8 = 0, FKLO_F32 = 1 };

enum fklo_read_kind {
    FKLO_READ_2D = 0,   /* PerThreadRead<_2D,T>: pitched array of cn-channel elements */
    FKLO_READ_NV12 = 1  /* ReadYUV<NV12>: luma plane + interleaved half-res chroma    */
};

enum fklo_aspect { FKLO_PRESERVE_AR = 0, FKLO_IGNORE_AR = 1 };

enum fklo_opcode {
    FKLO_MUL = 1,              /* out = in * p   (per channel, result float)           */
    FKLO_ADD = 2,              /* out = in + p                                         */
    FKLO_SUB = 3,              /* out = in - p                                         */
    FKLO_DIV = 4,              /* out = in / p   (IEEE division)                       */
    FKLO_REORDER = 5,          /* out[c] = in[idx[c]]  (BGR<->RGB is idx = 2,1,0)      */
    FKLO_SATCAST_U8 = 6,       /* float -> uchar: NaN->0, round-half-even, clamp       */
    FKLO_CAST_F32 = 7,         /* uchar -> float static_cast (no-op on float)          */
    FKLO_YUV2RGB_709_FULL = 8  /* uchar3 (Y,U,V) -> float3 RGB, BT.709 full range 8bit */
};

enum fklo_write_kind {
    FKLO_WRITE_2D = 0,      /* PerThreadWrite<_2D,T>; one fklo_write per plane when batched */
    FKLO_TENSOR_WRITE = 1,  /* TensorWrite<T>: AoS, plane z at z*plane_pitch*color_planes   */
    FKLO_TENSOR_SPLIT = 2   /* TensorSplit<T>: planar, channel c at +c*width*height elems   */
};

typedef struct {
    int32_t code;
    float p[4];
    int32_t idx[4];
} fklo_op;

typedef struct {
    int32_t kind;            /* fklo_read_kind */
    int32_t elem;            /* FKLO_U8 / FKLO_F32 (READ_2D); NV12 is always U8 */
    int32_t cn;              /* channels of one element (READ_2D); NV12 yields 3 */
    int32_t width, height;   /* READ_2D: element grid; NV12: luma size */
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
} fklo_read;

typedef struct {
    int32_t kind;            /* fklo_write_kind */
    int32_t elem;            /* element base type of the stored value */
    int32_t cn;              /* channels of the stored value */
    void *data;
    int32_t width, height, planes, color_planes;
    int32_t pitch;           /* bytes per row */
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
void fklo_yuv2rgb_709_full(const uint8_t yuv[3], float rgb[3]);
/* 4-tap bilinear of one channel given the four tap values already converted
 * to float; (sx, sy) is the source coordinate. */
float fklo_bilinear(float p00, float p10, float p01, float p11, float sx, float sy);

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

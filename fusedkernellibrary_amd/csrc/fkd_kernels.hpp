// fkd_kernels.hpp -- the gfx950 kernel skeletons of the fused data-parallel path and their launchers.
//
// Two skeletons cover every chain; which one a chain gets is decided from its read operation at compile time.
//
//  rows kernel    one thread produces V = 4 horizontally adjacent outputs of one row of plane z.  Reads and
//                 writes of 4 elements move as dwordx3 / dwordx4 accesses (12 bytes for uchar3, 16 for float,
//                 48 for float3) that consecutive lanes make contiguous, so a wave64 touches whole cache lines.
//                 Each thread handles ROWS rows so several independent loads are in flight per lane.
//                 Plane z = workgroup index in z: horizontal (batch) fusion, per-plane parameters are wave
//                 uniform and come out of the kernel-argument segment through scalar loads.
//
//  gather kernel  for chains whose read is a bilinear resize: a workgroup owns a tile of the output of one plane,
//                 a wave owns whole output rows of it, so source rows, vertical weights and all row addresses are
//                 wave uniform (scalar registers); a lane reads the four taps of each of its pixels straight from
//                 global memory as whole elements at byte granularity.  Whatever was fused into the read (colour
//                 conversion, per-plane arithmetic) is applied per tap, in the reference's order.  Workgroups are
//                 renumbered so each XCD works on a contiguous run of a plane's tiles and its L2 sees the source
//                 rows those tiles share.
//
// Reference being replaced: TransformDPP<GPU_NVIDIA>::exec and launchTransformDPP_Kernel,
// FK/core/execution_model/data_parallel_patterns.h:223-242 and executor_details/executor_kernels.h:26-30;
// launch geometry FK/core/execution_model/executors.h:242-351.
#pragma once

#if !defined(__HIPCC_RTC__)
#include <hip/hip_runtime.h>   // the run-time compiler provides the HIP device API without any header
#endif

#include <fkd/launch_info.hpp>
#include <fkd/ops.hpp>

namespace fkd {

template <int I> struct IntTag { static constexpr int value = I; };

// ---- chain classification ---------------------------------------------------------------------------

template <class R> struct ResizeRoot { static constexpr bool value = false; };
template <int AR, class Back> struct ResizeRoot<ResizeLinear<AR, Back>> {
    static constexpr bool value = true;
    static constexpr bool batched = false;
    using Resize = ResizeLinear<AR, Back>;
};
template <int N, int AR, class Back> struct ResizeRoot<BatchRead<N, ResizeLinear<AR, Back>>> {
    static constexpr bool value = true;
    static constexpr bool batched = true;
    using Resize = ResizeLinear<AR, Back>;
};

template <int N, int AR, class Back> struct ResizeRoot<BatchReadDefault<N, ResizeLinear<AR, Back>>> {
    static constexpr bool value = true;
    static constexpr bool batched = true;
    using Resize = ResizeLinear<AR, Back>;
};
template <class R> struct HasDefaultPlanes { static constexpr bool value = false; };
template <int N, class PlaneOp> struct HasDefaultPlanes<BatchReadDefault<N, PlaneOp>> { static constexpr bool value = true; };

// Reads whose taps are scattered gathers (warps): the rows kernel then keeps one element per thread.
template <class R> constexpr bool is_scattered_read() {
    if constexpr (requires { R::kGatherRead; }) return R::kGatherRead;
    else if constexpr (requires { typename R::Plane; }) return is_scattered_read<typename R::Plane>();
    else return false;
}

template <class Chain> constexpr bool is_gather_chain() {
    if constexpr (ResizeRoot<typename Chain::Read>::value)
        return ResizeRoot<typename Chain::Read>::Resize::BackOp::kTapCursor;
    else
        return false;
}

// Stores of a lane-masking writer (kLaneMasked); other writers never reach these calls, the indirection only keeps their
// instantiations from looking the members up.
template <class WP, class Plane> __device__ __forceinline__ u32 masked_row_offset(int y, const Plane& plane) {
    if constexpr (requires { WP::kLaneMasked; }) return WP::row_offset(y, plane); else return 0u;
}
template <class WP, class Plane, class V> __device__ __forceinline__ void masked_put(const Plane& plane, u32 row_off, u32 lane_off, const V& v) {
    if constexpr (requires { WP::kLaneMasked; }) WP::put_masked(plane, row_off, lane_off, v);
}

// (The geometry a launcher hands to kernels that renumber their workgroups -- TileGeom, division_magic, the limits that
// choose a form of grid -- is in fkd/launch_info.hpp, which the launchers of run-time compiled kernels share.)

// ---- rows kernel ---------------------------------------------------------------------------------------

constexpr int kRowsBX = 64;   // lanes along x: one wave per row segment
constexpr int kRowsBY = 4;    // waves per workgroup
constexpr unsigned long long kStreamElements = 1ull << 26;   // launches over more elements stream their input

// For the test of what run-time compilation does with a chain whose per-thread array cannot stay in registers: with
// FKD_TEST_UNRESOLVED_INDEX defined, the rows kernel indexes its values with an offset that is zero when the kernel runs
// but unknown when it is compiled (an index the optimiser cannot resolve keeps the array in memory).  Zero otherwise.
#ifdef FKD_TEST_UNRESOLVED_INDEX
#define FKD_TEST_INDEX_OFFSET int(p.active_w >> 31)
#else
#define FKD_TEST_INDEX_OFFSET 0
#endif

// The full-width part of the rows kernel: every lane has V elements in each of its ROWS rows.  MODE as in
// detail::load_run.
template <class Chain, int V, int ROWS, int MODE>
__device__ __forceinline__ void rows_full(const typename Chain::Params& p, u32 kernarg_offset, int x0, int ybase, int z, int ah) {
    using R = typename Chain::Read;
    using W = typename Chain::Write;

    // All loads first, unconditionally (rows past the end re-read the last row, which is in bounds), so every
    // lane has ROWS independent wide loads in flight before the first use; only the stores are predicated.
    Slot<typename R::Out> in[ROWS * V];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int y = ybase + r < ah ? ybase + r : ah - 1;
        Slot<typename R::Out> row[V];
        R::template exec_row<V, MODE>(x0, y, z, p.read, row);
#pragma unroll
        for (int i = 0; i < V; ++i) in[r * V + i].v = row[i].v;
    }
    // all ROWS*V elements go through the chain together, operation by operation
    Slot<typename Chain::Value> out[ROWS * V];
    if constexpr (Chain::kLongChain) Chain::template compute_run_kernarg<ROWS * V>(in, out, (const FKD_CONSTANT char*)__builtin_amdgcn_kernarg_segment_ptr() + kernarg_offset);
    else Chain::template compute_run<ROWS * V>(in, out, p.ops);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int y = ybase + r;
        Slot<typename Chain::Value> row[V];
#pragma unroll
        for (int i = 0; i < V; ++i) row[i].v = out[r * V + i + FKD_TEST_INDEX_OFFSET].v;
        if (y < ah) W::template exec_row<V, MODE>(x0, y, z, row, p.write);
    }
}

// Chains whose read gathers its taps from wherever the coordinates fall (warps, bilinear reads without a tap cursor): their
// larger launches number the workgroups of a plane so that each XCD works on a contiguous band of the output.
template <class Chain> constexpr bool rows_in_bands() {
    return ResizeRoot<typename Chain::Read>::value || is_scattered_read<typename Chain::Read>();
}
// The workgroups of a plane, bands form: the grid is one-dimensional, 8 * ceil(blocks / 8) workgroups per plane.  The
// hardware deals consecutive workgroup numbers round-robin to the 8 XCDs; XCD k takes the k-th contiguous eighth of the
// plane's blocks (row-major), so that neighbouring blocks, whose taps share source lines, share an L2.  With the
// workgroups in plain row-major order a warp fetched its source 2.5 to 3.2 times, once into nearly every L2; in bands it
// is fetched once (rocprofv3 FETCH_SIZE), and a 3840 x 2160 warp takes 25.1 instead of 30.8 us.  Launches of fewer than
// kRowsBandBlocks blocks per plane keep the two-dimensional grid: their source comes out of the last-level cache either
// way, and the 1080p warp measured 5 % slower in bands (9.27 against 8.83 us).  (rows_band_chunk and kRowsBandBlocks:
// fkd/launch_info.hpp.)

// `kernarg_offset`: where p sits inside the kernel-argument segment (0 when the chain's parameter block is the
// kernel's first argument); long chains fetch their operations' parameters from there.  BANDS: the launch has the bands
// form of grid (see rows_band_chunk).
template <class Chain, int V, int ROWS, bool ALIGNED, bool BANDS = false>
__device__ __forceinline__ void rows_body(const typename Chain::Params& p, u32 kernarg_offset = 0, const TileGeom* bands = nullptr) {
    using R = typename Chain::Read;
    using W = typename Chain::Write;
    const int z = blockIdx.z;
    const int aw = int(p.active_w), ah = int(p.active_h);
    u32 block_x = blockIdx.x, block_y = blockIdx.y;
    if constexpr (BANDS) {
        // (blocks per row and per column, and the multiplier that divides by the former, come from the launcher, which
        // leaves them zero for a two-dimensional grid; wave uniform)
        const u32 gx = bands->tiles_x, blocks = gx * bands->tiles_y;
        if (blocks != 0u) {
            const u32 tin = (blockIdx.x % 8u) * rows_band_chunk(blocks) + blockIdx.x / 8u;
            if (tin >= blocks) return;
            block_y = bands->tiles_x_magic ? u32(((unsigned long long)tin * bands->tiles_x_magic) >> 32) : tin / gx;
            block_x = tin - block_y * gx;
        }
    }
    const int x0 = (block_x * kRowsBX + threadIdx.x) * V;
    const int ybase = (block_y * kRowsBY + threadIdx.y) * ROWS;
    if (x0 >= aw || ybase >= ah) return;
    // Wave-cooperative accesses (mode 2 of load_run / store_run) need every lane of the wave on a full run.
    constexpr bool kExchange = ALIGNED && (detail::wave_exchange_ok<typename R::Out>(V) || detail::wave_exchange_ok<typename W::In>(V));
    if constexpr (kExchange) {
        if (int(block_x * kRowsBX + kRowsBX) * V <= aw) {
            rows_full<Chain, V, ROWS, 2>(p, kernarg_offset, x0, ybase, z, ah);
            return;
        }
    }
    // A launch over more elements than the last-level cache could hold between two launches reads them with the
    // non-temporal hint (100 images of 1920x1080 uchar3: 225 -> 209 us); smaller inputs are left to the caches, where a
    // pipeline's previous stage may have put them (the hint costs 15 % on a 33 MB image that is still cached).
    constexpr bool kMayStream = ALIGNED && !Chain::kLongChain && !kExchange;
    if constexpr (kMayStream) {
        if (x0 + V <= aw && (unsigned long long)(u32(aw)) * u32(ah) * gridDim.z > kStreamElements) {
            rows_full<Chain, V, ROWS, 1 | 4>(p, kernarg_offset, x0, ybase, z, ah);
            return;
        }
    }
    if (x0 + V <= aw) {
        rows_full<Chain, V, ROWS, ALIGNED ? 1 : 0>(p, kernarg_offset, x0, ybase, z, ah);
    } else {
        for (int r = 0; r < ROWS; ++r) {
            const int y = ybase + r;
            if (y >= ah) break;
            for (int x = x0; x < aw; ++x) {
                Slot<typename R::Out> in[1];
                Slot<typename Chain::Value> out[1];
                in[0].v = R::exec(x, y, z, p.read);
                if constexpr (Chain::kLongChain) Chain::template compute_run_kernarg<1>(in, out, (const FKD_CONSTANT char*)__builtin_amdgcn_kernarg_segment_ptr() + kernarg_offset);
                else Chain::template compute_run<1>(in, out, p.ops);
                W::exec(x, y, z, out[0].v, p.write);
            }
        }
    }
}

template <class Chain, int V, int ROWS, bool ALIGNED>
__global__ __launch_bounds__(kRowsBX * kRowsBY) void k_rows(const typename Chain::Params p, const TileGeom g) {
    rows_body<Chain, V, ROWS, ALIGNED, rows_in_bands<Chain>()>(p, 0u, &g);
}

// Whether the rows of plane z of the read and of the write all start on dword boundaries, decided on the device
// (wave uniform, a handful of scalar instructions).  Kernels compiled at run time use this instead of the
// launcher's host-side check, because their launcher does not know the chain's type.
template <class Op, class P> FKD_DEV bool read_plane_aligned(const P& p, int z) {
    if constexpr (requires { Op::plane_rows_aligned(p, z, 0); }) return Op::plane_rows_aligned(p, z, 0);
    else return Op::rows_aligned(p, 0);
}
template <class Op, class P> FKD_DEV bool write_plane_aligned(const P& p, int z) {
    if constexpr (requires { Op::plane_rows_aligned(p, z); }) return Op::plane_rows_aligned(p, z);
    else return Op::rows_aligned(p);
}
template <class Chain, int V, int ROWS, bool BANDS = false>
__device__ __forceinline__ void rows_auto_body(const typename Chain::Params& p, u32 kernarg_offset = 0, const TileGeom* bands = nullptr) {
    const int z = blockIdx.z;
    const bool aligned = read_plane_aligned<typename Chain::Read>(p.read, z) && write_plane_aligned<typename Chain::Write>(p.write, z);
    if (aligned) rows_body<Chain, V, ROWS, true, BANDS>(p, kernarg_offset, bands);
    else rows_body<Chain, V, ROWS, false, BANDS>(p, kernarg_offset, bands);
}

// ---- gather bilinear kernel ----------------------------------------------------------------------------

#ifndef FKD_GATHER_XI
#define FKD_GATHER_XI 2
#endif
#ifndef FKD_GATHER_YI
#define FKD_GATHER_YI 2
#endif
#ifndef FKD_GATHER_ADJ
#define FKD_GATHER_ADJ 0
#endif
#ifndef FKD_GATHER_BY
#define FKD_GATHER_BY 4
#endif
#ifndef FKD_GATHER_DEPTH
#define FKD_GATHER_DEPTH 2
#endif
constexpr int kGatherBX = 64;
constexpr int kGatherBY = FKD_GATHER_BY;

// A workgroup owns a (64*XI) x (4*YI) tile of the output of one plane; wave w owns rows w*YI .. w*YI+YI-1 of it, so
// everything that depends on the row (source rows, vertical weights, row addresses of source and destination) is
// wave uniform and lives in scalar registers.  A lane produces XI pixels (64 apart, so stores of a wave are
// contiguous) in each of its YI rows; the horizontal coordinate work is shared by the rows.  The four taps of a
// pixel are read straight from global memory as whole elements (a uchar3 comes in as one dword whose top byte is
// ignored); neighbouring lanes and rows hit the same cache lines, so HBM sees each source line about once.
// All loads of a lane are issued before the first use and are unconditional (coordinates are clamped into the
// source); only stores are predicated.
// The tile's work once the plane's parameters are in registers: q (the plane's read), ops, wpar (the plane's write), the
// output extent aw x ah, the plane z, the tile's first column tx0 and its row of tiles.
template <class Chain, int XI, int YI, class Q, class OPS, class WPAR>
__device__ __forceinline__ void gather_tile(const typename Chain::Params& p, const Q& q, const OPS& ops, const WPAR& wpar,
                                            int aw, int ah, int z, int tx0, u32 tile_row) {
    using Root = ResizeRoot<typename Chain::Read>;
    using RZ = typename Root::Resize;
    using Back = typename RZ::BackOp;
    using Raw = typename Back::Raw;
    using W = typename Chain::Write;
    using WP = typename W::Plane;
    constexpr int TH = kGatherBY * YI;
    const int wy = __builtin_amdgcn_readfirstlane(int(threadIdx.y));
    const int y0 = int(tile_row) * TH + wy * YI;
    if (y0 >= ah) return;
    if constexpr (HasDefaultPlanes<typename Chain::Read>::value) {
        // BatchRead<CONDITIONAL_WITH_DEFAULT>: planes at or beyond `used` read nothing; every element is the default
        // value, which still goes through the chain's compute operations and the write.
        if (z >= p.read.used) {
            const typename RZ::Out def = p.read.def;
            const typename Chain::Value r = Chain::compute_checked_ops(def, ops);
            for (int y = y0; y < (y0 + YI < ah ? y0 + YI : ah); ++y) {
                const typename WP::RowRef orow = WP::row(y, z, wpar);
#pragma unroll
                for (int i = 0; i < XI; ++i) {
                    const int x = tx0 + int(threadIdx.x) + kGatherBX * i;
                    if (x < aw) WP::put(orow, x, r);
                }
            }
            return;
        }
    }
    int ox = 0, oy = 0;
    if constexpr (RZ::kAR != IGNORE_AR) { ox = q.x1; oy = q.y1; }
    const int sw = Back::width(q.back), sh = Back::height(q.back);

    // Pixels of a lane: XI adjacent ones (their results leave as one wide store per plane), or 64 apart.
    auto xof = [&](int i) {
        if constexpr (FKD_GATHER_ADJ) return tx0 + int(threadIdx.x) * XI + i;
        else return tx0 + int(threadIdx.x) + kGatherBX * i;
    };
    // Horizontal part, per lane, shared by the YI rows.  float(x1) and float(x1 + 1) are taken as floor(sx) and
    // floor(sx) + 1, the same numbers (exact integers below 2^24).
    int x1[XI], x2[XI];
    f32 ax[XI], bx[XI];
    bool xin[XI], clamped[XI];
    bool lane_clamped = false;
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        int x = xof(i);
        x = x < aw ? x : aw - 1;                                   // idle lanes shadow the last column
        xin[i] = true;
        if constexpr (RZ::kAR != IGNORE_AR) xin[i] = x >= q.x1 && x <= q.x2;
        const f32 sx = f32(x - ox) * q.fx;
        const f32 f1 = __builtin_floorf(sx);
        ax[i] = (f1 + 1.0f) - sx;
        bx[i] = sx - f1;
        const int xi = int(f1);
        x1[i] = xi < 0 ? 0 : (xi < sw - 1 ? xi : sw - 1);       // no-op wherever the reference is in bounds
        x2[i] = x1[i] + 1 < sw - 1 ? x1[i] + 1 : sw - 1;
        clamped[i] = x1[i] + 1 > sw - 1;
        lane_clamped = lane_clamped || clamped[i];
    }
    const bool any_clamped = __builtin_amdgcn_ballot_w64(lane_clamped) != 0;

    // Rows, software pipelined: the taps of row y+1 are requested before row y is blended, so once the first row
    // has arrived a wave always has data to work on while its next loads are in flight.  Two tap sets alternate
    // (the loop handles two rows per trip), so no registers are copied.
    // Three ways to fetch the taps of a row, chosen per wave:
    //   kPairs    the two horizontally adjacent taps of a pixel come in one access (possible when no lane of the
    //             wave has its right tap clamped to the last column), halving the number of gather instructions;
    //   kPairsSel the same for waves with clamped lanes: such a lane fetches the pair ending at the last column and
    //             uses its second element for both taps;
    //   kSingles  one access per tap, whole dwords;
    //   kSafe     one access per tap, never touching a byte outside the elements (channel by channel for 3- and
    //             6-byte elements): for waves whose taps reach the last row of the image.
    //   kPairsPrepared  kPairs for images whose rows all start at the same offset inside their dword (pitch a multiple
    //             of 4): the image is a buffer resource, a row a scalar offset, and the lane's window offset and byte
    //             shift are worked out once per column instead of once per tap;
    //   kWhole    both scale factors are whole numbers (4K -> 1080p): every source point is a pixel, the weights are
    //             1, 0, 0, 0, and the blend is the first tap; the others are not fetched.  Only for reads whose taps are
    //             always finite (a zero weight times them is a zero), and a lane whose first tap is a negative zero,
    //             where the zeros of the other three terms decide the sign of the sum, takes all four after all.
    constexpr int kSafe = 0, kSingles = 1, kPairs = 2, kPairsSel = 3, kPairsPrepared = 4, kWhole = 5;
    const int yend = y0 + YI < ah ? y0 + YI : ah;
    // STATIC: every quick operation of the chain takes its static form (decided once per wave, below).
    // Writers that can switch lanes off through their offset (kLaneMasked) store without an execution mask and with
    // 32-bit scalar row arithmetic; image planes too large for that (plane_maskable) take the plain stores.
    constexpr bool kCanMask = [] { if constexpr (requires { WP::kLaneMasked; }) return WP::kLaneMasked && !FKD_GATHER_ADJ; else return false; }();
    auto make_plane = [&] { if constexpr (kCanMask) return WP::plane_ref(z, wpar); else return 0; };
    const auto oplane = make_plane();
    u32 lane_off[XI];
#pragma unroll
    for (int i = 0; i < XI; ++i) { if constexpr (kCanMask) lane_off[i] = WP::lane_offset(xof(i), xof(i) < aw); else lane_off[i] = 0; }
    auto rows_with = [&](auto mode_tag, auto static_tag, auto masked_tag) {
        constexpr int MODE = decltype(mode_tag)::value;
        constexpr bool STATIC = decltype(static_tag)::value != 0;
        constexpr bool MASKED = decltype(masked_tag)::value != 0;
        constexpr bool PAIRED = MODE == kPairs || MODE == kPairsSel || MODE == kPairsPrepared;
        detail::PairPrep prep[XI];
        detail::TapImage image;
        if constexpr (MODE == kPairsPrepared) {
            image = Back::tap_image(z, q.back);
#pragma unroll
            for (int i = 0; i < XI; ++i) prep[i] = Back::pair_prepare(image, x1[i], q.back);
        }
        struct RowTaps {
            typename Back::TapBits a[PAIRED ? 1 : XI], b[PAIRED ? 1 : XI], c[PAIRED ? 1 : XI], d[PAIRED ? 1 : XI];
            typename Back::PairBits ab[PAIRED ? XI : 1], cd[PAIRED ? XI : 1];
            typename Back::TapRow ra, rb;
            f32 ay, by;
        };
        auto request = [&](int yrow, RowTaps& t) {
            const int y = yrow;
            const f32 sy = f32(y - oy) * q.fy;
            const f32 f1 = __builtin_floorf(sy);
            t.ay = (f1 + 1.0f) - sy;
            t.by = sy - f1;
            const int yi = __builtin_amdgcn_readfirstlane(int(f1));
            const int ya = yi < 0 ? 0 : (yi < sh - 1 ? yi : sh - 1);
            const int yb = ya + 1 < sh - 1 ? ya + 1 : sh - 1;
            if constexpr (MODE != kPairsPrepared) {
                t.ra = Back::tap_row(0, ya, z, q.back);
                t.rb = Back::tap_row(0, yb, z, q.back);
            } else {
                t.ra = typename Back::TapRow{};     // rows are scalar offsets into the image's buffer resource
                t.rb = typename Back::TapRow{};
            }
#pragma unroll
            for (int i = 0; i < XI; ++i) {
                if constexpr (MODE == kPairsPrepared) {
                    t.ab[i] = Back::pair_load_prepared(image, Back::tap_row_offset(ya, q.back), prep[i], q.back);
                    t.cd[i] = Back::pair_load_prepared(image, Back::tap_row_offset(yb, q.back), prep[i], q.back);
                } else if constexpr (PAIRED) {
                    const int xl = MODE == kPairsSel ? x1[i] - int(clamped[i]) : x1[i];
                    t.ab[i] = Back::pair_load(t.ra, xl, q.back);
                    t.cd[i] = Back::pair_load(t.rb, xl, q.back);
                } else if constexpr (MODE == kWhole) {
                    t.a[i] = Back::template tap_load<false>(t.ra, x1[i], q.back);
                } else {
                    t.a[i] = Back::template tap_load<MODE == kSingles>(t.ra, x1[i], q.back);
                    t.b[i] = Back::template tap_load<MODE == kSingles>(t.ra, x2[i], q.back);
                    t.c[i] = Back::template tap_load<MODE == kSingles>(t.rb, x1[i], q.back);
                    t.d[i] = Back::template tap_load<MODE == kSingles>(t.rb, x2[i], q.back);
                }
            }
        };
        auto produce = [&](int y, const RowTaps& t) {
            if (y >= yend) return;
            bool yin = true;
            if constexpr (RZ::kAR != IGNORE_AR) yin = y >= q.y1 && y <= q.y2;
            typename WP::RowRef orow;
            if constexpr (!MASKED) orow = WP::row(y, z, wpar);
            Slot<typename Chain::Value> res[XI];
#pragma unroll
            for (int i = 0; i < XI; ++i) {
                typename RZ::Taps tp;
                tp.w00 = ax[i] * t.ay; tp.w10 = bx[i] * t.ay; tp.w01 = ax[i] * t.by; tp.w11 = bx[i] * t.by;
                Raw a, b, c, d;
                if constexpr (MODE == kWhole) {
                    using Src = typename RZ::Src;
                    const Src first = Back::finish(Back::tap_value(t.a[i]), q.back);
                    typename RZ::Out v;
                    bool negative_zero = false;
                    auto take = [&](auto pa) {
                        const f32 f = f32(pa);
                        if constexpr (__is_same(base_t<Src>, f32) || __is_same(base_t<Src>, f64))
                            negative_zero = negative_zero || __builtin_bit_cast(u32, f) == 0x80000000u;
                        return f;
                    };
                    chan<0>(v) = take(chan<0>(first));
                    if constexpr (cn_v<Src> > 1) chan<1>(v) = take(chan<1>(first));
                    if constexpr (cn_v<Src> > 2) chan<2>(v) = take(chan<2>(first));
                    if constexpr (cn_v<Src> > 3) chan<3>(v) = take(chan<3>(first));
                    if (negative_zero) {
                        b = Back::tap_value(Back::template tap_load<false>(t.ra, x2[i], q.back));
                        c = Back::tap_value(Back::template tap_load<false>(t.rb, x1[i], q.back));
                        d = Back::tap_value(Back::template tap_load<false>(t.rb, x2[i], q.back));
                        v = RZ::blend(first, Back::finish(b, q.back), Back::finish(c, q.back), Back::finish(d, q.back), tp);
                    }
                    if constexpr (RZ::kAR != IGNORE_AR) { if (!(yin && xin[i])) v = q.bg; }
                    if constexpr (STATIC) res[i].v = Chain::compute_static_ops(v, ops);
                    else res[i].v = Chain::compute_checked_ops(v, ops);
                    continue;
                }
                if constexpr (PAIRED) {
                    const int xl = MODE == kPairsSel ? x1[i] - int(clamped[i]) : x1[i];
                    Back::pair_values(t.ab[i], t.ra, xl, a, b);
                    Back::pair_values(t.cd[i], t.rb, xl, c, d);
                    if constexpr (MODE == kPairsSel) { if (clamped[i]) { a = b; c = d; } }
                } else {
                    a = Back::tap_value(t.a[i]); b = Back::tap_value(t.b[i]);
                    c = Back::tap_value(t.c[i]); d = Back::tap_value(t.d[i]);
                }
                typename RZ::Out v = RZ::blend(Back::finish(a, q.back), Back::finish(b, q.back),
                                               Back::finish(c, q.back), Back::finish(d, q.back), tp);
                if constexpr (RZ::kAR != IGNORE_AR) { if (!(yin && xin[i])) v = q.bg; }
                if constexpr (STATIC) res[i].v = Chain::compute_static_ops(v, ops);
                else res[i].v = Chain::compute_checked_ops(v, ops);
            }
            if constexpr (MASKED) {
                const u32 row_off = masked_row_offset<WP>(y, oplane);
#pragma unroll
                for (int i = 0; i < XI; ++i) masked_put<WP>(oplane, row_off, lane_off[i], res[i].v);
            } else if constexpr (FKD_GATHER_ADJ && XI > 1) {
                if (xof(XI - 1) < aw) {
                    WP::template put_run<XI>(orow, xof(0), res);
                } else {
#pragma unroll
                    for (int i = 0; i < XI; ++i) if (xof(i) < aw) WP::put(orow, xof(i), res[i].v);
                }
            } else {
#pragma unroll
                for (int i = 0; i < XI; ++i) if (xof(i) < aw) WP::put(orow, xof(i), res[i].v);
            }
        };
        if constexpr (FKD_GATHER_DEPTH <= 2) {
            RowTaps t0, t1;
            request(y0, t0);
#pragma unroll 1
            for (int y = y0; y < yend; y += 2) {
                if (y + 1 < yend) request(y + 1, t1);      // wave uniform
                produce(y, t0);
                if (y + 2 < yend) request(y + 2, t0);
                produce(y + 1, t1);
            }
        } else {
            // A ring of DEPTH tap sets: DEPTH - 1 rows of loads stay in flight behind the row being blended.
            constexpr int D = FKD_GATHER_DEPTH;
            RowTaps t[D];
#pragma unroll
            for (int k = 0; k < D - 1; ++k) if (y0 + k < yend) request(y0 + k, t[k]);
#pragma unroll 1
            for (int y = y0; y < yend; y += D) {
#pragma unroll
                for (int k = 0; k < D; ++k) {
                    if (y + k + D - 1 < yend) request(y + k + D - 1, t[(k + D - 1) % D]);
                    produce(y + k, t[k]);
                }
            }
        }
    };
    auto rows = [&](auto mode_tag) {
        if constexpr (Chain::kQuick) {
            if (Chain::ops_static(ops)) { rows_with(mode_tag, IntTag<1>{}, IntTag<kCanMask ? 1 : 0>{}); return; }
        }
        rows_with(mode_tag, IntTag<0>{}, IntTag<kCanMask ? 1 : 0>{});
    };
    // Whole-dword reads of 3- and 6-byte elements (and pair reads) touch up to 3 bytes past what they need.  Inside
    // the image that is the next element or row; only in the image's last row it could leave the allocation.
    bool tail = false;
    if constexpr (Back::kTapOverread) {
        const int ylast = yend - 1;                                       // last row the wave requests
        const int yl = int(__builtin_floorf(f32(ylast - oy) * q.fy));
        const int yb = yl + 1 < sh - 1 ? yl + 1 : sh - 1;
        tail = Back::tap_last(Back::tap_row(0, yb < 0 ? 0 : yb, z, q.back));
    }
    if constexpr (kCanMask) {
        if (!WP::plane_maskable(wpar)) {
            if (tail) rows_with(IntTag<kSafe>{}, IntTag<0>{}, IntTag<0>{});
            else rows_with(IntTag<kSingles>{}, IntTag<0>{}, IntTag<0>{});
            return;
        }
    }
    if constexpr (finite_taps<Back>()) {
        // whole factors, and every source coordinate an exact float: decided on the host (ResizeLinear::whole_factors)
        if (q.whole) { rows(IntTag<kWhole>{}); return; }
    }
    if (tail) {
        rows(IntTag<kSafe>{});
    } else {
        if constexpr (Back::kTapPair) {
            if (!any_clamped) {
                if constexpr (detail::tap_prepared<Back>()) {
                    if (Back::tap_rows_share_alignment(q.back)) { rows(IntTag<kPairsPrepared>{}); return; }
                }
                rows(IntTag<kPairs>{});
                return;
            }
            if (sw >= 2) { rows(IntTag<kPairsSel>{}); return; }
        }
        rows(IntTag<kSingles>{});
    }
}

template <class Chain, int XI, int YI>
__device__ __forceinline__ void gather_body(const typename Chain::Params& p, const TileGeom& g) {
    using Root = ResizeRoot<typename Chain::Read>;
    using RZ = typename Root::Resize;
    using W = typename Chain::Write;
    using WP = typename W::Plane;
    constexpr int TW = kGatherBX * XI;
    // The plane is the grid's z index, known at wave start, so the plane's parameters are fetched together with the
    // first kernel arguments instead of after them.  Within a plane workgroups are renumbered: hardware deals
    // consecutive workgroup ids round-robin to the 8 XCDs (the grid's x extent is a multiple of 8); XCD k gets the
    // k-th contiguous eighth of the plane's tiles so neighbouring tiles (which share source rows) share an L2.
    const int z = int(blockIdx.z);
    const typename RZ::Params* rp;
    if constexpr (Root::batched) rp = &p.read.plane[z]; else rp = &p.read;
    // A scalar load from the kernel-argument segment takes several hundred cycles, and a wave that lives for a few
    // thousand cannot afford one round trip per first use: geometry, the plane's read parameters, the operations'
    // parameters and the write's are requested back to back and waited for once.
    TileGeom gg = g;
    typename RZ::Params q = *rp;
    typename Chain::OpParams ops = p.ops;
    typename WP::Params wpar = W::plane_params(p.write, z);
    detail::pin_scalars(gg);
    detail::pin_scalars(q);
    detail::pin_scalars(ops);
    detail::pin_scalars(wpar);
    u32 dims[2] = {p.active_w, p.active_h};
    asm volatile("" : "+s"(dims[0]), "+s"(dims[1]));
    const int aw = int(dims[0]), ah = int(dims[1]);

    const u32 per_plane = gg.tiles_x * gg.tiles_y;
    const u32 chunk = (per_plane + 7u) / 8u;
    const u32 tin = (blockIdx.x % 8u) * chunk + blockIdx.x / 8u;
    if (tin >= per_plane) return;
    const u32 tile_row = gg.tiles_x_magic ? u32(((unsigned long long)tin * gg.tiles_x_magic) >> 32) : tin / gg.tiles_x;
    const int tx0 = int(tin - tile_row * gg.tiles_x) * TW;
    gather_tile<Chain, XI, YI>(p, q, ops, wpar, aw, ah, z, tx0, tile_row);
}

// ---- strip form of the bilinear kernel: narrow outputs (batches of small planes) -------------------------------------
//
// A workgroup of four waves owns 8 whole output rows of one plane, up to 256 pixels wide.  A HALF wave (32 lanes) owns
// one row and each lane the columns lane, lane + 32, lane + 64, ...: a 224-pixel row is seven such steps with no idle
// lane, where 128-pixel tiles leave one lane in eight without work.  What depends on the column (horizontal weights,
// the byte offset of the tap window and the bytes to drop from it) is worked out ONCE per workgroup, one column per
// thread, and handed round through 4 KB of LDS; what depends on the row is worked out once per lane and serves all its
// pixels.  So the fixed work of a wave is spread over seven pixels per lane instead of four, nearly all of it on the
// vector unit (the scalar unit is shared by the four SIMDs of a compute unit and was as busy as they were).
// What the form asks of every plane -- source rows that share their alignment (pitch a multiple of 4), source smaller
// than 2 GB and at least two columns wide, output plane smaller than 2 GB -- is checked on the host when the parameter
// block is made (Chain::finalize_write, bit 0 of Params::reserved); launchers take the tile form when the bit is clear.
// Taps come through a buffer resource whose extent ends with the image, so windows that reach past the last row read
// zeros in bytes nobody uses and no lane needs a narrower access; the row is part of the lane's offset.
// Wave priorities of the strip form.  A SIMD serves its oldest wave first, so in a launch that fits the chip in one round
// (every workgroup resident from the start: configuration 3's 1 792) the seven waves of a SIMD do not advance side by side:
// the wave that was started last is held back at every stage and ends up walking its steps nearly alone, each step exposed
// to the full latency of its taps (measured with per-wave time stamps: the first wave of a SIMD issues its last stores 3.6 us
// after the launch's first wave entered, the seventh 7.5 us).  Such a launch therefore starts every wave at priority 3 and
// lowers it as the wave advances (2 from step 3, 1 from step 5), which makes the waves of a SIMD advance together; and
// workgroups that were started late (the dispatcher hands consecutive workgroup numbers round the compute units, so a
// workgroup's number divided by the number of compute units says roughly how many were on its unit before it) keep each
// level one step longer, which is what keeps the last wave of a SIMD from finishing alone.  Configuration 3: 8.15 -> 7.85 us.
// A launch of several rounds is left alone: the fresh waves of a later round would outrank the last steps of the round
// before (twice the rows: 14.1 -> 15.4 us with the priorities on).  Priorities change the order of issue, never a result.
// The launcher decides and hands the kernel one number: the number of the first workgroup that counts as started late, or
// 0 for a launch whose waves keep the default priority.
// (strip_first_late_workgroup, fkd/launch_info.hpp)
constexpr int kStripRows = kGatherBY * FKD_GATHER_YI, kStripStep = 32, kStripMaxWidth = 256;
constexpr int kStripThreads = kStripRows * kStripStep, kStripMaxSteps = kStripMaxWidth / kStripStep;
static_assert(kStripThreads == kGatherBX * kGatherBY, "the two forms of the bilinear kernel share their workgroup shape");
static_assert(kStripThreads == kStripMaxWidth, "one table column per thread");

template <class Chain> constexpr bool strip_capable() {
    using Root = ResizeRoot<typename Chain::Read>;
    if constexpr (!Root::value) return false;
    else if constexpr (HasDefaultPlanes<typename Chain::Read>::value) return false;
    else {
        using Back = typename Root::Resize::BackOp;
        using WP = typename Chain::Write::Plane;
        if constexpr (!detail::tap_prepared<Back>()) return false;
        else if constexpr (!Back::kTapPair) return false;
        else if constexpr (requires { WP::kLaneMasked; }) return WP::kLaneMasked;
        else return false;
    }
}

template <class Chain>
__device__ __forceinline__ void strip_body(const typename Chain::Params& p, const u32 first_late_workgroup) {
    using Root = ResizeRoot<typename Chain::Read>;
    using RZ = typename Root::Resize;
    using Back = typename RZ::BackOp;
    using Raw = typename Back::Raw;
    using W = typename Chain::Write;
    using WP = typename W::Plane;
    // per column: ax, bx, window offset, bytes to drop from the window (bits 0-1) | flags
    __shared__ detail::u32x4_t column[kStripMaxWidth];
    __shared__ u32 wave_clamped[kStripThreads / 64];
    constexpr u32 kClamped = 0x80000000u, kOutsideX = 0x40000000u;

    const int z = int(blockIdx.z);
    // every wave starts at the highest priority, before its arguments are there: a launch of more than one round drops
    // it again below, once they say so
    __builtin_amdgcn_s_setprio(3);
    const typename RZ::Params* rp;
    if constexpr (Root::batched) rp = &p.read.plane[z]; else rp = &p.read;
    typename RZ::Params q = *rp;
    typename Chain::OpParams ops = p.ops;
    typename WP::Params wpar = W::plane_params(p.write, z);
    u32 dims[4] = {p.active_w, p.active_h, first_late_workgroup, gridDim.x};
    detail::pin_scalars(q);
    detail::pin_scalars(ops);
    detail::pin_scalars(wpar);
    // (the grid's width with the rest: fetched where it is used, it would be a second trip to the kernel-argument segment)
    asm volatile("" : "+s"(dims[0]), "+s"(dims[1]), "+s"(dims[2]), "+s"(dims[3]));
    const int aw = int(dims[0]), ah = int(dims[1]);
    // the steps at which this wave's priority falls to 2 and to 1, as two scalars (wave uniform)
    int falls[2] = {3, 5};
    if (dims[2] == 0u) {
        __builtin_amdgcn_s_setprio(0);
        falls[0] = falls[1] = kStripMaxSteps;                           // never
    } else if (blockIdx.z * dims[3] + blockIdx.x >= dims[2]) {
        falls[0] = 4;
        falls[1] = 6;
    }
    asm volatile("" : "+s"(falls[0]), "+s"(falls[1]));
    int ox = 0, oy = 0;
    if constexpr (RZ::kAR != IGNORE_AR) { ox = q.x1; oy = q.y1; }
    const int sw = Back::width(q.back), sh = Back::height(q.back);
    const detail::TapImage image = Back::tap_image_bounded(z, q.back);
    const int steps = (aw + kStripStep - 1) / kStripStep;
    if (steps == 0) return;                                             // no columns: nothing to write (the whole workgroup leaves)

    const int t = int(threadIdx.y) * 64 + int(threadIdx.x);
    // What depends on the column: the horizontal weights, the window's byte offset in a row, and flags beside the bytes to drop.
    auto column_entry = [&](int col, bool& clamped) {
        const int x = col < aw ? col : aw - 1;                          // columns beyond the output shadow the last one
        const f32 sx = f32(x - ox) * q.fx;
        const f32 f1 = __builtin_floorf(sx);
        const f32 ax = (f1 + 1.0f) - sx, bx = sx - f1;
        const int xi = int(f1);
        const int x1 = xi < 0 ? 0 : (xi < sw - 1 ? xi : sw - 1);
        clamped = x1 + 1 > sw - 1;                                      // right tap is the last column again
        const detail::PairPrep pp = Back::pair_prepare(image, x1 - int(clamped), q.back);
        u32 flags = pp.shift | (clamped ? kClamped : 0u);
        if constexpr (RZ::kAR != IGNORE_AR) flags |= (x >= q.x1 && x <= q.x2) ? 0u : kOutsideX;
        detail::u32x4_t e;
        e.x = __builtin_bit_cast(u32, ax); e.y = __builtin_bit_cast(u32, bx); e.z = pp.off; e.w = flags;
        return e;
    };

    // ---- the lane's row ----
    const int g = t & (kStripStep - 1), r = t >> 5;
    const int y = int(blockIdx.x) * kStripRows + r;
    const bool yvalid = y < ah;
    const int yc = yvalid ? y : ah - 1;
    const f32 sy = f32(yc - oy) * q.fy;
    const f32 fy1 = __builtin_floorf(sy);
    const f32 ay = (fy1 + 1.0f) - sy, by = sy - fy1;
    const int yi = int(fy1);
    const int ya = yi < 0 ? 0 : (yi < sh - 1 ? yi : sh - 1);
    const int yb = ya + 1 < sh - 1 ? ya + 1 : sh - 1;
    const u32 row_a = Back::tap_row_offset(ya, q.back), row_b = Back::tap_row_offset(yb, q.back);
    bool yin = true;
    if constexpr (RZ::kAR != IGNORE_AR) yin = yc >= q.y1 && yc <= q.y2;

    struct StepTaps { detail::u32x4_t e; typename Back::PairBits ab, cd; };
    auto fetch = [&](StepTaps& s) {
        // (v_alignbyte_b32 takes the bytes to drop from bits 0-1 of its operand, so the flags may ride along)
        detail::PairPrep pa, pb;
        pa.off = s.e.z + row_a; pa.shift = s.e.w;
        pb.off = s.e.z + row_b; pb.shift = s.e.w;
        s.ab = Back::pair_load_prepared(image, 0u, pa, q.back);
        s.cd = Back::pair_load_prepared(image, 0u, pb, q.back);
    };
    auto request = [&](int k, StepTaps& s) {
        s.e = column[g + kStripStep * k];
        fetch(s);
        __builtin_amdgcn_sched_barrier(0);      // the next step's taps leave before anything waits for this step's
    };
    // The taps of step 0 are requested before the table exists, from the lane's own working out of its first column:
    // they are then on their way while the table is made and the workgroup meets at the barrier.
    StepTaps first;
    {
        bool unused;
        first.e = column_entry(g, unused);
        fetch(first);
    }

    // ---- the column table: one column per thread (the workgroup has as many threads as the form has columns).  Columns
    // of the steps after the last one hold a window offset of 2 GB: the image is smaller than that (checked on the host), so
    // the sum with the lane's row offset neither wraps nor comes back below the image's extent, and requesting such a
    // column touches no memory.  Each wave notes whether it met a clamped column. ----
    constexpr u32 kNoWindow = 0x80000000u;
    {
        bool clamped = false;
        detail::u32x4_t e = column_entry(t, clamped);
        if (t >= steps * kStripStep) { e.z = kNoWindow; clamped = false; }
        column[t] = e;
        const bool any = __builtin_amdgcn_ballot_w64(clamped) != 0ull;
        if (threadIdx.x == 0) wave_clamped[threadIdx.y] = any ? 1u : 0u;
    }
    __syncthreads();
    u32 met = 0;
#pragma unroll
    for (int w = 0; w < kStripThreads / 64; ++w) met |= wave_clamped[w];
    const bool some_clamped = __builtin_amdgcn_readfirstlane(met) != 0u;

    const auto oplane = WP::plane_ref(z, wpar);
    // the lane's store offset in step 0; a lane without a row carries an offset beyond the resource's extent
    const u32 out0 = yvalid ? WP::row_offset(y, oplane) + WP::lane_offset(g, true) : WP::kMaskedOut;
    const bool partial = (aw & (kStripStep - 1)) != 0;             // the last step has columns beyond the output

    auto run = [&](auto static_tag, auto clamp_tag) {
        constexpr bool STATIC = decltype(static_tag)::value != 0;
        constexpr bool CLAMP = decltype(clamp_tag)::value != 0;
        auto produce = [&](int k, const StepTaps& s) {
            // (k is known where the steps are written out: one comparison in four of the steps)
            if ((k == 3 || k == 4) && k == falls[0]) __builtin_amdgcn_s_setprio(2);
            if ((k == 5 || k == 6) && k == falls[1]) __builtin_amdgcn_s_setprio(1);
            // (the words are copied out first: a bit cast applied directly to an element of the vector reads element 0)
            const u32 ax_bits = s.e.x, bx_bits = s.e.y;
            const f32 ax = __builtin_bit_cast(f32, ax_bits), bx = __builtin_bit_cast(f32, bx_bits);
            typename RZ::Taps tp;
            tp.w00 = ax * ay; tp.w10 = bx * ay; tp.w01 = ax * by; tp.w11 = bx * by;
            Raw a, b, c, d;
            if constexpr (CLAMP) {
                const bool clamped = (s.e.w & kClamped) != 0u;
                Back::pair_values_dup(s.ab, clamped, a, b);
                Back::pair_values_dup(s.cd, clamped, c, d);
            } else {
                Back::pair_values(s.ab, typename Back::TapRow{}, 0, a, b);
                Back::pair_values(s.cd, typename Back::TapRow{}, 0, c, d);
            }
            typename RZ::Out v = RZ::blend(Back::finish(a, q.back), Back::finish(b, q.back),
                                           Back::finish(c, q.back), Back::finish(d, q.back), tp);
            if constexpr (RZ::kAR != IGNORE_AR) { if (!yin || (s.e.w & kOutsideX)) v = q.bg; }
            typename Chain::Value res;
            if constexpr (STATIC) res = Chain::compute_static_ops(v, ops);
            else res = Chain::compute_checked_ops(v, ops);
            u32 off = out0 + u32(k) * WP::lane_offset(kStripStep, true);
            if (partial && k == steps - 1) {                          // wave uniform, kept a branch
                asm volatile("" : "+v"(off));
                if (g + kStripStep * k >= aw) off = WP::kMaskedOut;
            }
            WP::put_masked(oplane, 0u, off, res);
        };
        // One step of taps is in flight behind the step being blended.  The steps are written out (a plane has at most
        // kStripMaxSteps of them) and the only branches leave the kernel: every step issues the same accesses in the same
        // order, so the compiler's wait for a step's taps leaves all later accesses in flight, table reads carry their step
        // in the instruction's immediate offset, and there is no loop bookkeeping.  The request behind the last step meets
        // a column without a window.
        StepTaps sa = first, sb;
        request(1, sb);
#pragma unroll
        for (int k = 0; k < kStripMaxSteps; k += 2) {
            if (k > 0) request(k + 1, sb);
            produce(k, sa);
            if (k + 1 >= steps) return;
            if (k + 2 < kStripMaxSteps) request(k + 2, sa);
            produce(k + 1, sb);
            if (k + 2 >= steps) return;
        }
    };
    auto run_static = [&](auto static_tag) {
        if (some_clamped) run(static_tag, IntTag<1>{});
        else run(static_tag, IntTag<0>{});
    };
    if constexpr (Chain::kQuick) {
        if (Chain::ops_static(ops)) { run_static(IntTag<1>{}); return; }
    }
    run_static(IntTag<0>{});
}

template <class Chain>
__global__ __launch_bounds__(kStripThreads) void k_strip(const typename Chain::Params p, const u32 first_late_workgroup) {
    if constexpr (strip_capable<Chain>()) strip_body<Chain>(p, first_late_workgroup);
}

template <class Chain, int XI, int YI>
__global__ __launch_bounds__(kGatherBX * kGatherBY) void k_gather(const typename Chain::Params p, const TileGeom g) {
    gather_body<Chain, XI, YI>(p, g);
}

// ---- per-chain constants shared by the ahead-of-time and the run-time launchers ---------------------------

template <class Chain> struct RowsConfig {
    // Four elements per thread; a bilinear resize without a tap cursor keeps one element per thread.  (Warps take four
    // as well: their taps are gathers either way, and four float3 results per lane leave as dense wave-wide stores:
    // 1080p 9.06 -> 8.83 us, 2160p in bands 27.1 -> 25.1 us.)
    static constexpr bool kScattered = ResizeRoot<typename Chain::Read>::value;
#ifndef FKD_ROWS
#define FKD_ROWS 2
#endif
#ifndef FKD_SCATTER_V
#define FKD_SCATTER_V 1
#endif
#ifndef FKD_SCATTER_ROWS
#define FKD_SCATTER_ROWS 1
#endif
    static constexpr int V = kScattered ? FKD_SCATTER_V : 4;
    // Two rows per thread; chains long enough to be bound by instruction issue rather than by memory (more than 128
    // bytes of operation parameters) take four, for the independent work per thread.
    static constexpr bool kManyOps = sizeof(typename Chain::Params) - sizeof(typename Chain::Read::Params) - sizeof(typename Chain::Write::Params) > 128 + 16;
#ifndef FKD_ROWS_MANY
#define FKD_ROWS_MANY (2 * FKD_ROWS)
#endif
    static constexpr int ROWS = (kScattered || is_scattered_read<typename Chain::Read>()) ? FKD_SCATTER_ROWS : (kManyOps ? FKD_ROWS_MANY : FKD_ROWS);
};

// ---- divergent batch kernel -------------------------------------------------------------------------------

// Several chains in one launch of the rows kernel's geometry: plane z runs chain select[z] (wave uniform: the plane is
// the grid's z index).  Every chain runs through the rows body, bilinear reads included, all with the same elements per
// thread; workgroups beyond a chain's own extent leave at once.
template <class... Chains> struct RowsConfig<Divergent<Chains...>> {
    // One geometry for every chain of the launch, gathering reads included (they then take their elements one after
    // the other): with the grid laid out for the finest chain, the planes of the coarser ones launched up to 16 times
    // the workgroups they needed, and those empty workgroups cost 4 us of a 31 us launch.
    static constexpr int V = 4;
    static constexpr int ROWS = FKD_ROWS;
};
template <int I, class First, class... Rest, class P>
__device__ __forceinline__ void divergent_run(u32 sel, const P& p, const Tup<typename First::Params, typename Rest::Params...>& seq) {
    if (sel == u32(I)) {
        const u32 offset = u32(reinterpret_cast<const char*>(&seq.head) - reinterpret_cast<const char*>(&p));
        rows_auto_body<First, 4, FKD_ROWS>(seq.head, offset);
    } else if constexpr (sizeof...(Rest) > 0) {
        divergent_run<I + 1, Rest...>(sel, p, seq.tail);
    }
}
template <class D> struct DivergentBody;
template <class... Chains> struct DivergentBody<Divergent<Chains...>> {
    __device__ __forceinline__ static void run(const typename Divergent<Chains...>::Params& p) {
        using D = Divergent<Chains...>;
        const u32 z = blockIdx.z < u32(D::kMaxPlanes) ? blockIdx.z : 0u;
        // The table entry is fetched from the kernel-argument segment itself (the parameter block is the kernel's first
        // argument): indexing the by-value copy with a run-time index would make the compiler keep that copy in
        // scratch memory, for every lane.
        const FKD_CONSTANT u32* words = (const FKD_CONSTANT u32*)__builtin_amdgcn_kernarg_segment_ptr();
        const u32 at = u32(__builtin_offsetof(typename D::Params, select)) + z;
        const u32 sel = __builtin_amdgcn_readfirstlane((words[at / 4u] >> ((at & 3u) * 8u)) & 0xffu);
        divergent_run<0, Chains...>(sel, p, p.seq);
    }
};
template <class D> __global__ __launch_bounds__(kRowsBX * kRowsBY) void k_divergent(const typename D::Params p) {
    DivergentBody<D>::run(p);
}

// The one kernel of a chain compiled at run time, and what its launcher needs to know about it.  A launcher that
// only has the parameter block as bytes reads the active grid from its first three words.
// (JitMeta: fkd/launch_info.hpp)
template <class Chain> constexpr JitMeta jit_meta() {
    if constexpr (IsDivergent<Chain>::value)
        return JitMeta{0u, u32(sizeof(typename Chain::Params)), u32(RowsConfig<Chain>::V), u32(RowsConfig<Chain>::ROWS), 0u, 0u, 0u, u32(Chain::kMaxPlanes), 0u, 0u};
    else
        return JitMeta{is_gather_chain<Chain>() ? 1u : 0u, u32(sizeof(typename Chain::Params)), u32(RowsConfig<Chain>::V),
                       u32(RowsConfig<Chain>::ROWS), u32(FKD_GATHER_XI), u32(FKD_GATHER_YI), u32(kGatherBY), 0u,
                       is_gather_chain<Chain>() && strip_capable<Chain>() ? u32(kStripMaxWidth) : 0u,
                       !is_gather_chain<Chain>() && rows_in_bands<Chain>() ? 1u : 0u};
}
template <class Chain> __device__ __forceinline__ void jit_body(const typename Chain::Params& p, const TileGeom& g) {
    if constexpr (IsDivergent<Chain>::value) DivergentBody<Chain>::run(p);
    else if constexpr (is_gather_chain<Chain>()) {
        if constexpr (strip_capable<Chain>()) {
            if (g.tiles_x == 0u) { strip_body<Chain>(p, g.n_tiles); return; }      // wave uniform: the launcher chose the strip form
        }
        gather_body<Chain, FKD_GATHER_XI, FKD_GATHER_YI>(p, g);
    }
    else rows_auto_body<Chain, RowsConfig<Chain>::V, RowsConfig<Chain>::ROWS, rows_in_bands<Chain>()>(p, 0u, &g);
}

} // namespace fkd

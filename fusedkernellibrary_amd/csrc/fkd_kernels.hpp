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
//  staged kernel  for chains whose read is a bilinear resize: a workgroup owns a TW x TH tile of the output of
//                 one plane, first copies the source rectangle its taps fall in into LDS (replicating the last
//                 column/row once, which reproduces the reference's clamp of the +1 taps), then interpolates
//                 out of LDS.  Source pixels are staged raw (as they lie in memory, one dword per uchar3) and
//                 whatever was fused into the read (colour conversion, per-plane arithmetic) is applied per tap,
//                 in the reference's order.  Workgroups are renumbered so each XCD works on a contiguous run of
//                 tiles and planes and its L2 sees one set of crops.
//
// Reference being replaced: TransformDPP<GPU_NVIDIA>::exec and launchTransformDPP_Kernel,
// FK/core/execution_model/data_parallel_patterns.h:223-242 and executor_details/executor_kernels.h:26-30;
// launch geometry FK/core/execution_model/executors.h:242-351.
#pragma once

#include <hip/hip_runtime.h>

#include <fkd/launch_info.hpp>
#include <fkd/ops.hpp>

namespace fkd {

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

template <class Chain> constexpr bool is_staged_chain() {
    if constexpr (ResizeRoot<typename Chain::Read>::value)
        return ResizeRoot<typename Chain::Read>::Resize::BackOp::kStageable;
    else
        return false;
}

// ---- rows kernel ---------------------------------------------------------------------------------------

constexpr int kRowsBX = 64;   // lanes along x: one wave per row segment
constexpr int kRowsBY = 4;    // waves per workgroup

template <class Chain, int V, int ROWS, bool ALIGNED>
__global__ __launch_bounds__(kRowsBX * kRowsBY) void k_rows(const typename Chain::Params p) {
    using R = typename Chain::Read;
    using W = typename Chain::Write;
    const int z = blockIdx.z;
    const int x0 = (blockIdx.x * kRowsBX + threadIdx.x) * V;
    const int ybase = (blockIdx.y * kRowsBY + threadIdx.y) * ROWS;
    const int aw = int(p.active_w), ah = int(p.active_h);
    if (x0 >= aw || ybase >= ah) return;
    if (x0 + V <= aw) {
        // All loads first, unconditionally (rows past the end re-read the last row, which is in bounds), so every
        // lane has ROWS independent wide loads in flight before the first use; only the stores are predicated.
        Slot<typename R::Out> in[ROWS][V];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int y = ybase + r < ah ? ybase + r : ah - 1;
            R::template exec_row<V, ALIGNED>(x0, y, z, p.read, in[r]);
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int y = ybase + r;
            Slot<typename Chain::Value> out[V];
#pragma unroll
            for (int i = 0; i < V; ++i) out[i].v = Chain::compute(in[r][i].v, p);
            if (y < ah) W::template exec_row<V, ALIGNED>(x0, y, z, out, p.write);
        }
    } else {
        for (int r = 0; r < ROWS; ++r) {
            const int y = ybase + r;
            if (y >= ah) break;
            for (int x = x0; x < aw; ++x) W::exec(x, y, z, Chain::compute(R::exec(x, y, z, p.read), p), p.write);
        }
    }
}

// ---- staged (LDS) bilinear kernel ----------------------------------------------------------------------

// One staged source element in LDS: whole dwords, so a tap is one ds_read_b32 (uchar3, uchar, uchar4), b64 or b96.
template <class Raw> struct LdsSlot {
    static constexpr int kWords = (int(sizeof(Raw)) + 3) / 4;
    u32 w[kWords];
};
template <class Raw> FKD_DEV LdsSlot<Raw> lds_pack(const Raw& r) {
    LdsSlot<Raw> s;
    if constexpr (sizeof(base_t<Raw>) < 4 && sizeof(Raw) <= 4) {
        // sub-dword element: assemble the dword in registers (bytes beyond the element are zero)
        u32 word = 0;
        if constexpr (sizeof(base_t<Raw>) == 1) {
            word = detail::to_bits(chan<0>(r));
            if constexpr (cn_v<Raw> > 1) word |= detail::to_bits(chan<1>(r)) << 8;
            if constexpr (cn_v<Raw> > 2) word |= detail::to_bits(chan<2>(r)) << 16;
            if constexpr (cn_v<Raw> > 3) word |= detail::to_bits(chan<3>(r)) << 24;
        } else {
            word = detail::to_bits(chan<0>(r));
            if constexpr (cn_v<Raw> > 1) word |= detail::to_bits(chan<1>(r)) << 16;
        }
        s.w[0] = word;
    } else {
#pragma unroll
        for (int i = 0; i < LdsSlot<Raw>::kWords; ++i) s.w[i] = 0;
        __builtin_memcpy(&s, &r, sizeof(Raw));
    }
    return s;
}
template <class Raw> FKD_DEV Raw lds_unpack(const LdsSlot<Raw>& s) {
    if constexpr (sizeof(base_t<Raw>) < 4 && sizeof(Raw) <= 4) {
        u32 w[1] = {s.w[0]};
        asm("" : "+v"(w[0]));   // keep the dword whole: one ds_read_b32, bytes come out with v_cvt_f32_ubyteN / v_bfe
        return detail::unpack_one<0, Raw>(w);
    } else {
        Raw r;
        __builtin_memcpy(&r, &s, sizeof(Raw));
        return r;
    }
}

#ifndef FKD_STAGED_XI
#define FKD_STAGED_XI 2
#endif
#ifndef FKD_STAGED_YI
#define FKD_STAGED_YI 2
#endif
constexpr int kStagedBX = 64;
constexpr int kStagedBY = 4;

struct StagedGeom {
    u32 tiles_x, tiles_y, n_tiles, lds_slots;
};

// XI, YI: outputs per thread along x (stride 64) and y (stride 4): tile = 64*XI by 4*YI outputs.
template <class Chain, int XI, int YI>
__global__ __launch_bounds__(kStagedBX * kStagedBY) void k_staged(const typename Chain::Params p, const StagedGeom g) {
    using Root = ResizeRoot<typename Chain::Read>;
    using RZ = typename Root::Resize;
    using Back = typename RZ::BackOp;
    using Raw = typename Back::Raw;
    using Slot = LdsSlot<Raw>;
    using W = typename Chain::Write;
    constexpr int TW = kStagedBX * XI, TH = kStagedBY * YI;
    extern __shared__ u32 lds_words[];
    Slot* lds = reinterpret_cast<Slot*>(lds_words);

    // Renumber workgroups: hardware deals consecutive workgroup ids round-robin to the 8 XCDs; give XCD k the
    // k-th contiguous eighth of the tile list so neighbouring tiles (which share source rows) share an L2.
    const u32 chunk = (g.n_tiles + 7u) / 8u;
    const u32 t = (blockIdx.x % 8u) * chunk + blockIdx.x / 8u;
    if (t >= g.n_tiles || blockIdx.x / 8u >= chunk) return;
    const u32 per_plane = g.tiles_x * g.tiles_y;
    const int z = int(t / per_plane);
    const u32 tin = t % per_plane;
    const int tx0 = int(tin % g.tiles_x) * TW;
    const int ty0 = int(tin / g.tiles_x) * TH;

    const typename RZ::Params* rp;
    if constexpr (Root::batched) rp = &p.read.plane[z]; else rp = &p.read;
    const typename RZ::Params& q = *rp;
    const int aw = int(p.active_w), ah = int(p.active_h);

    // Output range of this tile that actually interpolates (inside the letterbox), relative to its origin.
    int ox = 0, oy = 0, lx2 = aw - 1, ly2 = ah - 1;
    if constexpr (RZ::kAR != IGNORE_AR) { ox = q.x1; oy = q.y1; lx2 = q.x2 < lx2 ? q.x2 : lx2; ly2 = q.y2 < ly2 ? q.y2 : ly2; }
    const int xs = (tx0 > ox ? tx0 : ox) - ox;
    const int ys = (ty0 > oy ? ty0 : oy) - oy;
    const int xe = (tx0 + TW - 1 < lx2 ? tx0 + TW - 1 : lx2) - ox;
    const int ye = (ty0 + TH - 1 < ly2 ? ty0 + TH - 1 : ly2) - oy;
    const int sw = Back::width(q.back), sh = Back::height(q.back);

    int fx0 = 0, fy0 = 0, fw = 0, fh = 0;
    bool staged = false;
    if (xs <= xe && ys <= ye) {
        fx0 = int(__builtin_floorf(f32(xs) * q.fx));
        fy0 = int(__builtin_floorf(f32(ys) * q.fy));
        fw = int(__builtin_floorf(f32(xe) * q.fx)) + 1 - fx0 + 1;
        fh = int(__builtin_floorf(f32(ye) * q.fy)) + 1 - fy0 + 1;
        staged = fx0 >= 0 && fy0 >= 0 && fw > 0 && fh > 0 && u32(fw) * u32(fh) <= g.lds_slots;
        if (staged) {
            // RU x CU raw elements per thread and step: all their loads are issued before the first LDS write.
            // Coordinates are clamped into the source, so even the predicated-off positions load in bounds.
            constexpr int RU = 2, CU = 2;
            for (int r0 = threadIdx.y; r0 < fh; r0 += kStagedBY * RU) {
                typename Back::RawRow rows[RU];
#pragma unroll
                for (int i = 0; i < RU; ++i) {
                    const int r = r0 + kStagedBY * i;
                    rows[i] = Back::raw_row(fy0 + r < sh - 1 ? fy0 + r : sh - 1, z, q.back);
                }
                for (int c0 = threadIdx.x; c0 < fw; c0 += kStagedBX * CU) {
                    Raw v[RU][CU];
#pragma unroll
                    for (int j = 0; j < CU; ++j) {
                        const int c = c0 + kStagedBX * j;
                        const int sx = fx0 + c < sw - 1 ? fx0 + c : sw - 1;
#pragma unroll
                        for (int i = 0; i < RU; ++i) v[i][j] = Back::raw_at(rows[i], sx, q.back);
                    }
#pragma unroll
                    for (int i = 0; i < RU; ++i) {
                        const int r = r0 + kStagedBY * i;
#pragma unroll
                        for (int j = 0; j < CU; ++j) {
                            const int c = c0 + kStagedBX * j;
                            if (r < fh && c < fw) lds[r * fw + c] = lds_pack<Raw>(v[i][j]);
                        }
                    }
                }
            }
        }
    }
    __syncthreads();

    // Interpolation.  Everything that depends on the row only (source y, vertical weights, LDS row, output row
    // address) is formed once per row; per pixel remain the horizontal coordinate, four weights, four LDS reads,
    // the blend, the chain's compute operations and the store.  float(x1) and float(x1 + 1) are taken as floor(sx)
    // and floor(sx) + 1, which are the same numbers (exact integers below 2^24).
#pragma unroll
    for (int j = 0; j < YI; ++j) {
        const int y = ty0 + int(threadIdx.y) + kStagedBY * j;
        if (y >= ah) continue;
        const typename W::RowRef orow = W::row(y, z, p.write);
        bool yin = true;
        if constexpr (RZ::kAR != IGNORE_AR) yin = y >= q.y1 && y <= q.y2;
        const f32 sy = f32(y - oy) * q.fy;
        const f32 fy1 = __builtin_floorf(sy);
        const f32 ay = (fy1 + 1.0f) - sy, by = sy - fy1;
        const int y1 = int(fy1);
        const Slot* lrow0 = lds + (y1 - fy0) * fw - fx0;
        const Slot* lrow1 = lrow0 + fw;
#pragma unroll
        for (int i = 0; i < XI; ++i) {
            const int x = tx0 + int(threadIdx.x) + kStagedBX * i;
            if (x >= aw) continue;
            typename RZ::Out v;
            bool in = yin;
            if constexpr (RZ::kAR != IGNORE_AR) in = in && x >= q.x1 && x <= q.x2;
            if (!in) {
                v = q.bg;
            } else if (!staged) {
                v = RZ::exec(x, y, z, q);
            } else {
                const f32 sx = f32(x - ox) * q.fx;
                const f32 fx1 = __builtin_floorf(sx);
                const f32 ax = (fx1 + 1.0f) - sx, bx = sx - fx1;
                const int x1 = int(fx1);
                typename RZ::Taps tp;
                tp.w00 = ax * ay; tp.w10 = bx * ay; tp.w01 = ax * by; tp.w11 = bx * by;
                // Unclamped +1 taps: the staged rectangle carries one replicated column/row past the edge.
                const auto a = Back::finish(lds_unpack<Raw>(lrow0[x1]), q.back);
                const auto b = Back::finish(lds_unpack<Raw>(lrow0[x1 + 1]), q.back);
                const auto c = Back::finish(lds_unpack<Raw>(lrow1[x1]), q.back);
                const auto d = Back::finish(lds_unpack<Raw>(lrow1[x1 + 1]), q.back);
                v = RZ::blend(a, b, c, d, tp);
            }
            W::put(orow, x, Chain::compute(v, p));
        }
    }
}

// ---- host-side launchers -------------------------------------------------------------------------------

template <class Chain> struct RowsConfig {
    // Four elements per thread wherever the chain reads rows; a bilinear read that cannot be staged keeps one
    // element per thread (its taps are gathers, wider threads would only spread them further apart).
    static constexpr int V = ResizeRoot<typename Chain::Read>::value ? 1 : 4;
#ifndef FKD_ROWS
#define FKD_ROWS 4
#endif
    static constexpr int ROWS = ResizeRoot<typename Chain::Read>::value ? 1 : FKD_ROWS;
};

inline const char* aligned_name(bool aligned) { return aligned ? "rows" : "rows_unaligned"; }

template <class Chain>
hipError_t launch_rows(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info) {
    constexpr int V = RowsConfig<Chain>::V, ROWS = RowsConfig<Chain>::ROWS;
    const unsigned gx = (p.active_w + kRowsBX * V - 1) / (kRowsBX * V);
    const unsigned gy = (p.active_h + kRowsBY * ROWS - 1) / (kRowsBY * ROWS);
    const dim3 grid(gx, gy, p.active_z), block(kRowsBX, kRowsBY, 1);
    // Wide (dwordx3/x4) accesses need every row start dword aligned; checked here, once per launch, on the host.
    const bool aligned = Chain::Read::rows_aligned(p.read, 0) && Chain::Write::rows_aligned(p.write);
    if (info) *info = LaunchInfo{aligned_name(aligned), {grid.x, grid.y, grid.z}, {block.x, block.y, 1}, 0};
    if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;
    if (grid.y > 65535u || grid.z > 65535u) return hipErrorInvalidConfiguration;
    if (aligned) hipLaunchKernelGGL((k_rows<Chain, V, ROWS, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((k_rows<Chain, V, ROWS, false>), grid, block, 0, stream, p);
    return hipGetLastError();
}

template <class RZParams> inline void staged_need(const RZParams& q, int tw, int th, unsigned& slots) {
    // Upper bound of the staged rectangle of any tile of this plane (two extra columns/rows: the +1 tap and
    // float rounding of the two floor() calls).
    const long long fw = (long long)__builtin_ceilf(float(tw - 1) * q.fx) + 3;
    const long long fh = (long long)__builtin_ceilf(float(th - 1) * q.fy) + 3;
    const long long n = fw * fh;
    if (n > (long long)slots) slots = n > 0x7fffffffLL ? 0x7fffffffu : unsigned(n);
}

constexpr unsigned kStagedLdsBudget = 64u * 1024u;

template <class Chain>
hipError_t launch_staged(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info) {
    using Root = ResizeRoot<typename Chain::Read>;
    using Slot = LdsSlot<typename Root::Resize::BackOp::Raw>;
    constexpr int XI = FKD_STAGED_XI, YI = FKD_STAGED_YI;
    constexpr int TW = kStagedBX * XI, TH = kStagedBY * YI;
    unsigned slots = 0;
    if constexpr (Root::batched) {
        for (unsigned z = 0; z < p.active_z && z < unsigned(Root::batched ? Chain::Read::kBatch : 1); ++z)
            staged_need(p.read.plane[z], TW, TH, slots);
    } else {
        staged_need(p.read, TW, TH, slots);
    }
    const unsigned long long bytes = (unsigned long long)slots * sizeof(Slot);
    if (bytes > kStagedLdsBudget) return launch_rows<Chain>(p, stream, info);   // very strong downscale
    StagedGeom g;
    g.tiles_x = (p.active_w + TW - 1) / TW;
    g.tiles_y = (p.active_h + TH - 1) / TH;
    g.n_tiles = g.tiles_x * g.tiles_y * p.active_z;
    g.lds_slots = slots;
    const unsigned chunk = (g.n_tiles + 7u) / 8u;
    const dim3 grid(chunk * 8u, 1, 1), block(kStagedBX, kStagedBY, 1);
    if (info) *info = LaunchInfo{"staged", {grid.x, 1, 1}, {block.x, block.y, 1}, unsigned(bytes)};
    if (g.n_tiles == 0) return hipSuccess;
    hipLaunchKernelGGL((k_staged<Chain, XI, YI>), grid, block, unsigned(bytes), stream, p, g);
    return hipGetLastError();
}

template <class Chain>
hipError_t launch_chain(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info) {
    if constexpr (is_staged_chain<Chain>()) return launch_staged<Chain>(p, stream, info);
    else return launch_rows<Chain>(p, stream, info);
}

} // namespace fkd

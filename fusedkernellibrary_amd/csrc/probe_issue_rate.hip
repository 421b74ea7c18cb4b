// probe_issue_rate.hip -- stand-alone measurement of instruction issue on gfx950, the figures the gather kernel's
// floor is priced with.  No image, no library: registers only, bounded loops, one guarded store per lane.
//
//   1. the interval at which ONE wave can issue vector instructions (independent ones, and a dependent chain);
//   2. cycles per instruction per SIMD with 8 waves on every SIMD of the chip, for the instruction kinds the bilinear
//      pixel body is made of, and for scalar instructions beside them;
//   3. the bilinear pixel body itself -- window alignment, byte -> float, weights, the four-term blend of three
//      channels, (x - mean) / std in its two-instruction form, exactly the code the kernel runs (fkd::ResizeLinear::blend,
//      fkd::Div::exec_static) on register data -- as cycles per wave-wide pixel per SIMD.
//
// Build: hipcc --offload-arch=gfx950 with the library's flags (fusedkernellibrary_amd/build.py builds it as
// fusedkernellibrary_amd/probe_issue_rate); run: `python3 bench.py --issue-rate`.
#define FKD_DEVICE_CODE 1
#define FKD_NO_NAMES 1
#include <hip/hip_runtime.h>
#include <fkd/ops.hpp>

#include <cstdio>
#include <cstring>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("ERR %s at line %d: %s\n", #x, __LINE__, hipGetErrorString(e_)); fflush(stdout); return 1; } } while (0)

using fkd::u32;
using fkd::f32;

enum Kind { kMul, kCvt, kAlign, kMulSgpr, kFma, kSAdd, kMulCvt, kMulSAdd, kMulSAdd2, kDependent };

#define OP16(STR) _Pragma("unroll") for (int i = 0; i < 16; ++i) asm volatile(STR : "+v"(a[i]) : "v"(b), "v"(c), "s"(sb))
#define SOP(STR, k) asm volatile(STR : "+s"(s[(k) & 7]) : : "scc")

template <int KIND> __global__ __launch_bounds__(1024) void k_rate(u32* out, int iters, u32 binit, u32 cinit, u32 ainit, unsigned long long* clk) {
    u32 a[16], s[8];
    u32 b = binit, c = cinit;
    const u32 sb = __builtin_amdgcn_readfirstlane(binit);
    for (int i = 0; i < 16; ++i) a[i] = ainit + u32(i) * 0x00010000u + (threadIdx.x & 3u);
    for (int i = 0; i < 8; ++i) s[i] = __builtin_amdgcn_readfirstlane(binit + u32(i));
    __syncthreads();
    const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
        if constexpr (KIND == kMul) { OP16("v_mul_f32_e32 %0, %0, %1"); }
        if constexpr (KIND == kCvt) { OP16("v_cvt_f32_ubyte0_e32 %0, %0"); }
        if constexpr (KIND == kAlign) { OP16("v_alignbyte_b32 %0, %0, %1, %2"); }
        if constexpr (KIND == kMulSgpr) { OP16("v_mul_f32_e32 %0, %3, %0"); }
        if constexpr (KIND == kFma) { OP16("v_fma_f32 %0, %0, %1, %2"); }
        if constexpr (KIND == kSAdd) {
#pragma unroll
            for (int i = 0; i < 16; ++i) SOP("s_add_u32 %0, %0, 3", i);
        }
        if constexpr (KIND == kMulCvt) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                asm volatile("v_mul_f32_e32 %0, %0, %1" : "+v"(a[i]) : "v"(b));
                asm volatile("v_cvt_f32_ubyte0_e32 %0, %0" : "+v"(a[8 + i]));
            }
        }
        if constexpr (KIND == kMulSAdd || KIND == kMulSAdd2) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                asm volatile("v_mul_f32_e32 %0, %0, %1" : "+v"(a[i]) : "v"(b));
                SOP("s_add_u32 %0, %0, 3", i);
                if constexpr (KIND == kMulSAdd2) SOP("s_mul_i32 %0, %0, 5", i + 3);
            }
        }
        if constexpr (KIND == kDependent) {
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("v_mul_f32_e32 %0, %0, %1" : "+v"(a[0]) : "v"(b));
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    u32 r = 0;
    for (int i = 0; i < 16; ++i) r += a[i];
    for (int i = 0; i < 8; ++i) r += s[i];
    if (r == 0x12345678u) out[threadIdx.x] = r;
    if (blockIdx.x == 0 && (threadIdx.x & 63u) == 0) { clk[2 * (threadIdx.x / 64)] = t1 - t0; clk[2 * (threadIdx.x / 64) + 1] = w1 - w0; }
}

// The pixel body of configuration 3 on register data.  Four wave-wide pixels per trip (what one wave of the kernel
// produces); the windows of the next trip are derived from this trip's results so nothing can be hoisted.
using Px = fkd::Vec<fkd::u8, 3>;
using Out3 = fkd::Vec<f32, 3>;
using RZ = fkd::ResizeLinear<1, fkd::Crop<fkd::Read2D<Px>>>;
using DivOp = fkd::Div<Out3, Out3, Out3>;
using SubOp = fkd::Sub<Out3, Out3, Out3>;
using Swap = fkd::Reorder<Out3, 2, 1, 0, 3>;

__global__ __launch_bounds__(256) void k_pixel(u32* out, int iters, u32 seed, f32 ax, f32 ay, SubOp::Params sub, DivOp::Params div, unsigned long long* clk) {
    fkd::detail::PairWindow<Px> top[4], bot[4];
    for (int i = 0; i < 4; ++i) {
        for (int k = 0; k < 3; ++k) { top[i].w[k] = seed * (threadIdx.x + 1u) + u32(7 * i + k); bot[i].w[k] = top[i].w[k] ^ 0x5a5a5a5au; }
        top[i].shift = bot[i].shift = (threadIdx.x + u32(i)) & 3u;
    }
    f32 axs[4], bxs[4];
    for (int i = 0; i < 4; ++i) { axs[i] = ax + f32(threadIdx.x & 7u) * 0x1p-6f; bxs[i] = 1.0f - axs[i]; }
    const f32 by = 1.0f - ay;
    u32 acc = 0;
    const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            Px a, b, c, d;
            fkd::detail::pair_window_values(top[i], a, b);
            fkd::detail::pair_window_values(bot[i], c, d);
            RZ::Taps tp;
            tp.w00 = axs[i] * ay; tp.w10 = bxs[i] * ay; tp.w01 = axs[i] * by; tp.w11 = bxs[i] * by;
            Out3 v = RZ::blend(a, b, c, d, tp);
            v = Swap::exec(v, fkd::Empty{});
            v = SubOp::exec(v, sub);
            v = DivOp::exec_static(v, div);
            const u32 bits = __builtin_bit_cast(u32, fkd::chan<0>(v)) ^ __builtin_bit_cast(u32, fkd::chan<1>(v)) ^ __builtin_bit_cast(u32, fkd::chan<2>(v));
            acc ^= bits;
            top[i].w[0] ^= bits; bot[i].w[1] ^= bits;      // 3 of the body's instructions: the loop-carried dependence
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    if (acc == 0x12345678u) out[threadIdx.x] = acc;
    if (blockIdx.x == 0 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = w1 - w0; }
}

static int simds() {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) != hipSuccess) return 1024;
    return p.multiProcessorCount * 4;
}

template <int KIND> int chip(const char* name, int slots_per_trip, u32 binit, u32 cinit, u32 ainit) {
    u32* out; unsigned long long* clk;
    CK(hipMalloc(&out, 4096)); CK(hipMalloc(&clk, 512));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int iters = 2000, waves_per_simd = 8, blocks = simds() / 4 * waves_per_simd / 4;     // 1024 threads: 4 waves per SIMD of one CU
    for (int rep = 0; rep < 2; ++rep) hipLaunchKernelGGL(k_rate<KIND>, dim3(blocks), dim3(1024), 0, 0, out, iters, binit, cinit, ainit, clk);
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(k_rate<KIND>, dim3(blocks), dim3(1024), 0, 0, out, iters, binit, cinit, ainit, clk);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    unsigned long long h[2]; CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
    const double mhz = double(h[0]) / (double(h[1]) / 100.0);
    const double cycles = double(ms) * 1e-3 * mhz * 1e6 / (double(waves_per_simd) * iters * slots_per_trip);
    printf("  %-58s %8.1f us  %5.0f MHz  %6.2f cycles per %s per SIMD\n", name, ms * 1e3, mhz, cycles, slots_per_trip == 16 ? "instruction (slot)" : "slot");
    fflush(stdout);
    (void)hipFree(out); (void)hipFree(clk);
    return 0;
}

template <int KIND> int one_workgroup(const char* name, int threads) {
    u32* out; unsigned long long* clk;
    CK(hipMalloc(&out, 4096)); CK(hipMalloc(&clk, 512)); CK(hipMemset(clk, 0, 512));
    const int iters = 4000;
    for (int rep = 0; rep < 2; ++rep) hipLaunchKernelGGL(k_rate<KIND>, dim3(1), dim3(threads), 0, 0, out, iters, 0x3f800347u, 0u, 0x3f900000u, clk);
    CK(hipDeviceSynchronize());
    unsigned long long h[32]; CK(hipMemcpy(h, clk, sizeof(h), hipMemcpyDeviceToHost));
    printf("  %-34s %2d wave(s) on one CU: cycles per instruction seen by each wave:", name, threads / 64);
    for (int w = 0; w < threads / 64; ++w) printf(" %.2f", double(h[2 * w]) / (iters * 16.0));
    printf("\n"); fflush(stdout);
    (void)hipFree(out); (void)hipFree(clk);
    return 0;
}

int pixel_body() {
    u32* out; unsigned long long* clk;
    CK(hipMalloc(&out, 4096)); CK(hipMalloc(&clk, 64));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    SubOp::Params sub; DivOp::Params div;
    memset(&sub, 0, sizeof(sub)); memset(&div, 0, sizeof(div));
    const f32 mean[3] = {0.485f * 255.f, 0.456f * 255.f, 0.406f * 255.f}, stdv[3] = {0.229f * 255.f, 0.224f * 255.f, 0.225f * 255.f};
    f32 rcp[3], lo[3];
    for (int c = 0; c < 3; ++c) { rcp[c] = f32(1.0 / double(stdv[c])); lo[c] = f32((1.0 - double(stdv[c]) * double(rcp[c])) / double(stdv[c])); }
    memcpy(&sub.v, mean, sizeof(mean)); memcpy(&div.v, stdv, sizeof(stdv)); memcpy(&div.rcp, rcp, sizeof(rcp)); memcpy(&div.rcp_lo, lo, sizeof(lo));
    const int iters = 1000, waves_per_simd = 8, blocks = simds() / 4 * waves_per_simd;        // 256 threads: one wave per SIMD of one CU
    for (int rep = 0; rep < 2; ++rep) hipLaunchKernelGGL(k_pixel, dim3(blocks), dim3(256), 0, 0, out, iters, 2654435761u, 0.375f, 0.625f, sub, div, clk);
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(k_pixel, dim3(blocks), dim3(256), 0, 0, out, iters, 2654435761u, 0.375f, 0.625f, sub, div, clk);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    unsigned long long h[2]; CK(hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost));
    const double mhz = double(h[0]) / (double(h[1]) / 100.0);
    const double per_pixel = double(ms) * 1e-3 * mhz * 1e6 / (double(waves_per_simd) * iters * 4.0);
    // configuration 3: 64 * 224 * 224 pixels = 50 176 wave-wide pixels, 49 per SIMD on 1024 SIMDs; the kernel's 128-pixel
    // tiles make that 56 per SIMD (one lane in eight idle)
    printf("  bilinear pixel body (align, 12 cvt, 4 weights, 12 mul, 9 add, 3 sub, 3 mul + 3 fma):\n"
           "      %.1f us for %d wave-wide pixels per SIMD at %.0f MHz: %.1f cycles per wave-wide pixel per SIMD\n"
           "      configuration 3 at this rate, arithmetic only: %.2f us for its 49 wave-wide pixels per SIMD, %.2f us for the 56 of 128-pixel tiles\n",
           ms * 1e3, waves_per_simd * iters * 4, mhz, per_pixel, 49.0 * per_pixel / mhz, 56.0 * per_pixel / mhz);
    fflush(stdout);
    (void)hipFree(out); (void)hipFree(clk);
    return 0;
}

int main() {
    hipDeviceProp_t p;
    CK(hipGetDeviceProperties(&p, 0));
    printf("device %s, %d compute units (%d SIMDs)\n", p.gcnArchName, p.multiProcessorCount, p.multiProcessorCount * 4);
    printf("1. one workgroup on one compute unit, v_mul_f32, 16 independent accumulators per lane (waves 0-3, 4-7, ... share SIMDs 0-3):\n");
    for (int threads : {64, 256, 512, 1024}) if (one_workgroup<kMul>("v_mul_f32 independent", threads)) return 1;
    if (one_workgroup<kDependent>("v_mul_f32 dependent chain", 64)) return 1;
    if (one_workgroup<kSAdd>("s_add_u32 independent", 64)) return 1;
    printf("2. whole chip, 8 waves per SIMD:\n");
    if (chip<kMul>("v_mul_f32 v, v, v", 16, 0x3f800347u, 0u, 0x3f900000u)) return 1;
    if (chip<kFma>("v_fma_f32 v, v, v, v", 16, 0x3f800347u, 0x3a000000u, 0x3f900000u)) return 1;
    if (chip<kCvt>("v_cvt_f32_ubyte0 v, v", 16, 0u, 0u, 0x40404040u)) return 1;
    if (chip<kAlign>("v_alignbyte_b32 v, v, v, v", 16, 0x01020304u, 1u, 0xdeadbeefu)) return 1;
    if (chip<kMulSgpr>("v_mul_f32 v, s, v (scalar-register operand)", 16, 0x3f800347u, 0u, 0x3f900000u)) return 1;
    if (chip<kMulCvt>("v_mul_f32 and v_cvt_f32_ubyte0 alternating", 16, 0x3f800347u, 0u, 0x3f900000u)) return 1;
    if (chip<kSAdd>("s_add_u32 s, s, 3", 16, 5u, 0u, 777u)) return 1;
    if (chip<kMulSAdd>("v_mul_f32 + s_add_u32 per slot", 16, 0x3f800347u, 0u, 0x3f900000u)) return 1;
    if (chip<kMulSAdd2>("v_mul_f32 + s_add_u32 + s_mul_i32 per slot", 16, 0x3f800347u, 0u, 0x3f900000u)) return 1;
    printf("3. the pixel body of the bilinear chain, whole chip, 8 waves per SIMD:\n");
    return pixel_body();
}

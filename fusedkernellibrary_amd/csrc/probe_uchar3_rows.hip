// probe_uchar3_rows.hip -- stand-alone measurement (not part of the library): how should 100 images of 1920 x 1080 uchar3
// pixels move through a pointwise chain (x * m + a, saturate to uchar3)?  Each form is timed as a plain copy and with the
// arithmetic, on 1.24 GB per launch, with the cache hints the library uses for launches of this size (non-temporal loads
// and stores).  Forms:
//   A  one dwordx3 per lane (four pixels), two rows per thread: what the rows kernel does
//   B  three dwordx4 per lane (sixteen pixels, 48 bytes): wide accesses, 32-byte gaps between the lanes of an instruction
//   C  dense dwordx4 accesses (lane i takes 16 bytes at k * 1024 + i * 16) and a wave-private LDS exchange that hands every
//      lane four 12-byte pixel groups: 16-byte accesses without gaps
//   F  a float4 copy of the same bytes (no notion of pixels): the ceiling for this amount of data
// Bounded work on fixed-size buffers; every kernel's indices are checked against the image size.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("ERR %s line %d: %s\n", #x, __LINE__, hipGetErrorString(e_)); fflush(stdout); exit(1); } } while (0)

constexpr int W = 1920, H = 1080, NB = 100, PITCH = W * 3;
constexpr size_t kImage = size_t(W) * H * 3;     // 6 220 800 bytes: a multiple of 3072
struct Plane { const uint8_t* src; uint8_t* dst; float m[3], a[3]; };
struct Params { Plane p[NB]; };
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x3 u32x3_a4 __attribute__((aligned(4)));

// twelve bytes = four pixels: copy, or x * m + a saturated (v_cvt_pk_u8_f32 rounds to nearest even and clamps to 0..255)
template <bool MATH> __device__ __forceinline__ void four_pixels(const uint32_t (&in)[3], uint32_t (&out)[3], const Plane& pl) {
    if constexpr (!MATH) { out[0] = in[0]; out[1] = in[1]; out[2] = in[2]; return; }
    out[0] = out[1] = out[2] = 0;
#pragma unroll
    for (int i = 0; i < 12; ++i) {
        const int c = i % 3;
        const float v = float((in[i / 4] >> (8 * (i % 4))) & 0xffu) * pl.m[c] + pl.a[c];
        out[i / 4] = __builtin_amdgcn_cvt_pk_u8_f32(v, i % 4, out[i / 4]);
    }
}
template <bool MATH> __global__ __launch_bounds__(256) void form_a(const Params P) {
    const Plane& pl = P.p[blockIdx.z];
    const int x0 = (blockIdx.x * 64 + threadIdx.x) * 4, y0 = (blockIdx.y * 4 + threadIdx.y) * 2;
    if (x0 >= W) return;
    u32x3 in[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) if (y0 + r < H) in[r] = __builtin_nontemporal_load((const u32x3_a4*)(pl.src + size_t(y0 + r) * PITCH + x0 * 3));
#pragma unroll
    for (int r = 0; r < 2; ++r) if (y0 + r < H) {
        const uint32_t i[3] = {in[r].x, in[r].y, in[r].z}; uint32_t o[3];
        four_pixels<MATH>(i, o, pl);
        u32x3 v; v.x = o[0]; v.y = o[1]; v.z = o[2];
        __builtin_nontemporal_store(v, (u32x3_a4*)(pl.dst + size_t(y0 + r) * PITCH + x0 * 3));
    }
}
template <bool MATH> __global__ __launch_bounds__(256) void form_b(const Params P) {
    const Plane& pl = P.p[blockIdx.y];
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= kImage / 48) return;
    const u32x4* s = (const u32x4*)(pl.src + i * 48);
    const u32x4 a = __builtin_nontemporal_load(s), b = __builtin_nontemporal_load(s + 1), c = __builtin_nontemporal_load(s + 2);
    const uint32_t in[12] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w, c.x, c.y, c.z, c.w};
    uint32_t out[12];
#pragma unroll
    for (int k = 0; k < 4; ++k) { const uint32_t ti[3] = {in[3 * k], in[3 * k + 1], in[3 * k + 2]}; uint32_t to[3]; four_pixels<MATH>(ti, to, pl); out[3 * k] = to[0]; out[3 * k + 1] = to[1]; out[3 * k + 2] = to[2]; }
    u32x4* d = (u32x4*)(pl.dst + i * 48);
    u32x4 o0, o1, o2;
    o0.x = out[0]; o0.y = out[1]; o0.z = out[2]; o0.w = out[3]; o1.x = out[4]; o1.y = out[5]; o1.z = out[6]; o1.w = out[7]; o2.x = out[8]; o2.y = out[9]; o2.z = out[10]; o2.w = out[11];
    __builtin_nontemporal_store(o0, d); __builtin_nontemporal_store(o1, d + 1); __builtin_nontemporal_store(o2, d + 2);
}
template <bool MATH> __global__ __launch_bounds__(256) void form_c(const Params P) {
    __shared__ uint32_t lds[4][768];
    const Plane& pl = P.p[blockIdx.y];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const size_t base = (size_t(blockIdx.x) * 4 + wave) * 3072;      // a wave moves 3072 bytes = 256 groups of four pixels
    if (base >= kImage) return;
    const u32x4* s = (const u32x4*)(pl.src + base);
    uint32_t* L = lds[wave];
#pragma unroll
    for (int k = 0; k < 3; ++k) *(u32x4*)&L[k * 256 + lane * 4] = __builtin_nontemporal_load(s + k * 64 + lane);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    uint32_t out[12];
#pragma unroll
    for (int k = 0; k < 4; ++k) { const uint32_t* g = &L[(k * 64 + lane) * 3]; const uint32_t ti[3] = {g[0], g[1], g[2]}; uint32_t to[3]; four_pixels<MATH>(ti, to, pl); out[3 * k] = to[0]; out[3 * k + 1] = to[1]; out[3 * k + 2] = to[2]; }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int k = 0; k < 4; ++k) { uint32_t* g = &L[(k * 64 + lane) * 3]; g[0] = out[3 * k]; g[1] = out[3 * k + 1]; g[2] = out[3 * k + 2]; }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    u32x4* d = (u32x4*)(pl.dst + base);
#pragma unroll
    for (int k = 0; k < 3; ++k) __builtin_nontemporal_store(*(u32x4*)&L[k * 256 + lane * 4], d + k * 64 + lane);
}
__global__ __launch_bounds__(256) void form_f(const Params P) {
    const Plane& pl = P.p[blockIdx.y];
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < kImage / 16) __builtin_nontemporal_store(__builtin_nontemporal_load((const u32x4*)pl.src + i), (u32x4*)pl.dst + i);
}

template <class F> float time_us(F launch) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int i = 0; i < 3; ++i) launch();
    CK(hipEventRecord(e0));
    for (int i = 0; i < 20; ++i) launch();
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms = 0; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError());
    CK(hipEventDestroy(e0)); CK(hipEventDestroy(e1));
    return ms * 1e3f / 20;
}
int main() {
    Params P;
    for (int i = 0; i < NB; ++i) {
        uint8_t *s, *d;
        CK(hipMalloc(&s, kImage)); CK(hipMalloc(&d, kImage)); CK(hipMemset(s, 17 + i, kImage));
        P.p[i].src = s; P.p[i].dst = d;
        for (int c = 0; c < 3; ++c) { P.p[i].m[c] = 0.5f + 0.01f * i + 0.1f * c; P.p[i].a[c] = -10.f + c; }
    }
    const double bytes = 2.0 * kImage * NB;
    auto line = [&](const char* name, float us) { printf("%-64s %7.1f us  %6.0f GB/s  %4.1f %% of 8 TB/s\n", name, us, bytes / us / 1e3, bytes / us / 1e3 / 80.0); fflush(stdout); };
    printf("100 x 1920 x 1080 uchar3, 1 244 160 000 bytes per launch, 20 launches back to back after 3 warm-up launches\n");
    line("F  float4 copy (ceiling)", time_us([&] { hipLaunchKernelGGL(form_f, dim3(unsigned(kImage / 16 / 256 + 1), NB), dim3(256), 0, 0, P); }));
    line("A  dwordx3 per lane, two rows per thread: copy", time_us([&] { hipLaunchKernelGGL(form_a<false>, dim3(8, 135, NB), dim3(64, 4), 0, 0, P); }));
    line("A  dwordx3 per lane, two rows per thread: x*m+a, saturate", time_us([&] { hipLaunchKernelGGL(form_a<true>, dim3(8, 135, NB), dim3(64, 4), 0, 0, P); }));
    line("B  three dwordx4 per lane (48-byte runs): copy", time_us([&] { hipLaunchKernelGGL(form_b<false>, dim3(unsigned(kImage / 48 / 256 + 1), NB), dim3(256), 0, 0, P); }));
    line("B  three dwordx4 per lane (48-byte runs): x*m+a, saturate", time_us([&] { hipLaunchKernelGGL(form_b<true>, dim3(unsigned(kImage / 48 / 256 + 1), NB), dim3(256), 0, 0, P); }));
    line("C  dense dwordx4 + LDS exchange to 12-byte groups: copy", time_us([&] { hipLaunchKernelGGL(form_c<false>, dim3(unsigned(kImage / 3072 / 4 + 1), NB), dim3(256), 0, 0, P); }));
    line("C  dense dwordx4 + LDS exchange to 12-byte groups: x*m+a, sat.", time_us([&] { hipLaunchKernelGGL(form_c<true>, dim3(unsigned(kImage / 3072 / 4 + 1), NB), dim3(256), 0, 0, P); }));
    line("F  float4 copy (ceiling), again", time_us([&] { hipLaunchKernelGGL(form_f, dim3(unsigned(kImage / 16 / 256 + 1), NB), dim3(256), 0, 0, P); }));
    return 0;
}

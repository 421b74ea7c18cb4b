// fkd/ops.hpp -- the operations of the fused data-parallel path, as device-side static structs.
//
// Each operation is a type with
//   * Params : plain aggregate holding its run-time values (this part is also seen by the host compiler,
//              which fills it in; layouts therefore agree by construction),
//   * name() : the C++ spelling of the type inside namespace fkd (host only) -- the chain signature,
//   * exec() : the per-element body (device only).
// Semantics follow the reference library's CPU backend operation by operation; the file:line given with
// each operation is the reference definition it restates (FK/ = include/fused_kernel/ of the reference).
//
// Floating point: the device code is built with -ffp-contract=off and HIP's default correctly rounded
// fp32 division, so every + - * / below is one IEEE-754 binary32 rounding, as on the CPU backend.
#pragma once

#include "types.hpp"

namespace fkd {

enum : int { PRESERVE_AR = 0, IGNORE_AR = 1 };

#if defined(FKD_HOST_NAMES)
#define FKD_NAME(expr) static std::string name() { return expr; }
inline std::string istr(long long v) { return std::to_string(v); }
#else
#define FKD_NAME(expr)
#endif

// In-register home of one element inside per-thread arrays.  Elements whose size is not a multiple of 4 (uchar3,
// uchar, ushort3 ...) are padded to whole dwords: arrays of 3-byte structs make the optimiser form 24-bit integer
// vectors that the backend can only legalise through scratch or LDS.
template <class T> struct alignas(sizeof(T) % 4 != 0 ? 4 : alignof(T)) Slot { T v; };

// Facts about values that only types can vouch for, used where an operation may be shortened if its input is tame.
// finite_taps<B>: the taps of read B, after everything fused into it, are finite numbers whatever the image holds
// (integer pixels through operations without run-time parameters); a tap with weight zero then contributes a zero and can
// be left out of a blend.  finite_map<Op>: Op maps finite inputs of moderate size to finite outputs of moderate size and
// has no run-time parameters.  bounded_out<R>: what read R hands to the chain is finite and below 2^30 in magnitude.
template <class B> constexpr bool finite_taps() {
    if constexpr (requires { B::kFiniteTaps; }) return B::kFiniteTaps; else return false;
}
template <class Op> constexpr bool finite_map() {
    if constexpr (requires { Op::kFiniteMap; }) return Op::kFiniteMap; else return false;
}
template <class R> constexpr bool bounded_out() {
    if constexpr (requires { R::kBoundedOut; }) return R::kBoundedOut; else return false;
}
template <class T> constexpr bool small_integer_base() {
    return !(__is_same(base_t<T>, f32) || __is_same(base_t<T>, f64)) && sizeof(base_t<T>) <= 2;
}
// Type classes without the standard library (run-time compilation has no headers) and without compiler-specific builtins.
template <class T> constexpr bool is_float_v = __is_same(T, f32) || __is_same(T, f64);
template <class T> constexpr bool is_integer_v =
    __is_same(T, bool) || __is_same(T, char) || __is_same(T, signed char) || __is_same(T, unsigned char) || __is_same(T, short) ||
    __is_same(T, unsigned short) || __is_same(T, int) || __is_same(T, unsigned int) || __is_same(T, long) ||
    __is_same(T, unsigned long) || __is_same(T, long long) || __is_same(T, unsigned long long);
template <int I, class T, class... Ts> struct TypeAt { using type = typename TypeAt<I - 1, Ts...>::type; };
template <class T, class... Ts> struct TypeAt<0, T, Ts...> { using type = T; };

// FKD_EXEC_CODE: the element-wise bodies of the operations (exec, width, height) are compiled: always in device code, and
// in host code that defines FKD_HOST_EXEC (the host headers' CPU executor, which runs a chain element by element with
// exactly these bodies).  Everything that moves runs of elements, gathers taps or uses a gfx950 instruction stays under
// FKD_DEVICE_CODE.
#if defined(FKD_DEVICE_CODE) || defined(FKD_HOST_EXEC)
#define FKD_EXEC_CODE 1
#endif

#if defined(FKD_HOST_EXEC) && !defined(FKD_DEVICE_CODE)
namespace detail {
#define FKD_GLOBAL
template <class T> inline const T* gconst(const void* p) { return static_cast<const T*>(p); }
template <class T> inline T* gmut(void* p) { return static_cast<T*>(p); }
template <class T> inline T load_elem(const T* p) { return *p; }
template <class T> inline void store_elem(T* p, const T& v) { *p = v; }
template <class T> inline const T* row_ptr(const T* data, u32 pitch, int x, int y) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(data) + size_t(y) * pitch) + x;
}
template <class T> inline T* row_ptr(T* data, u32 pitch, int x, int y) {
    return reinterpret_cast<T*>(reinterpret_cast<char*>(data) + size_t(y) * pitch) + x;
}
inline bool dword_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }
inline bool none_in_wave(bool) { return false; }     // never reached: host code has no paired-tap paths
} // namespace detail
#endif

#if defined(FKD_DEVICE_CODE)
namespace detail {

// True when no lane of the wave holds `flag`.
FKD_DEV bool none_in_wave(bool flag) { return __builtin_amdgcn_ballot_w64(flag) == 0; }

// Every pointer this library dereferences on the device is device (global) memory.  Saying so at the access keeps
// the accesses global_load/global_store (scalar base + lane offset addressing, vmcnt only) even where the pointer
// value went through integer registers and the compiler can no longer infer its address space.
#define FKD_GLOBAL __attribute__((address_space(1)))
template <class T> FKD_DEV const FKD_GLOBAL T* gconst(const void* p) { return (const FKD_GLOBAL T*)p; }
template <class T> FKD_DEV FKD_GLOBAL T* gmut(void* p) { return (FKD_GLOBAL T*)p; }

// Dword vectors that may sit at any dword-aligned address: one global_load/store_dwordx{2,3,4} each.
typedef u32 u32x2_t __attribute__((ext_vector_type(2)));
typedef u32 u32x3_t __attribute__((ext_vector_type(3)));
typedef u32 u32x4_t __attribute__((ext_vector_type(4)));
typedef u32x2_t u32x2_a4 __attribute__((aligned(4)));
typedef u32x3_t u32x3_a4 __attribute__((aligned(4)));
typedef u32x4_t u32x4_a4 __attribute__((aligned(4)));

// One whole-dword store (1-4 dwords).  Output is written once and not read again by the kernel, so the stores carry
// the non-temporal hint: the L2s then hand the lines on early instead of keeping them dirty until the kernel ends,
// when all of them would have to be written back at once (a 3840x2160 float copy: 10.6 -> 9.9 us).
template <class Q> FKD_DEV void gstore(FKD_GLOBAL Q* p, const Q& v) { __builtin_nontemporal_store(v, p); }
// One element of 4 or 8 bytes written through the L2 (a relaxed store at system scope: global_store ... sc0 sc1), for
// writers whose lanes each store single elements: the planar writer of the bilinear kernel runs configuration 3 in
// 11.1 us with these, 11.5 us with the non-temporal hint and 12.9 us with plain stores.  Other sizes take gstore.
template <class B> FKD_DEV void gstore_through(FKD_GLOBAL B* p, const B& v) {
    if constexpr (sizeof(B) == 4) __hip_atomic_store(reinterpret_cast<FKD_GLOBAL u32*>(p), __builtin_bit_cast(u32, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    else if constexpr (sizeof(B) == 8) __hip_atomic_store(reinterpret_cast<FKD_GLOBAL unsigned long long*>(p), __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    else *p = v;
}
// One whole-dword load of a row run; STREAM marks data that no cache can hold until its next use (see the rows kernel).
template <bool STREAM, class Q> FKD_DEV Q gload_run(const FKD_GLOBAL Q* p) {
    if constexpr (STREAM) return __builtin_nontemporal_load(p);
    else return *p;
}
template <class T> FKD_DEV T load_elem(const T* p) {
    T v;
    if constexpr (cn_v<T> == 1) {
        v = *gconst<T>(p);
    } else {
        const FKD_GLOBAL base_t<T>* b = gconst<base_t<T>>(p);
        chan<0>(v) = b[0];
        chan<1>(v) = b[1];
        if constexpr (cn_v<T> > 2) chan<2>(v) = b[2];
        if constexpr (cn_v<T> > 3) chan<3>(v) = b[3];
    }
    return v;
}
template <class T> FKD_DEV void store_elem(T* p, const T& v) {
    if constexpr (cn_v<T> == 1) {
        if constexpr (sizeof(T) == 4) gstore(gmut<T>(p), v); else *gmut<T>(p) = v;
    } else {
        FKD_GLOBAL base_t<T>* b = gmut<base_t<T>>(p);
        b[0] = chan<0>(v);
        b[1] = chan<1>(v);
        if constexpr (cn_v<T> > 2) b[2] = chan<2>(v);
        if constexpr (cn_v<T> > 3) b[3] = chan<3>(v);
    }
}

template <int W, bool STREAM = false> FKD_DEV void load_words(const void* p, u32 (&w)[W]) {
    static_assert(W >= 1 && (W <= 4 || W % 4 == 0), "runs are 1-4 dwords or whole 16-byte groups");
    if constexpr (W == 1) {
        w[0] = gload_run<STREAM>(gconst<u32>(p));
    } else if constexpr (W == 2) {
        const u32x2_t v = gload_run<STREAM>(gconst<u32x2_a4>(p));
        w[0] = v.x; w[1] = v.y;
    } else if constexpr (W == 3) {
        const u32x3_t v = gload_run<STREAM>(gconst<u32x3_a4>(p));
        w[0] = v.x; w[1] = v.y; w[2] = v.z;
    } else {
#pragma unroll
        for (int i = 0; i < W / 4; ++i) {
            const u32x4_t v = gload_run<STREAM>(gconst<u32x4_a4>(p) + i);
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
    }
}
template <int W> FKD_DEV void store_words(void* p, const u32 (&w)[W]) {
    static_assert(W >= 1 && (W <= 4 || W % 4 == 0), "runs are 1-4 dwords or whole 16-byte groups");
    if constexpr (W == 1) {
        gstore(gmut<u32>(p), w[0]);
    } else if constexpr (W == 2) {
        u32x2_t v; v.x = w[0]; v.y = w[1];
        gstore(gmut<u32x2_a4>(p), v);
    } else if constexpr (W == 3) {
        u32x3_t v; v.x = w[0]; v.y = w[1]; v.z = w[2];
        gstore(gmut<u32x3_a4>(p), v);
    } else {
#pragma unroll
        for (int i = 0; i < W / 4; ++i) {
            u32x4_t v; v.x = w[4 * i]; v.y = w[4 * i + 1]; v.z = w[4 * i + 2]; v.w = w[4 * i + 3];
            gstore(gmut<u32x4_a4>(p) + i, v);
        }
    }
}

// Bit image of one base element as an unsigned integer of the same width, and back.
template <class B> FKD_DEV auto to_bits(B v) {
    if constexpr (sizeof(B) == 1) return u32(__builtin_bit_cast(u8, v));
    else if constexpr (sizeof(B) == 2) return u32(__builtin_bit_cast(u16, v));
    else if constexpr (sizeof(B) == 4) return __builtin_bit_cast(u32, v);
    else return __builtin_bit_cast(unsigned long long, v);
}
template <class T, int C> FKD_DEV base_t<T> chan_at(const T& v) { return chan<C>(v); }

// Elements <-> packed dwords.  Every index is a compile-time constant (integer sequences, no loops over arrays
// of sub-dword structs), so the element arrays never leave registers: byte extraction folds into
// v_cvt_f32_ubyteN / v_bfe, packing into v_lshl_or / v_perm.
template <class I, I... Is> struct IntSeq {};
template <int N> using MakeSeq = __make_integer_seq<IntSeq, int, N>;

template <int K, class T, int V> FKD_DEV base_t<T> run_elem(const Slot<T> (&in)[V]) {   // K-th base element of the run
    if constexpr (K < V * cn_v<T>) return chan<K % cn_v<T>>(in[K / cn_v<T>].v);
    else return base_t<T>(0);   // padding of a last, partly filled dword
}
template <int I, class T, int V> FKD_DEV u32 pack_word(const Slot<T> (&in)[V]) {        // I-th dword of the run
    using B = base_t<T>;
    if constexpr (sizeof(B) == 1) {
        return to_bits(run_elem<4 * I>(in)) | (to_bits(run_elem<4 * I + 1>(in)) << 8) |
               (to_bits(run_elem<4 * I + 2>(in)) << 16) | (to_bits(run_elem<4 * I + 3>(in)) << 24);
    } else if constexpr (sizeof(B) == 2) {
        return to_bits(run_elem<2 * I>(in)) | (to_bits(run_elem<2 * I + 1>(in)) << 16);
    } else if constexpr (sizeof(B) == 4) {
        return to_bits(run_elem<I>(in));
    } else {
        return u32(to_bits(run_elem<I / 2>(in)) >> (32 * (I % 2)));
    }
}
template <class T, int V, int W, int... Is> FKD_DEV void pack_words_impl(const Slot<T> (&in)[V], u32 (&w)[W], IntSeq<int, Is...>) {
    ((w[Is] = pack_word<Is>(in)), ...);
}
template <class T, int V, int W> FKD_DEV void pack_words(const Slot<T> (&in)[V], u32 (&w)[W]) {
    pack_words_impl<T, V, W>(in, w, MakeSeq<W>{});
}

template <int K, class B, int W> FKD_DEV B unpack_elem(const u32 (&w)[W]) {       // K-th base element of the run
    if constexpr (sizeof(B) == 1) return __builtin_bit_cast(B, u8((w[K / 4] >> (8 * (K % 4))) & 0xffu));
    else if constexpr (sizeof(B) == 2) return __builtin_bit_cast(B, u16((w[K / 2] >> (16 * (K % 2))) & 0xffffu));
    else if constexpr (sizeof(B) == 4) return __builtin_bit_cast(B, w[K]);
    else return __builtin_bit_cast(B, (unsigned long long)w[2 * K] | ((unsigned long long)w[2 * K + 1] << 32));
}
template <int I, class T, int W> FKD_DEV T unpack_one(const u32 (&w)[W]) {        // I-th element of the run
    using B = base_t<T>;
    constexpr int N = cn_v<T>;
    T o;
    chan<0>(o) = unpack_elem<I * N, B>(w);
    if constexpr (N > 1) chan<1>(o) = unpack_elem<I * N + 1, B>(w);
    if constexpr (N > 2) chan<2>(o) = unpack_elem<I * N + 2, B>(w);
    if constexpr (N > 3) chan<3>(o) = unpack_elem<I * N + 3, B>(w);
    return o;
}
template <class T, int V, int W, int... Is> FKD_DEV void unpack_words_impl(const u32 (&w)[W], Slot<T> (&out)[V], IntSeq<int, Is...>) {
    ((out[Is].v = unpack_one<Is, T>(w)), ...);
}
template <class T, int V, int W> FKD_DEV void unpack_words(const u32 (&w)[W], Slot<T> (&out)[V]) {
    unpack_words_impl<T, V, W>(w, out, MakeSeq<V>{});
}

// V consecutive elements starting at p.  ALIGNED promises that p is dword aligned (the launcher checks every
// row start of every plane on the host before it picks the kernel variant): the run then moves as one wide
// access per <= 16 bytes (global_load_dwordx3 for four uchar3, dwordx4 for four floats), which consecutive
// lanes make contiguous.  Without the promise, or when the run is not a whole number of dwords, elements move
// one by one.
template <class T> constexpr bool wide_ok(int v) {
    const int bytes = int(sizeof(T)) * v;
    return v > 1 && bytes % 4 == 0 && (bytes <= 16 || bytes % 16 == 0) && sizeof(T) == sizeof(base_t<T>) * cn_v<T>;
}
// Runs of 32, 48 or 64 bytes per lane (four float2/float3/float4) as wide accesses would leave gaps between the lanes
// of one instruction: lane i moves 16 bytes at i * 48, and the memory pipeline sees three sparse passes over the
// same 3 KiB.  When the whole wave is active on consecutive runs (mode 2) the wave instead moves its segment as
// dense instructions, lane i taking 16 bytes at k * 1024 + i * 16, and exchanges the dwords through a wave-private
// piece of LDS.  The exchange is between lanes of one wave, whose LDS accesses complete in order, so a compiler
// fence is all the synchronisation it needs.
constexpr int kRowsWaves = 4;            // waves per workgroup of the rows kernels
constexpr int kStageDwords = 64 * 16 + 64;
template <class T> constexpr bool wave_exchange_ok(int v) {
    const int bytes = int(sizeof(T)) * v;
    return wide_ok<T>(v) && sizeof(base_t<T>) <= 4 && (bytes == 32 || bytes == 48 || bytes == 64);
}
FKD_DEV u32* wave_stage() {
    __shared__ __attribute__((aligned(16))) u32 stage[kRowsWaves * kStageDwords];
    return stage + threadIdx.y * kStageDwords;
}
// Where dword f of the wave's segment sits in the stage: runs of 32 and 64 bytes get 16 bytes of padding per 256 so
// that the 16 lanes of one LDS pass fall on distinct banks; runs of 48 bytes already do.
template <int W> FKD_DEV u32 stage_at(u32 f) { return W == 12 ? f : f + (f >> 6) * 4u; }
FKD_DEV void wave_exchange_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}
template <int W, bool STREAM> FKD_DEV void load_words_wave(const void* p, u32 (&w)[W]) {
    const u32 lane = threadIdx.x;
    u32* stage = wave_stage();
    // p is this lane's run; the segment starts W dwords per lane earlier
    const char* seg = reinterpret_cast<const char*>(p) - size_t(lane) * (W * 4);
    u32x4_t q[W / 4];
#pragma unroll
    for (int k = 0; k < W / 4; ++k) q[k] = gload_run<STREAM>(gconst<u32x4_a4>(seg + k * 1024 + lane * 16));
    wave_exchange_fence();   // the previous exchange's reads come first
#pragma unroll
    for (int k = 0; k < W / 4; ++k) *reinterpret_cast<u32x4_t*>(stage + stage_at<W>(u32(k) * 256u + lane * 4u)) = q[k];
    wave_exchange_fence();
#pragma unroll
    for (int j = 0; j < W / 4; ++j) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(stage + stage_at<W>(lane * W + u32(j) * 4u));
        w[4 * j] = v.x; w[4 * j + 1] = v.y; w[4 * j + 2] = v.z; w[4 * j + 3] = v.w;
    }
}
template <int W> FKD_DEV void store_words_wave(void* p, const u32 (&w)[W]) {
    const u32 lane = threadIdx.x;
    u32* stage = wave_stage();
    char* seg = reinterpret_cast<char*>(p) - size_t(lane) * (W * 4);
    wave_exchange_fence();
#pragma unroll
    for (int j = 0; j < W / 4; ++j) {
        u32x4_t v; v.x = w[4 * j]; v.y = w[4 * j + 1]; v.z = w[4 * j + 2]; v.w = w[4 * j + 3];
        *reinterpret_cast<u32x4_t*>(stage + stage_at<W>(lane * W + u32(j) * 4u)) = v;
    }
    wave_exchange_fence();
#pragma unroll
    for (int k = 0; k < W / 4; ++k)
        gstore(gmut<u32x4_a4>(seg + k * 1024 + lane * 16), *reinterpret_cast<const u32x4_t*>(stage + stage_at<W>(u32(k) * 256u + lane * 4u)));
}

// Low two bits of the mode: 0: nothing is known about p.  1: p is dword aligned.  2: as 1, and all 64 lanes of the
// wave are in this call with consecutive runs (lane i at p0 + i * V elements).  Bit 2 (value 4): the launch reads more
// than the caches hold, loads carry the non-temporal hint.
template <class T, int V, int MODE_BITS> FKD_DEV void load_run(const T* p, Slot<T> (&out)[V]) {
    constexpr int MODE = MODE_BITS & 3;
    constexpr bool STREAM = (MODE_BITS & 4) != 0;
    constexpr bool ALIGNED = MODE != 0;
    if constexpr (MODE == 2 && wave_exchange_ok<T>(V)) {
        constexpr int W = int(sizeof(T)) * V / 4;
        u32 w[W];
        load_words_wave<W, STREAM>(p, w);
        unpack_words<T, V, W>(w, out);
    } else if constexpr (ALIGNED && wide_ok<T>(V)) {
        constexpr int W = int(sizeof(T)) * V / 4;
        u32 w[W];
        load_words<W, STREAM>(p, w);
        if constexpr (sizeof(base_t<T>) < 4) {
            // Keep each dword an opaque scalar: otherwise the optimiser rewrites "shift and mask a vector lane"
            // into byte-vector extracts (<12 x i8>), which the backend can only legalise through scratch memory.
#pragma unroll
            for (int i = 0; i < W; ++i) asm("" : "+v"(w[i]));
        }
        unpack_words<T, V, W>(w, out);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = load_elem(p + i);
    }
}
template <class T, int V, int MODE_BITS> FKD_DEV void store_run(T* p, const Slot<T> (&in)[V]) {
    constexpr int MODE = MODE_BITS & 3;
    constexpr bool ALIGNED = MODE != 0;
    if constexpr (MODE == 2 && wave_exchange_ok<T>(V)) {
        constexpr int W = int(sizeof(T)) * V / 4;
        u32 w[W];
        pack_words<T, V, W>(in, w);
        store_words_wave<W>(p, w);
    } else if constexpr (ALIGNED && wide_ok<T>(V)) {
        constexpr int W = int(sizeof(T)) * V / 4;
        u32 w[W];
        pack_words<T, V, W>(in, w);
        if constexpr (sizeof(base_t<T>) < 4) {
            // Same reason as in load_run: keep the packed dwords opaque so the store stays one dwordx{2,3,4}
            // instead of becoming a vector of 24-bit elements.
#pragma unroll
            for (int i = 0; i < W; ++i) asm("" : "+v"(w[i]));
        }
        store_words<W>(p, w);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) store_elem(p + i, in[i].v);
    }
}

// V consecutive elements (V = 1 or 2) at byte offset `off` of a (typically wave-uniform) base address: the form a
// gather wants, because the base stays in scalar registers and the lane supplies a 32-bit offset.  The run arrives
// as raw dwords (RunBits) and is taken apart later, at its point of use (run_value), so a consumer can keep many
// such loads in flight.  The hardware takes global accesses at any byte alignment, so a run of 1, 2 or a multiple
// of 4 bytes (up to 16) moves as one access.  Runs of 3 and 6 bytes (uchar3, a uchar3 pair, ushort3) move as one or
// two whole dwords when OVERREAD allows touching up to 3 bytes past the run (the caller guarantees those bytes are
// inside the allocation); otherwise channel by channel.
typedef u16 u16_a1 __attribute__((aligned(1)));
typedef u32 u32_a1 __attribute__((aligned(1)));
typedef u32x2_t u32x2_a1 __attribute__((aligned(1)));
typedef u32x3_t u32x3_a1 __attribute__((aligned(1)));
typedef u32x4_t u32x4_a1 __attribute__((aligned(1)));
template <class T, int V = 1> constexpr int overread_bytes() {
    constexpr int n = int(sizeof(T)) * V;
    return (n == 1 || n == 2 || n % 4 == 0 || n > 16) ? 0 : (n + 3) / 4 * 4 - n;
}
template <class T, int V = 1> struct RunBits {
    static_assert(sizeof(T) == sizeof(base_t<T>) * cn_v<T>, "elements are packed channel arrays");
    static constexpr int kWords = (int(sizeof(T)) * V + 3) / 4;
    u32 w[kWords];
};
template <class T, int V, bool OVERREAD> FKD_DEV RunBits<T, V> load_bits_at(const char* base, u32 off) {
    constexpr int n = int(sizeof(T)) * V;
    constexpr int W = RunBits<T, V>::kWords;
    // Keeps the offset a 32-bit per-lane value next to the access, so base + offset selects the scalar-base
    // addressing form instead of a hoisted 64-bit per-lane pointer.
    asm volatile("" : "+v"(off));
    const char* a = base + off;
    RunBits<T, V> e;
    if constexpr (n == 1) {
        e.w[0] = u32(*gconst<u8>(a));
    } else if constexpr (n == 2) {
        e.w[0] = u32(*gconst<u16_a1>(a));
    } else if constexpr (n > 16 || (overread_bytes<T, V>() > 0 && !OVERREAD)) {
        Slot<T> run[V];
#pragma unroll
        for (int i = 0; i < V; ++i) run[i].v = load_elem(reinterpret_cast<const T*>(a) + i);
        pack_words<T, V, W>(run, e.w);
    } else if constexpr (W == 1) {
        e.w[0] = *gconst<u32_a1>(a);
    } else if constexpr (W == 2) {
        const u32x2_t v = *gconst<u32x2_a1>(a); e.w[0] = v.x; e.w[1] = v.y;
    } else if constexpr (W == 3) {
        const u32x3_t v = *gconst<u32x3_a1>(a); e.w[0] = v.x; e.w[1] = v.y; e.w[2] = v.z;
    } else {
        const u32x4_t v = *gconst<u32x4_a1>(a); e.w[0] = v.x; e.w[1] = v.y; e.w[2] = v.z; e.w[3] = v.w;
    }
    return e;
}
template <int K, class T, int V> FKD_DEV T run_value(const RunBits<T, V>& e) {    // K-th element of the run
    constexpr int W = RunBits<T, V>::kWords;
    u32 w[W];
#pragma unroll
    for (int i = 0; i < W; ++i) w[i] = e.w[i];
    if constexpr (sizeof(base_t<T>) < 4) {
#pragma unroll
        for (int i = 0; i < W; ++i) asm("" : "+v"(w[i]));   // keep dwords whole: bytes leave through v_cvt_f32_ubyteN / v_bfe
    }
    return unpack_one<K, T>(w);
}

// Two consecutive elements for a gather, fetched as ONE dword-aligned window.  A vector-L1 access that starts on a
// dword boundary costs the same whether it is 4 or 16 bytes wide, while a wide access at a byte address costs about
// twice as much; so for elements whose size is not a multiple of 4 the window starts at the dword boundary at or
// below the first element (at most 3 bytes early: same dword, so same page, as a byte that is needed) and the two
// elements are shifted into place with v_alignbyte_b32 where they are used.  The window may end up to 6 bytes past
// the second element; the caller guarantees those bytes are inside the allocation.
template <class T> struct PairWindow {
    static_assert(sizeof(T) == sizeof(base_t<T>) * cn_v<T>, "elements are packed channel arrays");
    static constexpr int kBytes = 2 * int(sizeof(T));
    static constexpr bool kShift = sizeof(T) % 4 != 0;
    static constexpr int kOut = (kBytes + 3) / 4;                          // dwords holding the aligned pair
    static constexpr int kWords = kShift ? (kBytes + 3 + 3) / 4 : kOut;    // dwords fetched
    static constexpr bool kSupported = kWords <= 4;
    u32 w[kWords];
    u32 shift;      // bytes between the window start and the first element
};
template <class T> FKD_DEV PairWindow<T> load_pair_window(const char* row, u32 off) {
    using PW = PairWindow<T>;
    PW p;
    const char* base = row;
    if constexpr (PW::kShift) {
        const u32 lo = u32(reinterpret_cast<uintptr_t>(row)) & 3u;     // wave uniform
        base = row - lo;
        off += lo;
        p.shift = off & 3u;
        off &= ~3u;
    } else {
        p.shift = 0;
    }
    asm volatile("" : "+v"(off));
    const char* a = base + off;
    constexpr int W = PW::kWords;
    if constexpr (W == 1) { p.w[0] = *gconst<u32_a1>(a); }
    else if constexpr (W == 2) { const u32x2_t v = *gconst<u32x2_a4>(a); p.w[0] = v.x; p.w[1] = v.y; }
    else if constexpr (W == 3) { const u32x3_t v = *gconst<u32x3_a4>(a); p.w[0] = v.x; p.w[1] = v.y; p.w[2] = v.z; }
    else { const u32x4_t v = *gconst<u32x4_a4>(a); p.w[0] = v.x; p.w[1] = v.y; p.w[2] = v.z; p.w[3] = v.w; }
    return p;
}
// The same window through a buffer resource, for images whose rows all start at the same offset inside their dword
// (pitch a multiple of 4) and that are smaller than 4 GB.  The image is described once per wave as a raw buffer
// starting at the dword at or below its first byte; a row is then a 32-bit SCALAR byte offset and a column a 32-bit
// per-lane one (window start and bytes to drop, prepared once per column because they no longer depend on the row), so
// a tap costs one buffer_load with no address arithmetic at all.  The resource's size field is left open: staying
// inside the allocation is the caller's business exactly as for the global-memory loads.
struct PairPrep { u32 off, shift; };
template <class B> constexpr bool tap_prepared() {
    if constexpr (requires { B::kTapPrepared; }) return B::kTapPrepared; else return false;
}
struct TapImage {
#if defined(FKD_DEVICE_CODE)
    __amdgpu_buffer_rsrc_t rsrc;
#endif
    u32 lo;       // bytes between the resource's base and the image's first byte
};
#if defined(FKD_DEVICE_CODE)
FKD_DEV TapImage make_tap_image(const void* data) {
    TapImage im;
    im.lo = u32(reinterpret_cast<uintptr_t>(data)) & 3u;
    // word 3 = 0x00020000: 32-bit raw data format of the gfx9 family, no swizzle, no index stride
    im.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(reinterpret_cast<const char*>(data)) - im.lo, 0, 0xffffffffu, 0x00020000);
    return im;
}
// `bytes` of image behind `data` (less than 4 GB): the extent ends with the dword that holds the last of them.  That dword
// starts inside the image, so it lies in a mapped page whatever follows the allocation.
FKD_DEV TapImage make_tap_image(const void* data, size_t bytes) {
    TapImage im;
    im.lo = u32(reinterpret_cast<uintptr_t>(data)) & 3u;
    const u32 extent = (u32(bytes) + im.lo + 3u) & ~3u;
    im.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(reinterpret_cast<const char*>(data)) - im.lo, 0, extent, 0x00020000);
    return im;
}
template <class T> FKD_DEV PairPrep prepare_pair_window(const TapImage& im, u32 off) {
    PairPrep pp;
    if constexpr (PairWindow<T>::kShift) {
        off += im.lo;
        pp.shift = off & 3u;
        pp.off = off & ~3u;
    } else {
        pp.shift = 0;
        pp.off = off + im.lo;
    }
    return pp;
}
template <class T> FKD_DEV PairWindow<T> load_prepared_pair_window(const TapImage& im, u32 row_off, const PairPrep& pp) {
    using PW = PairWindow<T>;
    PW p;
    p.shift = pp.shift;
    constexpr int W = PW::kWords;
    if constexpr (W == 1) { p.w[0] = __builtin_amdgcn_raw_buffer_load_b32(im.rsrc, pp.off, row_off, 0); }
    else if constexpr (W == 2) { const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(im.rsrc, pp.off, row_off, 0); p.w[0] = v.x; p.w[1] = v.y; }
    else if constexpr (W == 3) { const u32x3_t v = __builtin_amdgcn_raw_buffer_load_b96(im.rsrc, pp.off, row_off, 0); p.w[0] = v.x; p.w[1] = v.y; p.w[2] = v.z; }
    else { const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(im.rsrc, pp.off, row_off, 0); p.w[0] = v.x; p.w[1] = v.y; p.w[2] = v.z; p.w[3] = v.w; }
    return p;
}
#endif
// DUP: lanes with `dup` set take the window's SECOND element for both values (a tap pair that ends at the image's last
// column).  For 3-byte elements that is one byte permutation and one select on the aligned dwords (bytes 3,4,5,3 of the
// first two dwords replace the first one; the second dword, which holds the second element's last two channels, stays);
// for elements that are whole dwords it is a select per dword; other sizes select the unpacked values.
template <bool DUP = false, class T> FKD_DEV void pair_window_values(const PairWindow<T>& p, T& first, T& second, bool dup = false) {
    using PW = PairWindow<T>;
    u32 v[PW::kOut];
#pragma unroll
    for (int i = 0; i < PW::kOut; ++i) {
        if constexpr (PW::kShift) v[i] = __builtin_amdgcn_alignbyte(p.w[i + 1 < PW::kWords ? i + 1 : i], p.w[i], p.shift);
        else v[i] = p.w[i];
        if constexpr (sizeof(base_t<T>) < 4) asm("" : "+v"(v[i]));   // keep dwords whole: v_cvt_f32_ubyteN / v_bfe
    }
    constexpr bool kDupBytes = DUP && sizeof(T) == 3, kDupWords = DUP && sizeof(T) % 4 == 0;
    if constexpr (kDupBytes) {
        const u32 twice = __builtin_amdgcn_perm(v[1], v[0], 0x03050403u);
        v[0] = dup ? twice : v[0];
        asm("" : "+v"(v[0]));
    } else if constexpr (kDupWords) {
        constexpr int E = int(sizeof(T)) / 4;
#pragma unroll
        for (int i = 0; i < E; ++i) v[i] = dup ? v[E + i] : v[i];
    }
    // channel by channel: copying whole 3-byte elements makes the compiler gather each into one register first
    // (v_perm_b32), although every channel leaves its dword through v_cvt_f32_ubyteN anyway
    constexpr int N = cn_v<T>;
    using B = base_t<T>;
    chan<0>(first) = unpack_elem<0, B>(v);
    chan<0>(second) = unpack_elem<N, B>(v);
    if constexpr (N > 1) { chan<1>(first) = unpack_elem<1, B>(v); chan<1>(second) = unpack_elem<N + 1, B>(v); }
    if constexpr (N > 2) { chan<2>(first) = unpack_elem<2, B>(v); chan<2>(second) = unpack_elem<N + 2, B>(v); }
    if constexpr (N > 3) { chan<3>(first) = unpack_elem<3, B>(v); chan<3>(second) = unpack_elem<N + 3, B>(v); }
    if constexpr (DUP && !kDupBytes && !kDupWords) { if (dup) first = second; }
}

// Store counterpart of load_bits_at: element sizes 2 and multiples of 4 (up to 16) leave as one access.
template <class T> FKD_DEV void store_elem_at(char* base, u32 off, const T& v) {
    constexpr int n = int(sizeof(T));
    constexpr bool packed = sizeof(T) == sizeof(base_t<T>) * cn_v<T>;
    asm volatile("" : "+v"(off));   // as in load_bits_at: keep the scalar-base addressing form
    char* a = base + off;
    if constexpr (!packed || n > 16 || (n % 4 != 0 && n != 2) || cn_v<T> == 1) {
        store_elem(reinterpret_cast<T*>(a), v);
    } else {
        Slot<T> one[1];
        one[0].v = v;
        constexpr int W = (n + 3) / 4;
        u32 w[W];
        if constexpr (n == 2) {
            w[0] = to_bits(chan<0>(v)) | (to_bits(chan<1>(v)) << 8);
            *gmut<u16_a1>(a) = u16(w[0]);
        } else {
            pack_words<T, 1, W>(one, w);
            if constexpr (W == 1) { gstore(gmut<u32_a1>(a), w[0]); }
            else if constexpr (W == 2) { u32x2_t q; q.x = w[0]; q.y = w[1]; gstore(gmut<u32x2_a1>(a), q); }
            else if constexpr (W == 3) { u32x3_t q; q.x = w[0]; q.y = w[1]; q.z = w[2]; gstore(gmut<u32x3_a1>(a), q); }
            else { u32x4_t q; q.x = w[0]; q.y = w[1]; q.z = w[2]; q.w = w[3]; gstore(gmut<u32x4_a1>(a), q); }
        }
    }
}

// V consecutive elements to byte offset `off` of a wave-uniform base, as one wide access when the run is a whole
// number of dwords (any byte alignment), else element by element.
template <class T, int V> FKD_DEV void store_run_at(char* base, u32 off, const Slot<T> (&v)[V]) {
    constexpr int n = int(sizeof(T)) * V;
    constexpr bool packed = sizeof(T) == sizeof(base_t<T>) * cn_v<T>;
    if constexpr (packed && n % 4 == 0 && n <= 16) {
        constexpr int W = n / 4;
        u32 w[W];
        pack_words<T, V, W>(v, w);
        if constexpr (sizeof(base_t<T>) < 4) {
#pragma unroll
            for (int i = 0; i < W; ++i) asm("" : "+v"(w[i]));
        }
        asm volatile("" : "+v"(off));
        char* a = base + off;
        if constexpr (W == 1) { gstore(gmut<u32_a1>(a), w[0]); }
        else if constexpr (W == 2) { u32x2_t q; q.x = w[0]; q.y = w[1]; gstore(gmut<u32x2_a1>(a), q); }
        else if constexpr (W == 3) { u32x3_t q; q.x = w[0]; q.y = w[1]; q.z = w[2]; gstore(gmut<u32x3_a1>(a), q); }
        else { u32x4_t q; q.x = w[0]; q.y = w[1]; q.z = w[2]; q.w = w[3]; gstore(gmut<u32x4_a1>(a), q); }
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) store_elem_at<T>(base, off + u32(i) * u32(sizeof(T)), v[i].v);
    }
}

// A copy of a (wave-uniform) parameter object that is pinned into scalar registers right here: all its scalar loads
// are issued together and waited for once, instead of one load-and-wait round trip per first use further down.
template <class T> FKD_DEV T scalar_copy(const T& src) {
    if constexpr (sizeof(T) % 4 != 0 || sizeof(T) > 256) {
        return src;
    } else {
        constexpr int N = int(sizeof(T)) / 4;
        u32 w[N];
        __builtin_memcpy(w, &src, sizeof(T));
#pragma unroll
        for (int i = 0; i < N; ++i) asm volatile("" : "+s"(w[i]));
        T out;
        __builtin_memcpy(&out, w, sizeof(T));
        return out;
    }
}

// Pins an object that is wave uniform into scalar registers where it stands (objects whose size is not a whole number
// of dwords, or that are larger than 256 bytes, are left to the compiler).
template <class T> FKD_DEV void pin_scalars(T& v) {
    if constexpr (sizeof(T) % 4 == 0 && sizeof(T) <= 256 && __is_trivially_copyable(T)) {
        constexpr int N = int(sizeof(T)) / 4;
        u32 w[N];
        __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
        for (int i = 0; i < N; ++i) asm volatile("" : "+s"(w[i]));
        __builtin_memcpy(&v, w, sizeof(T));
    }
}

FKD_HD bool dword_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

template <class T> FKD_DEV const T* row_ptr(const T* data, u32 pitch, int x, int y) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(data) + size_t(y) * pitch) + x;
}
template <class T> FKD_DEV T* row_ptr(T* data, u32 pitch, int x, int y) {
    return reinterpret_cast<T*>(reinterpret_cast<char*>(data) + size_t(y) * pitch) + x;
}

} // namespace detail
#endif // FKD_DEVICE_CODE

// ===================================================================================================
// Compute operations: In -> Out
// ===================================================================================================

// Add/Sub/Mul/Div<I,P,O,BinaryType>::exec: FK/algorithms/basic_ops/arithmetic.h:26-124, evaluated per channel
// with the usual C++ promotions (FK/core/utils/vector_utils.h:508-563); a scalar P is broadcast.
#define FKD_BINARY_OP(NAME, EXPR)                                                                         \
    template <class I, class P, class O> struct NAME {                                                    \
        using In = I; using Out = O;                                                                      \
        struct Params { P v; };                                                                           \
        static constexpr bool kValueParams = true;   /* nothing but operands: see vector_params */          \
        FKD_NAME(#NAME "<" + type_name<I>() + "," + type_name<P>() + "," + type_name<O>() + ">")       \
        FKD_DEV static O exec(const I& a, const Params& p) {                                              \
            return map2<O>(a, p.v, [](auto x, auto y) { return static_cast<base_t<O>>(EXPR); });          \
        }                                                                                                 \
    };
FKD_BINARY_OP(Add, x + y)
FKD_BINARY_OP(Sub, x - y)
FKD_BINARY_OP(Mul, x * y)
#undef FKD_BINARY_OP

// Div<I,P,O>: FK/algorithms/basic_ops/arithmetic.h:96-124, x / y per channel, correctly rounded.
//
// The divisor is a launch-time constant, the same for every element, so for all-fp32 divisions the host also
// stores r = RN(1/y) and the device replaces the generic division (two scalings, a reciprocal estimate, its
// refinement, fix-ups: ~10 instructions) by five:
//     q0 = x*r;  e0 = fma(-y, q0, x);  q1 = fma(e0, r, q0);  e1 = fma(-y, q1, x);  q = fma(e1, r, q1)
// q0 is within 1.5 ulp of x/y, so q1 is within 0.5 ulp + 2^-23 ulp (faithful), e1 is then exact and, r being the
// correctly rounded reciprocal, the last step yields RN(x/y) (Markstein's theorem on the final division step).
// That argument needs every intermediate free of underflow and overflow: the host enables the path only for
// 2^-40 <= |y| <= 2^40, and the device takes it only for elements with 2^-60 <= |x| <= 2^60 in every channel;
// everything else (zeros, denormals, infinities, NaNs, extreme magnitudes) goes through the generic division.
//
// For most divisors two instructions are enough (fast == 2): with the reciprocal held in two floats, r = RN(1/y) and
// l = RN(1/y - r),
//     q = fma(x, r, x*l)
// is computed from t = x*r + RN(x*l), and |t - x/y| < 1.5 * 2^-47 |x/y|, i.e. less than 1.5 * 2^-23 ulp of the
// quotient.  RN(t) can differ from RN(x/y) only if x/y lies that close to the midpoint of two floats.  Write
// |x| = X 2^a, |y| = Y 2^b with 24-bit integers X, Y; the midpoints of the quotient's binade are (2Q+1) / 2^(25+s)
// (s = 0 for X >= Y, 1 otherwise) and the distance of X/Y from one of them is |2^(24+s) X - (2Q+1) Y| / (2Y) ulp.  The
// integer D = 2^(24+s) X - (2Q+1) Y is never 0 and must be below 6 in magnitude for a failure, so for a given y all
// candidate numerators are the solutions X of 2^(24+s) X = D (mod Y), |D| <= 8, a few dozen at most.  The host
// finds them with a modular inverse and runs the two instructions on each one; if every result equals the correctly
// rounded quotient the sequence is exact for that divisor and ALL x (powers of two only shift exponents; the range
// conditions above, with 2^-30 <= |y| <= 2^30, keep every intermediate normal or harmlessly small), otherwise the divisor
// keeps the five-instruction form.
//
// The per-element range test (7 instructions per pixel) goes away when the chain proves the range, which it can for the
// usual normalisation (x - mean) / std: see Chain::finalize.  A division with both proofs (fast == 2 | kInputProven) is
// "static": exec_static is the two instructions and nothing else, and kernels pick the code path built from it once per
// wave, because a test of `fast` inside the per-element code costs as much as the shorter sequence saves.
template <class I, class P, class O> struct Div {
    using In = I; using Out = O;
    static constexpr bool kReciprocal = __is_same(base_t<I>, f32) && __is_same(base_t<P>, f32) && __is_same(base_t<O>, f32);
    struct Params { P v; P rcp; P rcp_lo; i32 fast; };
    // `fast`: low two bits 0 generic division, 1 five instructions, 2 two instructions; kInputProven: the chain has
    // shown that every element reaching this division is zero or has 2^-60 <= |x| <= 2^60 (Chain::finalize).
    static constexpr i32 kInputProven = 4;
    FKD_NAME("Div<" + type_name<I>() + "," + type_name<P>() + "," + type_name<O>() + ">")

#if !defined(FKD_DEVICE_CODE)
    // RN(1/d) for a normal d: the double quotient rounded to float is off by at most one float; 1 - d*c is exact in
    // double for the three candidates, so the smallest residual names the correctly rounded one.
    static f32 exact_reciprocal(f32 d) {
        const f32 c0 = f32(1.0 / double(d));
        f32 best = c0;
        double err = __builtin_fabs(1.0 - double(d) * double(c0));
        for (const f32 c : {__builtin_nextafterf(c0, -__builtin_inff()), __builtin_nextafterf(c0, __builtin_inff())}) {
            const double e = __builtin_fabs(1.0 - double(d) * double(c));
            if (e < err) { err = e; best = c; }
        }
        return best;
    }
    // The low part of the reciprocal: 1 - d*r is exact in double, its quotient by d is rounded once to double and once
    // to float (the second rounding can cost one more unit in the last place of l, which the proof's margin covers).
    static f32 reciprocal_low(f32 d, f32 r) { return f32((1.0 - double(d) * double(r)) / double(d)); }
    // What the device computes, with the same roundings.
    static f32 two_step(f32 x, f32 r, f32 l) {
        volatile f32 low = x * l;
        return __builtin_fmaf(x, r, low);
    }
    // True when two_step(x, r, l) == RN(x/d) for every x whose quotient neither overflows nor underflows (see above).
    static bool two_step_proven(f32 d, f32 r, f32 l) {
        using u64 = unsigned long long; using i64 = long long;
        int e = 0;
        const f32 m = __builtin_frexpf(__builtin_fabsf(d), &e);       // |d| = m 2^e, m in [0.5, 1)
        const u64 Y = u64(__builtin_ldexpf(m, 24));                   // |d| = Y 2^(e-24), Y in [2^23, 2^24)
        const int v = __builtin_ctzll(Y);
        const u64 Yo = Y >> v;                                        // odd part
        if (Yo == 1) return true;                                     // a power of two: the quotient is exact
        auto inverse = [](u64 a, u64 mod) {                           // a^-1 mod an odd modulus, a odd or even but coprime
            i64 t = 0, nt = 1, rr = i64(mod), nr = i64(a % mod);
            while (nr != 0) { const i64 q = rr / nr; i64 k = t - q * nt; t = nt; nt = k; k = rr - q * nr; rr = nr; nr = k; }
            return u64(t < 0 ? t + i64(mod) : t);
        };
        for (int s = 0; s < 2; ++s) {
            const u64 N = 1ull << (24 + s);
            const u64 inv = inverse((N >> v) % Yo, Yo);
            for (int D = -8; D <= 8; ++D) {
                if (D == 0 || (D % (1 << v)) != 0) continue;          // 2^v divides Y and N, so it must divide D (v <= 3 here)
                if (v > 3) continue;
                const i64 Dg = D / (1 << v);
                const u64 res = u64(((Dg % i64(Yo)) + i64(Yo)) % i64(Yo));
                const u64 X0 = res * inv % Yo;
                for (u64 X = X0; X < (1ull << 24); X += Yo) {
                    if (X < (1ull << 23)) continue;
                    const f32 x = __builtin_ldexpf(f32(X), e - 24);    // x/|d| = X/Y
                    const f32 want = f32(double(x) / double(d));       // correctly rounded: double carries 2*24+2 bits
                    if (two_step(x, r, l) != want || two_step(-x, r, l) != -want) return false;
                }
            }
        }
        return true;
    }
    // What the host works out for one divisor: the reciprocal in two floats, and which sequence it licenses
    // (0 none: outside the accepted range; 1 five instructions; 2 two instructions).  A pure function of d that costs
    // about half a microsecond, and applications divide by the same constants launch after launch (a normalisation's
    // standard deviations), so each thread remembers the last divisors it analysed.
    struct Analysis { f32 d, r, l; i32 mode; };
    static Analysis analyse(f32 d) {
        Analysis a{d, 0.0f, 0.0f, 0};
        const f32 m = __builtin_fabsf(d);
        if (!(m >= 0x1p-40f && m <= 0x1p40f)) return a;
        a.r = exact_reciprocal(d);
        a.l = reciprocal_low(d, a.r);
        a.mode = (m >= 0x1p-30f && m <= 0x1p30f && two_step_proven(d, a.r, a.l)) ? 2 : 1;
        return a;
    }
    static Analysis analyse_cached(f32 d) {
        constexpr u32 kSlots = 16;
        thread_local Analysis slot[kSlots] = {};        // d = 0 in an unused slot: zero is never analysed (mode 0)
        const u32 bits = __builtin_bit_cast(u32, d);
        Analysis& s = slot[(bits ^ (bits >> 9) ^ (bits >> 18)) % kSlots];
        if (__builtin_bit_cast(u32, s.d) != bits || bits == 0u) s = analyse(d);
        return s;
    }
    static Params make(const P& v) {
        Params p{};
        p.v = v;
        p.fast = 0;
        if constexpr (kReciprocal) {
            i32 mode = 2;
            auto one = [&](f32 d, f32& r, f32& l) {
                const Analysis a = analyse_cached(d);
                r = a.r; l = a.l;
                mode = a.mode < mode ? a.mode : mode;
            };
            one(chan<0>(v), chan<0>(p.rcp), chan<0>(p.rcp_lo));
            if constexpr (cn_v<P> > 1) one(chan<1>(v), chan<1>(p.rcp), chan<1>(p.rcp_lo));
            if constexpr (cn_v<P> > 2) one(chan<2>(v), chan<2>(p.rcp), chan<2>(p.rcp_lo));
            if constexpr (cn_v<P> > 3) one(chan<3>(v), chan<3>(p.rcp), chan<3>(p.rcp_lo));
            if (mode == 0) { p.rcp = P{}; p.rcp_lo = P{}; }       // as before: no reciprocal is published for a refused divisor
            p.fast = mode;
        }
        return p;
    }
#endif

    FKD_DEV static O exec(const I& a, const Params& p) {
        return map2<O>(a, p.v, [](auto x, auto y) { return static_cast<base_t<O>>(x / y); });
    }
#if defined(FKD_DEVICE_CODE)
    FKD_DEV static f32 quick1(f32 x, f32 y, f32 r) {
        const f32 q0 = x * r;
        const f32 e0 = __builtin_fmaf(-y, q0, x);
        const f32 q1 = __builtin_fmaf(e0, r, q0);
        const f32 e1 = __builtin_fmaf(-y, q1, x);
        return __builtin_fmaf(e1, r, q1);
    }
    FKD_DEV static f32 quick2(f32 x, f32 r, f32 l) { return __builtin_fmaf(x, r, x * l); }
    FKD_DEV static bool is_static(const Params& p) { return p.fast == (2 | kInputProven); }
    FKD_DEV static O exec_static(const I& a, const Params& p) {
        O o;
        chan<0>(o) = quick2(chan<0>(a), chan_or_scalar<0>(p.rcp), chan_or_scalar<0>(p.rcp_lo));
        if constexpr (cn_v<O> > 1) chan<1>(o) = quick2(chan<1>(a), chan_or_scalar<1>(p.rcp), chan_or_scalar<1>(p.rcp_lo));
        if constexpr (cn_v<O> > 2) chan<2>(o) = quick2(chan<2>(a), chan_or_scalar<2>(p.rcp), chan_or_scalar<2>(p.rcp_lo));
        if constexpr (cn_v<O> > 3) chan<3>(o) = quick2(chan<3>(a), chan_or_scalar<3>(p.rcp), chan_or_scalar<3>(p.rcp_lo));
        return o;
    }
    // Straight-line variant: always returns the short sequence's result and clears `ok` when that result may not be
    // the correctly rounded quotient for this element; the caller then recomputes the element with exec().
    static constexpr bool kQuick = kReciprocal;
    FKD_DEV static O exec_quick(const I& a, const Params& p, bool& ok) {
        // sum of magnitudes <= 2^60 bounds every channel from above and is false for NaN and infinity
        f32 sum = __builtin_fabsf(chan<0>(a)), least = sum;
        if constexpr (cn_v<I> > 1) { sum += __builtin_fabsf(chan<1>(a)); least = __builtin_fminf(least, __builtin_fabsf(chan<1>(a))); }
        if constexpr (cn_v<I> > 2) { sum += __builtin_fabsf(chan<2>(a)); least = __builtin_fminf(least, __builtin_fabsf(chan<2>(a))); }
        if constexpr (cn_v<I> > 3) { sum += __builtin_fabsf(chan<3>(a)); least = __builtin_fminf(least, __builtin_fabsf(chan<3>(a))); }
        ok = ok && (p.fast & 3) != 0 && sum <= 0x1p60f && least >= 0x1p-60f;
        O o;
        if ((p.fast & 3) == 2) {      // launch constant: a scalar branch
            chan<0>(o) = quick2(chan<0>(a), chan_or_scalar<0>(p.rcp), chan_or_scalar<0>(p.rcp_lo));
            if constexpr (cn_v<O> > 1) chan<1>(o) = quick2(chan<1>(a), chan_or_scalar<1>(p.rcp), chan_or_scalar<1>(p.rcp_lo));
            if constexpr (cn_v<O> > 2) chan<2>(o) = quick2(chan<2>(a), chan_or_scalar<2>(p.rcp), chan_or_scalar<2>(p.rcp_lo));
            if constexpr (cn_v<O> > 3) chan<3>(o) = quick2(chan<3>(a), chan_or_scalar<3>(p.rcp), chan_or_scalar<3>(p.rcp_lo));
            return o;
        }
        chan<0>(o) = quick1(chan<0>(a), chan_or_scalar<0>(p.v), chan_or_scalar<0>(p.rcp));
        if constexpr (cn_v<O> > 1) chan<1>(o) = quick1(chan<1>(a), chan_or_scalar<1>(p.v), chan_or_scalar<1>(p.rcp));
        if constexpr (cn_v<O> > 2) chan<2>(o) = quick1(chan<2>(a), chan_or_scalar<2>(p.v), chan_or_scalar<2>(p.rcp));
        if constexpr (cn_v<O> > 3) chan<3>(o) = quick1(chan<3>(a), chan_or_scalar<3>(p.v), chan_or_scalar<3>(p.rcp));
        return o;
    }
#endif
};

// StaticLoop<Operation, ITERATIONS>: Operation applied ITERATIONS times with the same parameters.
// FK/algorithms/basic_ops/static_loop.h:21-44.
template <class Op, int N> struct StaticLoop {
    using In = typename Op::In; using Out = typename Op::Out;
    using Params = typename Op::Params;
    static_assert(N >= 1 && __is_same(In, Out), "the looped operation maps a type onto itself");
    FKD_NAME("StaticLoop<" + Op::name() + "," + istr(N) + ">")
    FKD_DEV static Out exec(const In& a, const Params& p) {
        Out v = Op::exec(a, p);
#pragma unroll
        for (int i = 1; i < N; ++i) v = Op::exec(v, p);
        return v;
    }
};

// Cast<I,O>: per-channel static_cast.  FK/algorithms/basic_ops/cast.h:22-33.
template <class I, class O> struct Cast {
    using In = I; using Out = O; using Params = Empty;
    static constexpr bool kFiniteMap = __is_same(base_t<O>, f32) && sizeof(base_t<I>) <= 4 && !__is_same(base_t<I>, f64);
    FKD_NAME("Cast<" + type_name<I>() + "," + type_name<O>() + ">")
    FKD_DEV static O exec(const I& a, const Params&) {
        return map1<O>(a, [](auto x) { return static_cast<base_t<O>>(x); });
    }
};

// ---- the per-channel functions of the reference's basic_ops headers that a chain may hold between read and write ----
// math.h:26-170 (Abs, Sqr, Sqrt, Ln, Exp, AbsDiff), logical.h:37-88 (Max, Min), bitwise.h:23-157 (BwAnd, BwOr, BwXor,
// BwNot, ShiftLeft, ShiftRight).  Each is a C++ expression on one channel (and on the matching channel of a launch
// constant, a scalar constant being broadcast), evaluated in the types the expression promotes to and converted to the
// output's channel type: FK/core/constexpr_libs/constexpr_vector_exec.h:24-108 (cxp::Exec) and the channel-wise operators
// of FK/core/utils/vector_utils.h:508-600.  Map1 / Map2 carry the function as a type.
namespace fn {
#define FKD_FN(text) FKD_NAME(text)
struct Abs {      // s < 0 ? -s : s for signed channel types, s for unsigned ones (so -0.f and NaN come back unchanged)
    FKD_FN("fn::Abs")
    template <class T> FKD_HD static auto apply(T s) {
        if constexpr (T(-1) < T(0)) return s < T(0) ? static_cast<T>(-s) : s;
        else return s;
    }
};
struct Sqr { FKD_FN("fn::Sqr") template <class T> FKD_HD static auto apply(T s) { return s * s; } };
// sqrtf / logf / expf of the channel converted to float.  The square root is correctly rounded on both sides; the
// logarithm and the exponential are the platform's, so device and host agree to a few units in the last place.
struct Sqrt { FKD_FN("fn::Sqrt") template <class T> FKD_HD static f32 apply(T s) { return __builtin_sqrtf(static_cast<f32>(s)); } };
struct Ln { FKD_FN("fn::Ln") template <class T> FKD_HD static f32 apply(T s) { return __builtin_logf(static_cast<f32>(s)); } };
struct Exp { FKD_FN("fn::Exp") template <class T> FKD_HD static f32 apply(T s) { return __builtin_expf(static_cast<f32>(s)); } };
struct BwNot { FKD_FN("fn::BwNot") template <class T> FKD_HD static auto apply(T s) { return ~s; } };
// std::max / std::min of two values of ONE type: (a < b) ? b : a and (b < a) ? b : a, so a NaN input comes back and a NaN
// constant never does.
struct Max { FKD_FN("fn::Max") template <class T> FKD_HD static T apply(T a, T b) { return (a < b) ? b : a; } };
struct Min { FKD_FN("fn::Min") template <class T> FKD_HD static T apply(T a, T b) { return (b < a) ? b : a; } };
struct AbsDiff {
    FKD_FN("fn::AbsDiff")
    template <class A, class B> FKD_HD static auto apply(A a, B b) {
        const auto d = a - b;
        return d < decltype(d)(0) ? -d : d;
    }
};
struct Add { FKD_FN("fn::Add") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a + b; } };
struct Sub { FKD_FN("fn::Sub") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a - b; } };
struct Mul { FKD_FN("fn::Mul") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a * b; } };
struct Div { FKD_FN("fn::Div") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a / b; } };
struct BwAnd { FKD_FN("fn::BwAnd") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a & b; } };
struct BwOr { FKD_FN("fn::BwOr") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a | b; } };
struct BwXor { FKD_FN("fn::BwXor") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a ^ b; } };
struct ShiftLeft { FKD_FN("fn::ShiftLeft") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a << b; } };
struct ShiftRight { FKD_FN("fn::ShiftRight") template <class A, class B> FKD_HD static auto apply(A a, B b) { return a >> b; } };
#undef FKD_FN
} // namespace fn
template <class F, class I, class O> struct Map1 {
    static_assert(cn_v<I> == cn_v<O>, "one output channel per input channel");
    using In = I; using Out = O; using Params = Empty;
    FKD_NAME("Map1<" + F::name() + "," + type_name<I>() + "," + type_name<O>() + ">")
    FKD_DEV static O exec(const I& a, const Params&) {
        return map1<O>(a, [](auto x) { return static_cast<base_t<O>>(F::apply(x)); });
    }
};
template <class F, class I, class P, class O> struct Map2 {
    static_assert(cn_v<I> == cn_v<O> && (cn_v<P> == cn_v<I> || cn_v<P> == 1), "a constant per channel, or one for all");
    using In = I; using Out = O;
    struct Params { P v; };
    static constexpr bool kValueParams = true;
    FKD_NAME("Map2<" + F::name() + "," + type_name<I>() + "," + type_name<P>() + "," + type_name<O>() + ">")
    FKD_DEV static O exec(const I& a, const Params& p) {
        return map2<O>(a, p.v, [](auto x, auto y) { return static_cast<base_t<O>>(F::apply(x, y)); });
    }
};

// The two-input forms of the same operations (Add<I1, I2, O, UnaryType> ... in arithmetic.h:26-124, bitwise.h, logical.h,
// math.h): the value is a pair, as DualRead2D hands it over, and the function is applied to its two halves channel by
// channel (a scalar half is broadcast).
template <class F, class A, class B, class O> struct Zip {
    static_assert(cn_v<A> == cn_v<O> || cn_v<B> == cn_v<O>, "one output channel per input channel");
    using In = Two<A, B>; using Out = O; using Params = Empty;
    FKD_NAME("Zip<" + F::name() + "," + type_name<A>() + "," + type_name<B>() + "," + type_name<O>() + ">")
    FKD_DEV static O exec(const In& v, const Params&) {
        return map2<O>(v.a, v.b, [](auto x, auto y) { return static_cast<base_t<O>>(F::apply(x, y)); });
    }
};

// MxVFloat3<BinaryType>: a float3 times a 3x3 matrix held row by row, per row three products summed as (a + b) + c.
// FK/algorithms/basic_ops/algebraic.h:25-40.
struct MxV3 {
    using In = Vec<f32, 3>; using Out = Vec<f32, 3>;
    struct Params { f32 m[9]; };
    FKD_NAME("MxV3")
    FKD_DEV static Out exec(const In& a, const Params& p) {
        Out o;
        o.x = (a.x * p.m[0] + a.y * p.m[1]) + a.z * p.m[2];
        o.y = (a.x * p.m[3] + a.y * p.m[4]) + a.z * p.m[5];
        o.z = (a.x * p.m[6] + a.y * p.m[7]) + a.z * p.m[8];
        return o;
    }
};

// IsEven<I>: per channel, whether an integer is even; the answer is a byte holding 0 or 1 (the layout of a host bool).
// FK/algorithms/basic_ops/logical.h:23-35.
template <class I> struct IsEven {
    static_assert(base_t<I>(1) / base_t<I>(2) == base_t<I>(0), "integer channels only");
    using In = I; using Out = vec_t<u8, cn_v<I>>; using Params = Empty;
    FKD_NAME("IsEven<" + type_name<I>() + ">")
    FKD_DEV static Out exec(const I& a, const Params&) {
        return map1<Out>(a, [](auto x) { return u8((x & 1) == 0 ? 1 : 0); });
    }
};

// VectorReorder<T,i0,i1,i2,i3>: out[c] = in[idx[c]] (BGR<->RGB is 2,1,0).  FK/algorithms/basic_ops/vector_ops.h:43-56,
// reached through ColorConversion<COLOR_BGR2RGB,...>, FK/algorithms/image_processing/color_conversion.h:472-476.
template <class T, int I0, int I1, int I2 = 2, int I3 = 3> struct Reorder {
    using In = T; using Out = T; using Params = Empty;
    static constexpr bool kFiniteMap = true;
    FKD_NAME("Reorder<" + type_name<T>() + "," + istr(I0) + "," + istr(I1) + "," + istr(I2) + "," + istr(I3) + ">")
    FKD_DEV static T exec(const T& a, const Params&) {
        T o;
        chan<0>(o) = chan<I0>(a);
        chan<1>(o) = chan<I1>(a);
        if constexpr (cn_v<T> > 2) chan<2>(o) = chan<I2>(a);
        if constexpr (cn_v<T> > 3) chan<3>(o) = chan<I3>(a);
        return o;
    }
};

// SaturateCast<I,O>: FK/algorithms/image_processing/saturate.h:25-36 -> cxp::saturate_cast,
// FK/core/constexpr_libs/constexpr_saturate.h:68-150.  float -> integer: NaN -> 0, round half to even,
// clamp; integer -> integer: clamp; float -> float / widening: plain cast.
template <class I, class O> struct SaturateCast {
    using In = I; using Out = O; using Params = Empty;
    FKD_NAME("SaturateCast<" + type_name<I>() + "," + type_name<O>() + ">")
#if defined(FKD_EXEC_CODE)
    template <class D> struct Lim {
        static constexpr bool is_signed = D(-1) < D(0);
        static constexpr long long hi = is_signed ? (long long)((1ull << (8 * sizeof(D) - 1)) - 1)
                                                  : (long long)(sizeof(D) >= 8 ? ~0ull >> 1 : (1ull << (8 * (sizeof(D) % 8))) - 1);
        static constexpr long long lo = is_signed ? -(long long)(1ull << (8 * sizeof(D) - 1)) : 0ll;
    };
    template <class S, class D> FKD_DEV static D sat(S s) {
        if constexpr (__is_same(S, D)) {
            return s;
#if defined(FKD_DEVICE_CODE)
        } else if constexpr (__is_same(S, f32) && __is_same(D, u8)) {
            // v_cvt_pk_u8_f32: round half to even, clamp to [0, 255], NaN -> 0 in one instruction.  Checked against
            // the reference rule for all 2^32 float bit patterns (tests/test_gpu_exhaustive.py).
            return u8(__builtin_amdgcn_cvt_pk_u8_f32(s, 0u, 0u));
#endif
        } else if constexpr (is_float_v<S> && is_integer_v<D>) {
            // Branch free.  Round half to even under the default rounding mode (v_rndne_f32 / v_rndne_f64), then
            // clamp: fmax/fmin return the non-NaN operand, so NaN leaves the clamp as lo; for destination types whose
            // bounds are exact in S (8/16-bit) the clamp alone is the saturation.
            S r;
            if constexpr (sizeof(S) == 4) r = __builtin_rintf(s); else r = __builtin_rint(s);
            if constexpr (sizeof(D) <= 2) {
                if constexpr (sizeof(S) == 4) r = __builtin_fminf(__builtin_fmaxf(r, S(Lim<D>::lo)), S(Lim<D>::hi));
                else r = __builtin_fmin(__builtin_fmax(r, S(Lim<D>::lo)), S(Lim<D>::hi));
                const D v = static_cast<D>(static_cast<int>(r));
                return (s != s) ? D(0) : v;
            } else {
                const bool over = r >= S(Lim<D>::hi), under = r <= S(Lim<D>::lo), nan = s != s;
                const S safe = (over || under || nan) ? S(0) : r;
                const D v = static_cast<D>(safe);
                return nan ? D(0) : (over ? D(Lim<D>::hi) : (under ? D(Lim<D>::lo) : v));
            }
        } else if constexpr (is_integer_v<S> && is_integer_v<D>) {
            const long long v = (long long)s;
            return v > Lim<D>::hi ? D(Lim<D>::hi) : (v < Lim<D>::lo ? D(Lim<D>::lo) : D(s));
        } else {
            return static_cast<D>(s);
        }
    }
#endif
    FKD_DEV static O exec(const I& a, const Params&) {
#if defined(FKD_EXEC_CODE)
        return map1<O>(a, [](auto x) { return sat<decltype(x), base_t<O>>(x); });
#else
        (void)a; return O{};
#endif
    }
};

// Codes of the colour vocabulary: the enumerator values of fk::ColorDepth, fk::ColorRange and fk::ColorPrimitives
// (FK/algorithms/image_processing/itu_color.h:26-29).
enum : int { CD_P8 = 0, CD_P10 = 1, CD_P12 = 2, CD_FN8 = 3, CD_FN10 = 4, CD_FN12 = 5 };
enum : int { CR_LIMITED = 0, CR_FULL = 1 };
enum : int { CP_BT601 = 0, CP_BT709 = 1, CP_BT2020 = 2 };

// Per-depth constants: sample type, largest value, the luma/chroma offsets and the limited-range spans.
// FK/algorithms/image_processing/itu_color.h:103-183; the normalised-float depths divide the integer constants by the
// integer depth's largest value, in binary32.
template <int CD> struct DepthConsts;
template <> struct DepthConsts<CD_P8>  { using base = u8;  static constexpr f32 max_v = 255.f,  luma = 16.f,  chroma = 128.f,  limit_y = 219.f,  limit_c = 224.f; };
template <> struct DepthConsts<CD_P10> { using base = u16; static constexpr f32 max_v = 1023.f, luma = 64.f,  chroma = 512.f,  limit_y = 876.f,  limit_c = 896.f; };
template <> struct DepthConsts<CD_P12> { using base = u16; static constexpr f32 max_v = 4095.f, luma = 256.f, chroma = 2048.f, limit_y = 3504.f, limit_c = 3584.f; };
template <> struct DepthConsts<CD_FN8> {
    using base = f32;
    static constexpr f32 max_v = 1.f, luma = 16.f / 255.f, chroma = 128.f / 255.f, limit_y = 219.f / 255.f, limit_c = 224.f / 255.f;
};
template <> struct DepthConsts<CD_FN10> {
    using base = f32;
    static constexpr f32 max_v = 1.f, luma = 64.f / 1023.f, chroma = 512.f / 1023.f, limit_y = 876.f / 1023.f, limit_c = 896.f / 1023.f;
};
template <> struct DepthConsts<CD_FN12> {
    using base = f32;
    static constexpr f32 max_v = 1.f, luma = 256.f / 4095.f, chroma = 2048.f / 4095.f, limit_y = 3504.f / 4095.f, limit_c = 3584.f / 4095.f;
};

// computeMatrix<CR, CP, dir, CD>, FK/algorithms/image_processing/itu_color.h:185-265: the ITU matrix from the luma
// weights Kr, Kb of the primaries (itu_color.h:150-158), then the limited-range scaling of the luma and chroma
// columns (to RGB) or rows (to YCbCr).  All binary32, in the reference's expression order, evaluated at compile time.
struct ColorMatrix { f32 m[9]; };
constexpr f32 luma_weight_red(int cp) { return cp == CP_BT601 ? 0.299f : (cp == CP_BT709 ? 0.2126f : 0.2627f); }
constexpr f32 luma_weight_blue(int cp) { return cp == CP_BT601 ? 0.114f : (cp == CP_BT709 ? 0.0722f : 0.0593f); }
template <int CD, int CR, int CP, bool TO_RGB> constexpr ColorMatrix color_matrix() {
    static_assert(CP >= 0 && CP <= 2 && (CR == CR_LIMITED || CR == CR_FULL), "unknown colour primaries or range");
    constexpr f32 Kr = luma_weight_red(CP), Kb = luma_weight_blue(CP);
    constexpr f32 Kg = 1.0f - Kr - Kb;
    using D = DepthConsts<CD>;
    ColorMatrix c{};
    f32 (&m)[9] = c.m;
    if constexpr (TO_RGB) {
        m[0] = 1.0f; m[1] = 0.0f;                            m[2] = 2.0f * (1.0f - Kr);
        m[3] = 1.0f; m[4] = -2.0f * Kb * (1.0f - Kb) / Kg;   m[5] = -2.0f * Kr * (1.0f - Kr) / Kg;
        m[6] = 1.0f; m[7] = 2.0f * (1.0f - Kb);              m[8] = 0.0f;
        if constexpr (CR == CR_LIMITED) {
            constexpr f32 scale_y = D::max_v / D::limit_y, scale_c = D::max_v / D::limit_c;
            for (int r = 0; r < 3; ++r) { m[3 * r] *= scale_y; m[3 * r + 1] *= scale_c; m[3 * r + 2] *= scale_c; }
        }
    } else {
        m[0] = Kr;                          m[1] = Kg;                          m[2] = Kb;
        m[3] = -Kr / (2.0f * (1.0f - Kb));  m[4] = -Kg / (2.0f * (1.0f - Kb));  m[5] = 0.5f;
        m[6] = 0.5f;                        m[7] = -Kg / (2.0f * (1.0f - Kr));  m[8] = -Kb / (2.0f * (1.0f - Kr));
        if constexpr (CR == CR_LIMITED) {
            constexpr f32 scale_y = D::limit_y / D::max_v, scale_c = D::limit_c / D::max_v;
            for (int i = 0; i < 3; ++i) { m[i] *= scale_y; m[3 + i] *= scale_c; m[6 + i] *= scale_c; }
        }
    }
    return c;
}
// MxVFloat3<UnaryType>, FK/algorithms/basic_ops/algebraic.h:42-56: per row three products, (a + b) + c.
FKD_DEV Vec<f32, 3> color_mxv(const ColorMatrix& c, f32 a, f32 b, f32 d) {
    Vec<f32, 3> o;
    o.x = (a * c.m[0] + b * c.m[1]) + d * c.m[2];
    o.y = (a * c.m[3] + b * c.m[4]) + d * c.m[5];
    o.z = (a * c.m[6] + b * c.m[7]) + d * c.m[8];
    return o;
}

// ConvertYUVToRGB<CD, CR, CP>: FK/algorithms/image_processing/color_conversion.h:150-174.  (Y, Cb, Cr) minus the
// depth's offsets (luma only for limited range) times the matrix; no clamp.
template <int CD, int CR, int CP> struct YUV2RGB {
    using In = Vec<typename DepthConsts<CD>::base, 3>; using Out = Vec<f32, 3>; using Params = Empty;
    static constexpr bool kFiniteMap = true;
    FKD_NAME("YUV2RGB<" + istr(CD) + "," + istr(CR) + "," + istr(CP) + ">")
    FKD_DEV static Out exec(const In& a, const Params&) {
        using D = DepthConsts<CD>;
        constexpr ColorMatrix c = color_matrix<CD, CR, CP, true>();
        const f32 y = CR == CR_LIMITED ? f32(a.x) - D::luma : f32(a.x);
        return color_mxv(c, y, f32(a.y) - D::chroma, f32(a.z) - D::chroma);
    }
};

// ConvertRGBToYUV<CD, CR, CP>: FK/algorithms/image_processing/color_conversion.h:176-201.  Matrix times (R, G, B),
// then the depth's offsets are added (luma only for limited range); no rounding, no clamp.
template <int CD, int CR, int CP> struct RGB2YUV {
    using In = Vec<typename DepthConsts<CD>::base, 3>; using Out = Vec<f32, 3>; using Params = Empty;
    FKD_NAME("RGB2YUV<" + istr(CD) + "," + istr(CR) + "," + istr(CP) + ">")
    FKD_DEV static Out exec(const In& a, const Params&) {
        using D = DepthConsts<CD>;
        constexpr ColorMatrix c = color_matrix<CD, CR, CP, false>();
        Out o = color_mxv(c, f32(a.x), f32(a.y), f32(a.z));
        if constexpr (CR == CR_LIMITED) o.x = o.x + D::luma;
        o.y = o.y + D::chroma;
        o.z = o.z + D::chroma;
        return o;
    }
};

// RGB2Gray<I, O, CCIR_601>: FK/algorithms/image_processing/color_conversion.h:49-80.  (R*0.299f + G*0.587f) + B*0.114f in
// binary32, rounded to the nearest integer (ties to even) for EVERY output type: the reference tests is_unsigned,
// then is_signed, and float is a signed type, so its float branch is never taken and a float output holds the
// rounded value too.  Integer outputs then convert like a C cast of the rounded value.  A fourth input channel is
// ignored.
template <class I, class O> struct RGB2Gray {
    static_assert(cn_v<I> >= 3 && cn_v<O> == 1, "three or four channels in, one out");
    using In = I; using Out = O; using Params = Empty;
    FKD_NAME("RGB2Gray<" + type_name<I>() + "," + type_name<O>() + ">")
    FKD_DEV static O exec(const I& a, const Params&) {
        const f32 l = (f32(a.x) * 0.299f + f32(a.y) * 0.587f) + f32(a.z) * 0.114f;
        if constexpr (__is_same(O, f32) || __is_same(O, f64)) return O(__builtin_rintf(l));
        else if constexpr (O(-1) < O(0)) return O(int(__builtin_rintf(l)));
        else return O(u32(__builtin_rintf(l)));
    }
};

// AddLast<I, O> with a run-time value and AddOpaqueAlpha<I, CD> (value = largest of the depth):
// FK/algorithms/basic_ops/vector_ops.h:94-118, FK/algorithms/image_processing/color_conversion.h:81-93.
template <class I> struct AddLast {
    static_assert(cn_v<I> <= 3, "at most three channels in");
    using In = I; using Out = vec_t<base_t<I>, cn_v<I> + 1>;
    struct Params { base_t<I> last; };
    FKD_NAME("AddLast<" + type_name<I>() + ">")
    FKD_DEV static Out exec(const I& a, const Params& p) {
        Out o;
        chan<0>(o) = chan<0>(a);
        if constexpr (cn_v<I> > 1) chan<1>(o) = chan<1>(a);
        if constexpr (cn_v<I> > 2) chan<2>(o) = chan<2>(a);
        chan<cn_v<I>>(o) = p.last;
        return o;
    }
};

// VectorReduce<T, Operation>: the channels of the input folded left to right with a binary operation,
// op(op(x, y), z): FK/algorithms/basic_ops/vector_ops.h:82-92 -> cxp::vector_reduce, FK/core/constexpr_libs/
// constexpr_vector.h:94-110.  BinOp is one of Add/Sub/Mul on scalars (its parameter is the right-hand operand).
template <class T, class BinOp> struct VectorReduce {
    static_assert(cn_v<T> >= 2 && cn_v<typename BinOp::In> == 1 && cn_v<typename BinOp::Out> == 1, "a vector in, a scalar operation");
    using In = T; using Out = typename BinOp::Out; using Params = Empty;
    FKD_NAME("VectorReduce<" + type_name<T>() + "," + BinOp::name() + ">")
    FKD_DEV static Out exec(const T& a, const Params&) {
        using P = typename BinOp::Params;
        Out r = BinOp::exec(a.x, P{a.y});
        if constexpr (cn_v<T> > 2) r = BinOp::exec(r, P{a.z});
        if constexpr (cn_v<T> > 3) r = BinOp::exec(r, P{a.w});
        return r;
    }
};

// Discard<I, O>: the first cn<O> channels of the input.  FK/algorithms/basic_ops/vector_ops.h:22-41.
template <class I, class O> struct Discard {
    static_assert(cn_v<I> > cn_v<O> && __is_same(base_t<I>, base_t<O>), "fewer channels out, same sample type");
    using In = I; using Out = O; using Params = Empty;
    FKD_NAME("Discard<" + type_name<I>() + "," + type_name<O>() + ">")
    FKD_DEV static O exec(const I& a, const Params&) {
        O o;
        chan<0>(o) = chan<0>(a);
        if constexpr (cn_v<O> > 1) chan<1>(o) = chan<1>(a);
        if constexpr (cn_v<O> > 2) chan<2>(o) = chan<2>(a);
        return o;
    }
};

// Fold of compute operations over a value, left to right.  FK/core/execution_model/data_parallel_patterns.h:75-78.
// Saturate<T>: every channel clamped to [lo, hi] with the comparisons of cxp::clamp, (v < lo) ? lo : ((hi < v) ? hi : v),
// so a NaN channel stays NaN.  FK/algorithms/image_processing/saturate.h:38-49, FK/core/constexpr_libs/
// constexpr_cmath.h:60-62.  SaturateDepth<T, CD> is this with lo = 0 and hi = the depth's largest value
// (FK/algorithms/image_processing/color_conversion.h:96-107).
template <class T> struct Saturate {
    using In = T; using Out = T;
    struct Params { base_t<T> lo, hi; };
    FKD_NAME("Saturate<" + type_name<T>() + ">")
    FKD_DEV static T exec(const T& a, const Params& p) {
        return map1<T>(a, [&](auto v) { return (v < p.lo) ? p.lo : ((p.hi < v) ? p.hi : v); });
    }
};

// SaturateFloat<T>: every float channel through fmaxf(0, fminf(s, 1)), spelled with comparisons so that the special cases
// come out as on the reference's CPU backend (x86-64, glibc): NaN -> 1 (fminf returns its other operand), -0 stays -0
// (of two zeros fmaxf returns its second operand there), everything else clamped to [0, 1].
// FK/algorithms/image_processing/saturate.h:51-64, FK/core/constexpr_libs/constexpr_saturate.h:152-168.
template <class T> struct SaturateFloat {
    static_assert(__is_same(base_t<T>, f32), "Saturate float only works with float base types.");
    using In = T; using Out = T; using Params = Empty;
    FKD_NAME("SaturateFloat<" + type_name<T>() + ">")
    FKD_DEV static f32 unit(f32 s) {
        const f32 t = (s < 1.f) ? s : 1.f;
        return (t < 0.f) ? 0.f : t;
    }
    FKD_DEV static T exec(const T& a, const Params&) { return map1<T>(a, [](f32 v) { return unit(v); }); }
};

// DenormalizePixel<O, CD>: float channels times the depth's largest value, converted to O's channel type like a C cast
// (truncation toward zero; the product must be representable, which it is for inputs in [0, 1]).
// FK/algorithms/image_processing/color_conversion.h:109-121.
template <class O, int CD> struct DenormalizePixel {
    using In = vec_t<f32, cn_v<O>>; using Out = O; using Params = Empty;
    FKD_NAME("DenormalizePixel<" + type_name<O>() + "," + istr(CD) + ">")
    FKD_DEV static O exec(const In& a, const Params&) {
        return map1<O>(a, [](f32 v) { return static_cast<base_t<O>>(v * DepthConsts<CD>::max_v); });
    }
};

// SaturateDenormalizePixel<I, O, CD>: SaturateFloat, then DenormalizePixel.
// FK/algorithms/image_processing/color_conversion.h:136-148.
template <class I, class O, int CD> struct SaturateDenormalizePixel {
    static_assert(__is_same(base_t<I>, f32) && cn_v<I> == cn_v<O>, "SaturateDenormalizePixel only works with float base types.");
    using In = I; using Out = O; using Params = Empty;
    FKD_NAME("SaturateDenormalizePixel<" + type_name<I>() + "," + type_name<O>() + "," + istr(CD) + ">")
    FKD_DEV static O exec(const I& a, const Params&) {
        return map1<O>(a, [](f32 v) { return static_cast<base_t<O>>(SaturateFloat<f32>::unit(v) * DepthConsts<CD>::max_v); });
    }
};

template <class... Ops> struct OpList {
    using Params = Tup<typename Ops::Params...>;
#if defined(FKD_HOST_NAMES)
    static std::string names() { std::string s; ((s += "," + Ops::name()), ...); return s; }
#endif
};
template <class In, class... Ops> struct FoldOut { using type = In; };
template <class In, class Op, class... Rest> struct FoldOut<In, Op, Rest...> {
    using type = typename FoldOut<typename Op::Out, Rest...>::type;
    using first_in = typename Op::In;
};
#if defined(FKD_EXEC_CODE)
template <class V> FKD_DEV V fold(const V& v, const Tup<>&) { return v; }
template <class Op, class... Rest, class V>
FKD_DEV auto fold(const V& v, const Tup<typename Op::Params, typename Rest::Params...>& p) {
    static_assert(__is_same(V, typename Op::In), "operation input type does not match the value it receives");
    if constexpr (sizeof...(Rest) == 0) return Op::exec(v, p.head);
    else return fold<Rest...>(Op::exec(v, p.head), p.tail);
}
#endif
#if defined(FKD_DEVICE_CODE)

// The same fold through each operation's straight-line variant where it has one (see Div).  `ok` comes back false
// when some operation could not vouch for its quick result; the value must then be recomputed with fold().
template <class Op> constexpr bool has_quick() {
    if constexpr (requires { Op::kQuick; }) return Op::kQuick; else return false;
}
template <class... Ops> constexpr bool any_quick() { return (false || ... || has_quick<Ops>()); }
template <class V> FKD_DEV V fold_quick(const V& v, const Tup<>&, bool&) { return v; }
template <class Op, class... Rest, class V>
FKD_DEV auto fold_quick(const V& v, const Tup<typename Op::Params, typename Rest::Params...>& p, bool& ok) {
    auto step = [&] {
        if constexpr (has_quick<Op>()) return Op::exec_quick(v, p.head, ok); else return Op::exec(v, p.head);
    };
    if constexpr (sizeof...(Rest) == 0) return step();
    else return fold_quick<Rest...>(step(), p.tail, ok);
}

// The fold with every quick operation in its static form (see Div), and whether the parameters allow it.
template <class V> FKD_DEV V fold_static(const V& v, const Tup<>&) { return v; }
template <class Op, class... Rest, class V>
FKD_DEV auto fold_static(const V& v, const Tup<typename Op::Params, typename Rest::Params...>& p) {
    auto step = [&] {
        if constexpr (has_quick<Op>()) return Op::exec_static(v, p.head); else return Op::exec(v, p.head);
    };
    if constexpr (sizeof...(Rest) == 0) return step();
    else return fold_static<Rest...>(step(), p.tail);
}
FKD_DEV bool all_static(const Tup<>&) { return true; }
template <class Op, class... Rest>
FKD_DEV bool all_static_of(const Tup<typename Op::Params, typename Rest::Params...>& p) {
    bool here = true;
    if constexpr (has_quick<Op>()) here = Op::is_static(p.head);
    if constexpr (sizeof...(Rest) == 0) return here;
    else return here && all_static_of<Rest...>(p.tail);
}

// The fold over a run of N elements, operation by operation: every element goes through operation k before any
// goes through operation k+1.  A long chain then needs each operation's parameters (scalar registers) only once and
// only briefly, instead of all parameters of the chain at the same time for every element.
// QUICK: 0 every operation as written, 1 quick forms that report doubtful elements through `ok`, 2 static forms.
//
// An instruction with a scalar-register operand issues at half the rate of one whose operands are all vector registers
// (4.7 against 2.45 cycles per SIMD on this chip), and an operation's launch constants arrive in scalar registers.  A
// thread that puts N >= 4 elements through the operation therefore copies constants that are nothing but operands
// (Add, Sub, Mul: kValueParams) into vector registers first: one half-rate copy per constant and wave buys N full-rate
// instructions.  (The 50- and 100-operation float chains over a 4K image were bound by exactly this: 15.5 -> 11.6 us and 26.7 -> 18.2 us;
// what remains is 4.7 us of launch, first loads and last stores plus 0.135 us per operation, the full issue rate.)
template <class Op, int N> constexpr bool vector_params() {
    if constexpr (requires { Op::kValueParams; })
        return Op::kValueParams && N >= 4 && sizeof(typename Op::Params) % 4 == 0 && sizeof(typename Op::Params) <= 16;
    else return false;
}
#if defined(FKD_DEVICE_CODE)
template <class P> FKD_DEV P in_vector_registers(const P& p) {
    constexpr int W = int(sizeof(P)) / 4;
    u32 w[W];
    __builtin_memcpy(w, &p, sizeof(P));
#pragma unroll
    for (int i = 0; i < W; ++i) asm volatile("" : "+v"(w[i]));
    P o;
    __builtin_memcpy(&o, w, sizeof(P));
    return o;
}
#endif
template <int QUICK, int N, class V> FKD_DEV void fold_run(const Slot<V> (&in)[N], Slot<V> (&out)[N], const Tup<>&, bool&) {
#pragma unroll
    for (int i = 0; i < N; ++i) out[i].v = in[i].v;
}
template <int QUICK, class Op, class... Rest, int N, class V, class O>
FKD_DEV void fold_run(const Slot<V> (&in)[N], Slot<O> (&out)[N], const Tup<typename Op::Params, typename Rest::Params...>& p, bool& ok) {
    static_assert(__is_same(V, typename Op::In), "operation input type does not match the value it receives");
    typename Op::Params head = p.head;
#if defined(FKD_DEVICE_CODE)
    if constexpr (vector_params<Op, N>()) head = in_vector_registers(head);
#endif
    auto step = [&](const V& v) {
        if constexpr (QUICK == 2 && has_quick<Op>()) return Op::exec_static(v, head);
        else if constexpr (QUICK == 1 && has_quick<Op>()) return Op::exec_quick(v, head, ok);
        else return Op::exec(v, head);
    };
    if constexpr (sizeof...(Rest) == 0) {
#pragma unroll
        for (int i = 0; i < N; ++i) out[i].v = step(in[i].v);
    } else {
        Slot<typename Op::Out> mid[N];
#pragma unroll
        for (int i = 0; i < N; ++i) mid[i].v = step(in[i].v);
        fold_run<QUICK, Rest...>(mid, out, p.tail, ok);
    }
}

// fold_run for long chains, reading the parameters from the kernel-argument segment where they are used.  Left to
// itself the compiler fetches every kernel argument at the top of the kernel; a chain of 100 operations then holds
// 100+ scalar registers at once and spills them into vector-register lanes (one v_readlane per use).  Here the
// pointer into the segment is made opaque every kGroup operations, so only one group's parameters are live.
#define FKD_CONSTANT __attribute__((address_space(4)))
constexpr int kParamGroup = 16;
template <class B> FKD_DEV void pin_base(B& b) {
    if constexpr (sizeof(B) == 4) { asm volatile("" : "+v"(b)); }
    else if constexpr (sizeof(B) < 4) { u32 w = detail::to_bits(b); asm volatile("" : "+v"(w)); b = __builtin_bit_cast(B, decltype(detail::to_bits(b))(w)); }
    else { unsigned long long w = __builtin_bit_cast(unsigned long long, b); asm volatile("" : "+v"(w)); b = __builtin_bit_cast(B, w); }
}
// A channel value the optimiser may not look behind (free to schedule, unlike pin_base): keeps it from gluing the channels
// of several 12-byte values into odd-sized vectors (<6 x float>) that it can then only shuffle through memory.
template <class B> FKD_DEV B opaque(B b) {
    if constexpr (sizeof(B) == 4) asm("" : "+v"(b));
    return b;
}
constexpr int kSharedValues = 8;      // access-mode bit: see TeeWrite
template <bool OPAQUE, class B> FKD_DEV B maybe_opaque(B b) {
    if constexpr (OPAQUE) return opaque(b); else return b;
}
template <class V> FKD_DEV void pin_value(V& v) {
    pin_base(chan<0>(v));
    if constexpr (cn_v<V> > 1) pin_base(chan<1>(v));
    if constexpr (cn_v<V> > 2) pin_base(chan<2>(v));
    if constexpr (cn_v<V> > 3) pin_base(chan<3>(v));
}
template <bool QUICK, int IDX, int N, class V> FKD_DEV void fold_run_k(const Slot<V> (&in)[N], Slot<V> (&out)[N], const FKD_CONSTANT Tup<>*, bool&) {
#pragma unroll
    for (int i = 0; i < N; ++i) out[i].v = in[i].v;
}
template <bool QUICK, int IDX, class Op, class... Rest, int N, class V, class O>
FKD_DEV void fold_run_k(const Slot<V> (&in)[N], Slot<O> (&out)[N],
                        const FKD_CONSTANT Tup<typename Op::Params, typename Rest::Params...>* pk, bool& ok) {
    static_assert(__is_same(V, typename Op::In), "operation input type does not match the value it receives");
    if constexpr (IDX % kParamGroup == 0) {
        // Every element finishes the previous group before the next group's parameters are touched: the values
        // pass through ordered opaque points, and so does the parameter pointer, which is then declared wave
        // uniform again so the reads stay scalar loads.
        if constexpr (IDX > 0) {
#pragma unroll
            for (int i = 0; i < N; ++i) pin_value(const_cast<Slot<V>&>(in[i]).v);
        }
        unsigned long long a = reinterpret_cast<unsigned long long>(pk);
        asm volatile("" : "+s"(a));
        const u32 lo = __builtin_amdgcn_readfirstlane(u32(a)), hi = __builtin_amdgcn_readfirstlane(u32(a >> 32));
        pk = reinterpret_cast<decltype(pk)>((unsigned long long)lo | ((unsigned long long)hi << 32));
    }
    typename Op::Params head;
    if constexpr (!__is_empty(typename Op::Params))
        __builtin_memcpy(&head, __builtin_assume_aligned((const void*)&pk->head, 4), sizeof(head));   // dword aligned: scalar loads
    if constexpr (vector_params<Op, N>()) head = in_vector_registers(head);
    auto step = [&](const V& v) {
        if constexpr (QUICK && has_quick<Op>()) return Op::exec_quick(v, head, ok); else return Op::exec(v, head);
    };
    if constexpr (sizeof...(Rest) == 0) {
#pragma unroll
        for (int i = 0; i < N; ++i) out[i].v = step(in[i].v);
    } else {
        Slot<typename Op::Out> mid[N];
#pragma unroll
        for (int i = 0; i < N; ++i) mid[i].v = step(in[i].v);
        fold_run_k<QUICK, IDX + 1, Rest...>(mid, out, &pk->tail, ok);
    }
}
#endif

// A run of compute operations packaged as one (host side: FusedOperation of compute IOps).
template <class... Ops> struct FusedCompute {
    using In = typename FoldOut<void, Ops...>::first_in;
    using Out = typename FoldOut<In, Ops...>::type;
    using Params = Tup<typename Ops::Params...>;
    FKD_NAME("FusedCompute<" + OpList<Ops...>::names().substr(1) + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static Out exec(const In& a, const Params& p) { return fold<Ops...>(a, p); }
#endif
};

// ===================================================================================================
// Read operations: (x, y, z) -> Out.  width()/height() give the extent a consumer may address.
// ===================================================================================================

// PerThreadRead<_2D,T>: FK/algorithms/basic_ops/memory_operations.h:26-67, addressing FK/core/data/rawptr.h:202-213.
template <class T> struct Read2D {
    using Out = T;
    using Params = RawPtr2D<const T>;
    static constexpr bool kTapCursor = true;
    static constexpr bool kFiniteTaps = !(__is_same(base_t<T>, f32) || __is_same(base_t<T>, f64));
    static constexpr bool kBoundedOut = small_integer_base<T>();
    FKD_NAME("Read2D<" + type_name<T>() + ">")
    // What the strip form of the bilinear kernel asks of a source image (checked on the host, see Chain::finalize): rows
    // that share their alignment, byte offsets below 2 GB (the offset 2 GB itself marks a column without a window), two
    // columns.
    FKD_HD static bool strip_ok(const Params& p) {
        return p.pitch % 4 == 0 && size_t(p.pitch) * p.height < 0x7ffffff0ull && p.width >= 2 && p.height >= 1;
    }
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return int(p.width); }
    FKD_DEV static int height(const Params& p) { return int(p.height); }
    FKD_DEV static T exec(int x, int y, int, const Params& p) {
        return detail::load_elem(detail::row_ptr(p.data, p.pitch, x, y));
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int, const Params& p, Slot<T> (&out)[V]) {
        detail::load_run<T, V, A>(detail::row_ptr(p.data, p.pitch, x, y), out);
    }
    // True when every row start (shifted by xoff elements) is dword aligned: the launcher's licence to use
    // the wide-access kernel variant.
    FKD_HD static bool rows_aligned(const Params& p, int xoff) {
        return detail::dword_aligned(reinterpret_cast<const char*>(p.data) + ptrdiff_t(xoff) * ptrdiff_t(sizeof(T))) && p.pitch % 4 == 0;
    }
    using Raw = T;
    FKD_DEV static T finish(const Raw& r, const Params&) { return r; }
    // Tap cursor for gathers: the address of element (x0, y), wave uniform when y is; tap_load adds a 32-bit byte
    // offset and returns the element's raw bits, tap_value takes them apart where they are used.  `last` marks
    // rows so close to the end of the image that reading a few bytes past an element could leave the allocation
    // (the last row, for any image wider than two pixels); kTapOverread says whether tap_load<true> or pair_load
    // read past elements at all.
    static constexpr bool kTapOverread = detail::overread_bytes<T, 1>() > 0 || detail::PairWindow<T>::kShift;
    struct TapRow { const char* p; bool last; };
    FKD_DEV static TapRow tap_row(int x0, int y, int, const Params& p) {
        // bytes of the image after this row's start that an over-reading access could lean on
        const bool last = size_t(int(p.height) - 1 - y) * p.pitch < 8;
        return TapRow{reinterpret_cast<const char*>(detail::row_ptr(p.data, p.pitch, x0, y)), last};
    }
    FKD_DEV static bool tap_last(const TapRow& r) { return r.last; }
    using TapBits = detail::RunBits<T, 1>;
    template <bool OVER> FKD_DEV static TapBits tap_load(const TapRow& r, int x, const Params&) {
        return detail::load_bits_at<T, 1, OVER>(r.p, u32(x) * u32(sizeof(T)));
    }
    FKD_DEV static Raw tap_value(const TapBits& b) { return detail::run_value<0>(b); }
    // Elements x and x+1 in one access (both must exist); may read up to 6 bytes past them.
    static constexpr bool kTapPair = detail::PairWindow<T>::kSupported;
    using PairBits = detail::PairWindow<T>;
    FKD_DEV static PairBits pair_load(const TapRow& r, int x, const Params&) {
        return detail::load_pair_window<T>(r.p, u32(x) * u32(sizeof(T)));
    }
    FKD_DEV static void pair_values(const PairBits& b, const TapRow&, int, Raw& first, Raw& second) {
        detail::pair_window_values<false, T>(b, first, second);
    }
    // The same with lanes (`dup`) that take the second element for both values.
    FKD_DEV static void pair_values_dup(const PairBits& b, bool dup, Raw& first, Raw& second) {
        detail::pair_window_values<true, T>(b, first, second, dup);
    }
    // Buffer-resource form of pair_load for images whose rows share their alignment (see detail::TapImage): the image
    // once per wave, a prepared column once per lane, a scalar offset per row.
    static constexpr bool kTapPrepared = true;
    FKD_DEV static bool tap_rows_share_alignment(const Params& p) { return p.pitch % 4 == 0 && size_t(p.pitch) * p.height < 0xfffffff0ull; }
    // Every byte offset inside the image fits 32 bits (the buffer-resource forms of the tap accesses).
    FKD_DEV static bool tap_offsets_fit(const Params& p) { return size_t(p.pitch) * p.height < 0xfffffff0ull; }
    using TapImage = detail::TapImage;
    using PairPrep = detail::PairPrep;
    FKD_DEV static TapImage tap_image(int, const Params& p) { return detail::make_tap_image(p.data); }
    // The same image with the resource's extent closed at the dword that holds the image's last byte: a window that
    // reaches past it reads zeros instead of memory (the address check works dword by dword), so lanes on the last
    // rows need no other form of access.
    FKD_DEV static TapImage tap_image_bounded(int, const Params& p) {
        return detail::make_tap_image(p.data, size_t(p.pitch) * (p.height - 1) + size_t(p.width) * sizeof(T));
    }
    FKD_DEV static u32 tap_row_offset(int y, const Params& p) { return u32(y) * p.pitch; }
    FKD_DEV static PairPrep pair_prepare(const TapImage& im, int x, const Params&) {
        return detail::prepare_pair_window<T>(im, u32(x) * u32(sizeof(T)));
    }
    FKD_DEV static PairBits pair_load_prepared(const TapImage& im, u32 row_off, const PairPrep& pp, const Params&) {
        return detail::load_prepared_pair_window<T>(im, row_off, pp);
    }
#endif
};

// TensorRead<T> / PerThreadRead<_3D,T>: FK/algorithms/basic_ops/memory_operations.h:124-157,
// addressing FK/core/data/rawptr.h:215-226.
template <class T> struct Read3D {
    using Out = T;
    using Params = RawPtr3D<const T>;
    static constexpr bool kTapCursor = false;
    static constexpr bool kBoundedOut = small_integer_base<T>();
    FKD_NAME("Read3D<" + type_name<T>() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return int(p.width); }
    FKD_DEV static int height(const Params& p) { return int(p.height); }
    FKD_DEV static const T* plane(const Params& p, int z) {
        return reinterpret_cast<const T*>(reinterpret_cast<const char*>(p.data) + size_t(p.plane_pitch) * p.color_planes * z);
    }
    FKD_DEV static T exec(int x, int y, int z, const Params& p) {
        return detail::load_elem(detail::row_ptr(plane(p, z), p.pitch, x, y));
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<T> (&out)[V]) {
        detail::load_run<T, V, A>(detail::row_ptr(plane(p, z), p.pitch, x, y), out);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) {
        return detail::dword_aligned(reinterpret_cast<const char*>(p.data) + ptrdiff_t(xoff) * ptrdiff_t(sizeof(T))) && p.pitch % 4 == 0 &&
               (size_t(p.plane_pitch) * p.color_planes) % 4 == 0;
    }
#endif
};

// Where the channel planes of a planar tensor lie.  Standard (TensorSplit / TensorPack, FK/core/data/rawptr.h:215-227):
// image z starts z * plane_pitch * color_planes bytes into the tensor and channel c of a pixel sits c * width * height
// elements after channel 0.  Transposed (TensorTSplit / TensorTPack, FK/core/data/rawptr.h:229-240): image z starts
// z * plane_pitch bytes in and channel c sits c * color_planes_pitch bytes after channel 0 (a multiple of the element
// size: rows are whole elements).
namespace detail {
template <class B, bool TRANSPOSED> struct PlanarGeometry;
template <class B> struct PlanarGeometry<B, false> {
    template <class E> using View = RawPtr3D<E>;
    template <class P> FKD_HD static size_t image_bytes(const P& p) { return size_t(p.plane_pitch) * p.color_planes; }
    template <class P> FKD_HD static size_t channel_elements(const P& p) { return size_t(p.width) * p.height; }
};
template <class B> struct PlanarGeometry<B, true> {
    template <class E> using View = RawPtrT3D<E>;
    template <class P> FKD_HD static size_t image_bytes(const P& p) { return size_t(p.plane_pitch); }
    template <class P> FKD_HD static size_t channel_elements(const P& p) { return size_t(p.color_planes_pitch) / sizeof(B); }
};
} // namespace detail

// TensorPack<T>: FK/algorithms/basic_ops/memory_operations.h:243-290, and TensorTPack<T> (TRANSPOSED), :292-327.  The
// planar layout TensorSplit / TensorTSplit writes, read back as a vector.
template <class T, bool TRANSPOSED = false> struct TensorPack {
    static_assert(cn_v<T> >= 2, "Wrong type for split tensor read. It must be one of <type>2, <type>3 or <type>4.");
    using Out = T;
    using B = base_t<T>;
    using G = detail::PlanarGeometry<B, TRANSPOSED>;
    using Params = typename G::template View<const B>;
    static constexpr bool kTapCursor = false;
    FKD_NAME((TRANSPOSED ? "TensorTPack<" : "TensorPack<") + type_name<T>() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return int(p.width); }
    FKD_DEV static int height(const Params& p) { return int(p.height); }
    FKD_DEV static const B* at(const Params& p, int x, int y, int z) {
        return reinterpret_cast<const B*>(reinterpret_cast<const char*>(p.data) + G::image_bytes(p) * z + size_t(y) * p.pitch) + x;
    }
    FKD_DEV static T exec(int x, int y, int z, const Params& p) {
        const FKD_GLOBAL B* g = detail::gconst<B>(at(p, x, y, z));
        const size_t px = G::channel_elements(p);
        T o;
        chan<0>(o) = g[0];
        chan<1>(o) = g[px];
        if constexpr (cn_v<T> > 2) chan<2>(o) = g[2 * px];
        if constexpr (cn_v<T> > 3) chan<3>(o) = g[3 * px];
        return o;
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<T> (&out)[V]) {
        const B* r = at(p, x, y, z);
        const size_t px = G::channel_elements(p);
        Slot<B> c[4][V];
        detail::load_run<B, V, A>(r, c[0]);
        detail::load_run<B, V, A>(r + px, c[1]);
        if constexpr (cn_v<T> > 2) detail::load_run<B, V, A>(r + 2 * px, c[2]);
        if constexpr (cn_v<T> > 3) detail::load_run<B, V, A>(r + 3 * px, c[3]);
#pragma unroll
        for (int i = 0; i < V; ++i) {
            chan<0>(out[i].v) = c[0][i].v;
            chan<1>(out[i].v) = c[1][i].v;
            if constexpr (cn_v<T> > 2) chan<2>(out[i].v) = c[2][i].v;
            if constexpr (cn_v<T> > 3) chan<3>(out[i].v) = c[3][i].v;
        }
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) {
        return detail::dword_aligned(reinterpret_cast<const char*>(p.data) + ptrdiff_t(xoff) * ptrdiff_t(sizeof(B))) && p.pitch % 4 == 0 &&
               G::image_bytes(p) % 4 == 0 && (G::channel_elements(p) * sizeof(B)) % 4 == 0;
    }
    using Raw = Out;
    FKD_DEV static Out finish(const Raw& r, const Params&) { return r; }
    struct TapRow {}; struct TapBits {}; struct PairBits {};
    static constexpr bool kTapOverread = false, kTapPair = false;
#endif
};

template <class T> using TensorTPack = TensorPack<T, true>;

// Plane index of a circular buffer of BATCH planes whose logical plane 0 is stored at `first`:
// computeCircularThreadIdx, FK/algorithms/basic_ops/memory_operations.h:422-432.  DIR 0 (Ascendent) walks forward from
// first, DIR 1 (Descendent) backward.
template <int DIR, int BATCH> FKD_HD int circular_plane(int z, int first) {
    if constexpr (DIR == 0) { const int c = z + first; return c >= BATCH ? c - BATCH : c; }
    else { const int c = first - z; return c < 0 ? BATCH + c : c; }
}

// CircularTensorRead<direction, Operation, BATCH>: FK/algorithms/basic_ops/memory_operations.h:505-552.
template <int DIR, int BATCH, class Back> struct CircularRead {
    using Out = typename Back::Out;
    struct Params { i32 first; typename Back::Params back; };
    static constexpr bool kTapCursor = false;
    FKD_NAME("CircularRead<" + istr(DIR) + "," + istr(BATCH) + "," + Back::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return Back::width(p.back); }
    FKD_DEV static int height(const Params& p) { return Back::height(p.back); }
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) { return Back::exec(x, y, circular_plane<DIR, BATCH>(z, p.first), p.back); }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        Back::template exec_row<V, A>(x, y, circular_plane<DIR, BATCH>(z, p.first), p.back, out);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return Back::rows_aligned(p.back, xoff); }
    using Raw = Out;
    FKD_DEV static Out finish(const Raw& r, const Params&) { return r; }
    struct TapRow {}; struct TapBits {}; struct PairBits {};
    static constexpr bool kTapOverread = false, kTapPair = false;
#endif
};

// CircularBatchRead<direction, Operation, BATCH>: FK/algorithms/basic_ops/memory_operations.h:434-474.  BATCH separate
// reads used as a circular buffer: logical plane z is read number circular_plane(z).
template <int DIR, int BATCH, class PlaneOp> struct CircularBatchRead {
    using Out = typename PlaneOp::Out;
    struct Params { i32 first; typename PlaneOp::Params plane[BATCH]; };
    static constexpr bool kTapCursor = false;
    FKD_NAME("CircularBatchRead<" + istr(DIR) + "," + istr(BATCH) + "," + PlaneOp::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return PlaneOp::width(p.plane[0]); }
    FKD_DEV static int height(const Params& p) { return PlaneOp::height(p.plane[0]); }
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        const int c = circular_plane<DIR, BATCH>(z, p.first);
        return PlaneOp::exec(x, y, c, p.plane[c]);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        const int c = circular_plane<DIR, BATCH>(z, p.first);
        PlaneOp::template exec_row<V, A>(x, y, c, p.plane[c], out);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) {
        for (int i = 0; i < BATCH; ++i) if (!PlaneOp::rows_aligned(p.plane[i], xoff)) return false;
        return true;
    }
    FKD_HD static bool plane_rows_aligned(const Params& p, int z, int xoff) {
        return PlaneOp::rows_aligned(p.plane[circular_plane<DIR, BATCH>(z, p.first)], xoff);
    }
#endif
};

// ReadYUV<NV12> and ReadYUV<NV21>: FK/algorithms/image_processing/color_conversion.h:219-253.  Y from the luma
// plane, the chroma pair from element x>>1 of chroma row y>>1; chroma base = data + pitch*height.  NV12 stores the
// pair as (U,V), NV21 as (V,U) (template argument VU); the value is (Y,U,V) either way.
template <bool VU> struct ReadNV {
    using Out = Vec<u8, 3>;
    using Params = RawNV12;
    static constexpr bool kTapCursor = true;
    static constexpr bool kFiniteTaps = true;
    static constexpr bool kBoundedOut = true;
    FKD_NAME(VU ? "ReadNV21" : "ReadNV12")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return int(p.width); }
    FKD_DEV static int height(const Params& p) { return int(p.height); }
    FKD_DEV static Out exec(int x, int y, int, const Params& p) {
        Out o;
        o.x = *detail::gconst<u8>(p.data + size_t(y) * p.pitch + x);
        const FKD_GLOBAL u8* c = detail::gconst<u8>(p.data + size_t(p.pitch) * p.height + size_t(y >> 1) * p.pitch + 2 * (x >> 1));
        o.y = c[VU ? 1 : 0];
        o.z = c[VU ? 0 : 1];
        return o;
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        if constexpr (V == 4 && (A & 3) != 0) {
            // four pixels: their luma is one dword, their two chroma pairs another (x is a multiple of four here)
            const u32 luma = *detail::gconst<u32>(p.data + size_t(y) * p.pitch + x);
            u32 uv = *detail::gconst<u32>(p.data + size_t(p.pitch) * p.height + size_t(y >> 1) * p.pitch + x);
            u32 l = luma;
            asm("" : "+v"(l), "+v"(uv));     // keep the dwords whole: bytes leave through v_cvt_f32_ubyteN / v_bfe
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32 pair = uv >> (16 * (i >> 1));
                out[i].v.x = u8((l >> (8 * i)) & 0xffu);
                out[i].v.y = u8((pair >> (VU ? 8 : 0)) & 0xffu);
                out[i].v.z = u8((pair >> (VU ? 0 : 8)) & 0xffu);
            }
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) out[i].v = exec(x + i, y, z, p);
        }
    }
    using Raw = Out;
    FKD_DEV static Out finish(const Raw& r, const Params&) { return r; }
    // Whole-dword row reads need luma and chroma rows that start on dword boundaries and a run that starts on a group of four.
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return detail::dword_aligned(p.data) && p.pitch % 4 == 0 && xoff % 4 == 0; }
    static constexpr bool kTapOverread = true;    // pair_load only; tap_load reads exact bytes
    struct TapRow { const char* luma; const char* chroma; int x0; bool last; };
    FKD_DEV static TapRow tap_row(int x0, int y, int, const Params& p) {
        const char* d = reinterpret_cast<const char*>(p.data);
        return TapRow{d + size_t(y) * p.pitch, d + size_t(p.pitch) * p.height + size_t(y >> 1) * p.pitch, x0,
                      (y >> 1) >= int(p.height >> 1) - 1};
    }
    FKD_DEV static bool tap_last(const TapRow& r) { return r.last; }
    struct TapBits { u32 y, uv; };
    template <bool OVER> FKD_DEV static TapBits tap_load(const TapRow& r, int x, const Params&) {
        u32 xs = u32(r.x0 + x), xc = xs & ~1u;
        asm volatile("" : "+v"(xs), "+v"(xc));      // 32-bit lane offsets against scalar row addresses
        TapBits b;
        b.y = u32(*detail::gconst<u8>(r.luma + xs));
        b.uv = u32(*detail::gconst<detail::u16_a1>(r.chroma + xc));   // (U,V) pair in one access
        return b;
    }
    FKD_DEV static Raw tap_value(const TapBits& b) {
        Out o;
        o.x = u8(b.y);
        o.y = u8(VU ? b.uv >> 8 : b.uv & 0xffu);
        o.z = u8(VU ? b.uv & 0xffu : b.uv >> 8);
        return o;
    }
    // Pixels x and x+1: two luma bytes in one access, and the dword at chroma pair x>>1, which holds the pair of
    // pixel x in its low half and, when x is odd, the pair of pixel x+1 in its high half (x even: same pair).  The
    // dword reaches one chroma pair past the one needed, hence the over-read flag on the last chroma row.
    static constexpr bool kTapPair = true;
    struct PairBits { u32 y, uv; };
    FKD_DEV static PairBits pair_load(const TapRow& r, int x, const Params&) {
        u32 xs = u32(r.x0 + x), xc = xs & ~1u;
        asm volatile("" : "+v"(xs), "+v"(xc));
        PairBits b;
        b.y = u32(*detail::gconst<detail::u16_a1>(r.luma + xs));
        b.uv = *detail::gconst<detail::u32_a1>(r.chroma + xc);
        return b;
    }
    FKD_DEV static void pair_values(const PairBits& b, const TapRow& r, int x, Raw& first, Raw& second) {
        first.x = u8(b.y & 0xffu);
        first.y = u8((b.uv >> (VU ? 8 : 0)) & 0xffu);
        first.z = u8((b.uv >> (VU ? 0 : 8)) & 0xffu);
        const u32 uv = b.uv >> ((u32(r.x0 + x) & 1u) * 16u);
        second.x = u8((b.y >> 8) & 0xffu);
        second.y = u8((uv >> (VU ? 8 : 0)) & 0xffu);
        second.z = u8((uv >> (VU ? 0 : 8)) & 0xffu);
    }
#endif
};
using ReadNV12 = ReadNV<false>;
using ReadNV21 = ReadNV<true>;

// Pixel-format codes: the enumerator values of fk::PixelFormat (FK/algorithms/image_processing/itu_color.h:51).
enum : int { PF_NV12 = 0, PF_NV21 = 1, PF_P010 = 3, PF_P210 = 6, PF_Y210 = 8, PF_UYVY = 10 };
template <int PF> struct PixelLayout {
    static_assert(PF == PF_NV12 || PF == PF_NV21 || PF == PF_P010 || PF == PF_P210 || PF == PF_Y210 || PF == PF_UYVY,
                  "pixel format without a reader/writer in the reference (YV12, P016, P216, Y216) or whose reader does not compile there (Y416)");
    static constexpr bool kSemiPlanar = PF == PF_NV12 || PF == PF_NV21 || PF == PF_P010 || PF == PF_P210;
    static constexpr bool k420 = PF == PF_NV12 || PF == PF_NV21 || PF == PF_P010;
    static constexpr bool kWide = PF == PF_P010 || PF == PF_P210 || PF == PF_Y210;     // 16-bit samples
    static constexpr bool kSwapUV = PF == PF_NV21;
};
template <int PF> struct PixelBase { using type = u8; };
template <> struct PixelBase<PF_P010> { using type = u16; };
template <> struct PixelBase<PF_P210> { using type = u16; };
template <> struct PixelBase<PF_Y210> { using type = u16; };

// ReadYUV<P010 | P210 | Y210 | UYVY>: FK/algorithms/image_processing/color_conversion.h:219-268.  Semi-planar formats
// (P010 4:2:0, P210 4:2:2): Y at (x, y) of the luma plane, the (U,V) pair at element x>>1 of chroma row y>>1 (4:2:0) or
// y (4:2:2), chroma base = data + pitch*height.  Packed 4:2:2: the four-sample group x>>1 of row y holds U Y0 V Y1
// (UYVY) or Y0 U Y1 V (Y210); even pixels take the first luma sample, odd ones the second.
template <int PF> struct ReadYUV {
    using L = PixelLayout<PF>;
    using B = typename PixelBase<PF>::type;
    using Out = Vec<B, 3>;
    using Params = RawYUV;
    static constexpr bool kTapCursor = false;
    FKD_NAME("ReadYUV<" + istr(PF) + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return int(p.width); }
    FKD_DEV static int height(const Params& p) { return int(p.height); }
    FKD_DEV static Out exec(int x, int y, int, const Params& p) {
        Out o;
        if constexpr (L::kSemiPlanar) {
            o.x = *detail::gconst<B>(p.data + size_t(y) * p.pitch + size_t(x) * sizeof(B));
            const int cy = L::k420 ? y >> 1 : y;
            const FKD_GLOBAL B* c = detail::gconst<B>(p.data + size_t(p.pitch) * p.height + size_t(cy) * p.pitch + size_t(x >> 1) * 2 * sizeof(B));
            o.y = c[L::kSwapUV ? 1 : 0];
            o.z = c[L::kSwapUV ? 0 : 1];
        } else {
            const FKD_GLOBAL B* g = detail::gconst<B>(p.data + size_t(y) * p.pitch + size_t(x >> 1) * 4 * sizeof(B));
            const B s0 = g[0], s1 = g[1], s2 = g[2], s3 = g[3];
            const bool even = (x & 1) == 0;
            if constexpr (PF == PF_UYVY) { o.x = even ? s1 : s3; o.y = s0; o.z = s2; }
            else { o.x = even ? s0 : s2; o.y = s1; o.z = s3; }
        }
        return o;
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        if constexpr (V == 4 && (A & 3) != 0) {
            // Four pixels as whole dwords (x is a multiple of four here): packed 4:2:2 holds them in two groups of four
            // samples, semi-planar formats in four luma samples and two chroma pairs.
            constexpr int S = int(sizeof(B));                 // bytes per sample
            constexpr int kBits = 8 * S;
            constexpr u32 kMask = S == 1 ? 0xffu : 0xffffu;
            auto sample = [&](const u32* w, int k) { return B((w[k * S / 4] >> ((k * kBits) & 31)) & kMask); };
            if constexpr (L::kSemiPlanar) {
                u32 l[S], c[S];
                const u8* lp = p.data + size_t(y) * p.pitch + size_t(x) * S;
                const u8* cp = p.data + size_t(p.pitch) * p.height + size_t(L::k420 ? y >> 1 : y) * p.pitch + size_t(x) * S;
                if constexpr (S == 1) { l[0] = *detail::gconst<u32>(lp); c[0] = *detail::gconst<u32>(cp); }
                else {
                    const detail::u32x2_t a = *detail::gconst<detail::u32x2_a4>(lp), b = *detail::gconst<detail::u32x2_a4>(cp);
                    l[0] = a.x; l[1] = a.y; c[0] = b.x; c[1] = b.y;
                }
#pragma unroll
                for (int i = 0; i < S; ++i) asm("" : "+v"(l[i]), "+v"(c[i]));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    out[i].v.x = sample(l, i);
                    out[i].v.y = sample(c, 2 * (i >> 1) + (L::kSwapUV ? 1 : 0));
                    out[i].v.z = sample(c, 2 * (i >> 1) + (L::kSwapUV ? 0 : 1));
                }
            } else {
                u32 g[2 * S];
                const u8* gp = p.data + size_t(y) * p.pitch + size_t(x) * 2 * S;
                if constexpr (S == 1) { const detail::u32x2_t a = *detail::gconst<detail::u32x2_a4>(gp); g[0] = a.x; g[1] = a.y; }
                else { const detail::u32x4_t a = *detail::gconst<detail::u32x4_a4>(gp); g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w; }
#pragma unroll
                for (int i = 0; i < 2 * S; ++i) asm("" : "+v"(g[i]));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int base = 4 * (i >> 1);            // first sample of the pixel's group: U Y0 V Y1 (UYVY) or Y0 U Y1 V (Y210)
                    const bool even = (i & 1) == 0;
                    if constexpr (PF == PF_UYVY) { out[i].v.x = sample(g, base + (even ? 1 : 3)); out[i].v.y = sample(g, base); out[i].v.z = sample(g, base + 2); }
                    else { out[i].v.x = sample(g, base + (even ? 0 : 2)); out[i].v.y = sample(g, base + 1); out[i].v.z = sample(g, base + 3); }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) out[i].v = exec(x + i, y, z, p);
        }
    }
    // Whole-dword row reads need rows that start on dword boundaries and a run that starts on a group of four pixels.
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return detail::dword_aligned(p.data) && p.pitch % 4 == 0 && xoff % 4 == 0; }
    // No tap cursor: a bilinear resize over this read takes its taps through exec().  The names below only let the
    // wrappers that forward a cursor (Crop, FusedRead) be formed around this read.
    using Raw = Out;
    FKD_DEV static Out finish(const Raw& r, const Params&) { return r; }
    struct TapRow {}; struct TapBits {}; struct PairBits {};
    static constexpr bool kTapOverread = false, kTapPair = false;
#endif
};

// Crop<BackIOp>: FK/algorithms/image_processing/crop.h:36-39.  Shifts by the rectangle origin, drops z,
// clips nothing.
// The tap interface of a read that wraps another one: the inner read's, or placeholders when the inner read has none
// (a bilinear resize, a warp: their elements are computed, not fetched), so that the wrapper's declarations still name
// types; nothing calls them then, because kTapCursor is false.
namespace detail {
template <class B> constexpr bool has_tap_types() {
    if constexpr (requires { typename B::TapRow; typename B::Raw; }) return true; else return false;
}
struct NoTapRaw {}; struct NoTapRow {}; struct NoTapBits {}; struct NoPairBits {};
template <class B, bool = has_tap_types<B>()> struct TapTypesOf {
    using Raw = typename B::Raw; using TapRow = typename B::TapRow; using TapBits = typename B::TapBits; using PairBits = typename B::PairBits;
    static constexpr bool kTapOverread = B::kTapOverread, kTapPair = B::kTapPair;
};
template <class B> struct TapTypesOf<B, false> {
    using Raw = NoTapRaw; using TapRow = NoTapRow; using TapBits = NoTapBits; using PairBits = NoPairBits;
    static constexpr bool kTapOverread = false, kTapPair = false;
};
} // namespace detail

template <class Back> struct Crop {
    using Out = typename Back::Out;
    struct Params { i32 x, y, w, h; typename Back::Params back; };
    static constexpr bool kTapCursor = Back::kTapCursor;
    static constexpr bool kBoundedOut = bounded_out<Back>();
    FKD_NAME("Crop<" + Back::name() + ">")
    FKD_HD static bool strip_ok(const Params& p) {
        if constexpr (requires { Back::strip_ok(p.back); }) return p.w >= 2 && p.h >= 1 && Back::strip_ok(p.back); else return false;
    }
#if defined(FKD_EXEC_CODE)
    static constexpr bool kFiniteTaps = finite_taps<Back>();
    FKD_DEV static int width(const Params& p) { return p.w; }
    FKD_DEV static int height(const Params& p) { return p.h; }
    FKD_DEV static Out exec(int x, int y, int, const Params& p) { return Back::exec(x + p.x, y + p.y, 0, p.back); }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int, const Params& p, Slot<Out> (&out)[V]) {
        Back::template exec_row<V, A>(x + p.x, y + p.y, 0, p.back, out);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return Back::rows_aligned(p.back, xoff + p.x); }
    using Raw = typename detail::TapTypesOf<Back>::Raw;
    FKD_DEV static Out finish(const Raw& r, const Params& p) { return Back::finish(r, p.back); }
    static constexpr bool kTapOverread = detail::TapTypesOf<Back>::kTapOverread;
    using TapRow = typename detail::TapTypesOf<Back>::TapRow;
    FKD_DEV static TapRow tap_row(int x0, int y, int, const Params& p) { return Back::tap_row(x0 + p.x, y + p.y, 0, p.back); }
    FKD_DEV static bool tap_last(const TapRow& r) { return Back::tap_last(r); }
    using TapBits = typename detail::TapTypesOf<Back>::TapBits;
    template <bool OVER> FKD_DEV static TapBits tap_load(const TapRow& r, int x, const Params& p) {
        return Back::template tap_load<OVER>(r, x, p.back);
    }
    FKD_DEV static Raw tap_value(const TapBits& b) { return Back::tap_value(b); }
    static constexpr bool kTapPair = detail::TapTypesOf<Back>::kTapPair;
    using PairBits = typename detail::TapTypesOf<Back>::PairBits;
    FKD_DEV static PairBits pair_load(const TapRow& r, int x, const Params& p) { return Back::pair_load(r, x, p.back); }
    FKD_DEV static void pair_values(const PairBits& b, const TapRow& r, int x, Raw& first, Raw& second) { Back::pair_values(b, r, x, first, second); }
    FKD_DEV static void pair_values_dup(const PairBits& b, bool dup, Raw& first, Raw& second) {
        if constexpr (requires { Back::pair_values_dup(b, dup, first, second); }) Back::pair_values_dup(b, dup, first, second);
        else { Back::pair_values(b, TapRow{}, 0, first, second); if (dup) first = second; }
    }
    static constexpr bool kTapPrepared = detail::tap_prepared<Back>();
    FKD_DEV static bool tap_rows_share_alignment(const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_rows_share_alignment(p.back); else return false;
    }
    FKD_DEV static bool tap_offsets_fit(const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_offsets_fit(p.back); else return false;
    }
    using TapImage = detail::TapImage;
    using PairPrep = detail::PairPrep;
    FKD_DEV static TapImage tap_image(int z, const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_image(z, p.back); else return TapImage{};
    }
    FKD_DEV static TapImage tap_image_bounded(int z, const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_image_bounded(z, p.back); else return TapImage{};
    }
    FKD_DEV static u32 tap_row_offset(int y, const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_row_offset(y + p.y, p.back); else return 0u;
    }
    FKD_DEV static PairPrep pair_prepare(const TapImage& im, int x, const Params& p) {
        if constexpr (kTapPrepared) return Back::pair_prepare(im, x + p.x, p.back); else return PairPrep{};
    }
    FKD_DEV static PairBits pair_load_prepared(const TapImage& im, u32 row_off, const PairPrep& pp, const Params& p) {
        if constexpr (kTapPrepared) return Back::pair_load_prepared(im, row_off, pp, p.back); else return PairBits{};
    }
#endif
};

// BorderReader<BT, Params, BackIOp>: FK/algorithms/image_processing/border_reader.h:177-327.  Coordinates outside the
// back operation's extent are folded back into it (BT = value of fk::BorderType: 1 REPLICATE aaa|abc|ccc, 2 REFLECT
// cba|abc|cba, 3 WRAP abc|abc|abc, 4 REFLECT_101 cb|abc|ba) or yield a constant (0 CONSTANT).  The index arithmetic
// is the reference's, in int: the high side is folded first, then the low side.  The extent it reports is the back
// operation's, so it changes nothing by itself; a Crop with a rectangle that leaves the image is what reaches outside.
template <int BT, class Back> struct Border {
    static_assert(BT >= 0 && BT <= 4, "border types: CONSTANT, REPLICATE, REFLECT, WRAP, REFLECT_101");
    using Out = typename Back::Out;
    struct Params { Out value; typename Back::Params back; };     // value: CONSTANT only
    static constexpr bool kTapCursor = false;
    FKD_NAME("Border<" + istr(BT) + "," + Back::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return Back::width(p.back); }
    FKD_DEV static int height(const Params& p) { return Back::height(p.back); }
    FKD_DEV static int iabs(int v) { return v < 0 ? -v : v; }
    // n = extent along the axis (last index = n - 1)
    // Within one image size of the image the reference's formulas below come to a single reflection or a single period,
    // and no division is needed (a pad, a crop that leans over an edge): fold_near gives that value and clears `near` for
    // an index further out, which takes the formulas as written.
    FKD_DEV static int fold_near(int i, int n, bool& near) {
        const int last = n - 1;
        if constexpr (BT == 2) { near = near && i >= -n && i <= 2 * last + 1; return i < 0 ? -i - 1 : (i > last ? 2 * last - i + 1 : i); }
        else if constexpr (BT == 3) { near = near && i >= -n && i < 2 * n; return i < 0 ? i + n : (i >= n ? i - n : i); }
        else if constexpr (BT == 4) { near = near && i >= -last && i <= 2 * last; return i < 0 ? -i : (i > last ? 2 * last - i : i); }
        else { return i < last ? (i > 0 ? i : 0) : last; }          // REPLICATE: the formula as written has no division
    }
    FKD_DEV static int fold(int i, int n) {
        if constexpr (BT >= 2) {
            bool near = true;
            const int near_value = fold_near(i, n, near);
            if (near) return near_value;
        }
        return fold_as_written(i, n);
    }
    FKD_DEV static int fold_as_written(int i, int n) {
        const int last = n - 1;
        if constexpr (BT == 1) {
            const int hi = i < last ? i : last;
            return hi > 0 ? hi : 0;
        } else if constexpr (BT == 2) {
            const int hi = last - iabs(last - i) + (i > last ? 1 : 0);
            return (iabs(hi) - (hi < 0 ? 1 : 0)) % (last + 1);
        } else if constexpr (BT == 3) {
            const int hi = i < n ? i : i % n;
            return hi >= 0 ? hi : hi - ((hi - n + 1) / n) * n;
        } else {
            const int hi = iabs(last - iabs(last - i)) % (last + 1);
            return iabs(hi) % (last + 1);
        }
    }
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        const int w = Back::width(p.back), h = Back::height(p.back);
        if constexpr (BT == 0) {
            const bool inside = x >= 0 && x < w && y >= 0 && y < h;
            // outside lanes read element (0, 0) instead of branching around the load; the select drops it
            const Out v = Back::exec(inside ? x : 0, inside ? y : 0, z, p.back);
            return inside ? v : p.value;
        } else {
            return Back::exec(fold(x, w), fold(y, h), z, p.back);
        }
    }
    // A lane whose whole run lies between the image's left and right edge reads it as the image itself would (one wide
    // access), from the folded row; lanes that touch an edge go element by element.  With a folding border the choice is
    // made for the wave (a wave with an edge lane goes element by element as a whole: running both forms one after the
    // other for their lanes cost a 16-pixel pad of a 2160p image 9.8 instead of 8.8 us); with a constant border it differs
    // from lane to lane.  Either way the wave-cooperative access mode is not handed on.
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        constexpr int kLaneMode = (A & 3) != 0 ? ((A & 4) | 1) : 0;
        const int w = Back::width(p.back), h = Back::height(p.back);
        const bool run_inside = x >= 0 && x + V <= w;
        if constexpr (BT == 0) {
            if (run_inside && y >= 0 && y < h) { Back::template exec_row<V, kLaneMode>(x, y, z, p.back, out); return; }
        } else {
            if (detail::none_in_wave(!run_inside)) { Back::template exec_row<V, kLaneMode>(x, fold(y, h), z, p.back, out); return; }
        }
#if defined(FKD_DEVICE_CODE)
        // A lane at the left or right edge: its elements come from wherever the border sends them, each as one access of
        // whole dwords (an element of three bytes as one dword, where the byte behind it is still inside the image's
        // allocation: everywhere but on the image's last rows), all of them requested before the first is taken apart.
        // Row and columns are folded without a branch first; a lane that has one of them further out than an image size
        // (no pad does) goes element by element.
        if constexpr (BT != 0 && requires(typename Back::TapRow r) { Back::template tap_load<true>(r, 0, p.back); Back::tap_last(r); }) {
            bool near = true;
            const int fy = fold_near(y, h, near);
            int fx[V];
#pragma unroll
            for (int i = 0; i < V; ++i) fx[i] = fold_near(x + i, w, near);
            if (near) {
                const auto row = Back::tap_row(0, fy, z, p.back);
                typename Back::TapBits bits[V];
                if (Back::tap_last(row)) {
#pragma unroll
                    for (int i = 0; i < V; ++i) bits[i] = Back::template tap_load<false>(row, fx[i], p.back);
                } else {
#pragma unroll
                    for (int i = 0; i < V; ++i) bits[i] = Back::template tap_load<true>(row, fx[i], p.back);
                }
#pragma unroll
                for (int i = 0; i < V; ++i) out[i].v = Back::finish(Back::tap_value(bits[i]), p.back);
                return;
            }
        }
#endif
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = exec(x + i, y, z, p);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return Back::rows_aligned(p.back, xoff); }
    using Raw = Out;
    FKD_DEV static Out finish(const Raw& r, const Params&) { return r; }
    struct TapRow {}; struct TapBits {}; struct PairBits {};
    static constexpr bool kTapOverread = false, kTapPair = false;
#endif
};

// FusedOperation<Read..., compute...> used as a Read: FK/core/execution_model/operation_model/fused_operation.h
// as produced by Fuser::fuse, FK/core/execution_model/operation_model/iop_fuser.h:99-106.
template <class Back, class... Ops> struct FusedRead {
    using Out = typename FoldOut<typename Back::Out, Ops...>::type;
    struct Params { typename Back::Params back; Tup<typename Ops::Params...> ops; };
    static constexpr bool kTapCursor = Back::kTapCursor;
    static constexpr bool kBoundedOut = bounded_out<Back>() && (finite_map<Ops>() && ...);
    FKD_NAME("FusedRead<" + Back::name() + OpList<Ops...>::names() + ">")
    FKD_HD static bool strip_ok(const Params& p) {
        if constexpr (requires { Back::strip_ok(p.back); }) return Back::strip_ok(p.back); else return false;
    }
#if defined(FKD_EXEC_CODE)
    static constexpr bool kFiniteTaps = finite_taps<Back>() && (finite_map<Ops>() && ...);
    FKD_DEV static int width(const Params& p) { return Back::width(p.back); }
    FKD_DEV static int height(const Params& p) { return Back::height(p.back); }
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        return fold<Ops...>(Back::exec(x, y, z, p.back), p.ops);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        Slot<typename Back::Out> t[V];
        Back::template exec_row<V, A>(x, y, z, p.back, t);
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = fold<Ops...>(t[i].v, p.ops);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return Back::rows_aligned(p.back, xoff); }
    using Raw = typename detail::TapTypesOf<Back>::Raw;
    FKD_DEV static Out finish(const Raw& r, const Params& p) { return fold<Ops...>(Back::finish(r, p.back), p.ops); }
    static constexpr bool kTapOverread = detail::TapTypesOf<Back>::kTapOverread;
    using TapRow = typename detail::TapTypesOf<Back>::TapRow;
    FKD_DEV static TapRow tap_row(int x0, int y, int z, const Params& p) { return Back::tap_row(x0, y, z, p.back); }
    FKD_DEV static bool tap_last(const TapRow& r) { return Back::tap_last(r); }
    using TapBits = typename detail::TapTypesOf<Back>::TapBits;
    template <bool OVER> FKD_DEV static TapBits tap_load(const TapRow& r, int x, const Params& p) {
        return Back::template tap_load<OVER>(r, x, p.back);
    }
    FKD_DEV static Raw tap_value(const TapBits& b) { return Back::tap_value(b); }
    static constexpr bool kTapPair = detail::TapTypesOf<Back>::kTapPair;
    using PairBits = typename detail::TapTypesOf<Back>::PairBits;
    FKD_DEV static PairBits pair_load(const TapRow& r, int x, const Params& p) { return Back::pair_load(r, x, p.back); }
    FKD_DEV static void pair_values(const PairBits& b, const TapRow& r, int x, Raw& first, Raw& second) { Back::pair_values(b, r, x, first, second); }
    FKD_DEV static void pair_values_dup(const PairBits& b, bool dup, Raw& first, Raw& second) {
        if constexpr (requires { Back::pair_values_dup(b, dup, first, second); }) Back::pair_values_dup(b, dup, first, second);
        else { Back::pair_values(b, TapRow{}, 0, first, second); if (dup) first = second; }
    }
    static constexpr bool kTapPrepared = detail::tap_prepared<Back>();
    FKD_DEV static bool tap_rows_share_alignment(const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_rows_share_alignment(p.back); else return false;
    }
    FKD_DEV static bool tap_offsets_fit(const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_offsets_fit(p.back); else return false;
    }
    using TapImage = detail::TapImage;
    using PairPrep = detail::PairPrep;
    FKD_DEV static TapImage tap_image(int z, const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_image(z, p.back); else return TapImage{};
    }
    FKD_DEV static TapImage tap_image_bounded(int z, const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_image_bounded(z, p.back); else return TapImage{};
    }
    FKD_DEV static u32 tap_row_offset(int y, const Params& p) {
        if constexpr (kTapPrepared) return Back::tap_row_offset(y, p.back); else return 0u;
    }
    FKD_DEV static PairPrep pair_prepare(const TapImage& im, int x, const Params& p) {
        if constexpr (kTapPrepared) return Back::pair_prepare(im, x, p.back); else return PairPrep{};
    }
    FKD_DEV static PairBits pair_load_prepared(const TapImage& im, u32 row_off, const PairPrep& pp, const Params& p) {
        if constexpr (kTapPrepared) return Back::pair_load_prepared(im, row_off, pp, p.back); else return PairBits{};
    }
#endif
};

// ResizeComplete<AR, Ternary<InterpolateComplete<INTER_LINEAR, Back>>>:
// FK/algorithms/image_processing/resize.h:86-98,117-123 (letterbox test, source coordinate = index * factor, no
// half-pixel offset) and FK/algorithms/image_processing/interpolation.h:70-104 (floor, clamp of x2/y2 only,
// weights from the unclamped x2/y2, four terms summed left to right).  Factors and letterbox rectangle are
// computed on the host (resize.h:164-233).
template <int AR, class Back> struct ResizeLinear {
    using Src = typename Back::Out;
    using Out = vec_t<f32, cn_v<Src>>;
    struct Params {
        i32 dst_w, dst_h;
        f32 fx, fy;
        i32 x1, y1, x2, y2;
        Out bg;
        i32 whole;      // whole_factors(dst_w, dst_h, fx, fy), filled by the host
        typename Back::Params back;
    };
    // Both scale factors are whole numbers and every source coordinate index * factor is an exact float: every source
    // point is then a pixel and the bilinear weights are exactly 1, 0, 0, 0.
    FKD_HD static i32 whole_factors(i32 dst_w, i32 dst_h, f32 fx, f32 fy) {
        // (whole numbers up to 2^24 survive the trip through an integer; no library call on the host)
        return fx >= 1.0f && fy >= 1.0f && fx <= 16777216.0f && fy <= 16777216.0f && fx == f32(i32(fx)) && fy == f32(i32(fy)) &&
               f32(dst_w) * fx <= 16777216.0f && f32(dst_h) * fy <= 16777216.0f;
    }
    static constexpr bool kTapCursor = false;
    static constexpr int kAR = AR;
    static constexpr bool kBoundedOut = AR == IGNORE_AR && bounded_out<Back>();   // a letterbox colour is a run-time value
    using BackOp = Back;
    FKD_NAME("ResizeLinear<" + istr(AR) + "," + Back::name() + ">")
    FKD_HD static bool strip_ok(const Params& p, u32 = 1u) {
        if constexpr (requires { Back::strip_ok(p.back); }) return Back::strip_ok(p.back); else return false;
    }
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return p.dst_w; }
    FKD_DEV static int height(const Params& p) { return p.dst_h; }

    struct Taps { int x1, y1, x2r, y2r; f32 w00, w10, w01, w11; };
    FKD_DEV static Taps taps(int x, int y, const Params& p, int sw, int sh) {
        const f32 sx = f32(x) * p.fx;
        const f32 sy = f32(y) * p.fy;
        Taps t;
        t.x1 = int(__builtin_floorf(sx));
        t.y1 = int(__builtin_floorf(sy));
        const int x2 = t.x1 + 1, y2 = t.y1 + 1;
        t.x2r = x2 < sw - 1 ? x2 : sw - 1;
        t.y2r = y2 < sh - 1 ? y2 : sh - 1;
        const f32 ax = f32(x2) - sx, bx = sx - f32(t.x1);
        const f32 ay = f32(y2) - sy, by = sy - f32(t.y1);
        t.w00 = ax * ay; t.w10 = bx * ay; t.w01 = ax * by; t.w11 = bx * by;
        return t;
    }
    FKD_DEV static Out blend(const Src& a, const Src& b, const Src& c, const Src& d, const Taps& t) {
        Out o;
        auto one = [&](auto pa, auto pb, auto pc, auto pd) {
            return ((f32(pa) * t.w00 + f32(pb) * t.w10) + f32(pc) * t.w01) + f32(pd) * t.w11;
        };
        chan<0>(o) = one(chan<0>(a), chan<0>(b), chan<0>(c), chan<0>(d));
        if constexpr (cn_v<Src> > 1) chan<1>(o) = one(chan<1>(a), chan<1>(b), chan<1>(c), chan<1>(d));
        if constexpr (cn_v<Src> > 2) chan<2>(o) = one(chan<2>(a), chan<2>(b), chan<2>(c), chan<2>(d));
        if constexpr (cn_v<Src> > 3) chan<3>(o) = one(chan<3>(a), chan<3>(b), chan<3>(c), chan<3>(d));
        return o;
    }
    FKD_DEV static bool inside(int x, int y, const Params& p) {
        if constexpr (AR == IGNORE_AR) return true;
        else return x >= p.x1 && x <= p.x2 && y >= p.y1 && y <= p.y2;
    }
    static constexpr bool kPairTaps = [] {
        if constexpr (requires { Back::kTapPair; }) return Back::kTapCursor && Back::kTapPair; else return false;
    }();
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        if constexpr (kPairTaps) {
            // The element-wise form of the bilinear read (kernels that keep one element per thread: several chains in
            // one launch).  Taps x1 and x1 + 1 of a source line come in one access each, issued by every lane (lanes
            // in the letterbox bars take the taps of pixel (0, 0) and drop them), so that no load waits behind a branch;
            // a wave that touches the image's last line, where such an access could reach past the allocation, takes
            // the tap-by-tap path below instead, all lanes together.
            const int sw = Back::width(p.back), sh = Back::height(p.back);
            const bool in = inside(x, y, p);
            int xs = in ? x : 0, ys = in ? y : 0;
            if constexpr (AR != IGNORE_AR) { if (in) { xs -= p.x1; ys -= p.y1; } }
            const Taps t = taps(xs, ys, p, sw, sh);
            const int x1 = t.x1 < 0 ? 0 : (t.x1 < sw - 1 ? t.x1 : sw - 1);      // no-ops wherever the reference is in bounds
            const int y1 = t.y1 < 0 ? 0 : (t.y1 < sh - 1 ? t.y1 : sh - 1);
            const int y2 = y1 + 1 < sh - 1 ? y1 + 1 : sh - 1;
            const auto ra = Back::tap_row(0, y1, z, p.back), rb = Back::tap_row(0, y2, z, p.back);
            const bool risky = sw < 2 || Back::tap_last(ra) || Back::tap_last(rb);
            if (detail::none_in_wave(risky)) {
                const bool edge = x1 >= sw - 1;           // x1 + 1 is past the line: both taps are the last pixel
                const int xp = edge ? sw - 2 : x1;
                const auto wa = Back::pair_load(ra, xp, p.back), wb = Back::pair_load(rb, xp, p.back);
                typename Back::Raw a0, a1, b0, b1;
                Back::pair_values(wa, ra, xp, a0, a1);
                Back::pair_values(wb, rb, xp, b0, b1);
                const Out v = blend(Back::finish(edge ? a1 : a0, p.back), Back::finish(a1, p.back),
                                    Back::finish(edge ? b1 : b0, p.back), Back::finish(b1, p.back), t);
                if constexpr (AR == IGNORE_AR) return v; else return in ? v : p.bg;
            }
        }
        if (!inside(x, y, p)) return p.bg;
        if constexpr (AR != IGNORE_AR) { x -= p.x1; y -= p.y1; }
        const Taps t = taps(x, y, p, Back::width(p.back), Back::height(p.back));
        const Src a = Back::exec(t.x1, t.y1, z, p.back);
        const Src b = Back::exec(t.x2r, t.y1, z, p.back);
        const Src c = Back::exec(t.x1, t.y2r, z, p.back);
        const Src d = Back::exec(t.x2r, t.y2r, z, p.back);
        return blend(a, b, c, d, t);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = exec(x + i, y, z, p);
    }
    FKD_HD static bool rows_aligned(const Params&, int) { return true; }
#endif
};

// Deinterlace<BLEND|INTER_LINEAR, Back>: FK/algorithms/image_processing/deinterlace.h:24-121.  BLEND (DT 0): line y > 0
// is (current + above + 1) * 0.5f, line 0 is current * 1.f.  INTER_LINEAR (DT 1): with use_even the odd lines
// except the last, otherwise the even lines except the first, are (above + below + 1) * 0.5f; all other lines are
// current * 1.f.  Sums follow the C++ promotions of the element type (uchar + uchar + 1 is an int).
template <int DT, class Back> struct Deinterlace {
    using Src = typename Back::Out;
    using Out = vec_t<f32, cn_v<Src>>;
    struct Params { i32 use_even; typename Back::Params back; };
    static constexpr bool kTapCursor = false;
    FKD_NAME("Deinterlace<" + istr(DT) + "," + Back::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return Back::width(p.back); }
    FKD_DEV static int height(const Params& p) { return Back::height(p.back); }
    // which lines take part for output line y: first, second, and whether they are averaged
    FKD_DEV static void lines(int y, const Params& p, int& ya, int& yb, bool& average) {
        const int h = Back::height(p.back);
        if constexpr (DT == 0) {
            average = y > 0;
            ya = y; yb = y > 0 ? y - 1 : y;
        } else {
            const bool even = (y & 1) == 0;
            average = p.use_even ? (!even && y != h - 1) : (even && y != 0);
            ya = average ? y - 1 : y; yb = average ? y + 1 : y;
            // The reference assumes an even number of lines; with an odd one and use_even == false its last line
            // would read one line past the image.  Here that read takes the last line instead.
            yb = yb < h ? yb : h - 1;
        }
    }
    FKD_DEV static Out mix(const Src& a, const Src& b, bool average) {
        return map2<Out>(a, b, [&](auto x, auto y) { return average ? (x + y + 1) * 0.5f : x * 1.f; });
    }
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        int ya, yb; bool average;
        lines(y, p, ya, yb, average);
        return mix(Back::exec(x, ya, z, p.back), Back::exec(x, yb, z, p.back), average);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        int ya, yb; bool average;
        lines(y, p, ya, yb, average);
        Slot<Src> ra[V], rb[V];
        Back::template exec_row<V, A>(x, ya, z, p.back, ra);
        Back::template exec_row<V, A>(x, yb, z, p.back, rb);
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = mix(ra[i].v, rb[i].v, average);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return Back::rows_aligned(p.back, xoff); }
#endif
};

namespace detail {
// The two-tap window type of a read that has one (Back::PairBits), else an empty stand-in.
template <class B> struct pair_bits_of { using type = Empty; };
template <class B> requires requires { typename B::PairBits; } struct pair_bits_of<B> { using type = typename B::PairBits; };
}

// Warping<Affine|Perspective, Back>: FK/algorithms/image_processing/warping.h:42-96.  Destination pixel (x, y) maps
// to source coordinate m * (x, y, 1) (row sums left to right, perspective divide as a multiplication by the
// reciprocal, as the reference writes it); outside [0,w) x [0,h) the result is 0, inside it is the bilinear
// interpolation of interpolation.h:70-104 at that coordinate (floor, +1 taps clamped, weights from the unclamped
// +1 coordinates).
template <int WT, class Back> struct Warp {
    using Src = typename Back::Out;
    using Out = vec_t<f32, cn_v<Src>>;
    struct Params {
        f32 m[9];
        i32 dst_w, dst_h;
        typename Back::Params back;
    };
    static constexpr bool kTapCursor = false;
    static constexpr bool kGatherRead = true;     // taps are scattered: one element per thread
    static constexpr bool kPairTaps = [] {
        if constexpr (requires { Back::kTapPair; }) return Back::kTapCursor && Back::kTapPair; else return false;
    }();
    FKD_NAME("Warp<" + istr(WT) + "," + Back::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return p.dst_w; }
    FKD_DEV static int height(const Params& p) { return p.dst_h; }
#if defined(FKD_DEVICE_CODE)
    // Images below 4 GB (wave uniform): the two line-pair taps through a buffer resource that ends with the image.
    // Row and column are one 32-bit byte offset per lane (no 64-bit address arithmetic on the vector unit), the
    // window starts at the dword at or below it, and a window that reaches past the image's last row reads zeros
    // in bytes nobody uses, so no wave needs the element-wise path.  Lanes whose source point lies outside take
    // the taps of pixel (0, 0) and drop them, so that no load waits behind a branch.  In two halves, so that a thread
    // with several elements has the taps of all of them on their way before it blends the first.
    struct BoundedTaps {
        typename detail::pair_bits_of<Back>::type wa, wb;
        f32 cx, cy, fx1, fy1;      // the source point (0, 0 for a lane outside) and its floor
        int xp;
        bool inside, edge;
    };
    // Whether the bounded form serves this image (wave uniform): at least two columns, every byte offset within 32 bits.
    // (Offsets by two 24-bit multiplications instead of the 32-bit ones the compiler picks were measured and are slower.)
    FKD_DEV static bool bounded_ok(int sw, const Params& p) { return sw >= 2 && Back::tap_offsets_fit(p.back); }
    FKD_DEV static BoundedTaps bounded_request(f32 sx, f32 sy, int sw, int sh, int z, const Params& p) {
        BoundedTaps t;
        t.inside = sx >= 0.f && sx < f32(sw) && sy >= 0.f && sy < f32(sh);
        t.cx = t.inside ? sx : 0.f; t.cy = t.inside ? sy : 0.f;
        t.fx1 = __builtin_floorf(t.cx); t.fy1 = __builtin_floorf(t.cy);
        const int x1 = int(t.fx1), y1 = int(t.fy1);
        const int y2r = y1 + 1 < sh - 1 ? y1 + 1 : sh - 1;
        t.edge = x1 >= sw - 1;                        // x1 + 1 is past the line: both taps are the last pixel
        t.xp = t.edge ? sw - 2 : x1;
        const detail::TapImage image = Back::tap_image_bounded(z, p.back);
        const detail::PairPrep col = Back::pair_prepare(image, t.xp, p.back);
        const u32 column_bytes = col.off + col.shift;             // from the resource's base
        const u32 ta = column_bytes + Back::tap_row_offset(y1, p.back), tb = column_bytes + Back::tap_row_offset(y2r, p.back);
        t.wa = Back::pair_load_prepared(image, 0u, detail::PairPrep{ta & ~3u, ta & 3u}, p.back);
        t.wb = Back::pair_load_prepared(image, 0u, detail::PairPrep{tb & ~3u, tb & 3u}, p.back);
        return t;
    }
    FKD_DEV static Out bounded_blend(const BoundedTaps& t, const Params& p) {
        // (x1 and x1 + 1 as floats are the floor and the floor plus one: coordinates are below 2^24.  Where the taps are
        // finite and not negative whatever the image holds, a lane outside gets horizontal weights of +0, hence four weights
        // of +0 and a result of +0 in every channel; otherwise its channels are replaced one by one)
        constexpr bool kZeroWeights = finite_taps<Back>() && is_integer_v<base_t<Src>> && base_t<Src>(-1) > base_t<Src>(0);
        f32 ax = (t.fx1 + 1.0f) - t.cx, bx = t.cx - t.fx1;
        const f32 ay = (t.fy1 + 1.0f) - t.cy, by = t.cy - t.fy1;
        if constexpr (kZeroWeights) { if (!t.inside) { ax = 0.f; bx = 0.f; } }
        const f32 w00 = ax * ay, w10 = bx * ay, w01 = ax * by, w11 = bx * by;
        typename Back::Raw a0, a1, b0, b1;
        if constexpr (requires { Back::pair_values_dup(t.wa, t.edge, a0, a1); }) {
            // (at the edge the left tap is the right one again: chosen inside the window, before the bytes are taken apart)
            Back::pair_values_dup(t.wa, t.edge, a0, a1);
            Back::pair_values_dup(t.wb, t.edge, b0, b1);
        } else {
            Back::pair_values(t.wa, typename Back::TapRow{}, t.xp, a0, a1);
            Back::pair_values(t.wb, typename Back::TapRow{}, t.xp, b0, b1);
            if (t.edge) { a0 = a1; b0 = b1; }
        }
        const Src a = Back::finish(a0, p.back), b = Back::finish(a1, p.back);
        const Src c = Back::finish(b0, p.back), d = Back::finish(b1, p.back);
        const bool inside = t.inside;
        auto one = [&](auto pa, auto pb, auto pc, auto pd) {
            const f32 v = ((f32(pa) * w00 + f32(pb) * w10) + f32(pc) * w01) + f32(pd) * w11;
            if constexpr (kZeroWeights) return v; else return inside ? v : 0.f;
        };
        Out o;
        chan<0>(o) = one(chan<0>(a), chan<0>(b), chan<0>(c), chan<0>(d));
        if constexpr (cn_v<Src> > 1) chan<1>(o) = one(chan<1>(a), chan<1>(b), chan<1>(c), chan<1>(d));
        if constexpr (cn_v<Src> > 2) chan<2>(o) = one(chan<2>(a), chan<2>(b), chan<2>(c), chan<2>(d));
        if constexpr (cn_v<Src> > 3) chan<3>(o) = one(chan<3>(a), chan<3>(b), chan<3>(c), chan<3>(d));
        return o;
    }
#endif
    // The source point of output pixel (x, y): warping.h:42-96 (each product and sum rounded on its own).
    FKD_DEV static void source_point(int x, int y, const Params& p, f32& sx, f32& sy) {
        const f32 fx = f32(x), fy = f32(y);
        sx = (p.m[0] * fx + p.m[1] * fy) + p.m[2];
        sy = (p.m[3] * fx + p.m[4] * fy) + p.m[5];
        if constexpr (WT == 1) {
            const f32 coeff = 1.0f / ((p.m[6] * fx + p.m[7] * fy) + p.m[8]);
            sx = coeff * sx;
            sy = coeff * sy;
        }
    }
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        f32 sx, sy;
        source_point(x, y, p, sx, sy);
        const int sw = Back::width(p.back), sh = Back::height(p.back);
        Out o;
#if defined(FKD_DEVICE_CODE)
        if constexpr (kPairTaps && detail::tap_prepared<Back>()) {
            if (bounded_ok(sw, p)) return bounded_blend(bounded_request(sx, sy, sw, sh, z, p), p);
        }
#endif
        if constexpr (kPairTaps) {
            // Taps x1 and x1 + 1 of a source line in one access each, issued by every lane (lanes whose source point
            // lies outside take the taps of pixel (0, 0) and drop them), so that no load waits behind a branch.  A wave
            // that touches the image's last line, where such an access could reach past the allocation, takes the
            // element-wise path below instead, all lanes together.
            const bool inside = sx >= 0.f && sx < f32(sw) && sy >= 0.f && sy < f32(sh);
            const f32 cx = inside ? sx : 0.f, cy = inside ? sy : 0.f;
            const int x1 = int(__builtin_floorf(cx)), y1 = int(__builtin_floorf(cy));
            const int y2r = y1 + 1 < sh - 1 ? y1 + 1 : sh - 1;
            const auto ra = Back::tap_row(0, y1, z, p.back), rb = Back::tap_row(0, y2r, z, p.back);
            const bool risky = sw < 2 || Back::tap_last(ra) || Back::tap_last(rb);
            if (detail::none_in_wave(risky)) {
                const bool edge = x1 >= sw - 1;           // x1 + 1 is past the line: both taps are the last pixel
                const int xp = edge ? sw - 2 : x1;
                const auto wa = Back::pair_load(ra, xp, p.back), wb = Back::pair_load(rb, xp, p.back);
                const f32 ax = f32(x1 + 1) - cx, bx = cx - f32(x1), ay = f32(y1 + 1) - cy, by = cy - f32(y1);
                const f32 w00 = ax * ay, w10 = bx * ay, w01 = ax * by, w11 = bx * by;
                typename Back::Raw a0, a1, b0, b1;
                Back::pair_values(wa, ra, xp, a0, a1);
                Back::pair_values(wb, rb, xp, b0, b1);
                const Src a = Back::finish(edge ? a1 : a0, p.back), b = Back::finish(a1, p.back);
                const Src c = Back::finish(edge ? b1 : b0, p.back), d = Back::finish(b1, p.back);
                auto one = [&](auto pa, auto pb, auto pc, auto pd) {
                    const f32 v = ((f32(pa) * w00 + f32(pb) * w10) + f32(pc) * w01) + f32(pd) * w11;
                    return inside ? v : 0.f;
                };
                chan<0>(o) = one(chan<0>(a), chan<0>(b), chan<0>(c), chan<0>(d));
                if constexpr (cn_v<Src> > 1) chan<1>(o) = one(chan<1>(a), chan<1>(b), chan<1>(c), chan<1>(d));
                if constexpr (cn_v<Src> > 2) chan<2>(o) = one(chan<2>(a), chan<2>(b), chan<2>(c), chan<2>(d));
                if constexpr (cn_v<Src> > 3) chan<3>(o) = one(chan<3>(a), chan<3>(b), chan<3>(c), chan<3>(d));
                return o;
            }
        }
        if (sx >= 0.f && sx < f32(sw) && sy >= 0.f && sy < f32(sh)) {
            const f32 f1x = __builtin_floorf(sx), f1y = __builtin_floorf(sy);
            const int x1 = int(f1x), y1 = int(f1y);
            const int x2 = x1 + 1, y2 = y1 + 1;
            const int x2r = x2 < sw - 1 ? x2 : sw - 1, y2r = y2 < sh - 1 ? y2 : sh - 1;
            const f32 ax = f32(x2) - sx, bx = sx - f32(x1), ay = f32(y2) - sy, by = sy - f32(y1);
            const f32 w00 = ax * ay, w10 = bx * ay, w01 = ax * by, w11 = bx * by;
            const Src a = Back::exec(x1, y1, z, p.back), b = Back::exec(x2r, y1, z, p.back);
            const Src c = Back::exec(x1, y2r, z, p.back), d = Back::exec(x2r, y2r, z, p.back);
            auto one = [&](auto pa, auto pb, auto pc, auto pd) {
                return ((f32(pa) * w00 + f32(pb) * w10) + f32(pc) * w01) + f32(pd) * w11;
            };
            chan<0>(o) = one(chan<0>(a), chan<0>(b), chan<0>(c), chan<0>(d));
            if constexpr (cn_v<Src> > 1) chan<1>(o) = one(chan<1>(a), chan<1>(b), chan<1>(c), chan<1>(d));
            if constexpr (cn_v<Src> > 2) chan<2>(o) = one(chan<2>(a), chan<2>(b), chan<2>(c), chan<2>(d));
            if constexpr (cn_v<Src> > 3) chan<3>(o) = one(chan<3>(a), chan<3>(b), chan<3>(c), chan<3>(d));
        } else {
            chan<0>(o) = 0.f;
            if constexpr (cn_v<Src> > 1) chan<1>(o) = 0.f;
            if constexpr (cn_v<Src> > 2) chan<2>(o) = 0.f;
            if constexpr (cn_v<Src> > 3) chan<3>(o) = 0.f;
        }
        return o;
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        if constexpr (kPairTaps && detail::tap_prepared<Back>()) {
            const int sw = Back::width(p.back), sh = Back::height(p.back);
            if (bounded_ok(sw, p)) {
                BoundedTaps taps[V];
#pragma unroll
                for (int i = 0; i < V; ++i) {
                    f32 sx, sy;
                    source_point(x + i, y, p, sx, sy);
                    taps[i] = bounded_request(sx, sy, sw, sh, z, p);
                }
                // (a variant without the selects for waves that have every source point inside and none on the last column
                // was measured: 1 % slower at 1080p, 1 % faster at 2160p, eleven registers more)
#pragma unroll
                for (int i = 0; i < V; ++i) out[i].v = bounded_blend(taps[i], p);
                return;
            }
        }
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = exec(x + i, y, z, p);
    }
    FKD_HD static bool rows_aligned(const Params&, int) { return true; }
#endif
};

// BatchRead<PROCESS_ALL, N, Op>: FK/core/execution_model/operation_model/batch_operations.h:164-219.  Plane z
// uses its own parameter set; z is the workgroup's grid-z index, so the selection is wave uniform.
template <int N, class PlaneOp> struct BatchRead {
    using Out = typename PlaneOp::Out;
    using Plane = PlaneOp;
    static constexpr int kBatch = N;
    struct Params { typename PlaneOp::Params plane[N]; };
    static constexpr bool kTapCursor = false;
    static constexpr bool kBoundedOut = bounded_out<PlaneOp>();
    FKD_NAME("BatchRead<" + istr(N) + "," + PlaneOp::name() + ">")
    FKD_HD static bool strip_ok(const Params& p, u32 planes) {
        if constexpr (requires { PlaneOp::strip_ok(p.plane[0]); }) {
            for (u32 z = 0; z < planes && z < u32(N); ++z) if (!PlaneOp::strip_ok(p.plane[z])) return false;
            return planes <= u32(N);
        } else {
            return false;
        }
    }
#if defined(FKD_EXEC_CODE)
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) { return PlaneOp::exec(x, y, z, p.plane[z]); }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        PlaneOp::template exec_row<V, A>(x, y, z, p.plane[z], out);
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) {
        for (int i = 0; i < N; ++i) if (!PlaneOp::rows_aligned(p.plane[i], xoff)) return false;
        return true;
    }
    FKD_HD static bool plane_rows_aligned(const Params& p, int z, int xoff) { return PlaneOp::rows_aligned(p.plane[z], xoff); }
#endif
};

// BatchRead<CONDITIONAL_WITH_DEFAULT, N, Op>: batch_operations.h:221-281.  Planes >= used yield a default.
template <int N, class PlaneOp> struct BatchReadDefault {
    using Out = typename PlaneOp::Out;
    using Plane = PlaneOp;
    static constexpr int kBatch = N;
    struct Params { typename PlaneOp::Params plane[N]; i32 used; Out def; };
    static constexpr bool kTapCursor = false;
    FKD_NAME("BatchReadDefault<" + istr(N) + "," + PlaneOp::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) {
        if (p.used <= z) return p.def;
        return PlaneOp::exec(x, y, z, p.plane[z]);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        if (p.used <= z) {
#pragma unroll
            for (int i = 0; i < V; ++i) out[i].v = p.def;
        } else {
            PlaneOp::template exec_row<V, A>(x, y, z, p.plane[z], out);
        }
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) {
        for (int i = 0; i < N && i < p.used; ++i) if (!PlaneOp::rows_aligned(p.plane[i], xoff)) return false;
        return true;
    }
    FKD_HD static bool plane_rows_aligned(const Params& p, int z, int xoff) {
        return z >= p.used || PlaneOp::rows_aligned(p.plane[z], xoff);
    }
#endif
};

// ReadSet<T>: constant fill source.  FK/algorithms/basic_ops/set.h:29-80.
template <class T> struct ReadSet {
    using Out = T;
    struct Params { T value; u32 width, height, planes; };
    static constexpr bool kTapCursor = false;
    FKD_NAME("ReadSet<" + type_name<T>() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static int width(const Params& p) { return int(p.width); }
    FKD_DEV static int height(const Params& p) { return int(p.height); }
    FKD_DEV static T exec(int, int, int, const Params& p) { return p.value; }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int, int, int, const Params& p, Slot<T> (&out)[V]) {
#pragma unroll
        for (int i = 0; i < V; ++i) out[i].v = map1<T>(p.value, [](auto c) { return opaque(c); });   // (see opaque)
    }
    FKD_HD static bool rows_aligned(const Params&, int) { return true; }
#endif
};

// ===================================================================================================
// Write operations: (x, y, z, value) -> memory
// ===================================================================================================

// PerThreadWrite<_2D,T>: FK/algorithms/basic_ops/memory_operations.h:84-107.
template <class T> struct Write2D {
    using In = T;
    using Params = RawPtr2D<T>;
    FKD_NAME("Write2D<" + type_name<T>() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static void exec(int x, int y, int, const T& v, const Params& p) {
        detail::store_elem(detail::row_ptr(p.data, p.pitch, x, y), v);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int, const Slot<T> (&v)[V], const Params& p) {
        detail::store_run<T, V, A>(detail::row_ptr(p.data, p.pitch, x, y), v);
    }
    FKD_HD static bool rows_aligned(const Params& p) { return detail::dword_aligned(p.data) && p.pitch % 4 == 0; }
    // Row cursor: one address computation per row, one add per element.
    // The part of the parameters one plane needs (all of them here).
    using Plane = Write2D;
    FKD_DEV static const Params& plane_params(const Params& p, int) { return p; }
    struct RowRef { T* p; };
    FKD_DEV static RowRef row(int y, int, const Params& p) { return RowRef{detail::row_ptr(p.data, p.pitch, 0, y)}; }
    // wave-uniform row address + 32-bit byte offset of the lane: the address form that needs no per-lane 64-bit add
    FKD_DEV static void put(const RowRef& r, int x, const T& v) {
        detail::store_elem_at<T>(reinterpret_cast<char*>(r.p), u32(x) * u32(sizeof(T)), v);
    }
    template <int V> FKD_DEV static void put_run(const RowRef& r, int x, const Slot<T> (&v)[V]) {
        detail::store_run_at<T, V>(reinterpret_cast<char*>(r.p), u32(x) * u32(sizeof(T)), v);
    }
#endif
};

// DualSourceRead<_2D, T>: the elements of two images at the same position, as a pair.
// FK/algorithms/basic_ops/memory_operations.h:585-640.  The extent is the first image's.
template <class T> struct DualRead2D {
    using Out = Two<T, T>;
    using One = Read2D<T>;
    struct Params { typename One::Params a, b; };
    FKD_NAME("DualRead2D<" + type_name<T>() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static Out exec(int x, int y, int z, const Params& p) { return Out{One::exec(x, y, z, p.a), One::exec(x, y, z, p.b)}; }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Params& p, Slot<Out> (&out)[V]) {
        Slot<T> ra[V], rb[V];
        One::template exec_row<V, A>(x, y, z, p.a, ra);
        One::template exec_row<V, A>(x, y, z, p.b, rb);
#pragma unroll
        for (int i = 0; i < V; ++i) { out[i].v.a = ra[i].v; out[i].v.b = rb[i].v; }
    }
    FKD_HD static bool rows_aligned(const Params& p, int xoff) { return One::rows_aligned(p.a, xoff) && One::rows_aligned(p.b, xoff); }
#endif
};

// SplitWrite<_2D, T>: channel c of every value goes to an image of its own, each with its own pitch.
// FK/algorithms/basic_ops/memory_operations.h:336-390.
template <class T> struct SplitWrite2D {
    static_assert(cn_v<T> >= 2, "two to four channels");
    using In = T;
    using B = base_t<T>;
    static constexpr int N = cn_v<T>;
    struct Params { RawPtr2D<B> c[N]; };
    FKD_NAME("SplitWrite2D<" + type_name<T>() + ">")
    template <int I> FKD_HD static B pick(const T& v) { return chan<I>(v); }
#if defined(FKD_EXEC_CODE)
    FKD_DEV static void exec(int x, int y, int, const T& v, const Params& p) {
        detail::store_elem(detail::row_ptr(p.c[0].data, p.c[0].pitch, x, y), pick<0>(v));
        detail::store_elem(detail::row_ptr(p.c[1].data, p.c[1].pitch, x, y), pick<1>(v));
        if constexpr (N > 2) detail::store_elem(detail::row_ptr(p.c[2].data, p.c[2].pitch, x, y), pick<2>(v));
        if constexpr (N > 3) detail::store_elem(detail::row_ptr(p.c[3].data, p.c[3].pitch, x, y), pick<3>(v));
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int, const Slot<T> (&v)[V], const Params& p) {
        // (the channels are taken apart in one pass over the values, as TensorSplit does: taken apart channel by channel
        // in separate passes, the value array stayed in memory)
        Slot<B> c0[V], c1[V];
#pragma unroll
        for (int i = 0; i < V; ++i) { c0[i].v = chan<0>(v[i].v); c1[i].v = chan<1>(v[i].v); }
        detail::store_run<B, V, A>(detail::row_ptr(p.c[0].data, p.c[0].pitch, x, y), c0);
        detail::store_run<B, V, A>(detail::row_ptr(p.c[1].data, p.c[1].pitch, x, y), c1);
        if constexpr (N > 2) {
            Slot<B> c2[V];
#pragma unroll
            for (int i = 0; i < V; ++i) c2[i].v = chan<2>(v[i].v);
            detail::store_run<B, V, A>(detail::row_ptr(p.c[2].data, p.c[2].pitch, x, y), c2);
        }
        if constexpr (N > 3) {
            Slot<B> c3[V];
#pragma unroll
            for (int i = 0; i < V; ++i) c3[i].v = chan<3>(v[i].v);
            detail::store_run<B, V, A>(detail::row_ptr(p.c[3].data, p.c[3].pitch, x, y), c3);
        }
    }
    FKD_HD static bool rows_aligned(const Params& p) {
        bool ok = true;
        for (int i = 0; i < N; ++i) ok = ok && detail::dword_aligned(p.c[i].data) && p.c[i].pitch % 4 == 0;
        return ok;
    }
    using Plane = SplitWrite2D;
    FKD_DEV static const Params& plane_params(const Params& p, int) { return p; }
    struct RowRef { B* p[N]; };
    FKD_DEV static RowRef row(int y, int, const Params& p) {
        RowRef r;
#pragma unroll
        for (int i = 0; i < N; ++i) r.p[i] = detail::row_ptr(p.c[i].data, p.c[i].pitch, 0, y);
        return r;
    }
    FKD_DEV static void put(const RowRef& r, int x, const T& v) {
        const u32 off = u32(x) * u32(sizeof(B));
        detail::store_elem_at<B>(reinterpret_cast<char*>(r.p[0]), off, pick<0>(v));
        detail::store_elem_at<B>(reinterpret_cast<char*>(r.p[1]), off, pick<1>(v));
        if constexpr (N > 2) detail::store_elem_at<B>(reinterpret_cast<char*>(r.p[2]), off, pick<2>(v));
        if constexpr (N > 3) detail::store_elem_at<B>(reinterpret_cast<char*>(r.p[3]), off, pick<3>(v));
    }
    template <int V> FKD_DEV static void put_run(const RowRef& r, int x, const Slot<T> (&v)[V]) {
#pragma unroll
        for (int i = 0; i < V; ++i) put(r, x + i, v[i].v);
    }
#endif
};

// TensorWrite<T> / PerThreadWrite<_3D,T>: FK/algorithms/basic_ops/memory_operations.h:159-179; plane z at
// z*plane_pitch*color_planes (FK/core/data/rawptr.h:215-226).
template <class T> struct TensorWrite {
    using In = T;
    using Params = RawPtr3D<T>;
    FKD_NAME("TensorWrite<" + type_name<T>() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static T* plane(const Params& p, int z) {
        return reinterpret_cast<T*>(reinterpret_cast<char*>(p.data) + size_t(p.plane_pitch) * p.color_planes * z);
    }
    FKD_DEV static void exec(int x, int y, int z, const T& v, const Params& p) {
        detail::store_elem(detail::row_ptr(plane(p, z), p.pitch, x, y), v);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<T> (&v)[V], const Params& p) {
        detail::store_run<T, V, A>(detail::row_ptr(plane(p, z), p.pitch, x, y), v);
    }
    FKD_HD static bool rows_aligned(const Params& p) {
        return detail::dword_aligned(p.data) && p.pitch % 4 == 0 && (size_t(p.plane_pitch) * p.color_planes) % 4 == 0;
    }
    // The part of the parameters one plane needs (all of them here).
    using Plane = TensorWrite;
    FKD_DEV static const Params& plane_params(const Params& p, int) { return p; }
    struct RowRef { T* p; };
    FKD_DEV static RowRef row(int y, int z, const Params& p) { return RowRef{detail::row_ptr(plane(p, z), p.pitch, 0, y)}; }
    FKD_DEV static void put(const RowRef& r, int x, const T& v) {
        detail::store_elem_at<T>(reinterpret_cast<char*>(r.p), u32(x) * u32(sizeof(T)), v);
    }
    template <int V> FKD_DEV static void put_run(const RowRef& r, int x, const Slot<T> (&v)[V]) {
        detail::store_run_at<T, V>(reinterpret_cast<char*>(r.p), u32(x) * u32(sizeof(T)), v);
    }
#endif
};

// TensorSplit<T>: FK/algorithms/basic_ops/memory_operations.h:181-212, and TensorTSplit<T> (TRANSPOSED), :214-241.
// Planar store: channel c of pixel (x,y) of image z goes to the address of (x,y,z) plus c channel planes
// (detail::PlanarGeometry).
template <class T, bool TRANSPOSED = false> struct TensorSplit {
    using In = T;
    using B = base_t<T>;
    using G = detail::PlanarGeometry<B, TRANSPOSED>;
    using Params = typename G::template View<B>;
    FKD_NAME((TRANSPOSED ? "TensorTSplit<" : "TensorSplit<") + type_name<T>() + ">")
    // An image plane with all its channel planes fits 31-bit byte offsets (stores through a buffer resource, see put_masked).
    FKD_HD static bool strip_ok(const Params& p) {
        return G::channel_elements(p) * sizeof(B) * cn_v<T> < size_t(0x7fffffffu) &&
               G::channel_elements(p) * sizeof(B) * (cn_v<T> - 1) + size_t(p.pitch) * p.height < size_t(0x7fffffffu);
    }
#if defined(FKD_EXEC_CODE)
    FKD_DEV static B* at(const Params& p, int x, int y, int z) {
        return reinterpret_cast<B*>(reinterpret_cast<char*>(p.data) + G::image_bytes(p) * z + size_t(y) * p.pitch) + x;
    }
    FKD_DEV static void exec(int x, int y, int z, const T& v, const Params& p) {
        B* w = at(p, x, y, z);
        const size_t px = G::channel_elements(p);
        FKD_GLOBAL B* gw = detail::gmut<B>(w);
        gw[0] = chan<0>(v);
        gw[px] = chan<1>(v);
        if constexpr (cn_v<T> > 2) gw[2 * px] = chan<2>(v);
        if constexpr (cn_v<T> > 3) gw[3 * px] = chan<3>(v);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<T> (&v)[V], const Params& p) {
        B* w = at(p, x, y, z);
        const size_t px = G::channel_elements(p);
        constexpr bool S = (A & kSharedValues) != 0;      // see TeeWrite
        Slot<B> c0[V], c1[V];
#pragma unroll
        for (int i = 0; i < V; ++i) { c0[i].v = maybe_opaque<S>(chan<0>(v[i].v)); c1[i].v = maybe_opaque<S>(chan<1>(v[i].v)); }
        detail::store_run<B, V, A>(w, c0);
        detail::store_run<B, V, A>(w + px, c1);
        if constexpr (cn_v<T> > 2) {
            Slot<B> c2[V];
#pragma unroll
            for (int i = 0; i < V; ++i) c2[i].v = maybe_opaque<S>(chan<2>(v[i].v));
            detail::store_run<B, V, A>(w + 2 * px, c2);
        }
        if constexpr (cn_v<T> > 3) {
            Slot<B> c3[V];
#pragma unroll
            for (int i = 0; i < V; ++i) c3[i].v = maybe_opaque<S>(chan<3>(v[i].v));
            detail::store_run<B, V, A>(w + 3 * px, c3);
        }
    }
    FKD_HD static bool rows_aligned(const Params& p) {
        return detail::dword_aligned(p.data) && p.pitch % 4 == 0 && G::image_bytes(p) % 4 == 0 && (G::channel_elements(p) * sizeof(B)) % 4 == 0;
    }
    // The part of the parameters one plane needs (all of them here).
    using Plane = TensorSplit;
    FKD_DEV static const Params& plane_params(const Params& p, int) { return p; }
    // Stores through a buffer resource, for kernels whose lanes keep their column while their wave walks down rows:
    // image plane z with all its channel planes is one resource, a row and a channel plane are a scalar offset, the
    // column is the lane's offset, and a lane outside the image carries an offset beyond the resource's extent, so the
    // address check drops its store and the wave needs no execution mask around the stores.  Scalar work per row: one
    // multiplication and one addition per channel, in 32 bits.  For image planes smaller than 2 GB (plane_maskable).
    static constexpr bool kLaneMasked = sizeof(B) == 4;
    static constexpr u32 kMaskedExtent = 0x7fffffffu, kMaskedOut = 0x80000000u;
    struct PlaneRef { __amdgpu_buffer_rsrc_t rsrc; u32 chan_bytes, pitch; };
    FKD_DEV static bool plane_maskable(const Params& p) { return strip_ok(p); }
    FKD_DEV static PlaneRef plane_ref(int z, const Params& p) {
        char* base = reinterpret_cast<char*>(p.data) + G::image_bytes(p) * z;
        PlaneRef r;
        r.rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, kMaskedExtent, 0x00020000);   // raw 32-bit data, as detail::make_tap_image
        r.chan_bytes = u32(G::channel_elements(p) * sizeof(B));
        r.pitch = p.pitch;
        return r;
    }
    FKD_DEV static u32 lane_offset(int x, bool valid) { return valid ? u32(x) * u32(sizeof(B)) : kMaskedOut; }
    FKD_DEV static u32 row_offset(int y, const PlaneRef& r) { return u32(y) * r.pitch; }
    FKD_DEV static void put_masked(const PlaneRef& r, u32 row_off, u32 lane_off, const T& v) {
#ifndef FKD_STORE_AUX
#define FKD_STORE_AUX (1 | 16)
#endif
        constexpr int kThrough = FKD_STORE_AUX;     // sc0 sc1: written through the L2, as gstore_through
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(u32, chan<0>(v)), r.rsrc, lane_off, row_off, kThrough);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(u32, chan<1>(v)), r.rsrc, lane_off, row_off + r.chan_bytes, kThrough);
        if constexpr (cn_v<T> > 2) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(u32, chan<2>(v)), r.rsrc, lane_off, row_off + 2u * r.chan_bytes, kThrough);
        if constexpr (cn_v<T> > 3) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(u32, chan<3>(v)), r.rsrc, lane_off, row_off + 3u * r.chan_bytes, kThrough);
    }
    struct RowRef { B* p; size_t px; };
    FKD_DEV static RowRef row(int y, int z, const Params& p) { return RowRef{at(p, 0, y, z), G::channel_elements(p)}; }
    FKD_DEV static void put(const RowRef& r, int x, const T& v) {
        u32 off = u32(x) * u32(sizeof(B));   // one lane offset, four wave-uniform plane row addresses
        asm volatile("" : "+v"(off));
        detail::gstore_through(detail::gmut<B>(reinterpret_cast<char*>(r.p) + off), chan<0>(v));
        detail::gstore_through(detail::gmut<B>(reinterpret_cast<char*>(r.p + r.px) + off), chan<1>(v));
        if constexpr (cn_v<T> > 2) detail::gstore_through(detail::gmut<B>(reinterpret_cast<char*>(r.p + 2 * r.px) + off), chan<2>(v));
        if constexpr (cn_v<T> > 3) detail::gstore_through(detail::gmut<B>(reinterpret_cast<char*>(r.p + 3 * r.px) + off), chan<3>(v));
    }
    template <int V> FKD_DEV static void put_run(const RowRef& r, int x, const Slot<T> (&v)[V]) {
        const u32 off = u32(x) * u32(sizeof(B));
        Slot<B> c[V];
#pragma unroll
        for (int i = 0; i < V; ++i) c[i].v = chan<0>(v[i].v);
        detail::store_run_at<B, V>(reinterpret_cast<char*>(r.p), off, c);
#pragma unroll
        for (int i = 0; i < V; ++i) c[i].v = chan<1>(v[i].v);
        detail::store_run_at<B, V>(reinterpret_cast<char*>(r.p + r.px), off, c);
        if constexpr (cn_v<T> > 2) {
#pragma unroll
            for (int i = 0; i < V; ++i) c[i].v = chan<2>(v[i].v);
            detail::store_run_at<B, V>(reinterpret_cast<char*>(r.p + 2 * r.px), off, c);
        }
        if constexpr (cn_v<T> > 3) {
#pragma unroll
            for (int i = 0; i < V; ++i) c[i].v = chan<3>(v[i].v);
            detail::store_run_at<B, V>(reinterpret_cast<char*>(r.p + 3 * r.px), off, c);
        }
    }
#endif
};

template <class T> using TensorTSplit = TensorSplit<T, true>;

// WriteYUV<NV12 | NV21 | P010 | P210 | Y210 | UYVY>: FK/algorithms/image_processing/color_conversion.h:298-389.  The value
// is (Y, U, V).  Semi-planar formats store Y at (x, y) and the chroma pair of a 2x2 (4:2:0) or 2x1 (4:2:2) block from
// ONE pixel of the block: the top-left one for NV12, P010 and P210 (the reference stores from even x / even y only).
// For NV21 the reference lets every pixel of the block store its own pair to the same place, so its result is the
// block's last pixel in z, y, x order on the CPU backend and whichever thread comes last on a GPU; here it is always
// the block's last pixel (odd x or the last column, odd y or the last row).  Packed 4:2:2 stores U, Y0, V from the
// even pixel of a pair and Y1 from the odd one (UYVY: U Y0 V Y1; Y210: Y0 U Y1 V).
template <int PF> struct WriteYUV {
    using L = PixelLayout<PF>;
    using B = typename PixelBase<PF>::type;
    using In = Vec<B, 3>;
    using Params = RawYUVOut;
    FKD_NAME("WriteYUV<" + istr(PF) + ">")
#if defined(FKD_EXEC_CODE)
    struct RowRef { char* row; char* crow; bool chroma_row; int last_x; };
    FKD_DEV static RowRef row(int y, int, const Params& p) {
        RowRef r;
        char* d = reinterpret_cast<char*>(p.data);
        r.row = d + size_t(y) * p.pitch;
        r.crow = d + size_t(p.pitch) * p.height + size_t(L::k420 ? y >> 1 : y) * p.pitch;
        if constexpr (!L::k420) r.chroma_row = true;
        else if constexpr (L::kSwapUV) r.chroma_row = (y & 1) != 0 || y == int(p.height) - 1;
        else r.chroma_row = (y & 1) == 0;
        r.last_x = int(p.width) - 1;
        return r;
    }
    FKD_DEV static void put(const RowRef& r, int x, const In& v) {
        if constexpr (L::kSemiPlanar) {
            *detail::gmut<B>(r.row + size_t(x) * sizeof(B)) = v.x;
            const bool mine = L::kSwapUV ? ((x & 1) != 0 || x == r.last_x) : (x & 1) == 0;
            if (r.chroma_row && mine) {
                FKD_GLOBAL B* c = detail::gmut<B>(r.crow + size_t(x >> 1) * 2 * sizeof(B));
                c[0] = L::kSwapUV ? v.z : v.y;
                c[1] = L::kSwapUV ? v.y : v.z;
            }
        } else {
            FKD_GLOBAL B* g = detail::gmut<B>(r.row + size_t(x >> 1) * 4 * sizeof(B));
            if ((x & 1) == 0) {
                if constexpr (PF == PF_UYVY) { g[0] = v.y; g[1] = v.x; g[2] = v.z; }
                else { g[0] = v.x; g[1] = v.y; g[3] = v.z; }
            } else {
                if constexpr (PF == PF_UYVY) g[3] = v.x; else g[2] = v.x;
            }
        }
    }
    FKD_DEV static void exec(int x, int y, int z, const In& v, const Params& p) { put(row(y, z, p), x, v); }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V> FKD_DEV static void put_run(const RowRef& r, int x, const Slot<In> (&v)[V]) {
#pragma unroll
        for (int i = 0; i < V; ++i) put(r, x + i, v[i].v);
    }
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<In> (&v)[V], const Params& p) {
        put_run<V>(row(y, z, p), x, v);
    }
    FKD_HD static bool rows_aligned(const Params&) { return true; }   // element-wise either way
    using Plane = WriteYUV;
    FKD_DEV static const Params& plane_params(const Params& p, int) { return p; }
#endif
};

// BatchWrite<N, Op>: FK/core/execution_model/operation_model/batch_operations.h:463-512.
template <int N, class W> struct BatchWrite {
    using In = typename W::In;
    struct Params { typename W::Params plane[N]; };
    FKD_NAME("BatchWrite<" + istr(N) + "," + W::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static void exec(int x, int y, int z, const In& v, const Params& p) { W::exec(x, y, z, v, p.plane[z]); }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<In> (&v)[V], const Params& p) {
        W::template exec_row<V, A>(x, y, z, v, p.plane[z]);
    }
    FKD_HD static bool rows_aligned(const Params& p) {
        for (int i = 0; i < N; ++i) if (!W::rows_aligned(p.plane[i])) return false;
        return true;
    }
    FKD_HD static bool plane_rows_aligned(const Params& p, int z) { return W::rows_aligned(p.plane[z]); }
    using Plane = W;
    FKD_DEV static const typename W::Params& plane_params(const Params& p, int z) { return p.plane[z]; }
    using RowRef = typename W::RowRef;
    FKD_DEV static RowRef row(int y, int z, const Params& p) { return W::row(y, z, p.plane[z]); }
    FKD_DEV static void put(const RowRef& r, int x, const In& v) { W::put(r, x, v); }
    template <int V> FKD_DEV static void put_run(const RowRef& r, int x, const Slot<In> (&v)[V]) { W::template put_run<V>(r, x, v); }
#endif
};

// CircularTensorWrite<direction, Operation, BATCH>: FK/algorithms/basic_ops/memory_operations.h:554-587.
template <int DIR, int BATCH, class W> struct CircularWrite {
    using In = typename W::In;
    struct Params { i32 first; typename W::Params w; };
    FKD_NAME("CircularWrite<" + istr(DIR) + "," + istr(BATCH) + "," + W::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static void exec(int x, int y, int z, const In& v, const Params& p) { W::exec(x, y, circular_plane<DIR, BATCH>(z, p.first), v, p.w); }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<In> (&v)[V], const Params& p) {
        W::template exec_row<V, A>(x, y, circular_plane<DIR, BATCH>(z, p.first), v, p.w);
    }
    FKD_HD static bool rows_aligned(const Params& p) { return W::rows_aligned(p.w); }
#endif
};

// CircularBatchWrite<direction, Operation, BATCH>: FK/algorithms/basic_ops/memory_operations.h:476-503.
template <int DIR, int BATCH, class W> struct CircularBatchWrite {
    using In = typename W::In;
    struct Params { i32 first; typename W::Params plane[BATCH]; };
    FKD_NAME("CircularBatchWrite<" + istr(DIR) + "," + istr(BATCH) + "," + W::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static void exec(int x, int y, int z, const In& v, const Params& p) {
        const int c = circular_plane<DIR, BATCH>(z, p.first);
        W::exec(x, y, c, v, p.plane[c]);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<In> (&v)[V], const Params& p) {
        const int c = circular_plane<DIR, BATCH>(z, p.first);
        W::template exec_row<V, A>(x, y, c, v, p.plane[c]);
    }
    FKD_HD static bool rows_aligned(const Params& p) {
        for (int i = 0; i < BATCH; ++i) if (!W::rows_aligned(p.plane[i])) return false;
        return true;
    }
    FKD_HD static bool plane_rows_aligned(const Params& p, int z) { return W::rows_aligned(p.plane[circular_plane<DIR, BATCH>(z, p.first)]); }
#endif
};

// A MidWrite operation directly before the chain's write (FK/core/execution_model/operation_model/
// instantiable_operations.h:219-262: it stores its input and hands it on unchanged): the same value goes to both.
template <class W1, class W2> struct TeeWrite {
    static_assert(__is_same(typename W1::In, typename W2::In), "both writes take the value the chain produces");
    using In = typename W2::In;
    struct Params { typename W1::Params first; typename W2::Params second; };
    FKD_NAME("TeeWrite<" + W1::name() + "," + W2::name() + ">")
#if defined(FKD_EXEC_CODE)
    FKD_DEV static void exec(int x, int y, int z, const In& v, const Params& p) {
        W1::exec(x, y, z, v, p.first);
        W2::exec(x, y, z, v, p.second);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    template <int V, int A> FKD_DEV static void exec_row(int x, int y, int z, const Slot<In> (&v)[V], const Params& p) {
        // Bit 8 of the access mode tells a planar write that another write reads the same values: it then takes the
        // channels apart behind opaque points (see opaque).  Without them the array of 12-byte values that two writes take
        // apart one after the other is kept in memory.
        W1::template exec_row<V, A | kSharedValues>(x, y, z, v, p.first);
        W2::template exec_row<V, A | kSharedValues>(x, y, z, v, p.second);
    }
    FKD_HD static bool rows_aligned(const Params& p) { return W1::rows_aligned(p.first) && W2::rows_aligned(p.second); }
#endif
};

// ===================================================================================================
// A fused chain: one read, a fold of compute operations, one write, over an active grid.
// ===================================================================================================
template <class T> struct IsSubOp { static constexpr bool value = false; };
template <class I, class P, class O> struct IsSubOp<Sub<I, P, O>> { static constexpr bool value = __is_same(base_t<I>, f32) && __is_same(base_t<P>, f32) && __is_same(base_t<O>, f32); };
template <class T> struct IsDivOp { static constexpr bool value = false; };
template <class I, class P, class O> struct IsDivOp<Div<I, P, O>> { static constexpr bool value = Div<I, P, O>::kReciprocal; };

template <class R, class Ops, class W> struct Chain;
template <class R, class... Ops, class W> struct Chain<R, OpList<Ops...>, W> {
    using Read = R;
    using Write = W;
    using Value = typename FoldOut<typename R::Out, Ops...>::type;
    struct Params {
        u32 active_w, active_h, active_z, reserved;
        typename R::Params read;
        Tup<typename Ops::Params...> ops;
        typename W::Params write;
    };
    FKD_NAME("Chain<" + R::name() + ",OpList<" + (sizeof...(Ops) ? OpList<Ops...>::names().substr(1) : std::string()) + ">," + W::name() + ">")
#if !defined(FKD_DEVICE_CODE)
    // Host, once the parameter block is filled: what only the whole chain knows about the values an operation receives.
    //
    // Normalisation, (x - m) / d with launch constants: when the read hands over finite values below 2^30 (integer pixels,
    // also bilinearly blended or colour converted) and only parameter-free finite maps sit between it and the
    // subtraction, then a = the subtraction's input is finite with |a| < 2^30, and for 2^-20 <= |m| <= 2^59 the
    // difference x = fl(a - m) is zero or has 2^-45 <= |x| < 2^60: if a and m have the same sign and lie within a factor of
    // two of each other the difference is exact (Sterbenz) and a multiple of the smaller unit in the last place, at least
    // 2^-24 * |m| / 2; otherwise |a - m| >= |m| / 2.  That is the range the division's short sequences need, so the
    // device may skip its per-element test.  x = 0 gives the right zero only for a positive divisor (0 * l has the sign of
    // l, and -0 + +0 is +0), hence d > 0 as well.
    template <int K> static void finalize_from(Params& p) {
        if constexpr (K + 1 < int(sizeof...(Ops))) {
            using A = typename TypeAt<K, Ops...>::type;
            using B = typename TypeAt<K + 1, Ops...>::type;
            if constexpr (IsSubOp<A>::value && IsDivOp<B>::value && bounded_out<R>() && prefix_finite<K>()) {
                const auto& sub = tup_get<K>(p.ops);
                auto& div = tup_get<K + 1>(p.ops);
                bool ok = (div.fast & 3) != 0;
                auto mean_ok = [&](f32 m) { const f32 a = __builtin_fabsf(m); if (!(a >= 0x1p-20f && a <= 0x1p59f)) ok = false; };
                auto div_ok = [&](f32 d) { if (!(d > 0.0f)) ok = false; };
                mean_ok(chan_or_scalar<0>(sub.v)); div_ok(chan_or_scalar<0>(div.v));
                if constexpr (cn_v<decltype(sub.v)> > 1) { mean_ok(chan<1>(sub.v)); }
                if constexpr (cn_v<decltype(sub.v)> > 2) { mean_ok(chan<2>(sub.v)); }
                if constexpr (cn_v<decltype(sub.v)> > 3) { mean_ok(chan<3>(sub.v)); }
                if constexpr (cn_v<decltype(div.v)> > 1) { div_ok(chan<1>(div.v)); }
                if constexpr (cn_v<decltype(div.v)> > 2) { div_ok(chan<2>(div.v)); }
                if constexpr (cn_v<decltype(div.v)> > 3) { div_ok(chan<3>(div.v)); }
                if (ok) div.fast |= B::kInputProven;
            }
            finalize_from<K + 1>(p);
        }
    }
    template <int K> static constexpr bool prefix_finite() {
        if constexpr (K == 0) return true;
        else return finite_map<typename TypeAt<K - 1, Ops...>::type>() && prefix_finite<K - 1>();
    }
    static void finalize(Params& p) { finalize_from<0>(p); }
    // Host, once read AND write are filled in: bit 0 of `reserved` tells the launcher that every active plane meets what
    // the strip form of the bilinear kernel asks of its source and destination (that form has no other way to decline a
    // plane).  A parameter block that never came through here keeps the bit clear and gets the tile form.
    static constexpr u32 kStripChecked = 1u;
    static void finalize_write(Params& p) {
        if constexpr (requires { R::strip_ok(p.read, p.active_z); W::strip_ok(p.write); }) {
            if (R::strip_ok(p.read, p.active_z) && W::strip_ok(p.write)) p.reserved |= kStripChecked;
        }
    }
#endif
#if defined(FKD_EXEC_CODE)
    static_assert(__is_same(Value, typename W::In), "the write operation does not take the type the chain produces");
    FKD_DEV static Value compute(const typename R::Out& v, const Params& p) {
        if constexpr (sizeof...(Ops) == 0) return v; else return fold<Ops...>(v, p.ops);
    }
#endif
#if defined(FKD_DEVICE_CODE)
    // compute() through the operations' straight-line variants, falling back to compute() for the (rare) elements
    // they cannot vouch for.  Same result as compute(), fewer instructions on the common path.
    static constexpr bool kQuick = any_quick<Ops...>();
    using OpParams = Tup<typename Ops::Params...>;
    FKD_DEV static Value compute_checked(const typename R::Out& v, const Params& p) { return compute_checked_ops(v, p.ops); }
    // N elements at once, operation-major (see fold_run); same results as compute() element by element.
    // Whether every quick operation of the chain can take its static form in this launch (wave uniform), and the
    // chain computed that way.
    FKD_DEV static bool ops_static(const OpParams& ops) {
        if constexpr (!kQuick) return false; else return all_static_of<Ops...>(ops);
    }
    FKD_DEV static Value compute_static_ops(const typename R::Out& v, const OpParams& ops) { return fold_static<Ops...>(v, ops); }
    template <int N> FKD_DEV static void compute_run(const Slot<typename R::Out> (&in)[N], Slot<Value> (&out)[N], const OpParams& ops) {
        bool ok = true;
        if constexpr (kQuick) {
            if (ops_static(ops)) { fold_run<2, Ops...>(in, out, ops, ok); return; }
        }
        fold_run<kQuick, Ops...>(in, out, ops, ok);
        if constexpr (kQuick) {
            if (__builtin_expect(!ok, 0)) fold_run<0, Ops...>(in, out, ops, ok);
        }
    }
    // The same for chains with many parameters; `kernarg` is the kernel-argument segment, holding a Params at offset 0.
    static constexpr bool kLongChain = sizeof(Tup<typename Ops::Params...>) > 128;
    template <int N> FKD_DEV static void compute_run_kernarg(const Slot<typename R::Out> (&in)[N], Slot<Value> (&out)[N],
                                                             const FKD_CONSTANT void* kernarg) {
        const auto* ops = reinterpret_cast<const FKD_CONSTANT OpParams*>(
            reinterpret_cast<const FKD_CONSTANT char*>(kernarg) + __builtin_offsetof(Params, ops));
        bool ok = true;
        fold_run_k<kQuick, 0, Ops...>(in, out, ops, ok);
        if constexpr (kQuick) {
            if (__builtin_expect(!ok, 0)) fold_run_k<false, 0, Ops...>(in, out, ops, ok);
        }
    }
    FKD_DEV static Value compute_checked_ops(const typename R::Out& v, const OpParams& ops) {
        if constexpr (sizeof...(Ops) == 0) {
            return v;
        } else if constexpr (!kQuick) {
            return fold<Ops...>(v, ops);
        } else {
            bool ok = true;
            Value r = fold_quick<Ops...>(v, ops, ok);
            if (__builtin_expect(!ok, 0)) r = fold<Ops...>(v, ops);
            return r;
        }
    }
#endif
};

// DivergentBatchTransformDPP: FK/core/execution_model/data_parallel_patterns.h:286-381.  Several chains share one launch;
// plane z of the grid (z counts over the planes of all chains together) runs chain select[z], with z handed to that
// chain's read and write unchanged.  select[] is SequenceSelector::at(z), evaluated on the host for every plane of
// the launch (it is a pure function of z), so user code never has to run on the device.  The grid covers the largest
// chain; each chain keeps its own active extent.
template <class... Chains> struct Divergent {
    static_assert(sizeof...(Chains) >= 1 && sizeof...(Chains) <= 255, "one to 255 operation sequences");
    static constexpr int kMaxPlanes = 256;
    static constexpr int kChains = int(sizeof...(Chains));
    struct Params {
        u32 active_w, active_h, active_z, reserved;     // the launch grid: largest width and height, planes of all chains
        u8 select[kMaxPlanes];
        Tup<typename Chains::Params...> seq;
    };
#if defined(FKD_HOST_NAMES)
    static std::string names() { std::string s; ((s += "," + Chains::name()), ...); return s.substr(1); }
#endif
    FKD_NAME("Divergent<" + names() + ">")
};
template <class T> struct IsDivergent { static constexpr bool value = false; };
template <class... Chains> struct IsDivergent<Divergent<Chains...>> { static constexpr bool value = true; };

} // namespace fkd

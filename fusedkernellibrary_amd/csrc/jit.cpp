// jit.cpp -- run-time compilation of chains that were not compiled ahead of time.
//
// A chain signature IS a device type expression (namespace fkd), so compiling a new chain needs nothing but the
// device headers, which the build embeds into this library as text: the signature is pasted into a four-line
// translation unit, hiprtc compiles it for the current device's architecture with the same flags as the
// ahead-of-time build, and the resulting kernel is registered under the signature like any other.  The reference
// gets the same effect from nvcc compiling the user's translation unit; here the user's translation unit is plain
// host C++, so the device compiler runs inside the library instead (once per signature and process, ~1 s).
//
// The generated kernel takes the chain's parameter block by value followed by a TileGeom, and publishes a JitMeta
// constant; the launcher below needs nothing else: the active grid is the first three words of the block.
#include <fklhip.h>
#include "registry.hpp"
#include <fkd/launch_info.hpp>

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace fklhip {
namespace {

// Mirrors of fkd::JitMeta and fkd::TileGeom (csrc/fkd_kernels.hpp): eight and three 32-bit words.
struct JitMeta {
    unsigned gather, params_bytes, v, rows, xi, yi, by, reserved;
};
struct TileGeom {
    unsigned tiles_x, tiles_y, n_tiles;
};

struct JitKernel {
    std::string signature;
    std::vector<char> code;
    JitMeta meta{};
    std::mutex mu;
    std::unordered_map<int, hipFunction_t> per_device;   // a module is loaded once per device that launches it
};

thread_local std::string g_log;
std::mutex g_compile_mu;

bool jit_enabled() {
    const char* v = getenv("FKLHIP_JIT");
    return !(v && v[0] == '0' && v[1] == 0);
}

std::string device_arch() {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
        std::string a = prop.gcnArchName;           // "gfx950:sramecc+:xnack-"
        const size_t colon = a.find(':');
        if (colon != std::string::npos) a.resize(colon);
        if (!a.empty()) return a;
    }
    return "gfx950";
}

// Only characters that occur in signatures pass: the text is pasted into a translation unit.
bool signature_is_clean(const char* s) {
    if (!*s) return false;
    for (; *s; ++s) {
        const char c = *s;
        const bool ok = (c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9') || c == '<' || c == '>' ||
                        c == ',' || c == '_' || c == ' ' || c == '-' || c == ':';
        if (!ok) return false;
    }
    return true;
}

int get_function(JitKernel* k, hipFunction_t* fn) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return int(e);
    std::lock_guard<std::mutex> lock(k->mu);
    const auto it = k->per_device.find(dev);
    if (it != k->per_device.end()) { *fn = it->second; return FKLHIP_OK; }
    hipModule_t mod = nullptr;
    if ((e = hipModuleLoadData(&mod, k->code.data())) != hipSuccess) return int(e);
    hipFunction_t f = nullptr;
    if ((e = hipModuleGetFunction(&f, mod, "fkd_jit_kernel")) != hipSuccess) return int(e);
    k->per_device.emplace(dev, f);   // the module stays loaded for the life of the process
    *fn = f;
    return FKLHIP_OK;
}

int jit_launch(const void* ctx, const void* blob, size_t bytes, void* stream, fkd::LaunchInfo* info) {
    JitKernel* k = const_cast<JitKernel*>(static_cast<const JitKernel*>(ctx));
    if (!blob) return FKLHIP_EINVAL;
    if (bytes != k->meta.params_bytes) return FKLHIP_EBLOB_SIZE;
    unsigned active[3];
    memcpy(active, blob, sizeof(active));   // Chain::Params starts with active_w, active_h, active_z
    const JitMeta& m = k->meta;
    TileGeom g{0, 0, 0};
    unsigned grid[3], block[3] = {64, 4, 1};
    if (m.gather) {
        const unsigned tw = 64 * m.xi, th = m.by * m.yi;
        g.tiles_x = (active[0] + tw - 1) / tw;
        g.tiles_y = (active[1] + th - 1) / th;
        g.n_tiles = g.tiles_x * g.tiles_y * active[2];
        grid[0] = (g.tiles_x * g.tiles_y + 7u) / 8u * 8u;
        grid[1] = 1;
        grid[2] = active[2];
        block[1] = m.by;
    } else {
        grid[0] = (active[0] + 64 * m.v - 1) / (64 * m.v);
        grid[1] = (active[1] + 4 * m.rows - 1) / (4 * m.rows);
        grid[2] = active[2];
    }
    if (info) *info = fkd::LaunchInfo{m.gather ? "gather_jit" : "rows_jit", {grid[0], grid[1], grid[2]}, {block[0], block[1], 1}, 0};
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return FKLHIP_OK;
    if (grid[1] > 65535u || grid[2] > 65535u) return int(hipErrorInvalidConfiguration);
    hipFunction_t fn = nullptr;
    const int rc = get_function(k, &fn);
    if (rc != FKLHIP_OK) return rc;
    // Kernel-argument segment: the parameter block, then the TileGeom at the next 4-byte boundary.  The runtime
    // copies the buffer during the call, so the caller's block may go away as soon as we return.
    const size_t geom_at = (bytes + 3) & ~size_t(3);
    std::vector<char> args(geom_at + sizeof(TileGeom));
    memcpy(args.data(), blob, bytes);
    memcpy(args.data() + geom_at, &g, sizeof(g));
    size_t arg_bytes = args.size();
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &arg_bytes, HIP_LAUNCH_PARAM_END};
    return int(hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0,
                                     static_cast<hipStream_t>(stream), nullptr, config));
}

} // namespace

const char* jit_last_log() { return g_log.c_str(); }

int jit_compile_and_register(const char* signature) {
    g_log.clear();
    if (!jit_enabled()) { g_log = "run-time compilation is switched off (FKLHIP_JIT=0)"; return FKLHIP_EUNKNOWN_SIGNATURE; }
    if (!signature_is_clean(signature)) { g_log = "not a chain signature"; return FKLHIP_EUNKNOWN_SIGNATURE; }
    std::lock_guard<std::mutex> lock(g_compile_mu);   // one compilation at a time; a second caller finds the entry
    {   // the entry may have appeared while this thread waited for the lock
        int count = 0;
        if (fklhip_signature_count(&count) == FKLHIP_OK) {
            for (int i = 0; i < count; ++i) {
                const char* s = nullptr;
                if (fklhip_signature_at(i, &s, nullptr) == FKLHIP_OK && s && strcmp(s, signature) == 0) return FKLHIP_OK;
            }
        }
    }
    std::string src = "#define FKD_DEVICE_CODE 1\n#define FKD_NO_NAMES 1\n#include \"fkd_kernels.hpp\"\nusing namespace fkd;\nusing JitChain = ";
    src += signature;
    src += ";\n"
           "extern \"C\" __device__ const JitMeta fkd_jit_meta = jit_meta<JitChain>();\n"
           "extern \"C\" __global__ __launch_bounds__(256) void fkd_jit_kernel(const JitChain::Params p, const TileGeom g) {\n"
           "    jit_body<JitChain>(p, g);\n"
           "}\n";
    hiprtcProgram prog = nullptr;
    hiprtcResult r = hiprtcCreateProgram(&prog, src.c_str(), "fkd_jit_chain.hip", kJitHeaderCount, kJitHeaderTexts, kJitHeaderNames);
    if (r != HIPRTC_SUCCESS) { g_log = hiprtcGetErrorString(r); return FKLHIP_EUNKNOWN_SIGNATURE; }
    const std::string arch = "--offload-arch=" + device_arch();
    std::vector<const char*> opts;
    opts.push_back(arch.c_str());
    for (int i = 0; i < kJitFlagCount; ++i) opts.push_back(kJitFlags[i]);
    r = hiprtcCompileProgram(prog, int(opts.size()), opts.data());
    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        g_log.resize(log_size);
        hiprtcGetProgramLog(prog, &g_log[0]);
    }
    if (r != HIPRTC_SUCCESS) {
        if (g_log.empty()) g_log = hiprtcGetErrorString(r);
        hiprtcDestroyProgram(&prog);
        return FKLHIP_EUNKNOWN_SIGNATURE;
    }
    JitKernel* k = new JitKernel();   // lives as long as the registry entry: for the life of the process
    k->signature = signature;
    size_t code_size = 0;
    hiprtcGetCodeSize(prog, &code_size);
    k->code.resize(code_size);
    hiprtcGetCode(prog, k->code.data());
    hiprtcDestroyProgram(&prog);
    // The metadata constant is read back from the module itself (on the current device).
    hipModule_t mod = nullptr;
    hipError_t e = hipModuleLoadData(&mod, k->code.data());
    hipDeviceptr_t meta_ptr = nullptr;
    size_t meta_bytes = 0;
    if (e == hipSuccess) e = hipModuleGetGlobal(&meta_ptr, &meta_bytes, mod, "fkd_jit_meta");
    if (e == hipSuccess && meta_bytes != sizeof(JitMeta)) e = hipErrorInvalidValue;
    if (e == hipSuccess) e = hipMemcpyDtoH(&k->meta, meta_ptr, sizeof(JitMeta));
    hipFunction_t fn = nullptr;
    if (e == hipSuccess) e = hipModuleGetFunction(&fn, mod, "fkd_jit_kernel");
    if (e != hipSuccess) {
        g_log = std::string("loading the compiled chain failed: ") + hipGetErrorString(e);
        delete k;
        return int(e);
    }
    int dev = 0;
    hipGetDevice(&dev);
    k->per_device.emplace(dev, fn);
    register_chain(k->signature.c_str(), k->meta.params_bytes, &jit_launch, k);
    return FKLHIP_OK;
}

} // namespace fklhip

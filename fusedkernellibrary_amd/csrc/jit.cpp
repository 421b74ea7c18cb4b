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
//
// With the environment variable FKLHIP_JIT_CACHE naming a directory, compiled code objects are kept there and reused
// by later processes.  A file's name is a hash of everything that went into it (signature, architecture, compiler
// flags, the text of the embedded headers), so a library rebuilt from changed headers never picks up a stale kernel.
#include <fklhip.h>
#include "registry.hpp"
#include <fkd/launch_info.hpp>

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace fklhip {
namespace {

// The launch geometry and the description of a compiled kernel are the kernels' own (fkd/launch_info.hpp).
using fkd::JitMeta;
using fkd::TileGeom;
using fkd::division_magic;
using fkd::kRowsBandBlocks;
using fkd::strip_first_late_workgroup;

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

// Extra preprocessor definitions for kernels compiled at run time, for tuning the kernels' compile-time constants
// (FKD_ROWS and the like) without rebuilding the library: FKLHIP_JIT_DEFINES="-DNAME=VALUE -DOTHER=VALUE".  Only tokens of
// that form pass (letters, digits, '_' and '='); anything else in the variable is ignored.
std::vector<std::string> extra_defines() {
    std::vector<std::string> out;
    const char* v = getenv("FKLHIP_JIT_DEFINES");
    if (!v) return out;
    std::string token;
    auto flush = [&] {
        bool ok = token.size() > 2 && token[0] == '-' && token[1] == 'D';
        for (size_t i = 2; ok && i < token.size(); ++i) {
            const char c = token[i];
            ok = (c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9') || c == '_' || c == '=';
        }
        if (ok) out.push_back(token);
        token.clear();
    };
    for (; *v; ++v) { if (*v == ' ') flush(); else token.push_back(*v); }
    flush();
    return out;
}

// ---- on-disk cache of code objects (opt in: FKLHIP_JIT_CACHE=<directory>) -----------------------------------------

unsigned long long fnv1a(unsigned long long h, const char* data, size_t n) {
    for (size_t i = 0; i < n; ++i) { h ^= static_cast<unsigned char>(data[i]); h *= 1099511628211ull; }
    return h;
}
unsigned long long fnv1a(unsigned long long h, const std::string& s) { return fnv1a(fnv1a(h, s.data(), s.size()), "\0", 1); }

// Path of the cache file for this signature on this architecture, or empty when the cache is off.
std::string cache_path(const char* signature, const std::string& arch) {
    const char* dir = getenv("FKLHIP_JIT_CACHE");
    if (!dir || !dir[0]) return std::string();
    unsigned long long a = fnv1a(14695981039346656037ull, std::string(signature));
    unsigned long long b = fnv1a(0x9e3779b97f4a7c15ull, arch);
    for (int i = 0; i < kJitFlagCount; ++i) b = fnv1a(b, std::string(kJitFlags[i]));
    for (const std::string& d : extra_defines()) b = fnv1a(b, d);
    for (int i = 0; i < kJitHeaderCount; ++i) { b = fnv1a(b, std::string(kJitHeaderNames[i])); b = fnv1a(b, std::string(kJitHeaderTexts[i])); }
    a = fnv1a(a, std::string(reinterpret_cast<const char*>(&b), sizeof(b)));
    char name[64];
    snprintf(name, sizeof(name), "/fklhip-%016llx%016llx.co", a, b);
    return std::string(dir) + name;
}
// Every compiled chain gets a kernel symbol of its own, so that profilers tell the chains apart: "fkd_jit_" and the
// FNV-1a hash of the signature text (terminating zero included) as 16 hex digits.
std::string kernel_symbol(const std::string& signature) {
    char name[32];
    snprintf(name, sizeof(name), "fkd_jit_%016llx", fnv1a(14695981039346656037ull, signature));
    return name;
}
// A cache file is a 24-byte header (magic, payload length, FNV-1a of the payload) followed by the code object: a file
// that was cut short, damaged or put there by something else fails the check and is recompiled, instead of being handed
// to the module loader, which takes a bare pointer and would run whatever loads.
constexpr char kCacheMagic[8] = {'F', 'K', 'L', 'H', 'I', 'P', 'C', '1'};
struct CacheHeader { char magic[8]; unsigned long long bytes, hash; };

bool read_file(const std::string& path, std::vector<char>* out) {
    const int fd = open(path.c_str(), O_RDONLY | O_NOFOLLOW | O_CLOEXEC);
    if (fd < 0) return false;
    bool ok = false;
    struct stat st;
    CacheHeader h;
    if (fstat(fd, &st) == 0 && S_ISREG(st.st_mode) && size_t(st.st_size) > sizeof(h) &&
        read(fd, &h, sizeof(h)) == ssize_t(sizeof(h)) && memcmp(h.magic, kCacheMagic, sizeof(kCacheMagic)) == 0 &&
        h.bytes == size_t(st.st_size) - sizeof(h)) {
        out->resize(size_t(h.bytes));
        size_t got = 0;
        while (got < out->size()) {
            const ssize_t n = read(fd, out->data() + got, out->size() - got);
            if (n <= 0) break;
            got += size_t(n);
        }
        ok = got == out->size() && fnv1a(14695981039346656037ull, out->data(), out->size()) == h.hash;
    }
    close(fd);
    if (!ok) out->clear();
    return ok;
}
// Written under a private name (created exclusively, owner-only, never through a symbolic link) and renamed into
// place, so a reader never sees half a file; failures are silent (the cache is an optimisation).
void write_file(const std::string& path, const std::vector<char>& data) {
    const std::string tmp = path + ".tmp" + std::to_string(long(getpid()));
    const int fd = open(tmp.c_str(), O_WRONLY | O_CREAT | O_EXCL | O_NOFOLLOW | O_CLOEXEC, 0600);
    if (fd < 0) return;
    CacheHeader h;
    memcpy(h.magic, kCacheMagic, sizeof(kCacheMagic));
    h.bytes = data.size();
    h.hash = fnv1a(14695981039346656037ull, data.data(), data.size());
    bool ok = write(fd, &h, sizeof(h)) == ssize_t(sizeof(h));
    size_t put = 0;
    while (ok && put < data.size()) {
        const ssize_t n = write(fd, data.data() + put, data.size() - put);
        if (n <= 0) ok = false; else put += size_t(n);
    }
    if (close(fd) != 0 || !ok || rename(tmp.c_str(), path.c_str()) != 0) unlink(tmp.c_str());
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
    if ((e = hipModuleGetFunction(&f, mod, kernel_symbol(k->signature).c_str())) != hipSuccess) return int(e);
    k->per_device.emplace(dev, f);   // the module stays loaded for the life of the process
    *fn = f;
    return FKLHIP_OK;
}

int jit_launch(const void* ctx, const void* blob, size_t bytes, void* stream, fkd::LaunchInfo* info) {
    JitKernel* k = const_cast<JitKernel*>(static_cast<const JitKernel*>(ctx));
    if (!blob) return FKLHIP_EINVAL;
    if (bytes != k->meta.params_bytes) return FKLHIP_EBLOB_SIZE;
    unsigned active[4];
    memcpy(active, blob, sizeof(active));   // Chain::Params starts with active_w, active_h, active_z, reserved (bit 0: strip form allowed)
    const JitMeta& m = k->meta;
    TileGeom g{0, 0, 0, 0};
    unsigned grid[3], block[3] = {64, 4, 1};
    const char* kind = m.gather ? "gather_jit" : "rows_jit";
    if (m.gather && m.strip_width != 0 && active[0] != 0 && active[0] <= m.strip_width && (active[3] & 1u) != 0 && strip_enabled()) {
        // strip form: one workgroup per m.by * m.yi output rows of a plane; tiles_x == 0 tells the kernel, and n_tiles
        // carries the launch's priority schedule
        kind = "strip_jit";
        grid[0] = (active[1] + m.by * m.yi - 1) / (m.by * m.yi);
        grid[1] = 1;
        grid[2] = active[2];
        block[1] = m.by;
        g.n_tiles = strip_first_late_workgroup((unsigned long long)grid[0] * grid[2]);
    } else if (m.gather) {
        const unsigned tw = 64 * m.xi, th = m.by * m.yi;
        g.tiles_x = (active[0] + tw - 1) / tw;
        g.tiles_y = (active[1] + th - 1) / th;
        g.n_tiles = g.tiles_x * g.tiles_y * active[2];
        g.tiles_x_magic = division_magic(g.tiles_x, g.tiles_x * g.tiles_y);
        grid[0] = (g.tiles_x * g.tiles_y + 7u) / 8u * 8u;
        grid[1] = 1;
        grid[2] = active[2];
        block[1] = m.by;
    } else {
        grid[0] = (active[0] + 64 * m.v - 1) / (64 * m.v);
        grid[1] = (active[1] + 4 * m.rows - 1) / (4 * m.rows);
        grid[2] = active[2];
        if (m.bands && (unsigned long long)grid[0] * grid[1] >= kRowsBandBlocks) {
            // as launch_rows_with: one-dimensional, eight equal runs of the plane's blocks
            if ((unsigned long long)grid[0] * grid[1] > 0x7fffff00ull) return int(hipErrorInvalidConfiguration);
            g.tiles_x = grid[0];
            g.tiles_y = grid[1];
            g.n_tiles = grid[0] * grid[1] * grid[2];
            g.tiles_x_magic = division_magic(g.tiles_x, g.tiles_x * g.tiles_y);
            grid[0] = (grid[0] * grid[1] + 7u) / 8u * 8u;
            grid[1] = 1;
        }
    }
    if (info) *info = fkd::LaunchInfo{kind, {grid[0], grid[1], grid[2]}, {block[0], block[1], 1}, 0};
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return FKLHIP_OK;
    if (grid[1] > 65535u || grid[2] > 65535u) return int(hipErrorInvalidConfiguration);
    if (m.max_planes != 0 && grid[2] > m.max_planes) return int(hipErrorInvalidConfiguration);   // as launch_divergent
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

// Compile (or fetch from the cache directory) and register; the caller holds g_compile_mu.
// `arrays_to_lds`: compile without the build's -disable-promote-alloca-to-lds, so that a per-thread array the optimiser
// cannot keep in registers goes to LDS instead of scratch memory (the second attempt for such a chain, see below).
static int build_and_register(const char* signature, bool may_read_cache, bool arrays_to_lds = false) {
    const std::string arch_name = device_arch();
    const std::string cached = cache_path(signature, arch_name);
    JitKernel* k = new JitKernel();   // lives as long as the registry entry: for the life of the process
    k->signature = signature;
    const bool from_cache = may_read_cache && !cached.empty() && read_file(cached, &k->code);
    if (!from_cache) {
        std::string src = "#define FKD_DEVICE_CODE 1\n#define FKD_NO_NAMES 1\n#include \"fkd_kernels.hpp\"\nusing namespace fkd;\nusing JitChain = ";
        src += signature;
        src += ";\n"
               "extern \"C\" __device__ const JitMeta fkd_jit_meta = jit_meta<JitChain>();\n"
               "extern \"C\" __global__ __launch_bounds__(256) void ";
        src += kernel_symbol(k->signature);
        src += "(const JitChain::Params p, const TileGeom g) {\n"
               "    jit_body<JitChain>(p, g);\n"
               "}\n";
        hiprtcProgram prog = nullptr;
        hiprtcResult r = hiprtcCreateProgram(&prog, src.c_str(), "fkd_jit_chain.hip", kJitHeaderCount, kJitHeaderTexts, kJitHeaderNames);
        if (r != HIPRTC_SUCCESS) { g_log = hiprtcGetErrorString(r); delete k; return FKLHIP_EUNKNOWN_SIGNATURE; }
        const std::string arch = "--offload-arch=" + arch_name;
        std::vector<const char*> opts;
        opts.push_back(arch.c_str());
        for (int i = 0; i < kJitFlagCount; ++i) {
            if (arrays_to_lds && strcmp(kJitFlags[i], "-mllvm") == 0 && i + 1 < kJitFlagCount &&
                strncmp(kJitFlags[i + 1], "-disable-promote-alloca-to-lds", 30) == 0) { ++i; continue; }
            opts.push_back(kJitFlags[i]);
        }
        const std::vector<std::string> defines = extra_defines();
        for (const std::string& d : defines) opts.push_back(d.c_str());
        r = hiprtcCompileProgram(prog, int(opts.size()), opts.data());
        size_t log_size = 0;
        if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
            g_log.resize(log_size);
            hiprtcGetProgramLog(prog, &g_log[0]);
        }
        if (r != HIPRTC_SUCCESS) {
            if (g_log.empty()) g_log = hiprtcGetErrorString(r);
            hiprtcDestroyProgram(&prog);
            delete k;
            return FKLHIP_EUNKNOWN_SIGNATURE;
        }
        size_t code_size = 0;
        hiprtcGetCodeSize(prog, &code_size);
        k->code.resize(code_size);
        hiprtcGetCode(prog, k->code.data());
        hiprtcDestroyProgram(&prog);
    }
    // The metadata constant is read back from the module itself (on the current device).
    hipModule_t mod = nullptr;
    hipError_t e = hipModuleLoadData(&mod, k->code.data());
    hipDeviceptr_t meta_ptr = nullptr;
    size_t meta_bytes = 0;
    if (e == hipSuccess) e = hipModuleGetGlobal(&meta_ptr, &meta_bytes, mod, "fkd_jit_meta");
    if (e == hipSuccess && meta_bytes != sizeof(JitMeta)) e = hipErrorInvalidValue;
    if (e == hipSuccess) e = hipMemcpyDtoH(&k->meta, meta_ptr, sizeof(JitMeta));
    hipFunction_t fn = nullptr;
    if (e == hipSuccess) e = hipModuleGetFunction(&fn, mod, kernel_symbol(k->signature).c_str());
    if (e != hipSuccess) {
        if (mod) hipModuleUnload(mod);
        delete k;
        if (from_cache) {
            // an unreadable or foreign file: compile afresh (which replaces it)
            return build_and_register(signature, false, arrays_to_lds);
        }
        g_log = std::string("loading the compiled chain failed: ") + hipGetErrorString(e);
        return int(e);
    }
    if (k->meta.params_bytes > unsigned(FKLHIP_MAX_BLOB_BYTES)) {
        // by-value kernel arguments beyond what the library passes on to the runtime: refused here, with a sentence,
        // instead of failing inside the launch call
        g_log = "the chain's parameter block is " + std::to_string(k->meta.params_bytes) + " bytes; a launch accepts at most " +
                std::to_string(FKLHIP_MAX_BLOB_BYTES) + " (FKLHIP_MAX_BLOB_BYTES): use a smaller batch per launch";
        hipModuleUnload(mod);
        delete k;
        return FKLHIP_EBLOB_SIZE;
    }
    // The ahead-of-time build refuses kernels that need scratch memory (a private array the optimiser could not keep in
    // registers, or spills: a silent slowdown of an order of magnitude).  A chain compiled here still runs: it is compiled
    // once more with such arrays moved to LDS, which is the faster of the two homes, and the note goes into the log; with
    // FKLHIP_JIT_STRICT=1 it is refused like there.
    int scratch_bytes = 0;
    if (hipFuncGetAttribute(&scratch_bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, fn) != hipSuccess) scratch_bytes = 0;
    if (scratch_bytes > 0) {
        const char* strict = getenv("FKLHIP_JIT_STRICT");
        const std::string note = "the compiled chain needs " + std::to_string(scratch_bytes) + " bytes of scratch memory per lane";
        if (strict && strict[0] == '1') {
            hipModuleUnload(mod);
            delete k;
            g_log = note + " (refused: FKLHIP_JIT_STRICT=1)";
            return FKLHIP_EUNKNOWN_SIGNATURE;
        }
        if (!arrays_to_lds) {
            hipModuleUnload(mod);
            delete k;
            const int rc = build_and_register(signature, false, true);
            g_log = note + "; compiled again with per-thread arrays in LDS" + (g_log.empty() ? std::string() : ": " + g_log);
            return rc;
        }
        g_log = note;
    } else if (from_cache) {
        g_log = "loaded from " + cached;
    }
    // (an object compiled with per-thread arrays in LDS is not kept: the file's name does not say how it was compiled, and
    // a later process running with FKLHIP_JIT_STRICT=1 would take it for a clean one)
    if (!from_cache && !cached.empty() && !arrays_to_lds) write_file(cached, k->code);
    int dev = 0;
    hipGetDevice(&dev);
    k->per_device.emplace(dev, fn);
    register_chain(k->signature.c_str(), k->meta.params_bytes, &jit_launch, k);
    return FKLHIP_OK;
}

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
    return build_and_register(signature, true);
}

} // namespace fklhip

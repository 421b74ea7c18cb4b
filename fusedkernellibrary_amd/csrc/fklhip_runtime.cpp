// fklhip_runtime.cpp -- implementation of the C ABI declared in include/fklhip.h.
//
// Thin by design: HIP runtime calls for streams, memory, copies and events, plus the lookup table that maps a
// chain signature to the launcher of its ahead-of-time compiled gfx950 kernel.
#include <fklhip.h>
#include "registry.hpp"
#include <fkd/launch_info.hpp>

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace fklhip {
namespace {

struct Table {
    std::mutex mu;
    std::vector<Entry> entries;
    std::unordered_map<std::string, size_t> index;
};

Table& table() {
    static Table* t = new Table();   // leaked on purpose: registrars run before and after other statics
    return *t;
}

thread_local fkd::LaunchInfo g_last = {"", {0, 0, 0}, {0, 0, 0}, 0};

// The environment is looked at once (a function-local static: thread safe), afterwards only the atomic is read.
std::atomic<int>& strip_setting() {
    static std::atomic<int> setting = [] {
        const char* e = getenv("FKLHIP_STRIP");
        return (e && e[0] == '0' && e[1] == 0) ? 0 : 1;
    }();
    return setting;
}

} // namespace

bool strip_enabled() { return strip_setting().load(std::memory_order_relaxed) != 0; }

void register_chain(const char* signature, size_t blob_bytes, LaunchFn fn, const void* ctx) {
    Table& t = table();
    std::lock_guard<std::mutex> lock(t.mu);
    if (t.index.count(signature)) return;
    t.index.emplace(signature, t.entries.size());
    t.entries.push_back(Entry{signature, blob_bytes, fn, ctx});
}

} // namespace fklhip

using namespace fklhip;

extern "C" {

int fklhip_abi_version(void) { return FKLHIP_ABI_VERSION; }

const char* fklhip_error_string(int code) {
    switch (code) {
    case FKLHIP_OK: return "success";
    case FKLHIP_EUNKNOWN_SIGNATURE:
        return "no kernel was compiled for this chain signature (add it to aot_signatures.txt and rebuild libfklhip.so)"
               " and it could not be compiled at run time (fklhip_jit_log has the compiler's messages)";
    case FKLHIP_EBLOB_SIZE:
        return "parameter block size does not match the chain signature, or exceeds FKLHIP_MAX_BLOB_BYTES (1 MiB less 64 bytes:"
               " the most the library passes on as by-value kernel arguments; split the batch into several launches)";
    case FKLHIP_EINVAL: return "invalid argument";
    default: return hipGetErrorString(static_cast<hipError_t>(code));
    }
}

int fklhip_get_device(int* device) { return device ? int(hipGetDevice(device)) : FKLHIP_EINVAL; }
int fklhip_set_device(int device) { return int(hipSetDevice(device)); }
int fklhip_device_count(int* count) { return count ? int(hipGetDeviceCount(count)) : FKLHIP_EINVAL; }

int fklhip_stream_create(void** stream) {
    if (!stream) return FKLHIP_EINVAL;
    hipStream_t s = nullptr;
    const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    *stream = s;
    return int(e);
}
int fklhip_stream_destroy(void* stream) { return int(hipStreamDestroy(static_cast<hipStream_t>(stream))); }
int fklhip_stream_sync(void* stream) { return int(hipStreamSynchronize(static_cast<hipStream_t>(stream))); }

int fklhip_malloc(void** ptr, size_t bytes) { return ptr ? int(hipMalloc(ptr, bytes)) : FKLHIP_EINVAL; }
int fklhip_malloc_pitch(void** ptr, size_t* pitch, size_t width_bytes, size_t height) {
    if (!ptr || !pitch) return FKLHIP_EINVAL;
    return int(hipMallocPitch(ptr, pitch, width_bytes, height));
}
int fklhip_free(void* ptr) { return int(hipFree(ptr)); }
int fklhip_host_alloc(void** ptr, size_t bytes) {
    return ptr ? int(hipHostMalloc(ptr, bytes, hipHostMallocDefault)) : FKLHIP_EINVAL;
}
int fklhip_host_free(void* ptr) { return int(hipHostFree(ptr)); }

static hipMemcpyKind to_kind(int kind) {
    switch (kind) {
    case FKLHIP_COPY_H2H: return hipMemcpyHostToHost;
    case FKLHIP_COPY_H2D: return hipMemcpyHostToDevice;
    case FKLHIP_COPY_D2H: return hipMemcpyDeviceToHost;
    case FKLHIP_COPY_D2D: return hipMemcpyDeviceToDevice;
    default: return hipMemcpyDefault;
    }
}

int fklhip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream) {
    return int(hipMemcpyAsync(dst, src, bytes, to_kind(kind), static_cast<hipStream_t>(stream)));
}
int fklhip_memcpy2d_async(void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t width_bytes,
                          size_t height, int kind, void* stream) {
    return int(hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width_bytes, height, to_kind(kind),
                                static_cast<hipStream_t>(stream)));
}
int fklhip_memset_async(void* dst, int value, size_t bytes, void* stream) {
    return int(hipMemsetAsync(dst, value, bytes, static_cast<hipStream_t>(stream)));
}

int fklhip_event_create(void** event) {
    if (!event) return FKLHIP_EINVAL;
    hipEvent_t e = nullptr;
    const hipError_t r = hipEventCreate(&e);
    *event = e;
    return int(r);
}
int fklhip_event_destroy(void* event) { return int(hipEventDestroy(static_cast<hipEvent_t>(event))); }
int fklhip_event_record(void* event, void* stream) {
    return int(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}
int fklhip_event_sync(void* event) { return int(hipEventSynchronize(static_cast<hipEvent_t>(event))); }
int fklhip_event_elapsed_ms(float* ms, void* start, void* stop) {
    return ms ? int(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop))) : FKLHIP_EINVAL;
}

int fklhip_lookup(const char* signature, const void** handle) {
    if (!signature || !handle) return FKLHIP_EINVAL;
    Table& t = table();
    std::unique_lock<std::mutex> lock(t.mu);
    auto it = t.index.find(signature);
    if (it == t.index.end()) {
        // Not compiled ahead of time: compile it now (once per process), outside the table lock.
        lock.unlock();
        const int rc = jit_compile_and_register(signature);
        lock.lock();
        if (rc != FKLHIP_OK) { *handle = nullptr; return rc; }
        it = t.index.find(signature);
        if (it == t.index.end()) { *handle = nullptr; return FKLHIP_EUNKNOWN_SIGNATURE; }
    }
    *handle = reinterpret_cast<const void*>(it->second + 1);   // index + 1: entries never move out of the table
    return FKLHIP_OK;
}

int fklhip_jit_log(const char** log) {
    if (!log) return FKLHIP_EINVAL;
    *log = jit_last_log();
    return FKLHIP_OK;
}

int fklhip_strip_form(int enable) {
    std::atomic<int>& s = strip_setting();
    if (enable < 0) return s.load(std::memory_order_relaxed);
    return s.exchange(enable != 0 ? 1 : 0, std::memory_order_relaxed);
}

int fklhip_launch_handle(const void* handle, const void* blob, size_t blob_bytes, void* stream) {
    if (blob_bytes > size_t(FKLHIP_MAX_BLOB_BYTES)) return FKLHIP_EBLOB_SIZE;   // before anything reaches the runtime
    const size_t idx = reinterpret_cast<size_t>(handle);
    Entry e;
    {
        Table& t = table();
        std::lock_guard<std::mutex> lock(t.mu);
        if (idx == 0 || idx > t.entries.size()) return FKLHIP_EINVAL;
        e = t.entries[idx - 1];
    }
    return e.launch(e.ctx, blob, blob_bytes, stream, &g_last);
}

int fklhip_launch(const char* signature, const void* blob, size_t blob_bytes, void* stream) {
    const void* h = nullptr;
    const int rc = fklhip_lookup(signature, &h);
    if (rc != FKLHIP_OK) return rc;
    return fklhip_launch_handle(h, blob, blob_bytes, stream);
}

int fklhip_last_launch(const char** kernel, unsigned grid[3], unsigned block[3], unsigned* lds_bytes) {
    if (kernel) *kernel = g_last.kernel;
    for (int i = 0; i < 3; ++i) {
        if (grid) grid[i] = g_last.grid[i];
        if (block) block[i] = g_last.block[i];
    }
    if (lds_bytes) *lds_bytes = g_last.lds_bytes;
    return FKLHIP_OK;
}

int fklhip_signature_count(int* count) {
    if (!count) return FKLHIP_EINVAL;
    Table& t = table();
    std::lock_guard<std::mutex> lock(t.mu);
    *count = int(t.entries.size());
    return FKLHIP_OK;
}

int fklhip_signature_at(int index, const char** signature, size_t* blob_bytes) {
    Table& t = table();
    std::lock_guard<std::mutex> lock(t.mu);
    if (index < 0 || size_t(index) >= t.entries.size()) return FKLHIP_EINVAL;
    if (signature) *signature = t.entries[size_t(index)].signature;
    if (blob_bytes) *blob_bytes = t.entries[size_t(index)].blob_bytes;
    return FKLHIP_OK;
}

} // extern "C"

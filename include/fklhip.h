/*
 * fklhip.h -- C ABI of libfklhip.so, the MI355X (gfx950) backend of the fused data-parallel path.
 *
 * This is the whole boundary between host code (plain C++20 headers under include/fused_kernel/, or any
 * language with a C FFI) and the HIP runtime + hand-written kernels.  Plain pointers and sizes only; no C++
 * types, no HIP types, no exceptions.  Every function returns 0 on success, a hipError_t value (1..9999) when
 * the HIP runtime reported an error, or one of the FKLHIP_E* codes below.  Functions are thread safe; none of
 * them synchronises the device unless its name says so.
 *
 * The reference library has no FFI: its device boundary is the CUDA runtime called from templates.  Each
 * declaration names the reference call site it stands in for (paths relative to the reference root,
 * FK/ = include/fused_kernel/).
 */
#ifndef FKLHIP_H
#define FKLHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FKLHIP_ABI_VERSION 1

enum {
    FKLHIP_OK = 0,
    FKLHIP_EUNKNOWN_SIGNATURE = 10001, /* no kernel was built for this chain signature */
    FKLHIP_EBLOB_SIZE = 10002,         /* parameter block size does not match the signature, or exceeds FKLHIP_MAX_BLOB_BYTES */
    FKLHIP_EINVAL = 10003              /* null pointer / malformed argument */
};

enum { FKLHIP_COPY_H2H = 0, FKLHIP_COPY_H2D = 1, FKLHIP_COPY_D2H = 2, FKLHIP_COPY_D2D = 3 };

/* Largest parameter block a launch accepts.  A chain's parameters travel as by-value kernel arguments, like the
 * reference's __grid_constant__ arguments (FK/core/execution_model/executor_details/executor_kernels.h:26-30), and
 * grow with the batch (FK/core/execution_model/operation_model/batch_operations.h:164-219: one entry per plane).
 * Measured on an MI355X with ROCm 7.2: the HIP runtime accepts 1 048 584 bytes of kernel arguments and the kernel reads
 * them correctly; with 4 MiB the launch call crashes inside the runtime.  The library therefore refuses anything above
 * 1 MiB less 64 bytes (room for its own trailing arguments) with FKLHIP_EBLOB_SIZE instead of passing it on. */
#define FKLHIP_MAX_BLOB_BYTES 1048512

/* Library identity: FKLHIP_ABI_VERSION the library was built with. */
int fklhip_abi_version(void);

/* Human readable text for any code the library returns (hipGetErrorString for runtime codes).
 * Replaces cudaGetErrorString inside gpuErrchk: FK/core/utils/utils.h:100-114. */
const char *fklhip_error_string(int code);

/* Device selection.  Replaces cudaGetDevice/cudaSetDevice around allocations: FK/core/data/ptr_nd.h:154-166. */
int fklhip_get_device(int *device);
int fklhip_set_device(int device);
int fklhip_device_count(int *count);

/* Streams (always default priority).  Replaces cudaStreamCreate/Destroy/Synchronize in Stream_<GPU_NVIDIA>:
 * FK/core/execution_model/stream.h:52-109. */
int fklhip_stream_create(void **stream);
int fklhip_stream_destroy(void *stream);
int fklhip_stream_sync(void *stream);

/* Memory.  Replaces cudaMalloc / cudaMallocPitch / cudaFree / cudaMallocHost / cudaFreeHost in PtrImpl and Ptr:
 * FK/core/data/ptr_nd.h:47-126,154-250. */
int fklhip_malloc(void **ptr, size_t bytes);
int fklhip_malloc_pitch(void **ptr, size_t *pitch, size_t width_bytes, size_t height);
int fklhip_free(void *ptr);
int fklhip_host_alloc(void **ptr, size_t bytes);   /* pinned */
int fklhip_host_free(void *ptr);

/* Asynchronous copies on a stream.  Replaces cudaMemcpyAsync / cudaMemcpy2DAsync in Ptr::copy:
 * FK/core/data/ptr_nd.h:253-269. */
int fklhip_memcpy_async(void *dst, const void *src, size_t bytes, int kind, void *stream);
int fklhip_memcpy2d_async(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t width_bytes,
                          size_t height, int kind, void *stream);
int fklhip_memset_async(void *dst, int value, size_t bytes, void *stream);

/* Events for timing.  Replaces the cudaEvent pairs of the reference benchmarks:
 * benchmarks/fkBenchmarksCommon.h:78-132. */
int fklhip_event_create(void **event);
int fklhip_event_destroy(void *event);
int fklhip_event_record(void *event, void *stream);
int fklhip_event_sync(void *event);
int fklhip_event_elapsed_ms(float *ms, void *start, void *stop);

/*
 * Launch one fused chain.  Replaces launchTransformDPP_Kernel<<<grid, block, 0, stream>>>(details, iOps...)
 * followed by gpuErrchk(cudaGetLastError()): FK/core/execution_model/executors.h:316-351.
 *
 *   signature   the chain's type, spelled as the device-side C++ type expression (for example
 *               "Chain<Read2D<f32>,OpList<Add<f32,f32,f32>>,Write2D<f32>>"); it selects the kernel.
 *   blob        the chain's parameter block (active grid, read, compute and write parameters), laid out as the
 *               device type <signature>::Params; it is copied before the call returns, like by-value kernel
 *               arguments, so the caller may free it immediately.
 *   stream      a stream from fklhip_stream_create, or NULL for the default stream.
 *
 * fklhip_lookup resolves a signature once; the handle stays valid for the life of the process.
 */
int fklhip_lookup(const char *signature, const void **handle);
int fklhip_launch_handle(const void *handle, const void *blob, size_t blob_bytes, void *stream);
int fklhip_launch(const char *signature, const void *blob, size_t blob_bytes, void *stream);

/* A signature that was not compiled ahead of time is compiled when fklhip_lookup / fklhip_launch first see it
 * (device headers are embedded in the library; about a second per new signature, once per process; switched off by
 * the environment variable FKLHIP_JIT=0).  This is the library's stand-in for nvcc compiling the user's translation
 * unit, FK/core/execution_model/executors.h:316-351 being instantiated for whatever chain the user wrote.  When the
 * lookup fails, fklhip_jit_log returns the device compiler's messages for the last attempt on this thread (valid
 * until the next lookup on the thread).  With the environment variable FKLHIP_JIT_CACHE naming an existing directory,
 * compiled code objects are kept there (file name = hash of signature, architecture, flags and header text) and
 * reused by later processes; after such a reuse the log reads "loaded from <file>". */
int fklhip_jit_log(const char **log);

/* The bilinear kernel has two forms that give identical results: tiles, and for outputs up to 256 pixels wide whole
 * rows ("strip").  fklhip_strip_form(0) makes every later launch of the process take the tile form, fklhip_strip_form(1)
 * restores the choice by shape, a negative argument changes nothing; the return value is the previous setting (0 or 1).
 * The initial setting is 1 unless the environment variable FKLHIP_STRIP is "0" when the library first needs it.  No
 * counterpart in the reference; it exists so that tests can compare the two forms in one process. */
int fklhip_strip_form(int enable);

/* Introspection for tests and benchmarks: what the last fklhip_launch* on this thread launched.
 * kernel receives "rows", "rows_unaligned", "gather", or "rows_jit" / "gather_jit" for chains compiled at run time; grid/block receive 3 values each. */
int fklhip_last_launch(const char **kernel, unsigned grid[3], unsigned block[3], unsigned *lds_bytes);

/* Number of chain signatures compiled into the library and the i-th of them with its parameter block size. */
int fklhip_signature_count(int *count);
int fklhip_signature_at(int index, const char **signature, size_t *blob_bytes);

#ifdef __cplusplus
}
#endif
#endif

// registry.hpp -- table of the chain signatures compiled ahead of time into libfklhip.so.
#pragma once

#include <stddef.h>
#include <stdlib.h>

namespace fkd { struct LaunchInfo; }

namespace fklhip {

// `ctx` is whatever the registrant passed to register_chain: nothing for kernels compiled ahead of time, the loaded
// module for kernels compiled at run time.
using LaunchFn = int (*)(const void* ctx, const void* blob, size_t bytes, void* stream, fkd::LaunchInfo* info);

struct Entry {
    const char* signature;   // owned by the registry (process lifetime)
    size_t blob_bytes;
    LaunchFn launch;
    const void* ctx;
};

// Narrow outputs of bilinear chains are launched in strip form unless that was switched off: by FKLHIP_STRIP=0 in the
// environment when the setting is first needed, or by fklhip_strip_form(0) (the two forms give identical results).
bool strip_enabled();

// Called from static initialisers of the generated instance files, and by the run-time compiler.
void register_chain(const char* signature, size_t blob_bytes, LaunchFn fn, const void* ctx = nullptr);

// Run-time compilation (jit.cpp).  jit_compile_and_register returns FKLHIP_OK after registering the chain, or
// FKLHIP_EUNKNOWN_SIGNATURE when run-time compilation is switched off or the signature does not compile (the
// compiler's messages are then available through jit_last_log).
int jit_compile_and_register(const char* signature);
const char* jit_last_log();

// Device headers and compiler flags embedded at build time (generated file aot/jit_sources.cpp).
extern const char* const kJitHeaderNames[];
extern const char* const kJitHeaderTexts[];
extern const int kJitHeaderCount;
extern const char* const kJitFlags[];
extern const int kJitFlagCount;

} // namespace fklhip

// registry.hpp -- table of the chain signatures compiled ahead of time into libfklhip.so.
#pragma once

#include <stddef.h>

namespace fkd { struct LaunchInfo; }

namespace fklhip {

using LaunchFn = int (*)(const void* blob, size_t bytes, void* stream, fkd::LaunchInfo* info);

struct Entry {
    const char* signature;   // owned by the registry (process lifetime)
    size_t blob_bytes;
    LaunchFn launch;
};

// Called from static initialisers of the generated instance files.
void register_chain(const char* signature, size_t blob_bytes, LaunchFn fn);

} // namespace fklhip

// aot_common.hpp -- glue included by the generated instance files (aot/aot_*.hip): one FKD_AOT_CHAIN(...) line
// instantiates the kernel of a chain for gfx950 and registers its launcher under the chain's signature.
#pragma once

#define FKD_DEVICE_CODE 1
#include "fkd_launch.hpp"
#include "registry.hpp"
#include <fklhip.h>

#include <stdint.h>
#include <string.h>
#include <string>

namespace fklhip {

template <class Chain> int aot_launch(const void*, const void* blob, size_t bytes, void* stream, fkd::LaunchInfo* info) {
    using Params = typename Chain::Params;
    static_assert(sizeof(Params) <= size_t(FKLHIP_MAX_BLOB_BYTES), "the chain's parameter block exceeds FKLHIP_MAX_BLOB_BYTES: use a smaller batch per launch");
    if (!blob) return FKLHIP_EINVAL;
    if (bytes != sizeof(Params)) return FKLHIP_EBLOB_SIZE;
    // The runtime copies the block into its kernel-argument buffer during the launch call, so the caller's block may go
    // away as soon as we return; a block that is not aligned for its type is copied to one that is first.
    if (reinterpret_cast<uintptr_t>(blob) % alignof(Params) == 0)
        return int(fkd::launch_chain<Chain>(*static_cast<const Params*>(blob), static_cast<hipStream_t>(stream), info));
    Params p;
    memcpy(&p, blob, sizeof(Params));
    return int(fkd::launch_chain<Chain>(p, static_cast<hipStream_t>(stream), info));
}

template <class Chain> struct Registrar {
    Registrar() {
        static const std::string sig = Chain::name();
        register_chain(sig.c_str(), sizeof(typename Chain::Params), &aot_launch<Chain>);
    }
};

} // namespace fklhip

#define FKD_AOT_CAT2(a, b) a##b
#define FKD_AOT_CAT(a, b) FKD_AOT_CAT2(a, b)
#define FKD_AOT_CHAIN(...) static ::fklhip::Registrar<__VA_ARGS__> FKD_AOT_CAT(fkd_aot_reg_, __COUNTER__);

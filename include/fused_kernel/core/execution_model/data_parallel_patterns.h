// TransformDPP: the data-parallel pattern "read -> fold of compute operations -> write, one work item per output
// element, grid z = batch plane".  On this backend the pattern's body is the gfx950 kernels of libfklhip.so; the
// type below only names the pattern, its architecture and the (result-neutral) thread-fusion switch.
// Interface counterpart: FK/core/execution_model/data_parallel_patterns.h:65-66.
#ifndef FK_AMD_DATA_PARALLEL_PATTERNS_H
#define FK_AMD_DATA_PARALLEL_PATTERNS_H

#include <fused_kernel/core/execution_model/parallel_architectures.h>
#include <fused_kernel/core/execution_model/thread_fusion.h>

namespace fk {

template <ParArch PA = defaultParArch, TF TFEN = TF::DISABLED, typename DPPDetails = void, bool THREAD_DIVISIBLE = true>
struct TransformDPP {
    static constexpr ParArch PAR_ARCH = PA;
    static constexpr TF THREAD_FUSION = TFEN;
};

} // namespace fk
#endif

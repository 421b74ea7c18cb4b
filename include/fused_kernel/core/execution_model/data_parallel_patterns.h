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


// DivergentBatchTransformDPP: several operation sequences in ONE launch; plane z of the launch (z counts over the
// planes of all sequences together) runs sequence SequenceSelector::at(z), and z reaches that sequence's read and
// write unchanged.  SequenceSelector is any type with a static `uint at(uint z)`; on this backend it is evaluated on
// the host for every plane of a launch and travels to the kernel as a table.
// Interface counterpart: FK/core/execution_model/data_parallel_patterns.h:286-381.
template <ParArch PA, typename SequenceSelector> struct DivergentBatchTransformDPP {
    static constexpr ParArch PAR_ARCH = PA;
};

} // namespace fk
#endif

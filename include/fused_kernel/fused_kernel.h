// Entry points: fk::executeOperations<DPP>(...), forwarding to Executor<DPP>.
// Interface counterpart: FK/fused_kernel.h:22-54 (same seven overloads, same argument order).
#ifndef FK_AMD_FUSED_KERNEL_H
#define FK_AMD_FUSED_KERNEL_H

#include <fused_kernel/core/execution_model/executors.h>

namespace fk {

template <typename DPPType, typename... Args>
inline void executeOperations(Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(stream, args...);
}
template <typename DPPType, ND D, typename I, typename... Args>
inline void executeOperations(const Ptr<D, I>& input, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, stream, args...);
}
template <typename DPPType, ND D, typename I, typename O, typename... Args>
inline void executeOperations(const Ptr<D, I>& input, const Ptr<D, O>& output, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, output, stream, args...);
}
template <typename DPPType, typename I, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                              Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, activeBatch, defaultValue, stream, args...);
}
template <typename DPPType, typename I, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, stream, args...);
}
template <typename DPPType, typename I, typename O, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                              const Tensor<O>& output, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, activeBatch, defaultValue, output, stream, args...);
}
template <typename DPPType, typename I, typename O, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const Tensor<O>& output,
                              Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, output, stream, args...);
}

} // namespace fk
#endif

// Executor<TransformDPP<ParArch::GPU_AMD, TF>>: turns an argument list of IOps into one launch of a gfx950 kernel.
// (Executor<TransformDPP<ParArch::CPU, TF>>, further down, runs the same lowered chain on the calling thread.)
//
//   1. BackFuser::fuse_back collapses the Read + ReadBack... prefix into one Read IOp (backwards vertical fusion).
//   2. Every IOp is lowered to its device counterpart; together they spell the type fkd::Chain<Read, OpList<...>,
//      Write>.  Its name() is the kernel signature; its Params, filled from the IOps' values, is the kernel argument.
//   3. fklhip_launch_handle copies the parameter block and enqueues the kernel on the stream (asynchronous, like the
//      CUDA backend's <<<>>> launch); a failure surfaces as std::runtime_error("GPU Error: ...").
//
// Interface counterpart: FK/core/execution_model/executors.h:53-143 (overload family), :311-358 (GPU executor).
#ifndef FK_AMD_EXECUTORS_H
#define FK_AMD_EXECUTORS_H

#include <string>

#include <fused_kernel/core/execution_model/data_parallel_patterns.h>
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/execution_model/stream.h>
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>

namespace fk {

namespace amd {

// The device chain type of a fused IOp list (read, compute..., write).
template <typename ReadIOp, typename... Rest> struct ChainOf;
template <typename ReadIOp, typename WriteIOp, typename... Compute>
struct ChainBuilder {
    using type = fkd::Chain<device_op_t<ReadIOp>, fkd::OpList<device_op_t<Compute>...>, device_op_t<WriteIOp>>;
};

template <typename Chain> const void* kernel_handle() {
    // Resolved once per chain type; thread-safe by the rules of function-local statics.
    static const void* handle = [] {
        const std::string sig = Chain::name();
        const void* h = nullptr;
        const int rc = fklhip_lookup(sig.c_str(), &h);
        if (rc != FKLHIP_OK) {
            throw std::runtime_error(std::string("GPU Error: ") + fklhip_error_string(rc) + "\n  signature: " + sig + "\n");
        }
        return h;
    }();
    return handle;
}

template <size_t... Is, typename Tuple>
auto lower_compute(std::index_sequence<Is...>, const Tuple& t) {
    return make_tup(lower_iop(std::get<Is + 1>(t))...);
}

// One fused IOp list (complete read, compute operations, [a MidWrite directly before] the write) as a device chain type
// and its parameter block.
template <typename... IOps> struct FusedChain {
    static constexpr size_t N = sizeof...(IOps);
    static_assert(N >= 2, "a chain needs at least a read and a write operation");
    using Tuple = std::tuple<const IOps&...>;
    template <size_t I> using At = std::decay_t<std::tuple_element_t<I, Tuple>>;
    using ReadIOp = At<0>;
    using WriteIOp = At<N - 1>;
    static_assert(isAnyCompleteReadType<ReadIOp>, "the first operation must be a complete Read or ReadBack operation");
    static_assert(opIs<WriteType, WriteIOp>, "the last operation must be a Write operation");
    // A MidWrite stores the value it receives and hands it on; directly before the final write both take the same value.
    static constexpr bool kTee = N >= 3 && opIs<MidWriteType, At<N >= 3 ? N - 2 : 0>>;
    static constexpr size_t kCompute = N - 2 - (kTee ? 1 : 0);
    template <typename Seq> struct Build;
    template <size_t... Is> struct Build<std::index_sequence<Is...>> {
        static_assert((isComputeType<At<Is + 1>> && ...),
                      "only Unary/Binary/Ternary operations may sit between the read and the write (a MidWrite only directly before the write)");
        using WriteOp = std::conditional_t<kTee, fkd::TeeWrite<device_op_t<At<kTee ? N - 2 : N - 1>>, device_op_t<WriteIOp>>, device_op_t<WriteIOp>>;
        using Chain = fkd::Chain<device_op_t<ReadIOp>, fkd::OpList<device_op_t<At<Is + 1>>...>, WriteOp>;
        static typename Chain::Params params(const Tuple& all) {
            typename Chain::Params p{};
            const ActiveThreads active = std::get<0>(all).getActiveThreads();
            p.active_w = active.x;
            p.active_h = active.y;
            p.active_z = active.z;
            p.read = lower_iop(std::get<0>(all));
            p.ops = make_tup(lower_iop(std::get<Is + 1>(all))...);
            Chain::finalize(p);
            if constexpr (kTee) {
                p.write.first = lower_iop(std::get<N - 2>(all));
                p.write.second = lower_iop(std::get<N - 1>(all));
            } else {
                p.write = lower_iop(std::get<N - 1>(all));
            }
            Chain::finalize_write(p);
            return p;
        }
    };
    using Builder = Build<std::make_index_sequence<kCompute>>;
    using Chain = typename Builder::Chain;
    static typename Chain::Params params(const IOps&... iOps) { return Builder::params(std::forward_as_tuple(iOps...)); }
};

template <typename... IOps> void launch_fused(void* stream, const IOps&... iOps) {
    using F = FusedChain<IOps...>;
    static_assert(!F::kTee, "a MidWrite operation is only supported inside the sequences of a DivergentBatchTransformDPP launch");
    static_assert(sizeof(typename F::Chain::Params) <= size_t(FKLHIP_MAX_BLOB_BYTES),
                  "the fused chain's parameters exceed FKLHIP_MAX_BLOB_BYTES (1 MiB of by-value kernel arguments): every plane of a "
                  "BatchRead or BatchWrite adds its own parameters, so use a smaller BATCH per launch");
    const typename F::Chain::Params p = F::params(iOps...);
    gpuErrchk(fklhip_launch_handle(kernel_handle<typename F::Chain>(), &p, sizeof(p), stream));
}

// Several already back-fused sequences in one launch.
template <typename SequenceSelector, typename... Seqs> void launch_divergent(void* stream, const Seqs&... seqs) {
    using D = fkd::Divergent<typename Seqs::Fused::Chain...>;
    static_assert(sizeof(typename D::Params) <= size_t(FKLHIP_MAX_BLOB_BYTES),
                  "the sequences' parameters together exceed FKLHIP_MAX_BLOB_BYTES (1 MiB of by-value kernel arguments)");
    typename D::Params p{};
    uint w = 0, h = 0, z = 0;
    auto fill = [&](auto& self, auto& node, const auto& first, const auto&... rest) -> void {
        node.head = first.params;
        w = first.params.active_w > w ? first.params.active_w : w;
        h = first.params.active_h > h ? first.params.active_h : h;
        z += first.params.active_z;
        if constexpr (sizeof...(rest) > 0) self(self, node.tail, rest...);
    };
    fill(fill, p.seq, seqs...);
    if (z > uint(D::kMaxPlanes))
        throw std::runtime_error("GPU Error: a DivergentBatchTransformDPP launch holds at most " + std::to_string(D::kMaxPlanes) + " planes");
    p.active_w = w; p.active_h = h; p.active_z = z;
    for (uint i = 0; i < z; ++i) {
        const uint sel = uint(SequenceSelector::at(i));
        // a plane no sequence claims runs nothing in the reference; the table entry then names no chain
        p.select[i] = static_cast<unsigned char>(sel < uint(D::kChains) ? sel : 255u);
    }
    gpuErrchk(fklhip_launch_handle(kernel_handle<D>(), &p, sizeof(p), stream));
}
template <typename... IOps> struct LoweredSequence {
    using Fused = FusedChain<IOps...>;
    typename Fused::Chain::Params params;
};

// ---- ParArch::CPU: the same lowered chain, run element by element on the calling thread ------------------------------
// Reference loop: FK/core/execution_model/data_parallel_patterns.h:271-283 (one pass over z, y, x; synchronous).  The
// element bodies are the device operations' own (fkd::...::exec, compiled for the host), so both architectures compute
// every element with the same source code; with floating-point contraction off on the host (-ffp-contract=off, and no
// -ffast-math) the results are the same bits.  Nothing on the GPU path ever comes here: the architecture is part of the
// DPP's type, chosen by the caller.
template <typename Chain> void run_plane_on_host(const typename Chain::Params& p, int z) {
    const int w = int(p.active_w), h = int(p.active_h);
    for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x)
            Chain::Write::exec(x, y, z, Chain::compute(Chain::Read::exec(x, y, z, p.read), p), p.write);
}
template <typename... IOps> void run_fused_on_host(const IOps&... iOps) {
    using F = FusedChain<IOps...>;
    const typename F::Chain::Params p = F::params(iOps...);
    for (int z = 0; z < int(p.active_z); ++z) run_plane_on_host<typename F::Chain>(p, z);
}
template <size_t I, typename First, typename... Rest> void run_selected_on_host(size_t sel, int z, const First& first, const Rest&... rest) {
    if (sel == I) run_plane_on_host<typename First::Fused::Chain>(first.params, z);
    else if constexpr (sizeof...(Rest) > 0) run_selected_on_host<I + 1>(sel, z, rest...);
}
template <typename SequenceSelector, typename... Seqs> void run_divergent_on_host(const Seqs&... seqs) {
    uint planes = 0;
    ((planes += seqs.params.active_z), ...);
    // plane z runs sequence SequenceSelector::at(z), with z handed on unchanged; a plane no sequence claims runs nothing
    for (uint z = 0; z < planes; ++z) run_selected_on_host<0>(size_t(SequenceSelector::at(z)), int(z), seqs...);
}

template <typename... IOps> auto lower_sequence(const IOpSequence<IOps...>& seq) {
    const auto fused = std::apply([](const auto&... iOps) { return BackFuser::fuse_back(iOps...); }, seq.iOps);
    return std::apply([](const auto&... f) {
        return LoweredSequence<std::decay_t<decltype(f)>...>{FusedChain<std::decay_t<decltype(f)>...>::params(f...)};
    }, fused);
}

} // namespace amd

template <typename Child> struct BaseExecutor {
    template <ParArch PA, typename... IOps> static void executeOperations(Stream_<PA>& stream, const IOps&... iOps) {
        const auto fused = BackFuser::fuse_back(iOps...);
        std::apply([&](const auto&... f) { Child::executeOperations_helper(stream, f...); }, fused);
    }
    template <ParArch PA, ND D, typename I, typename... IOps>
    static void executeOperations(const Ptr<D, I>& input, Stream_<PA>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<D, I>::build(input.ptr()), iOps...);
    }
    template <ParArch PA, ND D, typename I, typename O, typename... IOps>
    static void executeOperations(const Ptr<D, I>& input, const Ptr<D, O>& output, Stream_<PA>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<D, I>::build(input.ptr()), iOps..., PerThreadWrite<D, O>::build(output.ptr()));
    }
    template <ParArch PA, typename I, size_t BATCH, typename... IOps>
    static void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                                  Stream_<PA>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(activeBatch, defaultValue, input), iOps...);
    }
    template <ParArch PA, typename I, size_t BATCH, typename... IOps>
    static void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, Stream_<PA>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(input), iOps...);
    }
    template <ParArch PA, typename I, typename O, size_t Batch, typename... IOps>
    static void executeOperations(const std::array<Ptr2D<I>, Batch>& input, const int& activeBatch, const I& defaultValue,
                                  const Tensor<O>& output, Stream_<PA>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(activeBatch, defaultValue, input), iOps...,
                          PerThreadWrite<ND::_3D, O>::build(output.ptr()));
    }
    template <ParArch PA, typename I, typename O, size_t Batch, typename... IOps>
    static void executeOperations(const std::array<Ptr2D<I>, Batch>& input, const Tensor<O>& output, Stream_<PA>& stream,
                                  const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(input), iOps..., PerThreadWrite<ND::_3D, O>::build(output.ptr()));
    }
};

template <typename DataParallelPattern> struct Executor {
    static_assert(DataParallelPattern::PAR_ARCH == ParArch::GPU_AMD || DataParallelPattern::PAR_ARCH == ParArch::CPU,
                  "this build of the library provides the GPU_AMD (MI355X) and CPU architectures");
};

template <TF TFEN> struct Executor<TransformDPP<ParArch::GPU_AMD, TFEN, void>> : BaseExecutor<Executor<TransformDPP<ParArch::GPU_AMD, TFEN, void>>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::GPU_AMD; }

private:
    friend struct BaseExecutor<Executor<TransformDPP<ParArch::GPU_AMD, TFEN, void>>>;
    template <typename... IOps> static void executeOperations_helper(Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        amd::launch_fused(stream.getNativeStream(), iOps...);
    }
};


// TransformDPP<ParArch::CPU>: FK/core/execution_model/executors.h:163-189.  Synchronous; the stream is the reference's
// no-op Stream_<ParArch::CPU>.  Thread fusion changes nothing here either.
template <TF TFEN> struct Executor<TransformDPP<ParArch::CPU, TFEN, void>> : BaseExecutor<Executor<TransformDPP<ParArch::CPU, TFEN, void>>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::CPU; }

private:
    friend struct BaseExecutor<Executor<TransformDPP<ParArch::CPU, TFEN, void>>>;
    template <typename... IOps> static void executeOperations_helper(Stream_<ParArch::CPU>&, const IOps&... iOps) {
        amd::run_fused_on_host(iOps...);
    }
};

// Executor of DivergentBatchTransformDPP: every sequence is back-fused like a TransformDPP chain, then all of them go
// into one launch.  Interface counterpart: FK/core/execution_model/executors.h:360-411.
template <typename SequenceSelector> struct Executor<DivergentBatchTransformDPP<ParArch::GPU_AMD, SequenceSelector>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::GPU_AMD; }
    template <typename... IOpSequenceTypes>
    static void executeOperations(Stream_<ParArch::GPU_AMD>& stream, const IOpSequenceTypes&... iOpSequences) {
        amd::launch_divergent<SequenceSelector>(stream.getNativeStream(), lower(iOpSequences)...);
    }

private:
    template <typename... IOps> static auto lower(const IOpSequence<IOps...>& seq) { return amd::lower_sequence(seq); }
};

template <typename SequenceSelector> struct Executor<DivergentBatchTransformDPP<ParArch::CPU, SequenceSelector>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::CPU; }
    template <typename... IOpSequenceTypes>
    static void executeOperations(Stream_<ParArch::CPU>&, const IOpSequenceTypes&... iOpSequences) {
        amd::run_divergent_on_host<SequenceSelector>(amd::lower_sequence(iOpSequences)...);
    }
};

} // namespace fk
#endif

// Host-side fusion of IOps: Fuser::fuse (operator&, then()), fuse(a, b, ...), and BackFuser::fuse_back, which
// collapses the leading Read + ReadBack... prefix of an executeOperations argument list into one Read IOp.
// Interface counterpart: FK/core/execution_model/operation_model/iop_fuser.h:22-193.
#ifndef FK_AMD_IOP_FUSER_H
#define FK_AMD_IOP_FUSER_H

#ifndef FK_AMD_OPERATION_MODEL_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#else

namespace fk {

struct Fuser {
    template <typename SelfType, typename ContinuationIOp>
    static constexpr auto fuse(const SelfType& selfIOp, const ContinuationIOp& cIOp) {
        static_assert(isOperation<SelfType> && isOperation<ContinuationIOp>, "SelfType and ContinuationIOp should be IOps");
        using SelfOp = typename SelfType::Operation;
        using ContOp = typename ContinuationIOp::Operation;
        constexpr bool selfBatch = isBatchOperation<SelfOp>;
        constexpr bool contBatch = isBatchOperation<ContOp>;
        if constexpr (selfBatch && contBatch) {
            // plane i of the source feeds plane i of the continuation
            static_assert(SelfOp::BATCH == ContOp::BATCH, "Fusing two batch operations of different BATCH size is not allowed.");
            static_assert(opIs<IncompleteReadBackType, typename ContOp::Operation>,
                          "Read or ReadBack Operation as continuation is not allowed. It has to be an IncompleteReadBackOperation.");
            const auto back = BatchUtils::toArray(selfIOp);
            const auto fwd = BatchUtils::toArray(cIOp);
            using Builder = typename ContOp::Operation;
            if constexpr (SelfOp::PP == PlanePolicy::PROCESS_ALL && ContOp::PP == PlanePolicy::PROCESS_ALL) {
                return Builder::build(back, fwd);
            } else if constexpr (ContOp::PP == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
                return Builder::build(cIOp.params.usedPlanes, cIOp.params.default_value, back, fwd);
            } else {
                return Builder::build(selfIOp.params.usedPlanes, selfIOp.params.default_value, back, fwd);
            }
        } else if constexpr (!selfBatch && contBatch) {
            // one source shared by every plane of the continuation
            static_assert(opIs<IncompleteReadBackType, typename ContOp::Operation>,
                          "ReadOperation as continuation is not allowed. It has to be a ReadBackOperation.");
            constexpr size_t BATCH = size_t(ContOp::BATCH);
            const auto back = make_set_std_array<BATCH>(selfIOp);
            const auto fwd = BatchUtils::toArray(cIOp);
            using Builder = typename ContOp::Operation;
            if constexpr (ContOp::PP == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
                return Builder::build(cIOp.params.usedPlanes, cIOp.params.default_value, back, fwd);
            } else {
                return Builder::build(back, fwd);
            }
        } else if constexpr (selfBatch && !contBatch) {
            // the same continuation applied to every plane
            static_assert(!isAnyReadType<ContinuationIOp> || opIs<IncompleteReadBackType, ContinuationIOp>,
                          "ReadOperation as continuation is not allowed. It has to be a ReadBackOperation.");
            constexpr size_t BATCH = size_t(SelfOp::BATCH);
            const auto back = BatchUtils::toArray(selfIOp);
            const auto fwd = make_set_std_array<BATCH>(cIOp);
            if constexpr (opIs<IncompleteReadBackType, ContinuationIOp>) {
                using Builder = ContOp;
                if constexpr (SelfOp::PP == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
                    return Builder::build(selfIOp.params.usedPlanes, selfIOp.params.default_value, back, fwd);
                } else {
                    return Builder::build(back, fwd);
                }
            } else {
                const auto fused = fuse_planes(back, fwd);
                if constexpr (SelfOp::PP == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
                    return BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(fused, selfIOp.params.usedPlanes,
                                                                                   selfIOp.params.default_value);
                } else {
                    return BatchRead<PlanePolicy::PROCESS_ALL>::build(fused);
                }
            }
        } else {
            static_assert(!isAnyCompleteReadType<ContinuationIOp>,
                          "Complete Read Operations as continuations are not allowed. It has to be an IncompleteReadBackOperation.");
            if constexpr (opIs<IncompleteReadBackType, ContinuationIOp>) {
                return ContOp::build(selfIOp, cIOp);
            } else {
                return FusedOperation<>::build(selfIOp, cIOp);
            }
        }
    }

private:
    template <size_t BATCH, typename ThisIOp, typename ForwardIOp>
    static constexpr auto fuse_planes(const std::array<ThisIOp, BATCH>& self, const std::array<ForwardIOp, BATCH>& fwd) {
        using Result = decltype(FusedOperation<>::build(std::declval<ThisIOp>(), std::declval<ForwardIOp>()));
        std::array<Result, BATCH> out{};
        for (size_t i = 0; i < BATCH; ++i) out[i] = FusedOperation<>::build(self[i], fwd[i]);
        return out;
    }
};

// a & b & c : left fold of Fuser::fuse.
template <typename A, typename B, std::enable_if_t<isOperation<A> && isOperation<B> && op_detail::has_operation<A>::value &&
                                                   op_detail::has_operation<B>::value, int> = 0>
constexpr auto operator&(const A& a, const B& b) {
    return Fuser::fuse(a, b);
}

template <typename FirstIOp, typename... IOps> constexpr decltype(auto) fuse(FirstIOp&& firstIOp, IOps&&... iOps) {
    return (std::forward<FirstIOp>(firstIOp) & ... & std::forward<IOps>(iOps));
}

struct BackFuser {
protected:
    // 1-based position of the LAST ReadBack / IncompleteReadBack IOp in the list, 0 if there is none.
    template <typename... IOps> static constexpr size_t idxFirstNonBack() {
        size_t index = 0, result = 0;
        ((++index, (opIs<ReadBackType, IOps> || opIs<IncompleteReadBackType, IOps>) ? (result = index) : size_t(0)), ...);
        return result;
    }
    template <typename T, size_t... Is> static constexpr auto head(T&& t, const std::index_sequence<Is...>&) {
        return fuse(std::get<Is>(std::forward<T>(t))...);
    }
    template <size_t Offset, typename T, size_t... Is> static constexpr auto tail(T&& t, const std::index_sequence<Is...>&) {
        return std::make_tuple(std::get<Offset + Is>(std::forward<T>(t))...);
    }

public:
    // Everything up to and including the last read-back IOp is fused into one IOp; the rest is kept as is.
    template <typename... IOps> static constexpr auto fuse_back(IOps&&... iOps) {
        constexpr size_t split = idxFirstNonBack<std::decay_t<IOps>...>();
        if constexpr (split < 2) {
            return std::forward_as_tuple(std::forward<IOps>(iOps)...);
        } else {
            auto all = std::forward_as_tuple(std::forward<IOps>(iOps)...);
            auto fused = head(all, std::make_index_sequence<split>{});
            auto rest = tail<split>(all, std::make_index_sequence<sizeof...(IOps) - split>{});
            return std::tuple_cat(std::make_tuple(fused), rest);
        }
    }
};

} // namespace fk
#endif
#endif

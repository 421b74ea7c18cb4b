// FusedOperation<IOps...>: a left-to-right sequence of IOps packaged as one Operation.
//   first IOp is a Read / ReadBack  -> the package is a Read     (vertical fusion into the read)
//   only compute IOps               -> the package is a Unary (no parameters anywhere) or a Binary
// Interface counterpart: FK/core/execution_model/operation_model/fused_operation.h.
#ifndef FK_AMD_FUSED_OPERATION_H
#define FK_AMD_FUSED_OPERATION_H

#ifndef FK_AMD_OPERATION_MODEL_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#else

namespace fk {

namespace fused_detail {

template <typename... Ts> struct first_of;
template <typename T, typename... Ts> struct first_of<T, Ts...> { using type = T; };
template <typename... Ts> struct last_of;
template <typename T> struct last_of<T> { using type = T; };
template <typename T, typename... Ts> struct last_of<T, Ts...> { using type = typename last_of<Ts...>::type; };

enum class Kind { Read, Unary, Binary };
template <typename... IOps> constexpr Kind kind_of() {
    using F = typename first_of<IOps...>::type;
    if constexpr (opIs<ReadType, F> || opIs<ReadBackType, F>) return Kind::Read;
    else if constexpr ((opIs<UnaryType, IOps> && ...)) return Kind::Unary;
    else return Kind::Binary;
}

template <typename T> struct is_fused_iop : std::false_type {};

template <Kind K, typename Self, typename... IOps> struct Base;

template <typename Self, typename... IOps> struct Base<Kind::Read, Self, IOps...> {
    using FirstIOp = typename first_of<IOps...>::type;
    using LastIOp = typename last_of<IOps...>::type;
    using ParamsType = std::tuple<IOps...>;
    using ReadDataType = typename FirstIOp::Operation::ReadDataType;
    using OutputType = typename LastIOp::Operation::OutputType;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<Self>;
    using InstantiableType = Read<Self>;
    static constexpr bool IS_FUSED_OP = true;
    static constexpr bool THREAD_FUSION = false;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params) { return {{params}}; }
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) {
        return FirstIOp::Operation::num_elems_x(thread, std::get<0>(opData.params));
    }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) {
        return FirstIOp::Operation::num_elems_y(thread, std::get<0>(opData.params));
    }
    static constexpr uint num_elems_z(const Point thread, const OperationDataType& opData) {
        return FirstIOp::Operation::num_elems_z(thread, std::get<0>(opData.params));
    }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), num_elems_z(Point{0, 0, 0}, opData)};
    }
};

template <typename Self, typename... IOps> struct Base<Kind::Binary, Self, IOps...> {
    using FirstIOp = typename first_of<IOps...>::type;
    using LastIOp = typename last_of<IOps...>::type;
    using ParamsType = std::tuple<IOps...>;
    using InputType = typename FirstIOp::Operation::InputType;
    using OutputType = typename LastIOp::Operation::OutputType;
    using InstanceType = BinaryType;
    using OperationDataType = OperationData<Self>;
    using InstantiableType = Binary<Self>;
    static constexpr bool IS_FUSED_OP = true;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params) { return {{params}}; }
};

template <typename Self, typename... IOps> struct Base<Kind::Unary, Self, IOps...> {
    using FirstIOp = typename first_of<IOps...>::type;
    using LastIOp = typename last_of<IOps...>::type;
    using InputType = typename FirstIOp::Operation::InputType;
    using OutputType = typename LastIOp::Operation::OutputType;
    using InstanceType = UnaryType;
    using InstantiableType = Unary<Self>;
    static constexpr bool IS_FUSED_OP = true;
    static constexpr InstantiableType build() { return {}; }
    static constexpr InstantiableType build(const std::tuple<IOps...>&) { return {}; }
};

} // namespace fused_detail

template <typename... IOps>
struct FusedOperation : fused_detail::Base<fused_detail::kind_of<IOps...>(), FusedOperation<IOps...>, IOps...> {
    static_assert((isOperation<IOps> && ...), "FusedOperation takes instantiable operations");
    static_assert((!opIs<WriteType, IOps> && ...) && (!opIs<IncompleteReadBackType, IOps> && ...),
                  "Write and incomplete read-back operations cannot be packaged into a FusedOperation");
    using IOpList = TypeList<IOps...>;
};

namespace fused_detail {
template <typename... IOps> struct is_fused_iop<Read<FusedOperation<IOps...>>> : std::true_type {};
template <typename... IOps> struct is_fused_iop<Binary<FusedOperation<IOps...>>> : std::true_type {};
template <typename... IOps> struct is_fused_iop<Unary<FusedOperation<IOps...>>> : std::true_type {};

template <typename... IOps> constexpr std::tuple<IOps...> unpack(const Read<FusedOperation<IOps...>>& iop) { return iop.params; }
template <typename... IOps> constexpr std::tuple<IOps...> unpack(const Binary<FusedOperation<IOps...>>& iop) { return iop.params; }
template <typename... IOps> constexpr std::tuple<IOps...> unpack(const Unary<FusedOperation<IOps...>>&) { return {}; }
template <typename IOp, std::enable_if_t<!is_fused_iop<IOp>::value, int> = 0>
constexpr std::tuple<IOp> unpack(const IOp& iop) { return std::tuple<IOp>{iop}; }

template <typename... IOps> constexpr auto repack(const std::tuple<IOps...>& t) { return FusedOperation<IOps...>::build(t); }
} // namespace fused_detail

// FusedOperation<>::build(a, b, ...): concatenates (flattening packages that are already fused).
template <> struct FusedOperation<> {
    template <typename... IOps> static constexpr auto build(const IOps&... iops) {
        static_assert(sizeof...(IOps) >= 1);
        return fused_detail::repack(std::tuple_cat(fused_detail::unpack(iops)...));
    }
};

// Device side: fkd::FusedRead / fkd::FusedCompute over the lowered members.
namespace amd {
template <typename... Ps> fkd::Tup<Ps...> make_tup(const Ps&... ps) {
    fkd::Tup<Ps...> t{};
    if constexpr (sizeof...(Ps) > 0) {
        auto fill = [](auto& self, auto& node, const auto& head, const auto&... rest) -> void {
            node.head = head;
            if constexpr (sizeof...(rest) > 0) self(self, node.tail, rest...);
        };
        fill(fill, t, ps...);
    }
    return t;
}

template <typename First, typename... Rest>
struct Lower<FusedOperation<First, Rest...>, std::enable_if_t<opIs<ReadType, First> || opIs<ReadBackType, First>>> {
    static constexpr bool available = true;
    using type = fkd::FusedRead<device_op_t<First>, device_op_t<Rest>...>;
    static typename type::Params params(const OperationData<FusedOperation<First, Rest...>>& d) {
        typename type::Params p{};
        p.back = lower_iop(std::get<0>(d.params));
        p.ops = std::apply([](const First&, const Rest&... rest) { return make_tup(lower_iop(rest)...); }, d.params);
        return p;
    }
};
template <typename First, typename... Rest>
struct Lower<FusedOperation<First, Rest...>, std::enable_if_t<isComputeType<First>>> {
    static constexpr bool available = true;
    using Self = FusedOperation<First, Rest...>;
    using type = fkd::FusedCompute<device_op_t<First>, device_op_t<Rest>...>;
    static typename type::Params params(const OperationData<Self>& d) {
        if constexpr (opIs<UnaryType, Self>) {
            return make_tup(lower_iop(First{}), lower_iop(Rest{})...);
        } else {
            return std::apply([](const First& f, const Rest&... rest) { return make_tup(lower_iop(f), lower_iop(rest)...); }, d.params);
        }
    }
};
} // namespace amd

} // namespace fk
#endif
#endif

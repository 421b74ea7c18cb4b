// BorderReader<BT>: a read-back operation that folds coordinates outside the operation behind it back into its
// extent (REPLICATE, REFLECT, WRAP, REFLECT_101) or answers them with a constant (CONSTANT).  It reports the extent
// of the operation behind it, so it is what a later Crop with a rectangle reaching outside the image (padding) or any
// other read-back operation that addresses outside pixels lands on.
// Interface counterpart: FK/algorithms/image_processing/border_reader.h:24-330.  TRANSPARENT_ and ISOLATED are
// enumerators without an operation in the reference too.
#ifndef FK_AMD_BORDER_READER_H
#define FK_AMD_BORDER_READER_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>

namespace fk {

//! Border types, image boundaries are denoted with `|`
enum class BorderType : int {
    CONSTANT = 0,     //!< `iiiiii|abcdefgh|iiiiiii`  with some specified `i`
    REPLICATE = 1,    //!< `aaaaaa|abcdefgh|hhhhhhh`
    REFLECT = 2,      //!< `fedcba|abcdefgh|hgfedcb`
    WRAP = 3,         //!< `cdefgh|abcdefgh|abcdefg`
    REFLECT_101 = 4,  //!< `gfedcb|abcdefgh|gfedcba`
    TRANSPARENT_ = 5,
    DEFAULT = REFLECT_101,
    ISOLATED = 16
};

template <BorderType BT, typename ReadType = void> struct BorderReaderParameters;
template <BorderType BT> struct BorderReaderParameters<BT, void> {};
template <typename ReadType> struct BorderReaderParameters<BorderType::CONSTANT, ReadType> { ReadType value; };

template <BorderType BT, typename ParamsType = NullType, typename BackIOp = NullType, typename Enabler = void> struct BorderReader;

namespace border_detail {
// channel-wise static_cast between vector (or scalar) types of equal channel count
template <typename O, typename I> constexpr O cast_channels(const I& v) {
    static_assert(cn<O> == cn<I>, "the border value and the pixels behind the border have different channel counts");
    if constexpr (cn<O> == 1) {
        if constexpr (isVector<I>) return make_<O>(v.x); else return make_<O>(v);
    } else if constexpr (cn<O> == 2) return make_<O>(v.x, v.y);
    else if constexpr (cn<O> == 3) return make_<O>(v.x, v.y, v.z);
    else return make_<O>(v.x, v.y, v.z, v.w);
}
template <typename Self, typename P> struct Incomplete : IncompleteReadBackOperation<NullType, P, NullType, NullType, Self> {
    using Parent = IncompleteReadBackOperation<NullType, P, NullType, NullType, Self>;
    using typename Parent::OperationDataType;
    static constexpr uint num_elems_x(const Point, const OperationDataType&) { return 1; }
    static constexpr uint num_elems_y(const Point, const OperationDataType&) { return 1; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
};
} // namespace border_detail

// Complete form: a border around BackIOp_.
template <BorderType BT, typename P, typename BackIOp_>
struct BorderReader<BT, P, BackIOp_, std::enable_if_t<isAnyCompleteReadType<BackIOp_>, void>>
    : ReadBackOperation<typename BackIOp_::Operation::OutputType, P, BackIOp_, typename BackIOp_::Operation::OutputType,
                        BorderReader<BT, P, BackIOp_, void>> {
    static_assert(BT == BorderType::CONSTANT || BT == BorderType::REPLICATE || BT == BorderType::REFLECT || BT == BorderType::WRAP ||
                      BT == BorderType::REFLECT_101, "this border type has no operation");
    using Parent = ReadBackOperation<typename BackIOp_::Operation::OutputType, P, BackIOp_, typename BackIOp_::Operation::OutputType,
                                     BorderReader<BT, P, BackIOp_, void>>;
    using typename Parent::OperationDataType;
    using typename Parent::BackIOp;
    FK_STATIC_STRUCT(BorderReader, BorderReader)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) { return BackIOp::Operation::num_elems_x(thread, opData.backIOp); }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) { return BackIOp::Operation::num_elems_y(thread, opData.backIOp); }
    static constexpr uint num_elems_z(const Point thread, const OperationDataType& opData) { return BackIOp::Operation::num_elems_z(thread, opData.backIOp); }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), num_elems_z(Point{0, 0, 0}, opData)};
    }
    using Parent::build;
};

// BorderReader<CONSTANT>: build(value) keeps the value until a back operation arrives; build(back, value) completes.
template <> struct BorderReader<BorderType::CONSTANT, NullType, NullType, void>
    : border_detail::Incomplete<BorderReader<BorderType::CONSTANT, NullType, NullType, void>, NullType> {
    FK_STATIC_STRUCT(BorderReader, BorderReader)
    template <typename T> static constexpr auto build(const T& defaultValue) {
        using NewParamsType = BorderReaderParameters<BorderType::CONSTANT, T>;
        return BorderReader<BorderType::CONSTANT, NewParamsType>::build(NewParamsType{defaultValue}, NullType{});
    }
    template <typename BIOp> static constexpr auto build(const BIOp& backFunction, const typename BIOp::Operation::OutputType& defaultValue) {
        static_assert(isAnyCompleteReadType<BIOp>, "BIOp type is not of any complete Read Type.");
        using NewParamsType = BorderReaderParameters<BorderType::CONSTANT, typename BIOp::Operation::OutputType>;
        return BorderReader<BorderType::CONSTANT, NewParamsType, BIOp>::build(NewParamsType{defaultValue}, backFunction);
    }
};
template <typename T> struct BorderReader<BorderType::CONSTANT, BorderReaderParameters<BorderType::CONSTANT, T>, NullType, void>
    : border_detail::Incomplete<BorderReader<BorderType::CONSTANT, BorderReaderParameters<BorderType::CONSTANT, T>, NullType, void>,
                                BorderReaderParameters<BorderType::CONSTANT, T>> {
    using Parent = border_detail::Incomplete<BorderReader, BorderReaderParameters<BorderType::CONSTANT, T>>;
    using InstantiableType = typename Parent::InstantiableType;
    FK_STATIC_STRUCT(BorderReader, BorderReader)
    using Parent::build;
    template <typename BIOp, std::enable_if_t<isOperation<BIOp>, int> = 0>
    static constexpr auto build(const BIOp& backFunction, const InstantiableType& selfIOp) {
        static_assert(isAnyCompleteReadType<BIOp>, "BIOp type is not of any complete Read Type.");
        using O = typename BIOp::Operation::OutputType;
        using NewParamsType = BorderReaderParameters<BorderType::CONSTANT, O>;
        if constexpr (std::is_same_v<O, T>) {
            return BorderReader<BorderType::CONSTANT, NewParamsType, BIOp>::build(selfIOp.params, backFunction);
        } else {
            return BorderReader<BorderType::CONSTANT, NewParamsType, BIOp>::build(NewParamsType{border_detail::cast_channels<O>(selfIOp.params.value)}, backFunction);
        }
    }
};
// The other border types carry no parameters.
template <BorderType BT> struct BorderReader<BT, NullType, NullType, void>
    : border_detail::Incomplete<BorderReader<BT, NullType, NullType, void>, BorderReaderParameters<BT>> {
    using Parent = border_detail::Incomplete<BorderReader, BorderReaderParameters<BT>>;
    using InstantiableType = typename Parent::InstantiableType;
    using ParamsType = BorderReaderParameters<BT>;
    FK_STATIC_STRUCT(BorderReader, BorderReader)
    static constexpr auto build() { return InstantiableType{}; }
    template <typename BIOp, std::enable_if_t<isOperation<BIOp>, int> = 0> static constexpr auto build(const BIOp& backFunction) {
        static_assert(isAnyCompleteReadType<BIOp>, "BIOp type is not of any complete Read Type.");
        return BorderReader<BT, ParamsType, BIOp>::build(ParamsType{}, backFunction);
    }
    template <typename BIOp, std::enable_if_t<isOperation<BIOp>, int> = 0>
    static constexpr auto build(const BIOp& backFunction, const InstantiableType&) {
        static_assert(isAnyCompleteReadType<BIOp>, "BIOp type is not of any complete Read Type.");
        return BorderReader<BT, ParamsType, BIOp>::build(ParamsType{}, backFunction);
    }
};

namespace amd {
template <BorderType BT, typename P, typename BackIOp>
struct Lower<BorderReader<BT, P, BackIOp, void>, std::enable_if_t<isAnyCompleteReadType<BackIOp>>> {
    static constexpr bool available = true;
    using type = fkd::Border<int(BT), device_op_t<BackIOp>>;
    static typename type::Params params(const OperationData<BorderReader<BT, P, BackIOp, void>>& d) {
        typename type::Params p{};
        if constexpr (BT == BorderType::CONSTANT) p.value = to_dev(d.params.value);
        p.back = lower_iop(d.backIOp);
        return p;
    }
};
} // namespace amd

} // namespace fk
#endif

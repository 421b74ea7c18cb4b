// Parents of Operations and the DECLARE_*_PARENT macros a user-defined Operation pulls its parent's names in with.
// Interface counterpart: FK/core/execution_model/operation_model/parent_operations.h:49-326.  The parents themselves
// (UnaryOperation, BinaryOperation, ... WriteOperation) are defined in operation_model.h; the library's own Operations
// inherit from them instead of using the macros.
//
// What a user-defined Operation can do on this backend: it compiles, builds, fuses and type-checks exactly as in the
// reference (its exec body is ordinary host C++ and stays callable), but a launch needs its device counterpart: the
// executor stops at compile time with "this Operation has no MI355X lowering" until fk::amd::Lower<TheOperation> names a
// device operation (a struct in namespace fkd with In, Out, Params and a __device__ exec, see include/fkd/ops.hpp) and
// converts the parameters.  The host compiler never sees device code here, so the body cannot be taken from the host
// struct the way nvcc takes it in the reference.
#ifndef FK_AMD_PARENT_OPERATIONS_H
#define FK_AMD_PARENT_OPERATIONS_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>

// Pulls one member type of `Parent` into the Operation being declared.
#define FK_AMD_PARENT_TYPE(Name) using Name = typename Parent::Name;
#define FK_AMD_PARENT_FLAG(Name) static constexpr bool Name = Parent::Name;

#define DECLARE_UNARY_PARENT                                                                                        \
    FK_AMD_PARENT_TYPE(InputType) FK_AMD_PARENT_TYPE(OutputType) FK_AMD_PARENT_TYPE(InstanceType)                    \
    FK_AMD_PARENT_TYPE(InstantiableType) FK_AMD_PARENT_FLAG(IS_FUSED_OP)                                             \
    static constexpr InstantiableType build() { return Parent::build(); }

#define DECLARE_BINARY_PARENT                                                                                       \
    FK_AMD_PARENT_TYPE(InputType) FK_AMD_PARENT_TYPE(OutputType) FK_AMD_PARENT_TYPE(ParamsType)                      \
    FK_AMD_PARENT_TYPE(InstanceType) FK_AMD_PARENT_TYPE(OperationDataType) FK_AMD_PARENT_TYPE(InstantiableType)     \
    FK_AMD_PARENT_FLAG(IS_FUSED_OP)                                                                                  \
    static constexpr OutputType exec(const InputType input, const OperationDataType& opData) { return exec(input, opData.params); } \
    static constexpr InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }      \
    static constexpr InstantiableType build(const ParamsType& params) { return Parent::build(params); }

#define DECLARE_TERNARY_PARENT                                                                                      \
    FK_AMD_PARENT_TYPE(InputType) FK_AMD_PARENT_TYPE(OutputType) FK_AMD_PARENT_TYPE(ParamsType) FK_AMD_PARENT_TYPE(BackIOp) \
    FK_AMD_PARENT_TYPE(InstanceType) FK_AMD_PARENT_TYPE(OperationDataType) FK_AMD_PARENT_TYPE(InstantiableType)     \
    FK_AMD_PARENT_FLAG(IS_FUSED_OP)                                                                                  \
    static constexpr OutputType exec(const InputType input, const OperationDataType& opData) {                      \
        return exec(input, opData.params, opData.backIOp);                                                           \
    }                                                                                                                \
    static constexpr InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }      \
    static constexpr InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return Parent::build(params, backIOp); }

#define DECLARE_READ_PARENT_BASIC                                                                                   \
    FK_AMD_PARENT_TYPE(ParamsType) FK_AMD_PARENT_TYPE(ReadDataType) FK_AMD_PARENT_TYPE(InstanceType)                 \
    FK_AMD_PARENT_TYPE(OutputType) FK_AMD_PARENT_TYPE(OperationDataType) FK_AMD_PARENT_TYPE(InstantiableType)       \
    FK_AMD_PARENT_FLAG(IS_FUSED_OP) FK_AMD_PARENT_FLAG(THREAD_FUSION)                                                \
    static constexpr auto exec(const ::fk::Point thread, const OperationDataType& opData) { return exec(thread, opData.params); } \
    static constexpr InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }      \
    static constexpr InstantiableType build(const ParamsType& params) { return Parent::build(params); }

#define DECLARE_WRITE_PARENT_BASIC                                                                                  \
    FK_AMD_PARENT_TYPE(ParamsType) FK_AMD_PARENT_TYPE(InputType) FK_AMD_PARENT_TYPE(WriteDataType)                   \
    FK_AMD_PARENT_TYPE(InstanceType) FK_AMD_PARENT_TYPE(OperationDataType) FK_AMD_PARENT_TYPE(InstantiableType)     \
    FK_AMD_PARENT_FLAG(IS_FUSED_OP) FK_AMD_PARENT_FLAG(THREAD_FUSION)                                                \
    static constexpr void exec(const ::fk::Point thread, const InputType& input, const OperationDataType& opData) { \
        exec(thread, input, opData.params);                                                                          \
    }                                                                                                                \
    static constexpr InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }      \
    static constexpr InstantiableType build(const ParamsType& params) { return Parent::build(params); }

#define DECLARE_READBACK_PARENT_BASIC                                                                               \
    FK_AMD_PARENT_TYPE(ReadDataType) FK_AMD_PARENT_TYPE(OutputType) FK_AMD_PARENT_TYPE(ParamsType) FK_AMD_PARENT_TYPE(BackIOp) \
    FK_AMD_PARENT_TYPE(InstanceType) FK_AMD_PARENT_TYPE(OperationDataType) FK_AMD_PARENT_TYPE(InstantiableType)     \
    FK_AMD_PARENT_FLAG(IS_FUSED_OP) FK_AMD_PARENT_FLAG(THREAD_FUSION)                                                \
    static constexpr OutputType exec(const ::fk::Point thread, const OperationDataType& opData) {                   \
        return exec(thread, opData.params, opData.backIOp);                                                          \
    }                                                                                                                \
    static constexpr InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }      \
    static constexpr InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return Parent::build(params, backIOp); }

#endif

// Part of the operation model; the definitions live in operation_model.h.
#ifndef FK_AMD_FWD_PARENT_OPERATIONS_H
#define FK_AMD_FWD_PARENT_OPERATIONS_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#endif

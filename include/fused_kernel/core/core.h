#ifndef FK_AMD_CORE_H
#define FK_AMD_CORE_H
#include <fused_kernel/core/data/data.h>
#include <fused_kernel/core/utils/type_to_string.h>
#include <fused_kernel/core/utils/vlimits.h>
#include <fused_kernel/core/utils/type_lists.h>
#include <fused_kernel/core/execution_model/execution_model.h>
#endif

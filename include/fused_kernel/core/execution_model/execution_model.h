#ifndef FK_AMD_EXECUTION_MODEL_H
#define FK_AMD_EXECUTION_MODEL_H
#include <fused_kernel/core/execution_model/executors.h>
#include <fused_kernel/core/execution_model/stream.h>
#endif

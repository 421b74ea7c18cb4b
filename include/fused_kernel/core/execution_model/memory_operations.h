// The README of the reference includes the memory operations through this path.
#ifndef FK_AMD_EXEC_MEMORY_OPERATIONS_H
#define FK_AMD_EXEC_MEMORY_OPERATIONS_H
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>
#endif

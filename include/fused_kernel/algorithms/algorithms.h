#ifndef FK_AMD_ALGORITHMS_H
#define FK_AMD_ALGORITHMS_H
#include <fused_kernel/algorithms/basic_ops/basic_ops.h>
#include <fused_kernel/algorithms/image_processing/image_processing.h>
#endif

#ifndef FK_AMD_DATA_H
#define FK_AMD_DATA_H
#include <fused_kernel/core/data/array.h>
#include <fused_kernel/core/data/tuple.h>
#include <fused_kernel/core/data/point.h>
#include <fused_kernel/core/data/size.h>
#include <fused_kernel/core/data/rect.h>
#include <fused_kernel/core/data/rawptr.h>
#include <fused_kernel/core/data/ptr_nd.h>
#endif

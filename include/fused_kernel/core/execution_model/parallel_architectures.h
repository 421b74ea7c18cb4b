#ifndef FK_AMD_PARALLEL_ARCHITECTURES_H
#define FK_AMD_PARALLEL_ARCHITECTURES_H
#include <string_view>
namespace fk {
// Same enumerators, same order as FK/core/execution_model/parallel_architectures.h:23-48.  In this build the
// default architecture is GPU_AMD: TransformDPP<>, Stream and Ptr's default memory type follow it.
enum class ParArch { CPU, GPU_NVIDIA, GPU_NVIDIA_JIT, GPU_AMD, CPU_OMP, CPU_OMPSS, MULTI_GPU_NVIDIA, CLUSTER_GPU_NVIDIA, None };

constexpr inline std::string_view toStrView(const ParArch& arch) {
    switch (arch) {
    case ParArch::CPU: return "CPU";
    case ParArch::GPU_NVIDIA: return "GPU_NVIDIA";
    case ParArch::GPU_NVIDIA_JIT: return "GPU_NVIDIA_JIT";
    case ParArch::GPU_AMD: return "GPU_AMD";
    case ParArch::CPU_OMP: return "CPU_OMP";
    case ParArch::CPU_OMPSS: return "CPU_OMPSS";
    case ParArch::MULTI_GPU_NVIDIA: return "MULTI_GPU_NVIDIA";
    case ParArch::CLUSTER_GPU_NVIDIA: return "CLUSTER_GPU_NVIDIA";
    case ParArch::None: return "None";
    default: return "Unknown";
    }
}

constexpr ParArch defaultParArch = ParArch::GPU_AMD;
} // namespace fk
#endif

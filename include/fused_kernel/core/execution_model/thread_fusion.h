#ifndef FK_AMD_THREAD_FUSION_H
#define FK_AMD_THREAD_FUSION_H
namespace fk {
// Thread-fusion switch of TransformDPP (FK/core/execution_model/thread_fusion.h:23).  It only selects an access
// width in the reference and never changes results; this backend always moves four elements per lane where the
// chain reads rows, so both spellings run the same kernel.
enum class TF : bool { DISABLED = false, ENABLED = true };
} // namespace fk
#endif

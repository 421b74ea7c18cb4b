#ifndef FK_AMD_RAW_IMAGE_H
#define FK_AMD_RAW_IMAGE_H
#include <fused_kernel/algorithms/image_processing/itu_color.h>
#include <fused_kernel/core/data/rawptr.h>
namespace fk {
// POD view of a pixel-format image: the backing 2-D buffer plus the image size in pixels.
// Interface counterpart: FK/algorithms/image_processing/raw_image.h.
template <PixelFormat PF> struct RawImage {
    using BaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    RawPtr<ND::_2D, BaseType> data;
    uint width;
    uint height;
};
} // namespace fk
#endif

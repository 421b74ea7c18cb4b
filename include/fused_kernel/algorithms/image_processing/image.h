// Image<PF>: owner of a pixel-format image (NV12: width x height*3/2 bytes, luma rows then interleaved chroma rows).
// Interface counterpart: FK/algorithms/image_processing/image.h:25-95.
#ifndef FK_AMD_IMAGE_H
#define FK_AMD_IMAGE_H

#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/core/data/ptr_nd.h>

namespace fk {

template <PixelFormat PF> class Image {
public:
    using BaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    static constexpr PixelFormat pixelFormat = PF;

private:
    Ptr<ND::_2D, BaseType> data;
    uint width;
    uint height;

public:
    uint imageWidth() const { return width; }
    uint imageHeight() const { return height; }

    Image(const Ptr<ND::_2D, BaseType>& data_, const uint& width_, const uint& height_) : data(data_), width(width_), height(height_) {}
    Image(const uint width_, const uint height_, const MemType memType = defaultMemType, const uint deviceID = 0)
        : width(width_), height(height_) {
        const uint dataWidth = uint(width_ * PixelFormatTraits<PF>::rf.width_f);
        const uint dataHeight = uint(height_ * PixelFormatTraits<PF>::rf.height_f);
        data = Ptr<ND::_2D, BaseType>(dataWidth, dataHeight, 0, memType, int(deviceID));
    }

    RawImage<PF> ptr() const { return RawImage<PF>{data, width, height}; }
    Ptr<ND::_2D, BaseType> getData() const { return data; }
    RawImage<PF> operator()() const { return ptr(); }

    void upload(Stream_<ParArch::GPU_AMD>& stream) { data.upload(stream); }
    void download(Stream_<ParArch::GPU_AMD>& stream) { data.download(stream); }
    void upload(Stream_<ParArch::CPU>&) {}
    void download(Stream_<ParArch::CPU>&) {}
};

} // namespace fk
#endif

// Stream_<PA>: owner / non-owner of an execution queue.  Interface counterpart:
// FK/core/execution_model/stream.h:29-126.  Stream_<GPU_AMD> wraps a HIP stream obtained through the C ABI
// (void* on this side of the boundary); Stream_<CPU> is the reference's no-op.
#ifndef FK_AMD_STREAM_H
#define FK_AMD_STREAM_H

#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/core/data/ref_class.h>
#include <fused_kernel/core/execution_model/parallel_architectures.h>

namespace fk {

class BaseStream : public Ref {
public:
    BaseStream() : Ref() {}
    BaseStream(const BaseStream& other) : Ref(other) {}
    virtual ~BaseStream() = default;
    BaseStream(BaseStream&&) = delete;
    BaseStream& operator=(BaseStream&&) = delete;
    BaseStream& operator=(const BaseStream& other) {
        if (this != &other) Ref::operator=(other);
        return *this;
    }
    virtual void sync() = 0;
};

template <ParArch PA> class Stream_;

template <> class Stream_<ParArch::GPU_AMD> final : public BaseStream {
    void* m_stream{nullptr};   // hipStream_t behind the C ABI
    bool m_isMine{false};

    void release() {
        // Last copy of an owned stream: drain it and give it back.
        if (getRefCount() == 1 && m_stream != nullptr && m_isMine) {
            fklhip_stream_sync(m_stream);
            fklhip_stream_destroy(m_stream);
        }
    }
public:
    Stream_() : BaseStream() {
        gpuErrchk(fklhip_stream_create(&m_stream));
        m_isMine = true;
    }
    Stream_(const Stream_& other) : BaseStream(other), m_stream(other.m_stream), m_isMine(other.m_isMine) {}
    // Wraps a native stream (hipStream_t) without taking ownership.
    explicit Stream_(void* nativeStream) : BaseStream(), m_stream(nativeStream), m_isMine(false) {}
    Stream_& operator=(const Stream_& other) {
        if (this != &other) {
            release();
            BaseStream::operator=(other);
            m_stream = other.m_stream;
            m_isMine = other.m_isMine;
        }
        return *this;
    }
    Stream_(Stream_&&) = delete;
    Stream_& operator=(Stream_&&) = delete;
    ~Stream_() { release(); }

    void* operator()() const { return m_stream; }
    operator void*() const { return m_stream; }
    void* getNativeStream() const { return m_stream; }
    void sync() final { gpuErrchk(fklhip_stream_sync(m_stream)); }
    constexpr ParArch getParArch() const { return ParArch::GPU_AMD; }
    static constexpr ParArch parArch() { return ParArch::GPU_AMD; }
};

template <> class Stream_<ParArch::CPU> final : public BaseStream {
public:
    Stream_() : BaseStream() {}
    ~Stream_() = default;
    void sync() final {}
    constexpr ParArch getParArch() const { return ParArch::CPU; }
    static constexpr ParArch parArch() { return ParArch::CPU; }
};

using Stream = Stream_<defaultParArch>;

} // namespace fk
#endif

// ParArch, Stream_<PA> and Stream: counterpart of the reference's
// core/execution_model/parallel_architectures.h:22-59 and core/execution_model/stream.h:48-126.
// The GPU_AMD stream wraps a HIP stream obtained through the C runtime ABI; copies share it and the last owner
// destroys it.
#ifndef FK_CORE_STREAM_H
#define FK_CORE_STREAM_H

#include <memory>

#include "fk/core/utils.h"

namespace fk {

enum class ParArch {
    CPU = 0,
    GPU_NVIDIA = 1,
    GPU_NVIDIA_JIT = 2,
    GPU_AMD = 3,
    MULTI_GPU_NVIDIA = 4,
    CLUSTER_GPU_NVIDIA = 5,
    CPU_OMP = 6,
    CPU_OMPSS = 7,
    None = 8
};

// This library executes on one backend only.
constexpr ParArch defaultParArch = ParArch::GPU_AMD;

// What every stream can do (core/execution_model/stream.h:29-47).
class BaseStream {
public:
    BaseStream() = default;
    BaseStream(const BaseStream&) = default;
    BaseStream& operator=(const BaseStream&) = default;
    virtual ~BaseStream() = default;
    virtual void sync() = 0;
};

template <ParArch PA>
class Stream_ {
    static_assert(PA == ParArch::GPU_AMD || PA == ParArch::CPU, "Only ParArch::GPU_AMD and ParArch::CPU are implemented by this library.");
};

template <>
class Stream_<ParArch::GPU_AMD> final : public BaseStream {
    struct Owned {
        fkrt_stream handle{ nullptr };
        ~Owned() {
            if (handle != nullptr) {
                (void)fkrt_stream_sync(handle);
                (void)fkrt_stream_destroy(handle);
            }
        }
    };
    std::shared_ptr<Owned> m_owned; // empty when the handle is borrowed
    fkrt_stream m_stream{ nullptr };

public:
    Stream_() : m_owned(std::make_shared<Owned>()) {
        gpuErrchk(fkrt_stream_create(&m_owned->handle));
        m_stream = m_owned->handle;
    }
    // Borrow an existing native stream (a hipStream_t, or nullptr for the default stream); never destroyed here.
    explicit Stream_(fkrt_stream native) : m_stream(native) {}
    Stream_(const Stream_&) = default;
    Stream_& operator=(const Stream_&) = default;

    fkrt_stream operator()() const { return m_stream; }
    operator fkrt_stream() const { return m_stream; }
    fkrt_stream getHIPStream() const { return m_stream; }
    int getRefCount() const { return m_owned ? static_cast<int>(m_owned.use_count()) : 0; }
    void sync() final { gpuErrchk(fkrt_stream_sync(m_stream)); }
    constexpr ParArch getParArch() const { return ParArch::GPU_AMD; }
    static constexpr ParArch parArch() { return ParArch::GPU_AMD; }
};

// The host executor runs a chain before it returns: its stream has nothing to wait for (stream.h:112-124).
template <>
class Stream_<ParArch::CPU> final : public BaseStream {
public:
    Stream_() = default;
    void sync() final {}
    constexpr ParArch getParArch() const { return ParArch::CPU; }
    static constexpr ParArch parArch() { return ParArch::CPU; }
};

using Stream = Stream_<defaultParArch>;

} // namespace fk
#endif

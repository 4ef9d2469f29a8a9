// Umbrella header and the free executeOperations<DPP>(...) entry points of the library.
// Counterpart of the reference's include/fused_kernel/fused_kernel.h:22-54 and core/data/ptr_utils.h:23-45 (setTo).
#ifndef FK_FUSED_KERNEL_H
#define FK_FUSED_KERNEL_H

#include "fk/core/array.h"
#include "fk/core/parent_operations.h"
#include "fk/core/thread_fusion_info.h"
#include "fk/core/type_to_string.h"
#include "fk/exec/executor.h"
#include "fk/ops/yuv.h"
#include "fk/ops/border_reader.h"
#include "fk/ops/warping.h"
#include "fk/ops/static_loop.h"
#include "fk/ops/circular.h"
#include "fk/ops/deinterlace.h"

namespace fk {

template <typename DPPType, typename... Args>
inline void executeOperations(Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(stream, args...);
}
template <typename DPPType, ND D, typename I, typename... Args>
inline void executeOperations(const Ptr<D, I>& input, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, stream, args...);
}
template <typename DPPType, ND D, typename I, typename O, typename... Args>
inline void executeOperations(const Ptr<D, I>& input, const Ptr<D, O>& output, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, output, stream, args...);
}
template <typename DPPType, typename I, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                              Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, activeBatch, defaultValue, stream, args...);
}
template <typename DPPType, typename I, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, stream, args...);
}
template <typename DPPType, typename I, typename O, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                              const Tensor<O>& output, Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, activeBatch, defaultValue, output, stream, args...);
}
template <typename DPPType, typename I, typename O, size_t BATCH, typename... Args>
inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const Tensor<O>& output,
                              Stream_<DPPType::PAR_ARCH>& stream, const Args&... args) {
    Executor<DPPType>::executeOperations(input, output, stream, args...);
}

// Fills a buffer with one value: on the device through the fused executor, and its host mirror directly.
template <ND D, typename T>
inline void setTo(const T& value, Ptr<D, T>& outputPtr, Stream& stream) {
    const RawPtr<D, T> dev = outputPtr.ptr();
    const MemType type = outputPtr.getMemType();
    if (type == MemType::Device || type == MemType::DeviceAndPinned) {
        ActiveThreads extent(dev.dims.width);
        if constexpr (D == ND::_2D) extent = ActiveThreads(dev.dims.width, dev.dims.height);
        if constexpr (D == ND::_3D) extent = ActiveThreads(dev.dims.width, dev.dims.height * dev.dims.color_planes, dev.dims.planes);
        executeOperations<TransformDPP<>>(stream, ReadSet<T>::build(value, extent), PerThreadWrite<D, T>::build(dev));
    }
    if (type != MemType::Device) {
        const RawPtr<D, T> host = outputPtr.ptrPinned();
        uint rows = 1;
        if constexpr (D == ND::_2D) rows = host.dims.height;
        if constexpr (D == ND::_3D) rows = host.dims.height * host.dims.color_planes * host.dims.planes;
        for (uint y = 0; y < rows; ++y) {
            T* const row = reinterpret_cast<T*>(reinterpret_cast<char*>(host.data) + static_cast<size_t>(y) * host.dims.pitch);
            for (uint x = 0; x < host.dims.width; ++x) row[x] = value;
        }
    }
}

} // namespace fk
#endif

// Umbrella header and the free executeOperations<DPP>(...) entry points of the library.
// Counterpart of the reference's include/fused_kernel/fused_kernel.h:22-54 and core/data/ptr_utils.h:23-45 (setTo).
#ifndef FK_FUSED_KERNEL_H
#define FK_FUSED_KERNEL_H

#include "fk/core/array.h"
#include "fk/core/parent_operations.h"
#include "fk/core/thread_fusion_info.h"
#include "fk/core/string.h"
#include "fk/core/type_to_string.h"
#include "fk/exec/executor.h"
#include "fk/ops/yuv.h"
#include "fk/ops/border_reader.h"
#include "fk/ops/warping.h"
#include "fk/ops/static_loop.h"
#include "fk/ops/circular.h"
#include "fk/ops/deinterlace.h"
#include "fk/core/reference_surface.h"

namespace fk {

// executeOperations<DPP>(...) with any of the argument lists Executor<DPP>::executeOperations accepts: a stream and a
// chain of IOps; an input buffer (or an array of them, optionally with the number of used planes and a default value), an
// optional output buffer or tensor, the stream and the compute operations between them.
template <typename DPPType, typename... Args>
inline void executeOperations(Args&&... args) {
    Executor<DPPType>::executeOperations(std::forward<Args>(args)...);
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

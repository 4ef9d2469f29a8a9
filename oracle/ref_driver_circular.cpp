// ref_driver_circular.cpp — drives the REFERENCE's own headers (its CPU backend, built exactly as they lie under
// /root/reference, nothing copied, no stand-in headers) behind the C signatures of fk_oracle_circular.h, for the
// operations the reference can execute: the tensor layouts and the circular tensor read.  CircularTensor::update has
// no counterpart here: the reference has no executor for the divergent launch it asks for.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libfkref_circular.so.
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/fused_kernel.h>

#include <cstddef>

#include "fk_oracle_circular.h"

using namespace fk;

namespace {
using CPU = TransformDPP<ParArch::CPU>;

RawPtr<ND::_3D, float3> packed(const float* p, int w, int h, int n) {
    return RawPtr<ND::_3D, float3>{ reinterpret_cast<float3*>(const_cast<float*>(p)),
                                    PtrDims<ND::_3D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(n), 1u, static_cast<uint>(sizeof(float3) * w)) };
}
RawPtr<ND::_3D, float> split(const float* p, int w, int h, int n) {
    return RawPtr<ND::_3D, float>{ const_cast<float*>(p),
                                   PtrDims<ND::_3D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(n), 3u, static_cast<uint>(sizeof(float) * w)) };
}
RawPtr<ND::T3D, float> transposed(const float* p, int w, int h, int n) {
    PtrDims<ND::T3D> d(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(n), 3u);
    d.pitch = static_cast<uint>(sizeof(float) * w);
    d.plane_pitch = d.pitch * h;
    d.color_planes_pitch = d.plane_pitch * n;
    return RawPtr<ND::T3D, float>{ const_cast<float*>(p), d };
}

template <CircularDirection DIR, int N>
void circular_read(int first, const float* ring, int w, int h, float* dst) {
    Stream_<ParArch::CPU> stream;
    Read<CircularTensorRead<DIR, TensorRead<float3>, N>> read{};
    read.params.first = first;
    read.params.opData.params = packed(ring, w, h, N);
    executeOperations<CPU>(stream, read, Write<TensorWrite<float3>>{ { packed(dst, w, h, N) } });
}
template <int N>
int circular_read_dir(int direction, int first, const float* ring, int w, int h, float* dst) {
    if (direction == FKO_ASCENDENT) circular_read<CircularDirection::Ascendent, N>(first, ring, w, h, dst);
    else if (direction == FKO_DESCENDENT) circular_read<CircularDirection::Descendent, N>(first, ring, w, h, dst);
    else return 1;
    return 0;
}
} // namespace

extern "C" {

int fkr_tensor_relayout_f32c3(int mode, const float* src, int w, int h, int planes, float* dst) {
    Stream_<ParArch::CPU> stream;
    switch (mode) {
    case FKO_PACKED_TO_SPLIT:
        executeOperations<CPU>(stream, Read<TensorRead<float3>>{ { packed(src, w, h, planes) } }, Write<TensorSplit<float3>>{ { split(dst, w, h, planes) } });
        return 0;
    case FKO_PACKED_TO_TRANSPOSED:
        executeOperations<CPU>(stream, Read<TensorRead<float3>>{ { packed(src, w, h, planes) } }, Write<TensorTSplit<float3>>{ { transposed(dst, w, h, planes) } });
        return 0;
    case FKO_SPLIT_TO_PACKED:
        executeOperations<CPU>(stream, Read<TensorPack<float3>>{ { split(src, w, h, planes) } }, Write<TensorWrite<float3>>{ { packed(dst, w, h, planes) } });
        return 0;
    case FKO_TRANSPOSED_TO_PACKED:
        executeOperations<CPU>(stream, Read<TensorTPack<float3>>{ { transposed(src, w, h, planes) } }, Write<TensorWrite<float3>>{ { packed(dst, w, h, planes) } });
        return 0;
    default: return 1;
    }
}

// planes must be one of the instantiated ring sizes (2, 3, 4, 8)
int fkr_circular_tensor_read_f32c3(int direction, int first, const float* ring, int w, int h, int planes, float* dst) {
    switch (planes) {
    case 2: return circular_read_dir<2>(direction, first, ring, w, h, dst);
    case 3: return circular_read_dir<3>(direction, first, ring, w, h, dst);
    case 4: return circular_read_dir<4>(direction, first, ring, w, h, dst);
    case 8: return circular_read_dir<8>(direction, first, ring, w, h, dst);
    default: return 1;
    }
}

} // extern "C"

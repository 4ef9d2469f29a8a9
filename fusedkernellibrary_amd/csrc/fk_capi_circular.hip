// fk_capi_circular.hip — the tensor-layout and circular-tensor entry points of include/fk_capi.h, built with the fk::
// operator API.  Compiled by hipcc into libfk_capi.so.
#include "fk_capi_common.h"

using namespace fk;
using namespace fk_capi;

namespace {

RawPtr<ND::_3D, float3> packed(const float* p, int w, int h, int n) { return view3d<float3>(const_cast<float*>(p), w, h, n, 1); }
RawPtr<ND::_3D, float> split(const float* p, int w, int h, int n) { return view3d<float>(const_cast<float*>(p), w, h, n, 3); }
RawPtr<ND::T3D, float> transposed(const float* p, int w, int h, int n) {
    return TensorT<float>(const_cast<float*>(p), static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(n), 3u).ptr();
}

template <CircularDirection DIR, int N>
void circular_read(Stream& stream, int first, const float* ring, int w, int h, float* dst) {
    Read<CircularTensorRead<DIR, TensorRead<float3>, N>> read{};
    read.params.first = first;
    read.params.opData.params = packed(ring, w, h, N);
    executeOperations<TransformDPP<>>(stream, read, TensorWrite<float3>::build(packed(dst, w, h, N)));
}
template <int N>
int circular_read_dir(Stream& stream, int direction, int first, const float* ring, int w, int h, float* dst) {
    if (direction == FK_ASCENDENT) circular_read<CircularDirection::Ascendent, N>(stream, first, ring, w, h, dst);
    else if (direction == FK_DESCENDENT) circular_read<CircularDirection::Descendent, N>(stream, first, ring, w, h, dst);
    else return unsupported("direction must be ascendent or descendent");
    return FK_OK;
}

template <int N, CircularTensorOrder ORDER>
void circular_update(Stream& stream, const void* frame, int w, int h, size_t pitch, float mul_v, float* tensor, float* ring, int next_index) {
    CircularTensor<float, 3, N, ORDER, ColorPlanes::Standard> circular(tensor, ring, static_cast<uint>(w), static_cast<uint>(h), next_index);
    circular.update(stream, PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(frame, w, h, pitch)), Cast<uchar3, float3>::build(),
                    Mul<float3>::build(make_set<float3>(mul_v)), TensorSplit<float3>::build(circular.ptr()));
}
template <int N>
void circular_update_order(Stream& stream, int newest_first, const void* frame, int w, int h, size_t pitch, float mul_v, float* tensor, float* ring,
                           int next_index) {
    if (newest_first) circular_update<N, CircularTensorOrder::NewestFirst>(stream, frame, w, h, pitch, mul_v, tensor, ring, next_index);
    else circular_update<N, CircularTensorOrder::OldestFirst>(stream, frame, w, h, pitch, mul_v, tensor, ring, next_index);
}

#define FK_FOR_RING(n, CALL)                                                                                           \
    switch (n) {                                                                                                       \
    case 2: { constexpr int N = 2; CALL; break; }                                                                      \
    case 3: { constexpr int N = 3; CALL; break; }                                                                      \
    case 4: { constexpr int N = 4; CALL; break; }                                                                      \
    case 8: { constexpr int N = 8; CALL; break; }                                                                      \
    case 16: { constexpr int N = 16; CALL; break; }                                                                    \
    default: return unsupported("ring size has no instantiation (2, 3, 4, 8, 16)");                                    \
    }

} // namespace

extern "C" {

int fk_tensor_relayout_f32c3(int mode, const float* src, int w, int h, int planes, float* dst, void* stream) {
    if (src == nullptr || dst == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0 || planes <= 0) return bad_argument("empty tensor");
    return guarded([&]() -> int {
        Stream s(stream);
        switch (mode) {
        case FK_PACKED_TO_SPLIT:
            executeOperations<TransformDPP<>>(s, TensorRead<float3>::build(packed(src, w, h, planes)), TensorSplit<float3>::build(split(dst, w, h, planes)));
            break;
        case FK_PACKED_TO_TRANSPOSED:
            executeOperations<TransformDPP<>>(s, TensorRead<float3>::build(packed(src, w, h, planes)), TensorTSplit<float3>::build(transposed(dst, w, h, planes)));
            break;
        case FK_SPLIT_TO_PACKED:
            executeOperations<TransformDPP<>>(s, TensorPack<float3>::build(split(src, w, h, planes)), TensorWrite<float3>::build(packed(dst, w, h, planes)));
            break;
        case FK_TRANSPOSED_TO_PACKED:
            executeOperations<TransformDPP<>>(s, TensorTPack<float3>::build(transposed(src, w, h, planes)), TensorWrite<float3>::build(packed(dst, w, h, planes)));
            break;
        default: return unsupported("unknown layout conversion");
        }
        return FK_OK;
    });
}

int fk_circular_tensor_read_f32c3(int direction, int first, const float* ring, int w, int h, int planes, float* dst, void* stream) {
    if (ring == nullptr || dst == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0 || first < 0 || first >= planes) return bad_argument("empty tensor or first plane outside the ring");
    return guarded([&]() -> int {
        Stream s(stream);
        int rc = FK_OK;
        FK_FOR_RING(planes, (rc = circular_read_dir<N>(s, direction, first, ring, w, h, dst)))
        return rc;
    });
}

int fk_circular_tensor_update_u8c3_split_f32(const void* frame, int w, int h, size_t src_pitch, float mul_v, float* tensor, float* ring,
                                             int batch, int next_index, int newest_first, void* stream) {
    if (frame == nullptr || tensor == nullptr || ring == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0 || src_pitch < static_cast<size_t>(w) * 3) return bad_argument("empty frame or pitch shorter than a row");
    if (next_index < 0 || next_index >= batch) return bad_argument("next_index outside the ring");
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_RING(batch, (circular_update_order<N>(s, newest_first, frame, w, h, src_pitch, mul_v, tensor, ring, next_index)))
        return FK_OK;
    });
}

} // extern "C"

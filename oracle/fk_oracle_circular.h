/* fk_oracle_circular.h — CPU restatement of the planar / transposed tensor layouts, the circular (ring) reads and
 * CircularTensor::update of the Fused Kernel Library.
 *
 * TEST INFRASTRUCTURE ONLY (see fk_oracle.h): the checker the GPU library is compared with; nothing in the shipped
 * library links, loads or calls it.
 *
 * Layouts of a tensor of n images, c channels, h x w pixels (floats, rows tight):
 *   packed       n, h, w, c   TensorRead / TensorWrite of float3
 *   split        n, c, h, w   TensorSplit / TensorPack
 *   transposed   c, n, h, w   TensorTSplit / TensorTPack
 */
#ifndef FK_ORACLE_CIRCULAR_H
#define FK_ORACLE_CIRCULAR_H

#include "fk_oracle.h"

#ifdef __cplusplus
extern "C" {
#endif

enum { FKO_PACKED_TO_SPLIT = 0, FKO_PACKED_TO_TRANSPOSED = 1, FKO_SPLIT_TO_PACKED = 2, FKO_TRANSPOSED_TO_PACKED = 3 };
/* CircularDirection, core/execution_model/memory_operations.h:425 */
enum { FKO_ASCENDENT = 0, FKO_DESCENDENT = 1 };

/* TensorRead<float3> -> TensorSplit / TensorTSplit, or TensorPack / TensorTPack -> TensorWrite<float3> */
int fko_tensor_relayout_f32c3(int mode, const float* src, int w, int h, int planes, float* dst);
/* CircularTensorRead<direction, TensorRead<float3>, planes>{first} -> TensorWrite<float3>: plane z of dst is ring slot
 * first + z (ascendent) or first - z (descendent), modulo planes */
int fko_circular_tensor_read_f32c3(int direction, int first, const float* ring, int w, int h, int planes, float* dst);
/* CircularTensor<float, 3, batch, order, Standard>::update(PerThreadRead<_2D,uchar3>(frame), Cast<uchar3,float3>,
 * Mul<float3>(mul_v), TensorSplit<float3>(tensor)): tensor and ring are batch x 3 x h x w floats; next_index is the
 * ring slot this update fills (core/data/circular_tensor.h:107-155) */
int fko_circular_tensor_update_u8c3_split_f32(const uint8_t* frame, int w, int h, size_t pitch, float mul_v, float* tensor,
                                              float* ring, int batch, int next_index, int newest_first);

#ifdef __cplusplus
}
#endif
#endif

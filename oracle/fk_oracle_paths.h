/* fk_oracle_paths.h — CPU restatement of the chains that use the operator API's less common shapes: batch reads with
 * PlanePolicy::CONDITIONAL_WITH_DEFAULT, a write in the middle of a chain, a batch of separate output images and a
 * tensor as the source.
 *
 * TEST INFRASTRUCTURE ONLY (see fk_oracle.h): the checker the GPU library is compared with; nothing in the shipped
 * library links, loads or calls it.
 */
#ifndef FK_ORACLE_PATHS_H
#define FK_ORACLE_PATHS_H

#include "fk_oracle.h"

#ifdef __cplusplus
extern "C" {
#endif

/* executeOperations(std::array<Ptr2D<uchar3>, n> input, used, default, Tensor<uchar3> output, stream)
 * (fused_kernel.h:26-33 -> executors.h:77-84): PerThreadRead<_2D,uchar3>::build(used, default, input) ->
 * PerThreadWrite<_3D,uchar3>.  Planes z >= used hold `def` in every element (batch_operations.h:234-241).
 * out: n planes of h x w packed uchar3. */
int fko_conditional_copy_u8c3(const uint8_t* const* srcs, int w, int h, size_t pitch, int n, int used, const uint8_t def[3],
                              uint8_t* out);
/* PerThreadRead<_2D,uchar3>::build(array of n images) -> Resize<INTER_LINEAR, IGNORE_AR>::build(used, default, array of n
 * sizes) -> TensorWrite<float3>: the batch of resizes carries the policy (resize.h batch builders through
 * batch_operations.h:380-504), and the fused batch keeps it with its default (iop_fuser.h:57-62).  All sizes are
 * dst_w x dst_h.  out: n planes of dst_h x dst_w packed float3; planes z >= used hold `def`. */
int fko_conditional_resize_f32c3(const uint8_t* const* srcs, int w, int h, size_t pitch, int n, int used, const float def[3],
                                 int dst_w, int dst_h, int quirk_y1_from_x, float* out);
/* PerThreadRead<_2D,float3> -> Mul<float3>(mul_v) -> PerThreadWrite<_2D,float3>(mid) -> Add<float3>(add_v) ->
 * PerThreadWrite<_2D,float3>(out): the write in the middle stores the value and hands it on
 * (fused_operation.h:136-326, a MidWrite). */
int fko_muladd_midwrite_f32c3(const float* src, int w, int h, size_t src_pitch, float mul_v, float add_v, float* mid, size_t mid_pitch,
                              float* out, size_t out_pitch);
/* PerThreadRead<_2D,uchar3> -> Crop(rects[n]) -> Cast<uchar3,float3> -> PerThreadWrite<_2D,float3>::build(array of n images)
 * (a BatchWrite, batch_operations.h:43-75).  All rects have the same size; outs[i] is rects[i].height x rects[i].width. */
int fko_batch_crop_cast_images(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int n, float* const* outs,
                               size_t out_pitch);
/* TensorRead<float3> -> Mul<float3> -> TensorWrite<float3> (memory_operations.h:139-171). */
int fko_tensor_mul_f32c3(const float* src, int w, int h, int planes, const float mul[3], float* out);
/* The reference's horizontal-fusion benchmark chain (benchmarks/fusion/benchmark_horizontal_fusion.h:33-92): an array of n
 * windows of one uchar image, all of one size (there: Ptr2D::crop at (i, i), 60 x 120) -> SaturateCast<uchar,float> ->
 * Mul<float> -> Sub<float> -> Div<float> -> TensorWrite<float>.  out: n x rect.height x rect.width floats. */
int fko_batch_windows_saturate_muls_f32(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int n, float mul_v, float sub_v,
                                        float div_v, float* out);

#ifdef __cplusplus
}
#endif
#endif

/* fk_oracle_yuv.h — CPU restatement of the YUV front-end of the Fused Kernel Library's Transform path:
 * ReadYUV / WriteYUV / ConvertYUVToRGB and the chain ReadYUV -> ConvertYUVToRGB -> Crop -> Resize -> Div ->
 * TensorSplit.
 *
 * TEST INFRASTRUCTURE ONLY (see fk_oracle.h): the checker the GPU library is compared with; nothing in the shipped
 * library links, loads or calls it.  Plain C, FP32 in the reference's evaluation order, no FMA contraction.
 *
 * Buffers: a raw YUV image is one 2D allocation of `base` elements (uint8 for 8-bit formats, uint16 for 10-bit
 * ones, samples in the high bits) of fko_yuv_data_dims() elements, rows `pitch` bytes apart.  Semi-planar formats
 * hold `height` luma rows followed by the chroma rows.  Unpacked pixels are 3 (or 4) base elements, interleaved.
 */
#ifndef FK_ORACLE_YUV_H
#define FK_ORACLE_YUV_H

#include "fk_oracle.h"

#ifdef __cplusplus
extern "C" {
#endif

/* PixelFormat values of algorithms/image_processing/raw_image.h:48 (those whose read compiles in the reference). */
enum { FKO_PF_NV12 = 0, FKO_PF_NV21 = 1, FKO_PF_P010 = 3, FKO_PF_P210 = 6, FKO_PF_Y210 = 8, FKO_PF_UYVY = 10 };
/* ColorRange / ColorPrimitives, raw_image.h:27-28. */
enum { FKO_RANGE_LIMITED = 0, FKO_RANGE_FULL = 1 };
enum { FKO_BT601 = 0, FKO_BT709 = 1, FKO_BT2020 = 2 };

/* All return 0, or 1 for a format / matrix the reference does not define. */

/* bytes of one base element (1 or 2) through *base_bytes, data extent in base elements (raw_image.h:53-106) */
int fko_yuv_data_dims(int format, int width, int height, int* data_w, int* data_h, int* base_bytes);
/* ReadYUV<PF>::exec for every pixel: dst gets width x height pixels of 3 base elements */
int fko_read_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch);
/* WriteYUV<PF>::exec for every pixel in the reference's host order (z, y, x): src holds 3 base elements per pixel */
int fko_write_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch);
/* ReadYUV -> ConvertYUVToRGB<PF, range, primaries, alpha, base or float pixel> -> PerThreadWrite */
int fko_yuv_to_rgb(int format, int range, int primaries, int alpha, int float_out, const void* src, size_t src_pitch,
                   int width, int height, void* dst, size_t dst_pitch);
/* ReadYUV -> ConvertYUVToRGB<.., no alpha, base pixel> -> Crop(rect) -> Resize<INTER_LINEAR, IGNORE_AR>(dst size)
 * -> Div<float3>(div_v) -> TensorSplit<float3>: out is 3 planes of dst_h x dst_w floats */
int fko_yuv_crop_resize_norm_split(int format, int range, int primaries, const void* src, size_t src_pitch,
                                   int width, int height, fko_rect crop, int dst_w, int dst_h, float div_v,
                                   int quirk_y1_from_x, float* out);

#ifdef __cplusplus
}
#endif
#endif

/* fk_oracle_border_warp.h — CPU restatement of BorderReader, Warping and Deinterlace on the Fused Kernel Library's
 * Transform path.
 *
 * TEST INFRASTRUCTURE ONLY (see fk_oracle.h): the checker the GPU library is compared with; nothing in the shipped
 * library links, loads or calls it.  Plain C, FP32 in the reference's evaluation order, no FMA contraction.
 */
#ifndef FK_ORACLE_BORDER_WARP_H
#define FK_ORACLE_BORDER_WARP_H

#include "fk_oracle.h"

#ifdef __cplusplus
extern "C" {
#endif

/* BorderType values of algorithms/image_processing/border_reader.h:26-36 that have an implementation there. */
enum { FKO_BORDER_CONSTANT = 0, FKO_BORDER_REPLICATE = 1, FKO_BORDER_REFLECT = 2, FKO_BORDER_WRAP = 3, FKO_BORDER_REFLECT_101 = 4 };
/* WarpType, algorithms/image_processing/warping.h:25. */
enum { FKO_WARP_AFFINE = 0, FKO_WARP_PERSPECTIVE = 1 };

/* source index for coordinate i on an axis of n elements (REPLICATE, REFLECT, WRAP, REFLECT_101); -1 for CONSTANT
 * coordinates outside [0, n) */
int fko_border_index(int border_type, int i, int n);
/* PerThreadRead<_2D,uchar3> -> BorderReader<type>(value) -> Crop(Rect(-left, -top, dst_w, dst_h)) -> PerThreadWrite */
int fko_border_crop_u8c3(int border_type, const uint8_t* src, int w, int h, size_t src_pitch, int left, int top,
                         int dst_w, int dst_h, const uint8_t value[3], uint8_t* dst, size_t dst_pitch);
/* WarpingCoords<type>::exec: matrix is row-major 2x3 (affine) or 3x3 (perspective) */
void fko_warp_coords(int warp_type, const float* matrix, int x, int y, float out[2]);
/* PerThreadRead<_2D,uchar3> -> Warping<type>(matrix, dst size) -> PerThreadWrite<_2D,float3> */
int fko_warp_u8c3_f32c3(int warp_type, const float* matrix, const uint8_t* src, int w, int h, size_t src_pitch,
                        int dst_w, int dst_h, int quirk_y1_from_x, float* dst, size_t dst_pitch);

/* DeinterlaceType, algorithms/image_processing/deinterlace.h:25 */
enum { FKO_DEINTERLACE_BLEND = 0, FKO_DEINTERLACE_INTER_LINEAR = 1 };
/* PerThreadRead<_2D,uchar3> -> Deinterlace<type>(use_even_lines) -> PerThreadWrite<_2D,float3> */
int fko_deinterlace_u8c3_f32c3(int type, int use_even_lines, const uint8_t* src, int w, int h, size_t src_pitch, float* dst,
                               size_t dst_pitch);

#ifdef __cplusplus
}
#endif
#endif

/* fk_oracle.h — CPU restatement of the Fused Kernel Library's fused Transform path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker that the GPU library is compared
 * with; nothing in the shipped library links, loads or calls it.  Every function
 * is a serial, single-threaded restatement of what the reference CPU executor
 * computes for one chain (one output element at a time, z/y/x order,
 * core/execution_model/data_parallel_patterns.h:285-298), written in plain C with
 * FP32 arithmetic evaluated in the reference's order and no FMA contraction
 * (build with -ffp-contract=off).
 *
 * `quirk_y1_from_x`: the reference's host branch of the bilinear interpolation
 * takes the upper row index from the x coordinate
 * (algorithms/image_processing/interpolation.h:69-70) while its device branch
 * uses the y coordinate (:66-67).  0 selects the device-branch behaviour (the
 * canonical one that the GPU library implements), 1 the literal host behaviour.
 */
#ifndef FK_ORACLE_H
#define FK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Rect_<uint,int> of the reference (core/data/rect.h:23-32): x, y, width, height. */
typedef struct fko_rect {
    int x, y, width, height;
} fko_rect;

/* AspectRatio values of algorithms/image_processing/resize.h:42. */
enum { FKO_PRESERVE_AR = 0, FKO_IGNORE_AR = 1, FKO_PRESERVE_AR_RN_EVEN = 2, FKO_PRESERVE_AR_LEFT = 3 };

/* What Resize::build leaves in ResizeReadParams (resize.h:44-59). */
typedef struct fko_resize_params {
    int dst_w, dst_h;
    float fx, fy;
    int src_w, src_h;
    int x1, y1, x2, y2;
} fko_resize_params;

/* ---- seeded generators shared by oracle, fixtures and GPU runs ---- */
void fko_fill_bytes(uint64_t seed, uint8_t* dst, size_t n);
void fko_fill_unit_floats(uint64_t seed, float* dst, size_t n);
/* uniform integers in [lo, hi], one SplitMix64 word each */
void fko_fill_uniform_ints(uint64_t seed, int lo, int hi, int* dst, size_t n);
/* smooth gradient plus uniform noise in [-16, 16], uchar3, tight rows */
void fko_fill_gradient_noise_u8c3(uint64_t seed, uint8_t* dst, int w, int h);
uint64_t fko_fnv1a64(const void* data, size_t n);

/* ---- building blocks ---- */
float fko_round(float x);
void fko_resize_build(int aspect, int src_w, int src_h, int dst_w, int dst_h, fko_resize_params* out);
/* bilinear sample of an interleaved uchar image with `cn` channels; out gets cn floats */
void fko_bilinear_u8(const uint8_t* img, size_t pitch, int cn, int org_x, int org_y, int src_w, int src_h,
                     float sx, float sy, int quirk_y1_from_x, float* out);
uint8_t fko_saturate_int_to_u8(int v);
uint8_t fko_saturate_float_to_u8(float v);
uint8_t fko_rgb2gray_u8(uint8_t x, uint8_t y, uint8_t z);

/* ---- chains ---- */

/* PerThreadRead<_2D,uchar3> -> Crop(rects[n]) -> Resize<LINEAR,aspect>(dst, background)
 * -> Mul<float3> -> Sub<float3> -> Div<float3> -> RGB2BGR -> TensorWrite<float3>.
 * out: n planes of dst_h x dst_w packed float3. */
void fko_crop_resize_muls_bgr_tensor(const uint8_t* src, int src_w, int src_h, size_t src_pitch,
                                     const fko_rect* rects, int n, int dst_w, int dst_h, int aspect,
                                     const float background[3], const float mul[3], const float sub[3],
                                     const float div[3], int quirk_y1_from_x, float* out);

/* PerThreadRead<_2D,float3> -> depth alternating Mul(mul_v)/Add(add_v) (op 0 is Mul) -> PerThreadWrite. */
void fko_muladd_chain_f32c3(const float* src, int w, int h, size_t src_pitch, int depth, float mul_v,
                            float add_v, float* dst, size_t dst_pitch);
/* one unfused stage of the chain above: is_add==0 -> Mul, else Add */
void fko_single_op_f32c3(const float* src, int w, int h, size_t src_pitch, int is_add, float v, float* dst,
                         size_t dst_pitch);

/* PerThreadRead(array of n images) -> Crop(rects[n]) -> Resize<LINEAR,IGNORE_AR>(dst) -> Div<float3>
 * -> Sub<float3> -> Div<float3> -> RGB2BGR -> TensorSplit<float3>.
 * out: n x 3 x dst_h x dst_w planar float. */
void fko_batch_crop_resize_norm_split(const uint8_t* const* srcs, int src_w, int src_h, size_t src_pitch,
                                      const fko_rect* rects, int n, int dst_w, int dst_h, const float div1[3],
                                      const float sub[3], const float div2[3], int quirk_y1_from_x, float* out);

/* PerThreadRead<_2D,uchar3> -> Resize<LINEAR,IGNORE_AR>(rs_w x rs_h) -> Crop(rects[n]) -> Mul<float3>
 * -> TensorWrite<float3>.  The tensor is tile_w x tile_h x n; every (x,y) of the tile box is evaluated
 * for every plane, as the reference does (batch_operations.h:153-160). */
void fko_resize_crop_tiles(const uint8_t* src, int src_w, int src_h, size_t src_pitch, int rs_w, int rs_h,
                           const fko_rect* rects, int n, int tile_w, int tile_h, const float mul[3],
                           int quirk_y1_from_x, float* out);

/* The four chains of the divergent launch, each over a uchar4 image. */
void fko_rgba2gray_u8c4(const uint8_t* src, int w, int h, size_t src_pitch, uint8_t* dst, size_t dst_pitch);
void fko_resize_mul_u8c4_f32c4(const uint8_t* src, int w, int h, size_t src_pitch, int dst_w, int dst_h,
                               float mul_v, int quirk_y1_from_x, float* dst, size_t dst_pitch);
void fko_crop_mul_saturate_u8c4(const uint8_t* src, int w, int h, size_t src_pitch, fko_rect rect, int mul_v,
                                uint8_t* dst, size_t dst_pitch);
void fko_rgba2bgr_sub_u8c4_f32c3(const uint8_t* src, int w, int h, size_t src_pitch, float sub_v, float* dst,
                                 size_t dst_pitch);

/* Batch of crops written straight to a tensor (no resize): PerThreadRead -> Crop(rects[n]) -> Cast<uchar3,float3>
 * -> TensorWrite<float3>, tensor max_w x max_h x n.  `exec_all` != 0 evaluates the whole max box of every
 * plane like the reference (reads beyond a smaller rect; caller keeps them in bounds); 0 leaves elements
 * outside a plane's own rect untouched. */
void fko_batch_crop_cast_tensor(const uint8_t* src, int src_w, int src_h, size_t src_pitch, const fko_rect* rects,
                                int n, int max_w, int max_h, int exec_all, float* out);

#ifdef __cplusplus
}
#endif
#endif

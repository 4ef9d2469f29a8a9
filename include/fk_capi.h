/* fk_capi.h — C entry points for the fused chains of the Transform data-parallel path.
 *
 * The reference has no FFI: its operator API is C++17 templates, so a chain is fixed at compile time.  Each function
 * below is one such chain, instantiated from this library's fk:: templates (include/fk/) for a caller that cannot
 * compile templates (ctypes, cgo, JNI ...).  Device pointers and sizes only; `stream` is a hipStream_t (NULL = default
 * stream); work is enqueued asynchronously, the caller synchronises the stream.  Return value: 0 = enqueued,
 * FK_ERR_UNSUPPORTED = the depth / format / mode has no instantiation, FK_ERR_RUNTIME = the GPU runtime reported
 * an error (text from fk_last_error()), FK_ERR_ARGUMENT = inconsistent arguments.
 *
 * Reference interface each one stands for (paths below the reference's include/fused_kernel/ unless noted):
 *   every function: executeOperations<TransformDPP<>>(stream, sender, receiver), fused_kernel.h:22-25, with the chain
 *   built by .then() (core/execution_model/operation_model/instantiable_operations.h:44-52).
 */
#ifndef FK_CAPI_H
#define FK_CAPI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { FK_OK = 0, FK_ERR_UNSUPPORTED = 1, FK_ERR_RUNTIME = 2, FK_ERR_ARGUMENT = 3 };

/* Rect_<uint,int>, core/data/rect.h:23-32 */
typedef struct fk_rect {
    int x, y, width, height;
} fk_rect;

/* AspectRatio, algorithms/image_processing/resize.h:42 */
enum { FK_PRESERVE_AR = 0, FK_IGNORE_AR = 1, FK_PRESERVE_AR_RN_EVEN = 2, FK_PRESERVE_AR_LEFT = 3 };

const char* fk_last_error(void);
/* 0 when the library was built with the bilinear row index taken from y (the reference's device branch,
 * algorithms/image_processing/interpolation.h:66-67); 1 for a build that takes it from x (its host branch, :69-70). */
int fk_interpolate_y1_from_x(void);

/* The README pipeline (tests/examples/readme_test_code.h:26-72 of the reference):
 * PerThreadRead<_2D,uchar3> -> Crop(rects[n]) -> Resize<INTER_LINEAR, aspect>(dst_w x dst_h, background) ->
 * Mul<float3> -> Sub<float3> -> Div<float3> -> ColorConversion<COLOR_RGB2BGR> -> TensorWrite<float3>.
 * out: n planes of dst_h x dst_w packed float3.  Any n >= 1: the number of planes is a run-time value here (the reference
 * fixes it with BATCH; its benchmarks/fusion/benchmark_horizontal_fusion.h:27-31 sweeps 1 .. 46 and names 120), up to 64
 * planes per launch. */
int fk_crop_resize_muls_bgr_tensor(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n,
                                   int dst_w, int dst_h, int aspect, const float background[3], const float mul[3],
                                   const float sub[3], const float div[3], float* out, void* stream);

/* The same pipeline for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid it).  No counterpart in the reference, whose launches pass every parameter by value.  fk_crop_resize_muls_bgr_tensor
 * keeps the chain's plane table in the kernel arguments or, above the runtime's limit for those, in a block that it
 * allocates for the launch; this entry point keeps it in a fixed block of device memory that belongs to the library
 * (FK_NOALLOC_MAX_JOB_BYTES per GPU, held until the process ends) and calls no allocating or freeing routine.  Same
 * arguments and results; n <= FK_NOALLOC_MAX_PLANES, more returns FK_ERR_UNSUPPORTED.  All calls on one GPU share that
 * block: calls that overlap there (other streams or host threads) race; calls in one stream do not. */
#define FK_NOALLOC_MAX_PLANES 64
#define FK_NOALLOC_MAX_JOB_BYTES 32768
int fk_crop_resize_muls_bgr_tensor_noalloc(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n,
                                           int dst_w, int dst_h, int aspect, const float background[3], const float mul[3],
                                           const float sub[3], const float div[3], float* out, void* stream);

/* Vertical fusion: PerThreadRead<_2D,float3> -> depth x alternating Mul<float3>(mul_v) / Add<float3>(add_v)
 * (operation 0 is Mul) -> PerThreadWrite<_2D,float3>, one launch.  depth in {1,2,4,8,16,32,64,128}.
 * (algorithms/basic_ops/arithmetic.h:22-88; benchmarks/numinstructions/benchmark_numinstructions_x_operation.h:68-99
 * of the reference builds the same kind of chain.) */
int fk_muladd_chain_f32c3(const void* src, int w, int h, size_t src_pitch, int depth, float mul_v, float add_v, void* dst,
                          size_t dst_pitch, void* stream);
/* One unfused stage of that chain: read -> Mul or Add -> write. */
int fk_single_op_f32c3(const void* src, int w, int h, size_t src_pitch, int is_add, float v, void* dst, size_t dst_pitch,
                       void* stream);

/* Horizontal fusion: PerThreadRead(array of n images) -> Crop(rects[n]) -> Resize<INTER_LINEAR>(dst) -> Div<float3> ->
 * Sub<float3> -> Div<float3> -> COLOR_RGB2BGR -> TensorSplit<float3> (memory_operations.h:195-226).
 * srcs: host array of n device pointers.  out: n x 3 x dst_h x dst_w planar float.  Any n >= 1. */
int fk_batch_crop_resize_norm_split(const void* const* srcs, int src_w, int src_h, size_t src_pitch, const fk_rect* rects,
                                    int n, int dst_w, int dst_h, const float div1[3], const float sub[3],
                                    const float div2[3], float* out, void* stream);

/* Backwards vertical fusion: PerThreadRead<_2D,uchar3> -> Resize<INTER_LINEAR>(rs_w x rs_h) -> Crop(rects[n]) ->
 * Mul<float3> -> TensorWrite<float3>; no resized image is materialised.  out: n x tile_h x tile_w float3.  Any n >= 1. */
int fk_resize_crop_tiles(const void* src, int src_w, int src_h, size_t src_pitch, int rs_w, int rs_h, const fk_rect* rects,
                         int n, int tile_w, int tile_h, const float mul[3], float* out, void* stream);

/* The four chains of the divergent launch, runnable on their own ... */
int fk_rgba2gray_u8c4(const void* src, int w, int h, size_t src_pitch, void* dst, size_t dst_pitch, void* stream);
int fk_resize_mul_u8c4_f32c4(const void* src, int w, int h, size_t src_pitch, int dst_w, int dst_h, float mul_v, void* dst,
                             size_t dst_pitch, void* stream);
int fk_crop_mul_saturate_u8c4(const void* src, int w, int h, size_t src_pitch, fk_rect rect, int mul_v, void* dst,
                              size_t dst_pitch, void* stream);
int fk_rgba2bgr_sub_u8c4_f32c3(const void* src, int w, int h, size_t src_pitch, float sub_v, void* dst, size_t dst_pitch,
                               void* stream);
/* ... and as ONE launch (executeOperations<DivergentBatchTransformDPP<>>; the reference declares the pattern in
 * core/execution_model/data_parallel_patterns.h:301-353 but ships no executor for it):
 * (a) COLOR_RGBA2GRAY -> uchar; (b) Resize<INTER_LINEAR>(rs_w x rs_h) -> Mul<float4>(mul_b) -> float4;
 * (c) Crop(rect_c) -> Mul<uchar4,int,int4>(mul_c) -> SaturateCast<int4,uchar4>; (d) COLOR_RGBA2BGR -> Cast<float3> ->
 * Sub<float3>(sub_d).  Output rows are tight. */
int fk_divergent4_u8c4(const void* src, int w, int h, size_t src_pitch, void* gray_out, int rs_w, int rs_h, float mul_b,
                       void* resized_out, fk_rect rect_c, int mul_c, void* crop_out, float sub_d, void* bgr_out,
                       void* stream);

/* Ragged batch without resize: PerThreadRead -> Crop(rects[n]) -> Cast<uchar3,float3> -> TensorWrite<float3> into a
 * max_w x max_h x n tensor.  Every plane receives the box of the largest width and the largest height among the rects,
 * as the reference's thread grid covers it for every plane (batch_operations.h:153-160): beside its own rect a plane
 * holds the source image's pixels there, and zero where the box leaves the source image (the reference reads past the
 * image there).  Tensor elements outside that box are left untouched. */
int fk_batch_crop_cast_tensor(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n,
                              int max_w, int max_h, float* out, void* stream);

/* The reference's horizontal-fusion benchmark chain (benchmarks/fusion/benchmark_horizontal_fusion.h:55-72): a batch of
 * n windows of one uchar image, all of the size of the first (there Ptr2D::crop at (i, i), 60 x 120, batch 1 ... 46,
 * "120 in the paper") -> SaturateCast<uchar,float> -> Mul<float> -> Sub<float> -> Div<float> -> TensorWrite<float>, one
 * launch per 64 planes.  out: n x rects[0].height x rects[0].width floats.  Any n >= 1. */
int fk_batch_windows_saturate_muls_f32(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n,
                                       float mul_v, float sub_v, float div_v, float* out, void* stream);

/* ---- less common chain shapes ---------------------------------------------------------------------------------- */

/* executeOperations(std::array<Ptr2D<uchar3>, BATCH> input, activeBatch, defaultValue, Tensor<uchar3> output, stream)
 * (fused_kernel.h:26-33 -> executors.h:77-84): PerThreadRead<_2D,uchar3>::build(used, def, images) ->
 * PerThreadWrite<_3D,uchar3>, a batch read with PlanePolicy::CONDITIONAL_WITH_DEFAULT (batch_operations.h:218-241).
 * srcs: host array of n device pointers to w x h images; planes z >= used receive `def` in every element.
 * out: n planes of h x w packed uchar3.  1 <= n <= 64. */
int fk_conditional_copy_u8c3(const void* const* srcs, int w, int h, size_t pitch, int n, int used, const uint8_t def[3], void* out,
                             void* stream);
/* PerThreadRead<_2D,uchar3>::build(images) -> Resize<INTER_LINEAR>::build(used, def, sizes) -> TensorWrite<float3>: the
 * batch of resizes carries the policy and the fused batch keeps it (iop_fuser.h:57-62).  out: n planes of
 * dst_h x dst_w packed float3; planes z >= used receive `def`.  1 <= n <= 64. */
int fk_conditional_resize_f32c3(const void* const* srcs, int w, int h, size_t pitch, int n, int used, const float def[3], int dst_w,
                                int dst_h, float* out, void* stream);
/* PerThreadRead<_2D,float3> -> Mul<float3>(mul_v) -> PerThreadWrite<_2D,float3>(mid) -> Add<float3>(add_v) ->
 * PerThreadWrite<_2D,float3>(out): a write in the middle of a chain stores the value and hands it on
 * (fused_operation.h:49-62).  (The reference does this for a chain fused with .then(); given the same operations as
 * separate arguments of executeOperations it ends the chain at the first write, data_parallel_patterns.h:77-79.  This
 * library treats both forms alike.) */
int fk_muladd_midwrite_f32c3(const void* src, int w, int h, size_t src_pitch, float mul_v, float add_v, void* mid, size_t mid_pitch,
                             void* out, size_t out_pitch, void* stream);
/* PerThreadRead<_2D,uchar3> -> Crop(rects[n]) -> Cast<uchar3,float3> -> PerThreadWrite<_2D,float3>::build(array of n
 * images), a BatchWrite (batch_operations.h:43-75).  All rects have the size of the first; outs: host array of n device
 * pointers to images of that size, rows out_pitch bytes apart.  1 <= n <= 64. */
int fk_batch_crop_cast_images(const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, float* const* outs,
                              size_t out_pitch, void* stream);
/* TensorRead<float3> -> Mul<float3> -> TensorWrite<float3> (memory_operations.h:139-171, 173-193): planes x h x w packed
 * float3 on both sides. */
int fk_tensor_mul_f32c3(const void* src, int w, int h, int planes, const float mul[3], void* out, void* stream);
/* fk::setTo(value, Tensor<float3>, stream) for a tensor in device memory (core/data/ptr_utils.h:23-45): ReadSet<float3> ->
 * PerThreadWrite<_3D,float3>, a launch that only stores.  out: planes x h x w packed float3. */
int fk_set_to_f32c3_tensor(const float value[3], void* out, int w, int h, int planes, void* stream);

/* ---- YUV front-end ------------------------------------------------------------------------------------------
 * A raw YUV image is ONE 2D allocation of base elements (uint8 for the 8-bit formats, uint16 with the sample in the
 * high bits for the 10-bit ones), rows src_pitch bytes apart, as RawImage<PF> describes it
 * (algorithms/image_processing/raw_image.h:108-114): NV12/NV21/P010 hold `height` luma rows then height/2 rows of
 * interleaved chroma pairs, P210 `height` luma rows then `height` chroma rows, UYVY/Y210 2*width elements per row.
 * width and height must be even.  Unpacked pixels are 3 (or 4) base elements, interleaved. */

/* PixelFormat, raw_image.h:48 (the formats whose read compiles in the reference) */
enum { FK_PF_NV12 = 0, FK_PF_NV21 = 1, FK_PF_P010 = 3, FK_PF_P210 = 6, FK_PF_Y210 = 8, FK_PF_UYVY = 10 };
/* ColorRange and ColorPrimitives, raw_image.h:27-28.  A YCbCr -> RGB matrix exists for (FULL, BT601), (FULL, BT709),
 * (LIMITED, BT709) and (FULL, BT2020) (algorithms/image_processing/color_conversion.h:137-171); any other pair
 * returns FK_ERR_UNSUPPORTED. */
enum { FK_RANGE_LIMITED = 0, FK_RANGE_FULL = 1 };
enum { FK_BT601 = 0, FK_BT709 = 1, FK_BT2020 = 2 };

/* ReadYUV<PF> -> PerThreadWrite<_2D, base3> (color_conversion.h:315-400): the {Y, U, V} of every pixel. */
int fk_read_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch, void* stream);
/* PerThreadRead<_2D, base3> -> WriteYUV<PF> (color_conversion.h:402-513): {Y, U, V} pixels into a raw image; each
 * chroma sample takes the value of the last pixel that the reference's host loop lets write it. */
int fk_write_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch, void* stream);
/* ReadYUV<PF> -> ConvertYUVToRGB<PF, range, primaries, alpha, pixel> -> PerThreadWrite (color_conversion.h:250-310).
 * pixel = base3/base4 (float_out = 0) or float3/float4 (float_out = 1); alpha appends the depth's maximum. */
int fk_yuv_to_rgb(int format, int range, int primaries, int alpha, int float_out, const void* src, size_t src_pitch, int width,
                  int height, void* dst, size_t dst_pitch, void* stream);
/* The README's backwards-vertical-fusion example (README.md:155-163 of the reference): ReadYUV<PF> ->
 * ConvertYUVToRGB<PF, range, primaries, false> -> Crop(crop) -> Resize<INTER_LINEAR>(dst_w x dst_h) ->
 * Div<float3>(div_v) -> TensorSplit<float3>: dst receives 3 planes of dst_h x dst_w floats.  Only the YUV samples
 * that the interpolation of the crop touches are read. */
int fk_yuv_crop_resize_norm_split(int format, int range, int primaries, const void* src, size_t src_pitch, int width, int height,
                                  fk_rect crop, int dst_w, int dst_h, float div_v, float* dst, void* stream);

/* ---- BorderReader and Warping ------------------------------------------------------------------------------ */

/* BorderType, algorithms/image_processing/border_reader.h:26-36 (the types implemented there) */
enum { FK_BORDER_CONSTANT = 0, FK_BORDER_REPLICATE = 1, FK_BORDER_REFLECT = 2, FK_BORDER_WRAP = 3, FK_BORDER_REFLECT_101 = 4 };
/* WarpType, algorithms/image_processing/warping.h:25 */
enum { FK_WARP_AFFINE = 0, FK_WARP_PERSPECTIVE = 1 };

/* PerThreadRead<_2D,uchar3> -> BorderReader<border_type>(value) -> Crop(Rect(-left, -top, dst_w, dst_h)) ->
 * PerThreadWrite<_2D,uchar3> (border_reader.h:141-277, crop.h:35-38): a window of the image extended by its border
 * rule; with left, top >= 0 and a larger destination this is the image with a border around it.  `value` is used by
 * FK_BORDER_CONSTANT only. */
int fk_border_crop_u8c3(int border_type, const void* src, int w, int h, size_t src_pitch, int left, int top, int dst_w, int dst_h,
                        const uint8_t value[3], void* dst, size_t dst_pitch, void* stream);
/* PerThreadRead<_2D,uchar3> -> Warping<warp_type>(matrix, dst size) -> PerThreadWrite<_2D,float3> (warping.h:43-108):
 * matrix is row-major 2x3 (affine) or 3x3 (perspective) and maps destination to source coordinates; destinations whose
 * source point falls outside the image are zero. */
int fk_warp_u8c3_f32c3(int warp_type, const float* matrix, const void* src, int w, int h, size_t src_pitch, int dst_w, int dst_h,
                       void* dst, size_t dst_pitch, void* stream);

/* DeinterlaceType, algorithms/image_processing/deinterlace.h:25 */
enum { FK_DEINTERLACE_BLEND = 0, FK_DEINTERLACE_INTER_LINEAR = 1 };
/* PerThreadRead<_2D,uchar3> -> Deinterlace<type>(use_even_lines) -> PerThreadWrite<_2D,float3> (deinterlace.h:41-126):
 * BLEND averages each line with the one above; INTER_LINEAR keeps the even (use_even_lines != 0) or odd lines and
 * rebuilds the others from their two neighbours.  Sums are integer, + 1, times 0.5f. */
int fk_deinterlace_u8c3_f32c3(int type, int use_even_lines, const void* src, int w, int h, size_t src_pitch, void* dst, size_t dst_pitch,
                              void* stream);

/* ---- tensor layouts and circular tensors ---------------------------------------------------------------------
 * A tensor of `planes` images of h x w float3 pixels, rows tight: packed = planes, h, w, 3 (TensorRead / TensorWrite);
 * split = planes, 3, h, w (TensorSplit / TensorPack); transposed = 3, planes, h, w (TensorTSplit / TensorTPack). */
enum { FK_PACKED_TO_SPLIT = 0, FK_PACKED_TO_TRANSPOSED = 1, FK_SPLIT_TO_PACKED = 2, FK_TRANSPOSED_TO_PACKED = 3 };
/* CircularDirection, core/execution_model/memory_operations.h:425 */
enum { FK_ASCENDENT = 0, FK_DESCENDENT = 1 };

/* TensorRead<float3> -> TensorSplit / TensorTSplit, or TensorPack / TensorTPack -> TensorWrite<float3>
 * (memory_operations.h:195-348). */
int fk_tensor_relayout_f32c3(int mode, const float* src, int w, int h, int planes, float* dst, void* stream);
/* CircularTensorRead<direction, TensorRead<float3>, planes>{first} -> TensorWrite<float3> (memory_operations.h:527-566):
 * plane z of dst is ring plane first + z (ascendent) or first - z (descendent) modulo planes; planes in 2, 3, 4, 8, 16. */
int fk_circular_tensor_read_f32c3(int direction, int first, const float* ring, int w, int h, int planes, float* dst, void* stream);
/* CircularTensor<float, 3, batch, order, ColorPlanes::Standard>::update(stream, PerThreadRead<_2D,uchar3>(frame),
 * Cast<uchar3,float3>, Mul<float3>(mul_v), TensorSplit<float3>(tensor)) (core/data/circular_tensor.h:84-161) over memory
 * the caller owns: `tensor` and `ring` are batch x 3 x h x w floats each; next_index is the ring slot this update fills
 * (0 for the first update, then (next_index + 1) % batch).  After the call plane 0 (newest_first) or plane batch - 1 of
 * `tensor` holds this frame and the other planes the previous frames by age.  batch in 2, 3, 4, 8, 16. */
int fk_circular_tensor_update_u8c3_split_f32(const void* frame, int w, int h, size_t src_pitch, float mul_v, float* tensor, float* ring,
                                             int batch, int next_index, int newest_first, void* stream);

#ifdef __cplusplus
}
#endif
#endif

/* fk_oracle_yuv.c — CPU restatement of the reference's YUV front-end (see fk_oracle_yuv.h).
 *
 * TEST INFRASTRUCTURE ONLY.  Citations are paths below the reference's include/fused_kernel/.
 *
 * How each function is pinned (tests/test_oracle_yuv.py):
 *   - fko_read_yuv: the reference's own known-answer vectors for UYVY
 *     (utests/algorithm/image_processing/utest_color_conversion.h:226-324), hand-laid buffers for every other
 *     format, and the reference's headers compiled for its CPU backend (oracle/_ref) on random buffers;
 *   - fko_write_yuv: read(write(p)) == p on chroma-consistent input, and oracle/_ref;
 *   - fko_yuv_to_rgb: oracle/_ref bit for bit on every format x matrix x alpha x output type, the grey axis
 *     (U = V = centre gives R = G = B), and a double-precision evaluation of the same matrices;
 *   - fko_yuv_crop_resize_norm_split: oracle/_ref with the literal host interpolation (quirk = 1), and with
 *     quirk = 0 the composition fko_yuv_to_rgb -> crop -> bilinear of fk_oracle.c, which is pinned on its own.
 *
 * Semi-planar chroma rows start `pitch * height` bytes after the first luma row, `height` being the image
 * height.  The reference computes that offset from the height of the data extent
 * (algorithms/image_processing/color_conversion.h:337,353); both agree when the caller describes the buffer with
 * the image height, which is how oracle/_ref is driven.
 */
#include "fk_oracle_yuv.h"

#include <math.h>
#include <string.h>

typedef struct yuv_layout {
    int base_bytes;   /* 1: uint8 samples, 2: uint16 samples */
    int semi_planar;  /* luma plane + interleaved chroma plane, else packed 4:2:2 */
    int u, v;         /* position of U and V inside a chroma pair / a packed quad */
    int y0, y1;       /* packed: position of the even and the odd pixel's luma in the quad */
    int row_shift;    /* semi-planar: log2 of luma rows per chroma row */
    int shift;        /* shiftFactor<depth>, color_conversion.h:179-182 */
    float data_wf, data_hf; /* ResolutionFactors, raw_image.h:53-106 */
} yuv_layout;

static int layout_of(int format, yuv_layout* l) {
    memset(l, 0, sizeof *l);
    switch (format) {
    case FKO_PF_NV12: *l = (yuv_layout){1, 1, 0, 1, 0, 0, 1, 0, 1.f, 1.5f}; return 0;
    case FKO_PF_NV21: *l = (yuv_layout){1, 1, 1, 0, 0, 0, 1, 0, 1.f, 1.5f}; return 0;
    case FKO_PF_P010: *l = (yuv_layout){2, 1, 0, 1, 0, 0, 1, 6, 1.f, 1.5f}; return 0;
    case FKO_PF_P210: *l = (yuv_layout){2, 1, 0, 1, 0, 0, 0, 6, 1.f, 2.f}; return 0;
    case FKO_PF_Y210: *l = (yuv_layout){2, 0, 1, 3, 0, 2, 0, 6, 2.f, 1.f}; return 0;
    case FKO_PF_UYVY: *l = (yuv_layout){1, 0, 0, 2, 1, 3, 0, 0, 2.f, 1.f}; return 0;
    default: return 1;
    }
}

int fko_yuv_data_dims(int format, int width, int height, int* data_w, int* data_h, int* base_bytes) {
    yuv_layout l;
    if (layout_of(format, &l)) return 1;
    /* Image<PF> constructor, image.h:40-45: uint = uint * float */
    *data_w = (int)(unsigned)((float)(unsigned)width * l.data_wf);
    *data_h = (int)(unsigned)((float)(unsigned)height * l.data_hf);
    *base_bytes = l.base_bytes;
    return 0;
}

static inline unsigned sample(const void* row, int base_bytes, size_t i) {
    return base_bytes == 1 ? ((const uint8_t*)row)[i] : ((const uint16_t*)row)[i];
}
static inline void put(void* row, int base_bytes, size_t i, unsigned v) {
    if (base_bytes == 1) ((uint8_t*)row)[i] = (uint8_t)v;
    else ((uint16_t*)row)[i] = (uint16_t)v;
}

/* ReadYUV<PF>::exec, color_conversion.h:327-378: {Y, U, V} of pixel (x, y) */
static void read_pixel(const yuv_layout* l, const void* src, size_t pitch, int height, int x, int y, unsigned out[3]) {
    const char* base = (const char*)src;
    if (l->semi_planar) {
        out[0] = sample(base + (size_t)y * pitch, l->base_bytes, (size_t)x);
        const char* chroma = base + pitch * (size_t)height + (size_t)(y >> l->row_shift) * pitch;
        out[1] = sample(chroma, l->base_bytes, 2 * (size_t)(x >> 1) + l->u);
        out[2] = sample(chroma, l->base_bytes, 2 * (size_t)(x >> 1) + l->v);
    } else {
        const char* row = base + (size_t)y * pitch;
        const size_t q = 4 * (size_t)(x >> 1);
        out[0] = sample(row, l->base_bytes, q + ((x & 1) ? l->y1 : l->y0));
        out[1] = sample(row, l->base_bytes, q + l->u);
        out[2] = sample(row, l->base_bytes, q + l->v);
    }
}

int fko_read_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch) {
    yuv_layout l;
    if (layout_of(format, &l)) return 1;
    for (int y = 0; y < height; ++y) {
        void* drow = (char*)dst + (size_t)y * dst_pitch;
        for (int x = 0; x < width; ++x) {
            unsigned p[3];
            read_pixel(&l, src, src_pitch, height, x, y, p);
            for (int k = 0; k < 3; ++k) put(drow, l.base_bytes, 3 * (size_t)x + k, p[k]);
        }
    }
    return 0;
}

/* WriteYUV<PF>::exec, color_conversion.h:413-489, applied in the host executor's order (y outer, x inner), so a
 * sample that several pixels write keeps the last writer's value. */
int fko_write_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch) {
    yuv_layout l;
    if (layout_of(format, &l)) return 1;
    char* base = (char*)dst;
    for (int y = 0; y < height; ++y) {
        const void* srow = (const char*)src + (size_t)y * src_pitch;
        for (int x = 0; x < width; ++x) {
            const unsigned Y = sample(srow, l.base_bytes, 3 * (size_t)x);
            const unsigned U = sample(srow, l.base_bytes, 3 * (size_t)x + 1);
            const unsigned V = sample(srow, l.base_bytes, 3 * (size_t)x + 2);
            if (l.semi_planar) {
                put(base + (size_t)y * dst_pitch, l.base_bytes, (size_t)x, Y);
                int writes;
                if (format == FKO_PF_NV21) writes = 1;                                   /* :446, every pixel */
                else if (l.row_shift == 1) writes = (x & 1) == 0 && (y & 1) == 0;        /* :427-431 */
                else writes = (x & 1) == 0;                                              /* :433-436 */
                if (writes) {
                    char* chroma = base + dst_pitch * (size_t)height + (size_t)(y >> l.row_shift) * dst_pitch;
                    put(chroma, l.base_bytes, 2 * (size_t)(x >> 1) + l.u, U);
                    put(chroma, l.base_bytes, 2 * (size_t)(x >> 1) + l.v, V);
                }
            } else {
                char* row = base + (size_t)y * dst_pitch;
                const size_t q = 4 * (size_t)(x >> 1);
                if ((x & 1) == 0) {
                    put(row, l.base_bytes, q + l.y0, Y);
                    put(row, l.base_bytes, q + l.u, U);
                    put(row, l.base_bytes, q + l.v, V);
                } else {
                    put(row, l.base_bytes, q + l.y1, Y);
                }
            }
        }
    }
    return 0;
}

/* ccMatrix<range, primaries, YCbCr2RGB>, color_conversion.h:137-171 (rows x, y, z) */
static const float* matrix_of(int range, int primaries) {
    static const float full601[9] = {1.164383562f, 0.f, 1.596026786f, 1.164383562f, -0.39176229f, -0.812967647f,
                                     1.164383562f, 2.017232143f, 0.f};
    static const float full709[9] = {1.f, 0.f, 1.5748f, 1.f, -0.1873f, -0.4681f, 1.f, 1.8556f, 0.f};
    static const float limited709[9] = {1.f, 0.f, 1.402f, 1.f, -0.34414f, -0.71414f, 1.f, 1.772f, 0.f};
    static const float full2020[9] = {1.f, 0.f, 1.4746f, 1.f, -0.16455312684366f, -0.57135312684366f,
                                      1.f, 1.8814f, 0.f};
    if (range == FKO_RANGE_FULL && primaries == FKO_BT601) return full601;
    if (range == FKO_RANGE_FULL && primaries == FKO_BT709) return full709;
    if (range == FKO_RANGE_LIMITED && primaries == FKO_BT709) return limited709;
    if (range == FKO_RANGE_FULL && primaries == FKO_BT2020) return full2020;
    return NULL;
}

/* SaturateCastBase<float, uchar|ushort>, saturate.h:35-53 */
static unsigned saturate_to_base(float v, int base_bytes) {
    const float hi = base_bytes == 1 ? 255.0f : 65535.0f;
    if (v > hi) return (unsigned)hi;
    if (v < 0.0f) return 0;
    return (unsigned)fko_round(v);
}

typedef struct yuv_pixel {
    unsigned i[4]; /* integer output, already shifted back up */
    float f[4];    /* float output */
} yuv_pixel;

/* ConvertYUVToRGB::exec, color_conversion.h:262-310, on one {Y, U, V} as stored */
static void convert_pixel(const yuv_layout* l, const float* m, int primaries, int alpha, int float_out,
                          const unsigned stored[3], yuv_pixel* out) {
    const int ten_bit = l->shift != 0;
    const float chroma_sub = ten_bit ? 512.f : 128.f; /* subCoefficients, :92-96 */
    const float luma_sub = ten_bit ? 64.f : 16.f;
    const unsigned max_depth = ten_bit ? 1023u : 255u; /* :98-103 */
    /* ShiftRight on the storage type, :300 */
    const unsigned Y = stored[0] >> l->shift, U = stored[1] >> l->shift, V = stored[2] >> l->shift;
    /* computeRGB, :267-276: luma is offset for bt601 only */
    const float c0 = primaries == FKO_BT601 ? (float)Y - luma_sub : (float)Y;
    const float c1 = (float)U - chroma_sub;
    const float c2 = (float)V - chroma_sub;
    float rgb[3];
    for (int r = 0; r < 3; ++r) { /* MxVFloat3, basic_ops/algebraic.h:55-61: products, then (x + y) + z */
        const float px = c0 * m[3 * r], py = c1 * m[3 * r + 1], pz = c2 * m[3 * r + 2];
        rgb[r] = (px + py) + pz;
    }
    if (float_out) { /* :280-285 then NormalizeColorRangeDepth :218-228 on every channel */
        const float scale = ten_bit ? 64.f : 1.f;
        for (int r = 0; r < 3; ++r) out->f[r] = rgb[r] * scale;
        if (alpha) out->f[3] = (float)max_depth * scale;
    } else { /* :287-293 then ShiftLeft on the storage type :308 */
        const unsigned mask = l->base_bytes == 1 ? 0xFFu : 0xFFFFu;
        for (int r = 0; r < 3; ++r) out->i[r] = (saturate_to_base(rgb[r], l->base_bytes) << l->shift) & mask;
        if (alpha) out->i[3] = (max_depth << l->shift) & mask;
    }
}

int fko_yuv_to_rgb(int format, int range, int primaries, int alpha, int float_out, const void* src, size_t src_pitch,
                   int width, int height, void* dst, size_t dst_pitch) {
    yuv_layout l;
    const float* m = matrix_of(range, primaries);
    if (layout_of(format, &l) || m == NULL) return 1;
    const int cn = alpha ? 4 : 3;
    for (int y = 0; y < height; ++y) {
        void* drow = (char*)dst + (size_t)y * dst_pitch;
        for (int x = 0; x < width; ++x) {
            unsigned p[3];
            yuv_pixel o;
            read_pixel(&l, src, src_pitch, height, x, y, p);
            convert_pixel(&l, m, primaries, alpha, float_out, p, &o);
            for (int k = 0; k < cn; ++k) {
                if (float_out) ((float*)drow)[(size_t)cn * x + k] = o.f[k];
                else put(drow, l.base_bytes, (size_t)cn * x + k, o.i[k]);
            }
        }
    }
    return 0;
}

int fko_yuv_crop_resize_norm_split(int format, int range, int primaries, const void* src, size_t src_pitch,
                                   int width, int height, fko_rect crop, int dst_w, int dst_h, float div_v,
                                   int quirk_y1_from_x, float* out) {
    yuv_layout l;
    const float* m = matrix_of(range, primaries);
    if (layout_of(format, &l) || m == NULL) return 1;
    (void)width;
    fko_resize_params p;
    fko_resize_build(FKO_IGNORE_AR, crop.width, crop.height, dst_w, dst_h, &p);
    const size_t plane = (size_t)dst_w * dst_h;
    for (int y = 0; y < dst_h; ++y)
        for (int x = 0; x < dst_w; ++x) {
            /* Resize::exec_resize, resize.h:183-194, and Interpolate, interpolation.h:61-96, over the back read
             * Crop(ReadYUV -> ConvertYUVToRGB) */
            const float sx = (float)x * p.fx;
            const float sy = (float)y * p.fy;
            const int x1 = (int)floorf(sx);
            const int y1 = quirk_y1_from_x ? (int)floorf(sx) : (int)floorf(sy);
            const int x2 = x1 + 1, y2 = y1 + 1;
            const int x2r = x2 < p.src_w - 1 ? x2 : p.src_w - 1;
            const int y2r = y2 < p.src_h - 1 ? y2 : p.src_h - 1;
            const int tx[4] = {x1, x2r, x1, x2r}, ty[4] = {y1, y1, y2r, y2r};
            const float w[4] = {((float)x2 - sx) * ((float)y2 - sy), (sx - (float)x1) * ((float)y2 - sy),
                                ((float)x2 - sx) * (sy - (float)y1), (sx - (float)x1) * (sy - (float)y1)};
            yuv_pixel tap[4];
            for (int t = 0; t < 4; ++t) {
                unsigned s[3];
                read_pixel(&l, src, src_pitch, height, tx[t] + crop.x, ty[t] + crop.y, s);
                convert_pixel(&l, m, primaries, 0, 0, s, &tap[t]);
            }
            for (int k = 0; k < 3; ++k) {
                const float t0 = (float)tap[0].i[k] * w[0], t1 = (float)tap[1].i[k] * w[1];
                const float t2 = (float)tap[2].i[k] * w[2], t3 = (float)tap[3].i[k] * w[3];
                const float v = ((t0 + t1) + t2) + t3;
                /* Div<float3>, arithmetic.h:75-87; TensorSplit, memory_operations.h:207-218 */
                out[(size_t)k * plane + (size_t)y * dst_w + x] = v / div_v;
            }
        }
    return 0;
}

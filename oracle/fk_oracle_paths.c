/* fk_oracle_paths.c — see fk_oracle_paths.h.  TEST INFRASTRUCTURE ONLY.
 *
 * Every function walks the output in the reference CPU executor's z / y / x order and computes one element at a time.
 * Pinned by tests/test_oracle_paths.py: vectors written by the reference's own headers (tests/golden/
 * reference_paths_vectors.npz), side-by-side runs against oracle/_ref where that is built, and closed forms in numpy
 * (copies, casts, one multiplication and one addition per element; the resize through the pinned fko_bilinear_u8). */
#include "fk_oracle_paths.h"

int fko_conditional_copy_u8c3(const uint8_t* const* srcs, int w, int h, size_t pitch, int n, int used, const uint8_t def[3],
                              uint8_t* out) {
    if (n <= 0 || w <= 0 || h <= 0) return 1;
    for (int z = 0; z < n; ++z) {
        for (int y = 0; y < h; ++y) {
            for (int x = 0; x < w; ++x) {
                uint8_t* o = out + (((size_t)z * h + y) * w + x) * 3;
                /* batch_operations.h:234-241: usedPlanes <= thread.z yields the default value */
                const uint8_t* p = used <= z ? def : srcs[z] + (size_t)y * pitch + (size_t)x * 3;
                o[0] = p[0];
                o[1] = p[1];
                o[2] = p[2];
            }
        }
    }
    return 0;
}

int fko_conditional_resize_f32c3(const uint8_t* const* srcs, int w, int h, size_t pitch, int n, int used, const float def[3],
                                 int dst_w, int dst_h, int quirk_y1_from_x, float* out) {
    if (n <= 0 || w <= 0 || h <= 0 || dst_w <= 0 || dst_h <= 0) return 1;
    fko_resize_params p;
    fko_resize_build(FKO_IGNORE_AR, w, h, dst_w, dst_h, &p);
    for (int z = 0; z < n; ++z) {
        for (int y = 0; y < dst_h; ++y) {
            for (int x = 0; x < dst_w; ++x) {
                float* o = out + (((size_t)z * dst_h + y) * dst_w + x) * 3;
                if (used <= z) {
                    /* the default of the batch of resizes, which the fused batch keeps (iop_fuser.h:57-62) */
                    o[0] = def[0];
                    o[1] = def[1];
                    o[2] = def[2];
                } else {
                    /* resize.h:168-181: source position = destination position times the conversion factor */
                    fko_bilinear_u8(srcs[z], pitch, 3, 0, 0, w, h, (float)x * p.fx, (float)y * p.fy, quirk_y1_from_x, o);
                }
            }
        }
    }
    return 0;
}

int fko_muladd_midwrite_f32c3(const float* src, int w, int h, size_t src_pitch, float mul_v, float add_v, float* mid, size_t mid_pitch,
                              float* out, size_t out_pitch) {
    if (w <= 0 || h <= 0) return 1;
    for (int y = 0; y < h; ++y) {
        const float* s = (const float*)((const char*)src + (size_t)y * src_pitch);
        float* m = (float*)((char*)mid + (size_t)y * mid_pitch);
        float* o = (float*)((char*)out + (size_t)y * out_pitch);
        for (int i = 0; i < 3 * w; ++i) {
            const float v = s[i] * mul_v;
            m[i] = v;        /* the write in the middle stores what it receives ... */
            o[i] = v + add_v; /* ... and hands it on unchanged */
        }
    }
    return 0;
}

int fko_batch_crop_cast_images(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int n, float* const* outs,
                               size_t out_pitch) {
    if (n <= 0) return 1;
    for (int z = 0; z < n; ++z) {
        const fko_rect r = rects[z];
        if (r.width != rects[0].width || r.height != rects[0].height) return 1;
        if (r.x < 0 || r.y < 0 || r.x + r.width > w || r.y + r.height > h) return 1;
        for (int y = 0; y < r.height; ++y) {
            float* o = (float*)((char*)outs[z] + (size_t)y * out_pitch);
            const uint8_t* s = src + (size_t)(r.y + y) * pitch + (size_t)r.x * 3;
            for (int i = 0; i < 3 * r.width; ++i) o[i] = (float)s[i];
        }
    }
    return 0;
}

int fko_tensor_mul_f32c3(const float* src, int w, int h, int planes, const float mul[3], float* out) {
    if (w <= 0 || h <= 0 || planes <= 0) return 1;
    const size_t n = (size_t)w * h * planes;
    for (size_t i = 0; i < n; ++i) {
        out[3 * i] = src[3 * i] * mul[0];
        out[3 * i + 1] = src[3 * i + 1] * mul[1];
        out[3 * i + 2] = src[3 * i + 2] * mul[2];
    }
    return 0;
}

/* benchmark_horizontal_fusion.h:66-72: per element ((float)v * mul - sub) / div, each operation rounded to float
 * (SaturateCast<uchar,float> is the plain conversion: saturate.h:35-53 clamps nothing for a wider output type). */
int fko_batch_windows_saturate_muls_f32(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int n, float mul_v, float sub_v,
                                        float div_v, float* out) {
    if (n <= 0) return 1;
    for (int i = 0; i < n; ++i) {
        const fko_rect r = rects[i];
        if (r.x < 0 || r.y < 0 || r.width <= 0 || r.height <= 0 || r.x + r.width > w || r.y + r.height > h) return 1;
        if (r.width != rects[0].width || r.height != rects[0].height) return 1;
    }
    const int rw = rects[0].width, rh = rects[0].height;
    for (int z = 0; z < n; ++z) {
        for (int y = 0; y < rh; ++y) {
            const uint8_t* row = src + (size_t)(rects[z].y + y) * pitch + rects[z].x;
            float* o = out + ((size_t)z * rh + y) * rw;
            for (int x = 0; x < rw; ++x) {
                const float v = (float)row[x];
                const float m = v * mul_v;
                const float d = m - sub_v;
                o[x] = d / div_v;
            }
        }
    }
    return 0;
}

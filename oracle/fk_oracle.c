/* fk_oracle.c — CPU restatement of the reference's fused Transform path.
 *
 * TEST INFRASTRUCTURE ONLY (see fk_oracle.h).  Citations are paths below the reference's
 * include/fused_kernel/.  Build: gcc -O2 -ffp-contract=off (no -march=native, no fast-math).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   - against the reference's own headers compiled for its CPU backend (oracle/_ref, literal
 *     host semantics) on the same inputs, bit for bit, for every chain with quirk_y1_from_x=1 and
 *     for the resize-free chains;
 *   - quirk_y1_from_x=0 differs from that by one token (row index from sy instead of sx); it is pinned
 *     by the reference build on every element whose floor(sx)==floor(sy), by transposition symmetry,
 *     by the identity/constant/ramp closed forms and by a double-precision brute force;
 *   - against the known-answer vectors of the reference's unit tests (RGB2Gray, SaturateCast,
 *     cxp::round, BGR reorder) and the Resize parameters the reference's README chain produces.
 */
#include "fk_oracle.h"

#include <math.h>
#include <string.h>

/* ------------------------------------------------------------------ generators */

static inline uint64_t splitmix64_next(uint64_t* s) {
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void fko_fill_bytes(uint64_t seed, uint8_t* dst, size_t n) {
    uint64_t s = seed;
    size_t i = 0;
    for (; i + 8 <= n; i += 8) {
        uint64_t z = splitmix64_next(&s);
        for (int b = 0; b < 8; ++b) dst[i + b] = (uint8_t)(z >> (8 * b));
    }
    if (i < n) {
        uint64_t z = splitmix64_next(&s);
        for (int b = 0; i < n; ++i, ++b) dst[i] = (uint8_t)(z >> (8 * b));
    }
}

void fko_fill_unit_floats(uint64_t seed, float* dst, size_t n) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; ++i) dst[i] = (float)(splitmix64_next(&s) >> 40) * 0x1p-24f;
}

void fko_fill_uniform_ints(uint64_t seed, int lo, int hi, int* dst, size_t n) {
    uint64_t s = seed;
    const uint64_t span = (uint64_t)((int64_t)hi - (int64_t)lo + 1);
    for (size_t i = 0; i < n; ++i) dst[i] = lo + (int)(splitmix64_next(&s) % span);
}

void fko_fill_gradient_noise_u8c3(uint64_t seed, uint8_t* dst, int w, int h) {
    /* ramp weights in quarters: channel c gets (WX[c]*x/(w-1) + WY[c]*y/(h-1)) / 4 of full scale */
    static const int WX[3] = {2, 1, 3};
    static const int WY[3] = {2, 3, 1};
    uint64_t s = seed;
    const int64_t dw = w > 1 ? w - 1 : 1, dh = h > 1 ? h - 1 : 1;
    const int64_t den = 4 * dw * dh;
    for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x)
            for (int c = 0; c < 3; ++c) {
                const int64_t num = 255 * ((int64_t)x * WX[c] * dh + (int64_t)y * WY[c] * dw);
                int v = (int)((num + den / 2) / den) + (-16 + (int)(splitmix64_next(&s) % 33u));
                v = v < 0 ? 0 : (v > 255 ? 255 : v);
                dst[((size_t)y * w + x) * 3 + c] = (uint8_t)v;
            }
}

uint64_t fko_fnv1a64(const void* data, size_t n) {
    const uint8_t* p = (const uint8_t*)data;
    uint64_t hsh = 0xcbf29ce484222325ull;
    for (size_t i = 0; i < n; ++i) {
        hsh ^= p[i];
        hsh *= 0x100000001b3ull;
    }
    return hsh;
}

/* ------------------------------------------------------------------ building blocks */

/* cxp::round, core/constexpr_libs/constexpr_cmath.h:119-130: half away from zero through an int cast */
float fko_round(float x) {
    if (isnan(x) || isinf(x)) return x;
    return (x > 0.0f) ? (float)(int)(x + 0.5f) : (float)(int)(x - 0.5f);
}

/* Resize::compute_target_size, algorithms/image_processing/resize.h:196-221 */
static void compute_target_size(int aspect, int src_w, int src_h, int dst_w, int dst_h, int* tw, int* th) {
    const float scale = dst_h / (float)src_h;
    const int target_h = dst_h;
    const int target_w = (int)fko_round(scale * src_w);
    if (aspect == FKO_PRESERVE_AR_RN_EVEN) {
        const int even_w = target_w - (target_w % 2);
        if (even_w > dst_w) {
            const float scale2 = dst_w / (float)src_w;
            const int h2 = (int)fko_round(scale2 * src_h);
            *tw = dst_w;
            *th = h2 - (h2 % 2);
        } else {
            *tw = even_w;
            *th = target_h;
        }
    } else {
        if (target_w > dst_w) {
            const float scale2 = dst_w / (float)src_w;
            *tw = dst_w;
            *th = (int)fko_round(scale2 * src_h);
        } else {
            *tw = target_w;
            *th = target_h;
        }
    }
}

/* Resize::build, resize.h:105-119 (IGNORE_AR) and :121-166 (PRESERVE_AR*) */
void fko_resize_build(int aspect, int src_w, int src_h, int dst_w, int dst_h, fko_resize_params* out) {
    out->dst_w = dst_w;
    out->dst_h = dst_h;
    out->src_w = src_w;
    out->src_h = src_h;
    if (aspect == FKO_IGNORE_AR) {
        const double cfx = (double)dst_w / (double)src_w;
        const double cfy = (double)dst_h / (double)src_h;
        out->fx = (float)(1.0 / cfx);
        out->fy = (float)(1.0 / cfy);
        out->x1 = 0;
        out->y1 = 0;
        out->x2 = dst_w - 1;
        out->y2 = dst_h - 1;
        return;
    }
    int tw, th;
    compute_target_size(aspect, src_w, src_h, dst_w, dst_h, &tw, &th);
    const double cfx = (double)tw / src_w;
    const double cfy = (double)th / src_h;
    out->fx = (float)(1.0 / cfx);
    out->fy = (float)(1.0 / cfy);
    out->x1 = (aspect == FKO_PRESERVE_AR_LEFT) ? 0 : (dst_w - tw) / 2;
    out->y1 = (dst_h - th) / 2;
    out->x2 = out->x1 + tw - 1;
    out->y2 = out->y1 + th - 1;
}

/* Interpolate<INTER_LINEAR>::exec, algorithms/image_processing/interpolation.h:61-96, over a back read that is
 * Crop (crop.h:35-38: thread + rect origin) on PerThreadRead (memory_operations.h:79-83; rawptr.h:203-213). */
void fko_bilinear_u8(const uint8_t* img, size_t pitch, int cn, int org_x, int org_y, int src_w, int src_h,
                     float sx, float sy, int quirk_y1_from_x, float* out) {
    const int x1 = (int)floorf(sx);
    const int y1 = quirk_y1_from_x ? (int)floorf(sx) : (int)floorf(sy);
    const int x2 = x1 + 1;
    const int y2 = y1 + 1;
    const int x2r = x2 < src_w - 1 ? x2 : src_w - 1;
    const int y2r = y2 < src_h - 1 ? y2 : src_h - 1;
    const uint8_t* r0 = img + (size_t)(org_y + y1) * pitch;
    const uint8_t* r1 = img + (size_t)(org_y + y2r) * pitch;
    const uint8_t* a = r0 + (size_t)(org_x + x1) * cn;
    const uint8_t* b = r0 + (size_t)(org_x + x2r) * cn;
    const uint8_t* c = r1 + (size_t)(org_x + x1) * cn;
    const uint8_t* d = r1 + (size_t)(org_x + x2r) * cn;
    const float wa = ((float)x2 - sx) * ((float)y2 - sy);
    const float wb = (sx - (float)x1) * ((float)y2 - sy);
    const float wc = ((float)x2 - sx) * (sy - (float)y1);
    const float wd = (sx - (float)x1) * (sy - (float)y1);
    for (int k = 0; k < cn; ++k) {
        const float t0 = (float)a[k] * wa;
        const float t1 = (float)b[k] * wb;
        const float t2 = (float)c[k] * wc;
        const float t3 = (float)d[k] * wd;
        out[k] = ((t0 + t1) + t2) + t3;
    }
}

/* SaturateCastBase<int,uchar>, algorithms/image_processing/saturate.h:35-53 */
uint8_t fko_saturate_int_to_u8(int v) { return v > 255 ? 255 : (v < 0 ? 0 : (uint8_t)v); }

/* SaturateCastBase<float,uchar>: clamp, then cxp::round */
uint8_t fko_saturate_float_to_u8(float v) {
    if (v > 255.0f) return 255;
    if (v < 0.0f) return 0;
    return (uint8_t)fko_round(v);
}

/* RGB2Gray<I,uchar>, algorithms/image_processing/color_conversion.h:47-77 (device branch rounds to nearest
 * even with __float2uint_rn, host branch with nearbyint: the same value). */
uint8_t fko_rgb2gray_u8(uint8_t x, uint8_t y, uint8_t z) {
    const float g = ((float)x * 0.299f + (float)y * 0.587f) + (float)z * 0.114f;
    return (uint8_t)nearbyintf(g);
}

/* Resize::exec, resize.h:75-87 and exec_resize :183-194, for one destination element.
 * Returns 0 and leaves `out` untouched when the element lies outside the PRESERVE_AR region. */
static int resize_sample_u8(const uint8_t* img, size_t pitch, int cn, int org_x, int org_y,
                            const fko_resize_params* p, int x, int y, int quirk, float* out) {
    if (x < p->x1 || x > p->x2 || y < p->y1 || y > p->y2) return 0;
    const int tx = x - p->x1, ty = y - p->y1;
    const float sx = (float)tx * p->fx;
    const float sy = (float)ty * p->fy;
    fko_bilinear_u8(img, pitch, cn, org_x, org_y, p->src_w, p->src_h, sx, sy, quirk, out);
    return 1;
}

/* ------------------------------------------------------------------ chains */

void fko_crop_resize_muls_bgr_tensor(const uint8_t* src, int src_w, int src_h, size_t src_pitch,
                                     const fko_rect* rects, int n, int dst_w, int dst_h, int aspect,
                                     const float background[3], const float mul[3], const float sub[3],
                                     const float div[3], int quirk, float* out) {
    (void)src_w;
    (void)src_h;
    for (int z = 0; z < n; ++z) {
        fko_resize_params p;
        fko_resize_build(aspect, rects[z].width, rects[z].height, dst_w, dst_h, &p);
        for (int y = 0; y < dst_h; ++y)
            for (int x = 0; x < dst_w; ++x) {
                float v[3];
                if (!resize_sample_u8(src, src_pitch, 3, rects[z].x, rects[z].y, &p, x, y, quirk, v)) {
                    v[0] = background[0];
                    v[1] = background[1];
                    v[2] = background[2];
                }
                for (int k = 0; k < 3; ++k) {
                    v[k] = v[k] * mul[k]; /* arithmetic.h:61-73 */
                    v[k] = v[k] - sub[k]; /* :47-59 */
                    v[k] = v[k] / div[k]; /* :75-87 */
                }
                /* VectorReorder<float3,2,1,0>, basic_ops/cuda_vector.h:49-62; TensorWrite, memory_operations.h:181-184 */
                float* o = out + (((size_t)z * dst_h + y) * dst_w + x) * 3;
                o[0] = v[2];
                o[1] = v[1];
                o[2] = v[0];
            }
    }
}

void fko_muladd_chain_f32c3(const float* src, int w, int h, size_t src_pitch, int depth, float mul_v,
                            float add_v, float* dst, size_t dst_pitch) {
    for (int y = 0; y < h; ++y) {
        const float* s = (const float*)((const char*)src + (size_t)y * src_pitch);
        float* d = (float*)((char*)dst + (size_t)y * dst_pitch);
        for (int i = 0; i < w * 3; ++i) {
            float v = s[i];
            for (int k = 0; k < depth; ++k) v = (k & 1) ? v + add_v : v * mul_v;
            d[i] = v;
        }
    }
}

void fko_single_op_f32c3(const float* src, int w, int h, size_t src_pitch, int is_add, float val, float* dst,
                         size_t dst_pitch) {
    for (int y = 0; y < h; ++y) {
        const float* s = (const float*)((const char*)src + (size_t)y * src_pitch);
        float* d = (float*)((char*)dst + (size_t)y * dst_pitch);
        for (int i = 0; i < w * 3; ++i) d[i] = is_add ? s[i] + val : s[i] * val;
    }
}

void fko_batch_crop_resize_norm_split(const uint8_t* const* srcs, int src_w, int src_h, size_t src_pitch,
                                      const fko_rect* rects, int n, int dst_w, int dst_h, const float div1[3],
                                      const float sub[3], const float div2[3], int quirk, float* out) {
    (void)src_w;
    (void)src_h;
    const size_t plane = (size_t)dst_w * dst_h;
    for (int z = 0; z < n; ++z) {
        fko_resize_params p;
        fko_resize_build(FKO_IGNORE_AR, rects[z].width, rects[z].height, dst_w, dst_h, &p);
        for (int y = 0; y < dst_h; ++y)
            for (int x = 0; x < dst_w; ++x) {
                float v[3];
                resize_sample_u8(srcs[z], src_pitch, 3, rects[z].x, rects[z].y, &p, x, y, quirk, v);
                for (int k = 0; k < 3; ++k) {
                    v[k] = v[k] / div1[k];
                    v[k] = v[k] - sub[k];
                    v[k] = v[k] / div2[k];
                }
                /* RGB2BGR then TensorSplit (memory_operations.h:203-219): channel c at + c*W*H elements,
                 * plane z at + z*color_planes*W*H (rawptr.h:216-226 with ptr_nd.h:85-104) */
                float* o = out + (size_t)z * 3 * plane + (size_t)y * dst_w + x;
                o[0] = v[2];
                o[plane] = v[1];
                o[2 * plane] = v[0];
            }
    }
}

void fko_resize_crop_tiles(const uint8_t* src, int src_w, int src_h, size_t src_pitch, int rs_w, int rs_h,
                           const fko_rect* rects, int n, int tile_w, int tile_h, const float mul[3], int quirk,
                           float* out) {
    fko_resize_params p;
    fko_resize_build(FKO_IGNORE_AR, src_w, src_h, rs_w, rs_h, &p);
    for (int z = 0; z < n; ++z)
        for (int y = 0; y < tile_h; ++y)
            for (int x = 0; x < tile_w; ++x) {
                float v[3];
                /* Crop over Resize: the resize is asked for thread + rect origin (crop.h:35-38) */
                const int rx = x + rects[z].x, ry = y + rects[z].y;
                const float sx = (float)rx * p.fx;
                const float sy = (float)ry * p.fy;
                fko_bilinear_u8(src, src_pitch, 3, 0, 0, p.src_w, p.src_h, sx, sy, quirk, v);
                float* o = out + (((size_t)z * tile_h + y) * tile_w + x) * 3;
                for (int k = 0; k < 3; ++k) o[k] = v[k] * mul[k];
            }
}

void fko_rgba2gray_u8c4(const uint8_t* src, int w, int h, size_t src_pitch, uint8_t* dst, size_t dst_pitch) {
    for (int y = 0; y < h; ++y) {
        const uint8_t* s = src + (size_t)y * src_pitch;
        uint8_t* d = dst + (size_t)y * dst_pitch;
        for (int x = 0; x < w; ++x) d[x] = fko_rgb2gray_u8(s[4 * x], s[4 * x + 1], s[4 * x + 2]);
    }
}

void fko_resize_mul_u8c4_f32c4(const uint8_t* src, int w, int h, size_t src_pitch, int dst_w, int dst_h,
                               float mul_v, int quirk, float* dst, size_t dst_pitch) {
    fko_resize_params p;
    fko_resize_build(FKO_IGNORE_AR, w, h, dst_w, dst_h, &p);
    for (int y = 0; y < dst_h; ++y) {
        float* d = (float*)((char*)dst + (size_t)y * dst_pitch);
        for (int x = 0; x < dst_w; ++x) {
            float v[4];
            resize_sample_u8(src, src_pitch, 4, 0, 0, &p, x, y, quirk, v);
            for (int k = 0; k < 4; ++k) d[4 * x + k] = v[k] * mul_v;
        }
    }
}

void fko_crop_mul_saturate_u8c4(const uint8_t* src, int w, int h, size_t src_pitch, fko_rect rect, int mul_v,
                                uint8_t* dst, size_t dst_pitch) {
    (void)w;
    (void)h;
    for (int y = 0; y < rect.height; ++y) {
        const uint8_t* s = src + (size_t)(y + rect.y) * src_pitch + (size_t)rect.x * 4;
        uint8_t* d = dst + (size_t)y * dst_pitch;
        /* Mul<uchar4,int,int4>: uchar*int -> int per channel (core/utils/cuda_vector_utils.h:499-554),
         * then SaturateCast<int4,uchar4> */
        for (int i = 0; i < rect.width * 4; ++i) d[i] = fko_saturate_int_to_u8((int)s[i] * mul_v);
    }
}

void fko_rgba2bgr_sub_u8c4_f32c3(const uint8_t* src, int w, int h, size_t src_pitch, float sub_v, float* dst,
                                 size_t dst_pitch) {
    for (int y = 0; y < h; ++y) {
        const uint8_t* s = src + (size_t)y * src_pitch;
        float* d = (float*)((char*)dst + (size_t)y * dst_pitch);
        for (int x = 0; x < w; ++x) {
            /* COLOR_RGBA2BGR: VectorReorder<uchar4,2,1,0,3> then Discard<uchar4,uchar3>
             * (color_conversion.h:555-613), Cast<uchar3,float3>, Sub<float3> */
            d[3 * x + 0] = (float)s[4 * x + 2] - sub_v;
            d[3 * x + 1] = (float)s[4 * x + 1] - sub_v;
            d[3 * x + 2] = (float)s[4 * x + 0] - sub_v;
        }
    }
}

void fko_batch_crop_cast_tensor(const uint8_t* src, int src_w, int src_h, size_t src_pitch, const fko_rect* rects,
                                int n, int max_w, int max_h, int exec_all, float* out) {
    (void)src_w;
    (void)src_h;
    for (int z = 0; z < n; ++z)
        for (int y = 0; y < max_h; ++y)
            for (int x = 0; x < max_w; ++x) {
                if (!exec_all && (x >= rects[z].width || y >= rects[z].height)) continue;
                const uint8_t* s = src + (size_t)(y + rects[z].y) * src_pitch + (size_t)(x + rects[z].x) * 3;
                float* o = out + (((size_t)z * max_h + y) * max_w + x) * 3;
                o[0] = (float)s[0];
                o[1] = (float)s[1];
                o[2] = (float)s[2];
            }
}

/* fk_oracle_border_warp.c — CPU restatement of the reference's BorderReader and Warping (see the header).
 *
 * TEST INFRASTRUCTURE ONLY.  Citations are paths below the reference's include/fused_kernel/.
 *
 * How each function is pinned (tests/test_oracle_border_warp.py):
 *   - fko_border_index / fko_border_crop_u8c3: the border diagrams printed in the reference's header
 *     (`fedcba|abcdefgh|hgfedcb` ...), periodicity and symmetry identities far outside the image, and the
 *     reference's own headers compiled for its CPU backend (oracle/_ref) on random images and windows;
 *   - fko_warp_coords / fko_warp_u8c3_f32c3: oracle/_ref with the literal host interpolation (quirk = 1);
 *     with quirk = 0: identity and integer translations (the output is the shifted image), agreement with the
 *     literal result wherever floor(x) == floor(y), the pure-scaling affine warp against the separately pinned
 *     resize sample fko_bilinear_u8, and a double-precision evaluation.
 *   - fko_deinterlace_u8c3_f32c3: the BLEND known answers of the reference's own unit test
 *     (utests/algorithm/image_processing/utest_deinterlace.h:24-45; its INTER_LINEAR tables hold the truncated
 *     values 2 and 1 where the operation's code yields 2.5 and 1.5, and the code is what is followed), oracle/_ref
 *     on random images, and closed forms (constant image, kept lines unchanged, numpy averages).
 */
#include "fk_oracle_border_warp.h"

#include <math.h>
#include <stdlib.h>

/* idx_row = idx_row_low(idx_row_high(y)), border_reader.h:159-277 */
int fko_border_index(int border_type, int i, int n) {
    const int last = n - 1;
    switch (border_type) {
    case FKO_BORDER_REPLICATE: { /* :159-186 */
        const int high = i < last ? i : last;
        return high > 0 ? high : 0;
    }
    case FKO_BORDER_REFLECT: { /* :188-216 */
        const int high = last - abs(last - i) + (i > last);
        return (abs(high) - (high < 0)) % (last + 1);
    }
    case FKO_BORDER_WRAP: { /* :218-250 */
        const int high = i < n ? i : i % n;
        return high >= 0 ? high : high - ((high - n + 1) / n) * n;
    }
    case FKO_BORDER_REFLECT_101: { /* :252-277 */
        const int high = abs(last - abs(last - i)) % (last + 1);
        return abs(high) % (last + 1);
    }
    default: /* CONSTANT, :141-157 */
        return (i >= 0 && i < n) ? i : -1;
    }
}

int fko_border_crop_u8c3(int border_type, const uint8_t* src, int w, int h, size_t src_pitch, int left, int top,
                         int dst_w, int dst_h, const uint8_t value[3], uint8_t* dst, size_t dst_pitch) {
    if (border_type < FKO_BORDER_CONSTANT || border_type > FKO_BORDER_REFLECT_101) return 1;
    for (int y = 0; y < dst_h; ++y)
        for (int x = 0; x < dst_w; ++x) {
            /* Crop::exec, crop.h:35-38: thread + rect origin */
            const int sx = fko_border_index(border_type, x - left, w);
            const int sy = fko_border_index(border_type, y - top, h);
            uint8_t* o = dst + (size_t)y * dst_pitch + (size_t)x * 3;
            if (sx < 0 || sy < 0) {
                o[0] = value[0], o[1] = value[1], o[2] = value[2];
            } else {
                const uint8_t* p = src + (size_t)sy * src_pitch + (size_t)sx * 3;
                o[0] = p[0], o[1] = p[1], o[2] = p[2];
            }
        }
    return 0;
}

/* WarpingCoords::exec, warping.h:51-68: int coordinates converted to float in each product */
void fko_warp_coords(int warp_type, const float* m, int x, int y, float out[2]) {
    const float fx = (float)x, fy = (float)y;
    const float xs = (m[0] * fx + m[1] * fy) + m[2];
    const float ys = (m[3] * fx + m[4] * fy) + m[5];
    if (warp_type == FKO_WARP_PERSPECTIVE) {
        const float coeff = 1.0f / ((m[6] * fx + m[7] * fy) + m[8]);
        out[0] = coeff * xs;
        out[1] = coeff * ys;
    } else {
        out[0] = xs;
        out[1] = ys;
    }
}

int fko_warp_u8c3_f32c3(int warp_type, const float* matrix, const uint8_t* src, int w, int h, size_t src_pitch,
                        int dst_w, int dst_h, int quirk_y1_from_x, float* dst, size_t dst_pitch) {
    if (warp_type != FKO_WARP_AFFINE && warp_type != FKO_WARP_PERSPECTIVE) return 1;
    for (int y = 0; y < dst_h; ++y) {
        float* row = (float*)((char*)dst + (size_t)y * dst_pitch);
        for (int x = 0; x < dst_w; ++x) {
            float c[2];
            fko_warp_coords(warp_type, matrix, x, y, c);
            float* o = row + (size_t)x * 3;
            /* Warping::exec, warping.h:84-94 */
            if (c[0] >= 0.f && c[0] < (float)w && c[1] >= 0.f && c[1] < (float)h) {
                fko_bilinear_u8(src, src_pitch, 3, 0, 0, w, h, c[0], c[1], quirk_y1_from_x, o);
            } else {
                o[0] = o[1] = o[2] = 0.f;
            }
        }
    }
    return 0;
}

/* Deinterlace::exec, deinterlace.h:53-126: integer sums of the promoted channels, + 1, times 0.5f */
int fko_deinterlace_u8c3_f32c3(int type, int use_even_lines, const uint8_t* src, int w, int h, size_t src_pitch, float* dst,
                               size_t dst_pitch) {
    if (type != FKO_DEINTERLACE_BLEND && type != FKO_DEINTERLACE_INTER_LINEAR) return 1;
    for (int y = 0; y < h; ++y) {
        const uint8_t* cur = src + (size_t)y * src_pitch;
        const uint8_t* above = y > 0 ? cur - src_pitch : cur;
        const uint8_t* below = y + 1 < h ? cur + src_pitch : cur;
        float* out = (float*)((char*)dst + (size_t)y * dst_pitch);
        int mode; /* 0 pass through, 1 current + above, 2 above + below */
        if (type == FKO_DEINTERLACE_BLEND) {
            mode = y > 0 ? 1 : 0; /* :97-104 */
        } else {                  /* :118-125 */
            const int odd = y & 1;
            /* the last line never interpolates: for an odd number of lines the reference's USE_ODD case reads the line
             * past the image there (it assumes an even number, deinterlace.h:112) */
            const int interpolate = y != h - 1 && (use_even_lines ? odd : (!odd && y != 0));
            mode = interpolate ? 2 : 0;
        }
        for (int i = 0; i < 3 * w; ++i) {
            if (mode == 0) out[i] = (float)cur[i] * 1.f;
            else if (mode == 1) out[i] = (float)((int)cur[i] + (int)above[i] + 1) * 0.5f;
            else out[i] = (float)((int)above[i] + (int)below[i] + 1) * 0.5f;
        }
    }
    return 0;
}

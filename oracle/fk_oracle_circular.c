/* fk_oracle_circular.c — CPU restatement of tensor layouts, circular reads and CircularTensor::update (see the header).
 *
 * TEST INFRASTRUCTURE ONLY.  Citations are paths below the reference's include/fused_kernel/.
 *
 * How each function is pinned (tests/test_oracle_circular.py):
 *   - fko_tensor_relayout_f32c3, fko_circular_tensor_read_f32c3: the reference's own headers compiled for its CPU
 *     backend (oracle/_ref), numpy transposes / rolls (the layouts are permutations), and round trips;
 *   - fko_circular_tensor_update_u8c3_split_f32: the reference cannot run CircularTensor::update (it has no executor
 *     for the divergent launch the method asks for), so this function is pinned by what the class is for: after any
 *     number of updates the tensor holds the chain's output for the last `batch` frames in age order (newest first or
 *     oldest first), and by composing the two sequences the method builds out of operations pinned above.
 */
#include "fk_oracle_circular.h"

/* packed (n,h,w,3): rawptr.h:216-226 with color_planes 1; split (n,3,h,w): memory_operations.h:203-219;
 * transposed (3,n,h,w): rawptr.h:228-239 */
static size_t packed_at(int w, int h, int z, int y, int x, int c) { return (((size_t)z * h + y) * w + x) * 3 + c; }
static size_t split_at(int w, int h, int z, int y, int x, int c) { return (((size_t)z * 3 + c) * h + y) * w + x; }
static size_t transposed_at(int w, int h, int n, int z, int y, int x, int c) { return (((size_t)c * n + z) * h + y) * w + x; }

int fko_tensor_relayout_f32c3(int mode, const float* src, int w, int h, int planes, float* dst) {
    if (mode < FKO_PACKED_TO_SPLIT || mode > FKO_TRANSPOSED_TO_PACKED) return 1;
    for (int z = 0; z < planes; ++z)
        for (int y = 0; y < h; ++y)
            for (int x = 0; x < w; ++x)
                for (int c = 0; c < 3; ++c) {
                    const size_t p = packed_at(w, h, z, y, x, c), s = split_at(w, h, z, y, x, c), t = transposed_at(w, h, planes, z, y, x, c);
                    switch (mode) {
                    case FKO_PACKED_TO_SPLIT: dst[s] = src[p]; break;       /* TensorSplit, memory_operations.h:195-226 */
                    case FKO_PACKED_TO_TRANSPOSED: dst[t] = src[p]; break;  /* TensorTSplit, :228-255 */
                    case FKO_SPLIT_TO_PACKED: dst[p] = src[s]; break;       /* TensorPack, :257-302 */
                    default: dst[p] = src[t]; break;                        /* TensorTPack, :304-348 */
                    }
                }
    return 0;
}

/* computeCircularThreadIdx, memory_operations.h:433-443 */
static int ring_slot(int direction, int z, int first, int planes) {
    if (direction == FKO_ASCENDENT) {
        const int s = z + first;
        return s >= planes ? s - planes : s;
    }
    const int s = first - z;
    return s < 0 ? planes + s : s;
}

int fko_circular_tensor_read_f32c3(int direction, int first, const float* ring, int w, int h, int planes, float* dst) {
    if (direction != FKO_ASCENDENT && direction != FKO_DESCENDENT) return 1;
    const size_t plane = (size_t)w * h * 3;
    for (int z = 0; z < planes; ++z) {
        const float* s = ring + (size_t)ring_slot(direction, z, first, planes) * plane;
        float* d = dst + (size_t)z * plane;
        for (size_t i = 0; i < plane; ++i) d[i] = s[i];
    }
    return 0;
}

int fko_circular_tensor_update_u8c3_split_f32(const uint8_t* frame, int w, int h, size_t pitch, float mul_v, float* tensor,
                                              float* ring, int batch, int next_index, int newest_first) {
    if (batch < 1 || next_index < 0 || next_index >= batch) return 1;
    const size_t plane = (size_t)w * h * 3;
    /* SequenceSelectorType::at, circular_tensor.h:26-35: which plane runs the new frame's chain */
    const int new_plane = newest_first ? 0 : batch - 1;
    /* sequence 1 (circular_tensor.h:118-124): chain -> CircularTensorWrite<Ascendent>(ring, first = next) -> write */
    const int new_slot = ring_slot(FKO_ASCENDENT, new_plane, next_index, batch);
    for (int y = 0; y < h; ++y)
        for (int x = 0; x < w; ++x)
            for (int c = 0; c < 3; ++c) {
                const float v = (float)frame[(size_t)y * pitch + (size_t)x * 3 + c] * mul_v; /* Cast, then Mul */
                ring[split_at(w, h, new_slot, y, x, c)] = v;
                tensor[split_at(w, h, new_plane, y, x, c)] = v;
            }
    /* sequence 2 (:126-131): CircularTensorRead<Descendent for NewestFirst | Ascendent>(ring, first = next) -> write */
    const int direction = newest_first ? FKO_DESCENDENT : FKO_ASCENDENT;
    for (int z = 0; z < batch; ++z) {
        if (z == new_plane) continue;
        const float* s = ring + (size_t)ring_slot(direction, z, next_index, batch) * plane;
        float* d = tensor + (size_t)z * plane;
        for (size_t i = 0; i < plane; ++i) d[i] = s[i];
    }
    return 0;
}

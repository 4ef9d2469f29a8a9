// Host-only check of the launch plans that Executor builds (fk::exec::JobOf::make): no GPU call is made and no device memory
// is touched; the pointers are made up.  Compiled by hipcc for the host only.
#include <cstdio>
#include <vector>

#include "fk/fused_kernel.h"

using namespace fk;

namespace {
int failures = 0;
#define CHECK(cond)                                               \
    do {                                                          \
        if (!(cond)) {                                            \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond); \
            ++failures;                                           \
        }                                                         \
    } while (0)

template <typename T>
RawPtr<ND::_2D, T> image(size_t address, uint w, uint h, uint pitch) {
    return RawPtr<ND::_2D, T>{ reinterpret_cast<T*>(address), PtrDims<ND::_2D>(w, h, pitch) };
}

// a three-byte source whose window spans 4 GiB or more must not be addressed with 32-bit offsets: no tile is staged, no
// line is touched, the taps are read with 64-bit row addresses
void huge_windows_keep_64_bit_addressing() {
    const auto write = PerThreadWrite<ND::_2D, float3>::build(image<float3>(0x7000000000ull, 1000, 800, 12000));
    {
        const auto read = PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(0x1000000000ull, 40000, 40000, 120000))
                              .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(1000, 800)));
        const auto job = exec::JobOf<std::decay_t<decltype(read)>, std::decay_t<decltype(write)>>::make(read, write);
        CHECK((job.flags & exec::FLAG_OFFSETS_32) == 0u);
        CHECK((job.flags & (exec::FLAG_SOURCE_TILE | exec::FLAG_PACKED_TILE)) == 0u);
        CHECK(job.lds_bytes() == 0u);
    }
    {   // up-scaling from a huge source: the tile of float taps would be worth it, and is still refused
        const auto read = PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(0x1000000000ull, 40000, 40000, 120000))
                              .then(Crop<>::build(Rect(10, 10, 500, 39000)))
                              .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(1000, 800)));
        const auto job = exec::JobOf<std::decay_t<decltype(read)>, std::decay_t<decltype(write)>>::make(read, write);
        CHECK((job.flags & exec::FLAG_OFFSETS_32) == 0u);
        CHECK((job.flags & (exec::FLAG_SOURCE_TILE | exec::FLAG_PACKED_TILE)) == 0u);
    }
    {   // the same chains over an ordinary frame take the tiles
        const auto up = PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(0x1000000000ull, 3840, 2160, 11520))
                            .then(Crop<>::build(Rect(0, 0, 500, 400)))
                            .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(1000, 800)));
        const auto job = exec::JobOf<std::decay_t<decltype(up)>, std::decay_t<decltype(write)>>::make(up, write);
        CHECK((job.flags & exec::FLAG_OFFSETS_32) != 0u);
        CHECK((job.flags & exec::FLAG_SOURCE_TILE) != 0u);
        const auto down = PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(0x1000000000ull, 1500, 1200, 4500))
                              .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(1000, 800)));
        const auto job2 = exec::JobOf<std::decay_t<decltype(down)>, std::decay_t<decltype(write)>>::make(down, write);
        CHECK((job2.flags & exec::FLAG_PACKED_TILE) != 0u && job2.lds_bytes() > 0u);
        // a source that does not start at a whole dword, or whose rows are not whole dwords apart: no packed tile
        const auto odd = PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(0x1000000001ull, 1500, 1200, 4500))
                             .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(1000, 800)));
        const auto job3 = exec::JobOf<std::decay_t<decltype(odd)>, std::decay_t<decltype(write)>>::make(odd, write);
        CHECK((job3.flags & exec::FLAG_PACKED_TILE) == 0u);
        const auto odd_pitch = PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(0x1000000000ull, 1500, 1200, 4501))
                                   .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(1000, 800)));
        const auto job4 = exec::JobOf<std::decay_t<decltype(odd_pitch)>, std::decay_t<decltype(write)>>::make(odd_pitch, write);
        CHECK((job4.flags & exec::FLAG_PACKED_TILE) == 0u);
    }
}

// which launches fill their tiles of float taps from aligned groups of four pixels: three-byte images with dword-aligned
// rows, 64 x 32 tiles (launches of 1024 tiles and more), boxes of at most one group per thread
void tiles_are_filled_from_groups_of_four_where_planned() {
    const auto write = PerThreadWrite<ND::_2D, float3>::build(image<float3>(0x7000000000ull, 2880, 2160, 34560));
    const auto chain = [&](size_t address, uint pitch, const Rect& crop, const Size& to) {
        return PerThreadRead<ND::_2D, uchar3>::build(image<uchar3>(address, 3840, 2160, pitch)).then(Crop<>::build(crop)).then(
            Resize<InterpolationType::INTER_LINEAR>::build(to));
    };
    const auto flags_of = [&](const auto& read) { return exec::JobOf<std::decay_t<decltype(read)>, std::decay_t<decltype(write)>>::make(read, write); };
    // 1024x576 -> 2048x1152 (1152 tiles of 64 x 32): 34 x 18 source pixels per tile, ten groups per row, 180 groups
    const auto wide = flags_of(chain(0x1000000000ull, 11520, Rect(8, 8, 1024, 576), Size(2048, 1152)));
    CHECK(wide.wave_rows == 8u && (wide.flags & exec::FLAG_QUAD_FILL) != 0u && (wide.flags & exec::FLAG_SOURCE_TILE) != 0u);
    // 2048x1536 -> 2880x2160 (the factors of the headline's planes): 47 x 25 source pixels per tile, 325 groups: one pixel per thread
    const auto headline = flags_of(chain(0x1000000000ull, 11520, Rect(8, 8, 2048, 1536), Size(2880, 2160)));
    CHECK(headline.wave_rows == 8u && (headline.flags & exec::FLAG_QUAD_FILL) == 0u && (headline.flags & exec::FLAG_SOURCE_TILE) != 0u);
    // a small output: 64 x 16 tiles, one pixel per thread
    const auto small = flags_of(chain(0x1000000000ull, 11520, Rect(8, 8, 100, 60), Size(224, 224)));
    CHECK(small.wave_rows == 4u && (small.flags & exec::FLAG_QUAD_FILL) == 0u && (small.flags & exec::FLAG_SOURCE_TILE) != 0u);
    // rows that are not a whole number of dwords apart, an image that does not start at a whole dword
    CHECK((flags_of(chain(0x1000000000ull, 11521, Rect(8, 8, 1024, 576), Size(2048, 1152))).flags & exec::FLAG_QUAD_FILL) == 0u);
    CHECK((flags_of(chain(0x1000000002ull, 11520, Rect(8, 8, 1024, 576), Size(2048, 1152))).flags & exec::FLAG_QUAD_FILL) == 0u);
}

// a batch of windows of different sizes: every plane gets the extent of the batch's thread grid, and the wide (several
// pixels per thread) path only where the rows below the first are aligned too
void ragged_batches_take_their_alignment_from_the_whole_box() {
    // rows 131 bytes apart: a one-row window alone may use the wide path, the same window inside a taller box may not
    const auto source = image<uchar3>(0x1000000000ull, 41, 60, 131);
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(source);
    const auto plane = [&](const Rect& r) { return read.then(Crop<>::build(r)).then(Cast<uchar3, float3>::build()); };
    using Plane = decltype(plane(Rect()));
    const std::vector<Plane> planes{ plane(Rect(4, 7, 32, 1)), plane(Rect(0, 0, 16, 9)), plane(Rect(8, 20, 32, 5)) };
    const auto out = TensorWrite<float3>::build(RawPtr<ND::_3D, float3>{ reinterpret_cast<float3*>(0x7000000000ull), PtrDims<ND::_3D>(36, 12, 3, 1, 36 * 12) });
    const auto batch = BatchRead<8>::build_first(planes.data(), planes.size());
    const auto job = exec::JobOf<std::decay_t<decltype(batch)>, std::decay_t<decltype(out)>>::make(batch, out);
    for (int i = 0; i < 3; ++i) {
        CHECK(job.plane[i].prog.view.w == 32 && job.plane[i].prog.view.h == 9);
        CHECK((job.plane[i].flags & exec::FLAG_WHOLE_BOX) != 0u);
        CHECK((job.plane[i].flags & exec::FLAG_VECTOR_IO) == 0u); // 131-byte rows: no wide accesses below the first row
    }
    // alone, the one-row window is not ragged and keeps its own extent
    const auto single = BatchRead<8>::build_first(planes.data(), 1);
    const auto job1 = exec::JobOf<std::decay_t<decltype(single)>, std::decay_t<decltype(out)>>::make(single, out);
    CHECK(job1.plane[0].prog.view.w == 32 && job1.plane[0].prog.view.h == 1 && (job1.plane[0].flags & exec::FLAG_WHOLE_BOX) == 0u);
    // a part of a larger batch carries the whole batch's box
    const auto part = BatchRead<8>::build_first(planes.data() + 1, 2, 40, 11);
    const auto job2 = exec::JobOf<std::decay_t<decltype(part)>, std::decay_t<decltype(out)>>::make(part, out);
    for (int i = 0; i < 2; ++i) {
        CHECK(job2.plane[i].prog.view.w == 40 && job2.plane[i].prog.view.h == 11 && (job2.plane[i].flags & exec::FLAG_WHOLE_BOX) != 0u);
    }
}

// The dealing of tiles to launch positions is a permutation for every count, and puts the tiles 2k and 2k + 1 on launch
// positions that are 8 apart (the same XCD) wherever the count leaves room for it.
void tile_pairs_are_a_permutation_with_neighbours_eight_apart() {
    for (unsigned n = 1; n < 300; ++n) {
        std::vector<int> position(n, -1);
        for (unsigned l = 0; l < n; ++l) {
            const unsigned t = exec::dev::deal_pairs(l, n);
            CHECK(t < n && position[t < n ? t : 0] < 0);
            if (t < n) position[t] = static_cast<int>(l);
        }
        unsigned together = 0;
        for (unsigned t = 0; t + 1 < n; t += 2) together += (position[t + 1] - position[t] == 8) ? 1u : 0u;
        const unsigned last = n & 15u;
        CHECK(together == (n >> 4) * 8u + (last > 8u ? last - 8u : 0u));
    }
}
} // namespace

int main() {
    huge_windows_keep_64_bit_addressing();
    tile_pairs_are_a_permutation_with_neighbours_eight_apart();
    tiles_are_filled_from_groups_of_four_where_planned();
    ragged_batches_take_their_alignment_from_the_whole_box();
    if (failures == 0) std::printf("host plans: ok\n");
    return failures == 0 ? 0 : 1;
}

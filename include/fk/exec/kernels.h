// The fused Transform kernels for gfx950 (CDNA4, wave64), hand-written against the views of fk/exec/views.h.
//
// Every launch runs blocks of 256 threads (four wave64).  A "job" is one fused chain over all its planes:
//   PointwiseJob  element-wise chains over a PlainView: each thread owns K consecutive pixels of a row so that both the
//                 source and the destination bytes of a thread are whole 16-byte (or 8/4-byte) transactions;
//   ResizeJob     bilinear resize (with optional inner/outer crop and aspect-ratio border): a block owns a 32x8 output
//                 tile, stages the source bounding box of the tile in LDS with coalesced dword loads and takes the
//                 2x2 taps from LDS; tiles whose bounding box does not fit (strong down-scaling, no tap reuse) read
//                 their taps straight from memory;
//   GenericJob    one thread per output element through Operation::exec, for any chain the views cannot describe.
// blockIdx.z selects the plane of a batch; blocks that start outside their plane's own extent return at once.
// What one thread computes per element is the reference's TransformDPP::exec -> read -> compute... -> write
// (core/execution_model/data_parallel_patterns.h:120-181,254-268); the traversal, vector widths and LDS staging
// are this library's.  Build with -ffp-contract=off: results are compared bit for bit with an unfused evaluation.
#ifndef FK_EXEC_KERNELS_H
#define FK_EXEC_KERNELS_H

#include "fk/exec/views.h"

// clang emits a host-side stub for every __global__ function that refers to this runtime entry point; kernels are
// launched through fkrt_launch (which calls it with the stub's address), so only the declaration is needed here.
struct fk_launch_dim3 {
    unsigned x, y, z;
};
extern "C" int hipLaunchKernel(const void* function_address, fk_launch_dim3 grid, fk_launch_dim3 block, void** args,
                               size_t lds_bytes, struct ihipStream_t* stream);

namespace fk {
namespace exec {

constexpr int BLOCK_THREADS = 256;

namespace dev {
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ inline int thread_in_block() { return static_cast<int>(__builtin_amdgcn_workitem_id_x()); }
__device__ inline void block_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

constexpr int gcd(int a, int b) { return b == 0 ? a : gcd(b, a % b); }
// widest transaction (16, 8 or 4 bytes) that tiles NBYTES
constexpr int chunk_bytes(int nbytes) { return gcd(nbytes, 16); }

// NBYTES (a multiple of 4) from `p`, which is aligned to chunk_bytes(NBYTES)
template <int NBYTES>
__device__ inline void load_words(const void* p, unsigned int* w) {
    constexpr int C = chunk_bytes(NBYTES);
    static_assert(NBYTES % 4 == 0 && C >= 4, "vector I/O moves whole dwords");
    if constexpr (C == 16) {
#pragma unroll
        for (int i = 0; i < NBYTES / 16; ++i) {
            const u32x4 v = static_cast<const u32x4*>(p)[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
    } else if constexpr (C == 8) {
#pragma unroll
        for (int i = 0; i < NBYTES / 8; ++i) {
            const u32x2 v = static_cast<const u32x2*>(p)[i];
            w[2 * i] = v.x; w[2 * i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < NBYTES / 4; ++i) w[i] = static_cast<const unsigned int*>(p)[i];
    }
}
// STREAM: non-temporal stores.  Only for accesses where a wave writes whole cache lines (consecutive lanes,
// consecutive 16/8/4-byte pieces): they then leave the caches alone and measurably raise the write bandwidth;
// on partial lines they are a pessimisation.
template <bool STREAM, typename V>
__device__ inline void store_piece(V* p, const V& v) {
    if constexpr (STREAM) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}
template <int NBYTES, bool STREAM = false>
__device__ inline void store_words(void* p, const unsigned int* w) {
    constexpr int C = chunk_bytes(NBYTES);
    static_assert(NBYTES % 4 == 0 && C >= 4, "vector I/O moves whole dwords");
    if constexpr (C == 16) {
#pragma unroll
        for (int i = 0; i < NBYTES / 16; ++i) {
            u32x4 v;
            v.x = w[4 * i]; v.y = w[4 * i + 1]; v.z = w[4 * i + 2]; v.w = w[4 * i + 3];
            store_piece<STREAM>(static_cast<u32x4*>(p) + i, v);
        }
    } else if constexpr (C == 8) {
#pragma unroll
        for (int i = 0; i < NBYTES / 8; ++i) {
            u32x2 v;
            v.x = w[2 * i]; v.y = w[2 * i + 1];
            store_piece<STREAM>(static_cast<u32x2*>(p) + i, v);
        }
    } else {
#pragma unroll
        for (int i = 0; i < NBYTES / 4; ++i) store_piece<STREAM>(static_cast<unsigned int*>(p) + i, w[i]);
    }
}

template <typename Tail, typename V>
__device__ inline auto apply_tail(const Tail& tail, const V& v) {
    if constexpr (std::is_same_v<Tail, NoTail>) {
        return v;
    } else {
        return fk::detail::tuple_compute(v, tail);
    }
}

template <typename O>
__device__ inline void store_one(const PackedOut<O>& out, int x, int y, int z, const O& v) {
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
    reinterpret_cast<O*>(row)[x] = v;
}
template <typename O>
__device__ inline void store_one(const SplitOut<O>& out, int x, int y, int z, const O& v) {
    using B = VBase<O>;
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
    reinterpret_cast<B*>(row)[x] = v.x;
    reinterpret_cast<B*>(row + out.chan_stride)[x] = v.y;
    if constexpr (cn<O> >= 3) reinterpret_cast<B*>(row + 2 * out.chan_stride)[x] = v.z;
    if constexpr (cn<O> == 4) reinterpret_cast<B*>(row + 3 * out.chan_stride)[x] = v.w;
}

// K consecutive pixels starting at x0 (caller guarantees the alignment that chunk_bytes asks for)
template <int K, bool STREAM = false, typename O>
__device__ inline void store_group(const PackedOut<O>& out, int x0, int y, int z, const O* v) {
    constexpr int NB = K * static_cast<int>(sizeof(O));
    unsigned int w[NB / 4];
    __builtin_memcpy(w, v, NB);
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
    // a thread's K pixels are one transaction only when they fill exactly one piece
    store_words<NB, STREAM && NB == chunk_bytes(NB)>(row + static_cast<size_t>(x0) * sizeof(O), w);
}
template <int K, bool STREAM = false, typename O>
__device__ inline void store_group(const SplitOut<O>& out, int x0, int y, int z, const O* v) {
    using B = VBase<O>;
    constexpr int NB = K * static_cast<int>(sizeof(B));
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
#pragma unroll
    for (int c = 0; c < cn<O>; ++c) {
        B ch[K];
#pragma unroll
        for (int k = 0; k < K; ++k) ch[k] = vectorAt(c, v[k]);
        unsigned int w[NB / 4];
        __builtin_memcpy(w, ch, NB);
        store_words<NB, STREAM && NB == chunk_bytes(NB)>(row + c * out.chan_stride + static_cast<size_t>(x0) * sizeof(B), w);
    }
}
} // namespace dev

// Pixels per thread: the smallest power of two that makes the wider side a whole number of 16-byte transactions and
// the narrower side a whole number of dwords.
template <typename S, typename O, bool SPLIT>
constexpr int pixels_per_thread() {
    const int ss = static_cast<int>(sizeof(S));
    const int so = SPLIT ? static_cast<int>(sizeof(VBase<O>)) : static_cast<int>(sizeof(O));
    const int big = ss > so ? ss : so, small = ss > so ? so : ss;
    for (int k = 1; k <= 16; k *= 2) {
        if ((k * big) % 16 == 0 && (k * small) % 4 == 0) return k;
    }
    return 16;
}

// ---- pointwise ---------------------------------------------------------------------------------------------------
enum : unsigned { FLAG_VECTOR_IO = 1u, FLAG_STREAM_STORES = 2u };

template <typename Prog, size_t N, typename Out>
struct PointwiseJob {
    using View = decltype(Prog::view);
    using Src = typename View::Source;
    using OutPixel = typename Out::Pixel;
    static constexpr int K = pixels_per_thread<Src, OutPixel, Out::IS_SPLIT>();
    static constexpr int IN_BYTES = K * static_cast<int>(sizeof(Src));
    static constexpr int OUT_BYTES = Out::IS_SPLIT ? K * static_cast<int>(sizeof(VBase<OutPixel>)) : K * static_cast<int>(sizeof(OutPixel));
    // A thread's K pixels span more than one 16-byte transaction when pixels are 12 bytes wide (48 bytes per thread).
    // Lanes reading 48-byte runs touch every cache line three times; instead the block moves its contiguous
    // 256*K-pixel span with fully coalesced 16-byte accesses and redistributes pixels to threads through LDS.
    static constexpr bool STAGE_IN = IN_BYTES > 16 && IN_BYTES % 16 == 0;
    static constexpr bool STAGE_OUT = !Out::IS_SPLIT && OUT_BYTES > 16 && OUT_BYTES % 16 == 0;
    static constexpr int STAGE_BYTES = (STAGE_IN && STAGE_OUT) ? (IN_BYTES > OUT_BYTES ? IN_BYTES : OUT_BYTES)
                                       : STAGE_IN              ? IN_BYTES
                                       : STAGE_OUT             ? OUT_BYTES
                                                               : 0;
    static constexpr int LDS_BYTES = BLOCK_THREADS * STAGE_BYTES;
    static constexpr bool READ_IN_PLACE = N > 1 || sizeof(Prog) > 512; // run-time plane index, or a very long chain
    struct Plane {
        Prog prog;
        unsigned flags;
    };
    Plane plane[N];
    Out out;
    unsigned tx_shift; // log2 of the thread columns of a block; the other threads cover further rows
    unsigned grid_x, grid_y;

    __device__ static inline void run(const PointwiseJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char* lds) {
        const Plane& pl = job.plane[N == 1 ? 0u : bz];
        const View& v = pl.prog.view;
        const int tid = dev::thread_in_block();
        const int cols = 1 << job.tx_shift;
        const int x0 = (static_cast<int>(bx) * cols + (tid & (cols - 1))) * K;
        const int y = static_cast<int>(by) * (BLOCK_THREADS >> job.tx_shift) + (tid >> job.tx_shift);

        if constexpr (STAGE_IN || STAGE_OUT) {
            // block-uniform: the whole block lies on one row and its 256*K pixels are all inside the plane
            const bool whole = (pl.flags & FLAG_VECTOR_IO) != 0u && job.tx_shift == 8u && y < v.h &&
                               (static_cast<int>(bx) + 1) * BLOCK_THREADS * K <= v.w;
            if (whole) {
                const int bx0 = static_cast<int>(bx) * BLOCK_THREADS * K; // first pixel of the block
                dev::u32x4* const stage = reinterpret_cast<dev::u32x4*>(lds);
                Src in[K];
                if constexpr (STAGE_IN) {
                    const dev::u32x4* const g = reinterpret_cast<const dev::u32x4*>(
                        reinterpret_cast<const char*>(v.data) + static_cast<size_t>(v.oy + y) * v.pitch +
                        static_cast<size_t>(v.ox + bx0) * sizeof(Src));
#pragma unroll
                    for (int j = 0; j < IN_BYTES / 16; ++j) stage[j * BLOCK_THREADS + tid] = g[j * BLOCK_THREADS + tid];
                    dev::block_sync();
                    dev::u32x4 mine[IN_BYTES / 16];
#pragma unroll
                    for (int j = 0; j < IN_BYTES / 16; ++j) mine[j] = stage[tid * (IN_BYTES / 16) + j];
                    __builtin_memcpy(in, mine, IN_BYTES);
                } else {
                    const char* const srow = reinterpret_cast<const char*>(v.data) + static_cast<size_t>(v.oy + y) * v.pitch +
                                             static_cast<size_t>(v.ox) * sizeof(Src);
                    unsigned int w[IN_BYTES / 4];
                    dev::load_words<IN_BYTES>(srow + static_cast<size_t>(x0) * sizeof(Src), w);
                    __builtin_memcpy(in, w, IN_BYTES);
                }
                OutPixel o[K];
#pragma unroll
                for (int k = 0; k < K; ++k) o[k] = dev::apply_tail(pl.prog.tail, in[k]);
                if constexpr (STAGE_OUT) {
                    if constexpr (STAGE_IN) dev::block_sync(); // every thread has taken its input out of the buffer
                    dev::u32x4 mine[OUT_BYTES / 16];
                    __builtin_memcpy(mine, o, OUT_BYTES);
#pragma unroll
                    for (int j = 0; j < OUT_BYTES / 16; ++j) stage[tid * (OUT_BYTES / 16) + j] = mine[j];
                    dev::block_sync();
                    dev::u32x4* const g = reinterpret_cast<dev::u32x4*>(
                        reinterpret_cast<char*>(job.out.data) + static_cast<size_t>(bz) * job.out.z_stride +
                        static_cast<size_t>(y) * job.out.pitch + static_cast<size_t>(bx0) * sizeof(OutPixel));
                    if ((pl.flags & FLAG_STREAM_STORES) != 0u) {
#pragma unroll
                        for (int j = 0; j < OUT_BYTES / 16; ++j) dev::store_piece<true>(g + j * BLOCK_THREADS + tid, stage[j * BLOCK_THREADS + tid]);
                    } else {
#pragma unroll
                        for (int j = 0; j < OUT_BYTES / 16; ++j) g[j * BLOCK_THREADS + tid] = stage[j * BLOCK_THREADS + tid];
                    }
                } else {
                    if ((pl.flags & FLAG_STREAM_STORES) != 0u) dev::store_group<K, true>(job.out, x0, y, static_cast<int>(bz), o);
                    else dev::store_group<K>(job.out, x0, y, static_cast<int>(bz), o);
                }
                return;
            }
        }

        if (y >= v.h || x0 >= v.w) return; // also ends blocks that lie outside a smaller plane of a ragged batch
        const char* const srow = reinterpret_cast<const char*>(v.data) + static_cast<size_t>(v.oy + y) * v.pitch +
                                 static_cast<size_t>(v.ox) * sizeof(Src);
        if ((pl.flags & FLAG_VECTOR_IO) != 0u && x0 + K <= v.w) {
            unsigned int w[IN_BYTES / 4];
            dev::load_words<IN_BYTES>(srow + static_cast<size_t>(x0) * sizeof(Src), w);
            Src in[K];
            __builtin_memcpy(in, w, IN_BYTES);
            OutPixel o[K];
#pragma unroll
            for (int k = 0; k < K; ++k) o[k] = dev::apply_tail(pl.prog.tail, in[k]);
            if ((pl.flags & FLAG_STREAM_STORES) != 0u) dev::store_group<K, true>(job.out, x0, y, static_cast<int>(bz), o);
            else dev::store_group<K>(job.out, x0, y, static_cast<int>(bz), o);
        } else {
            const int xe = x0 + K < v.w ? x0 + K : v.w;
            for (int x = x0; x < xe; ++x) {
                const OutPixel o = dev::apply_tail(pl.prog.tail, reinterpret_cast<const Src*>(srow)[x]);
                dev::store_one(job.out, x, y, static_cast<int>(bz), o);
            }
        }
    }
};

// ---- resize ------------------------------------------------------------------------------------------------------
constexpr int RESIZE_TILE_W = 32;
constexpr int RESIZE_TILE_H = 8;
constexpr int RESIZE_LDS_DWORDS = 4096;

namespace dev {
// sizeof(T) bytes at byte offset `off` of a dword array in LDS
template <typename T>
__device__ inline T lds_pixel(const unsigned int* tile, unsigned off) {
    constexpr int ND = (static_cast<int>(sizeof(T)) + 3) / 4;
    const unsigned int* const p = tile + (off >> 2);
    const unsigned sh = off & 3u;
    unsigned int w[ND];
    if constexpr (sizeof(T) % 4 == 0 && alignof(T) % 4 == 0) {
#pragma unroll
        for (int i = 0; i < ND; ++i) w[i] = p[i]; // such pixels only ever sit at dword offsets
    } else {
#pragma unroll
        for (int i = 0; i < ND; ++i) w[i] = __builtin_amdgcn_alignbyte(p[i + 1], p[i], sh);
    }
    T out;
    __builtin_memcpy(&out, w, sizeof(T));
    return out;
}
} // namespace dev

template <typename Prog, size_t N, typename Out>
struct ResizeJob {
    using View = decltype(Prog::view);
    using Src = typename View::Source;
    using Pixel = typename View::Pixel;
    using OutPixel = typename Out::Pixel;
    static constexpr int LDS_BYTES = (RESIZE_LDS_DWORDS + 2) * 4;
    static constexpr bool READ_IN_PLACE = N > 1;
    Prog plane[N];
    Out out;
    unsigned grid_x, grid_y;

    __device__ static inline void run(const ResizeJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char* lds_raw) {
        const Prog& prog = job.plane[N == 1 ? 0u : bz];
        const View& v = prog.view;
        const PlainView<Src>& s = v.src;
        const int tx0 = static_cast<int>(bx) * RESIZE_TILE_W;
        const int ty0 = static_cast<int>(by) * RESIZE_TILE_H;
        if (tx0 >= v.w || ty0 >= v.h) return; // block outside this plane's own extent
        const int tid = dev::thread_in_block();
        const int x = tx0 + (tid & (RESIZE_TILE_W - 1));
        const int y = ty0 + (tid / RESIZE_TILE_W);

        // part of the tile that resamples the source, in resize coordinates (after the outer crop offset)
        int rx_lo = tx0 + v.off_x, rx_hi = (tx0 + RESIZE_TILE_W < v.w ? tx0 + RESIZE_TILE_W : v.w) - 1 + v.off_x;
        int ry_lo = ty0 + v.off_y, ry_hi = (ty0 + RESIZE_TILE_H < v.h ? ty0 + RESIZE_TILE_H : v.h) - 1 + v.off_y;
        if constexpr (View::HAS_ROI) {
            rx_lo = rx_lo > v.x1 ? rx_lo : v.x1;
            rx_hi = rx_hi < v.x2 ? rx_hi : v.x2;
            ry_lo = ry_lo > v.y1 ? ry_lo : v.y1;
            ry_hi = ry_hi < v.y2 ? ry_hi : v.y2;
        }
        const bool resamples = rx_lo <= rx_hi && ry_lo <= ry_hi;

        unsigned int* const tile = reinterpret_cast<unsigned int*>(lds_raw);
        bool staged = false;
        int sx_lo = 0, sy_lo = 0;
        unsigned stride_dw = 0;
        const unsigned base_lo = static_cast<unsigned>(reinterpret_cast<size_t>(s.data));
#ifndef FK_INTERPOLATE_Y1_FROM_X
        if (resamples) {
            // source bounding box of the tile: taps are floor(c) and min(floor(c) + 1, limit) for c in [lo, hi] * f
            sx_lo = fk::detail::floor_to_int((rx_lo - v.x1) * v.fx);
            sy_lo = fk::detail::floor_to_int((ry_lo - v.y1) * v.fy);
            int sx_hi = fk::detail::floor_to_int((rx_hi - v.x1) * v.fx) + 1;
            int sy_hi = fk::detail::floor_to_int((ry_hi - v.y1) * v.fy) + 1;
            sx_hi = sx_hi < s.w - 1 ? sx_hi : s.w - 1;
            sy_hi = sy_hi < s.h - 1 ? sy_hi : s.h - 1;
            sx_lo = sx_lo < sx_hi ? sx_lo : sx_hi;
            sy_lo = sy_lo < sy_hi ? sy_lo : sy_hi;
            const int rows = sy_hi - sy_lo + 1;
            const unsigned row_bytes = static_cast<unsigned>(sx_hi - sx_lo + 1) * sizeof(Src);
            stride_dw = ((row_bytes + 3u) >> 2) + 1u; // + up to 3 bytes of misalignment at the row start
            stride_dw |= 1u;                          // odd stride spreads rows over the LDS banks
            staged = static_cast<unsigned>(rows) * stride_dw <= static_cast<unsigned>(RESIZE_LDS_DWORDS);
            if (staged) {
                const int wave = tid >> 6, lane = tid & 63;
                const long valid_lo = -static_cast<long>(s.ox) * static_cast<long>(sizeof(Src));
                const long valid_hi = static_cast<long>(s.img_w - s.ox) * static_cast<long>(sizeof(Src));
                for (int r = wave; r < rows; r += BLOCK_THREADS / 64) {
                    const size_t row_off = static_cast<size_t>(s.oy + sy_lo + r) * s.pitch + static_cast<size_t>(s.ox) * sizeof(Src);
                    const char* const row = reinterpret_cast<const char*>(s.data) + row_off; // window x = 0 of this row
                    const long first = static_cast<long>(sx_lo) * static_cast<long>(sizeof(Src));
                    const unsigned mis = (base_lo + static_cast<unsigned>(row_off) + static_cast<unsigned>(first)) & 3u;
                    const unsigned need = (mis + row_bytes + 3u) >> 2;
                    for (unsigned c = static_cast<unsigned>(lane); c < need; c += 64u) {
                        const long b = first - static_cast<long>(mis) + 4l * static_cast<long>(c); // byte offset in the window row
                        unsigned int word;
                        if (b >= valid_lo && b + 4 <= valid_hi) {
                            word = *reinterpret_cast<const unsigned int*>(row + b);
                        } else { // dword straddles the end of the parent image row: take only the bytes that exist
                            word = 0u;
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                if (b + k >= valid_lo && b + k < valid_hi) {
                                    word |= static_cast<unsigned int>(static_cast<unsigned char>(row[b + k])) << (8 * k);
                                }
                            }
                        }
                        tile[static_cast<unsigned>(r) * stride_dw + c] = word;
                    }
                }
            }
        }
#endif
        dev::block_sync();
        if (x >= v.w || y >= v.h) return;

        Pixel value;
        const int rx = x + v.off_x, ry = y + v.off_y;
        bool inside = true;
        if constexpr (View::HAS_ROI) inside = rx >= v.x1 && rx <= v.x2 && ry >= v.y1 && ry <= v.y2;
        if (inside) {
            const float src_x = (rx - v.x1) * v.fx;
            const float src_y = (ry - v.y1) * v.fy;
            const fk::detail::BilinearTaps t = fk::detail::bilinear_taps(src_x, src_y, Size(s.w, s.h));
            Src a, b, c, d;
            if (staged) {
                const unsigned row0 = static_cast<unsigned>(t.y1 - sy_lo), row1 = static_cast<unsigned>(t.y2r - sy_lo);
                const unsigned first = static_cast<unsigned>(sx_lo) * static_cast<unsigned>(sizeof(Src));
                const unsigned org = base_lo + static_cast<unsigned>(s.ox) * static_cast<unsigned>(sizeof(Src)) + first;
                const unsigned mis0 = (org + static_cast<unsigned>(s.oy + t.y1) * s.pitch) & 3u;
                const unsigned mis1 = (org + static_cast<unsigned>(s.oy + t.y2r) * s.pitch) & 3u;
                const unsigned xa = static_cast<unsigned>(t.x1 - sx_lo) * static_cast<unsigned>(sizeof(Src));
                const unsigned xb = static_cast<unsigned>(t.x2r - sx_lo) * static_cast<unsigned>(sizeof(Src));
                a = dev::lds_pixel<Src>(tile, row0 * stride_dw * 4u + mis0 + xa);
                b = dev::lds_pixel<Src>(tile, row0 * stride_dw * 4u + mis0 + xb);
                c = dev::lds_pixel<Src>(tile, row1 * stride_dw * 4u + mis1 + xa);
                d = dev::lds_pixel<Src>(tile, row1 * stride_dw * 4u + mis1 + xb);
            } else {
                const char* const r0 = reinterpret_cast<const char*>(s.data) + static_cast<size_t>(s.oy + t.y1) * s.pitch;
                const char* const r1 = reinterpret_cast<const char*>(s.data) + static_cast<size_t>(s.oy + t.y2r) * s.pitch;
                a = reinterpret_cast<const Src*>(r0)[s.ox + t.x1];
                b = reinterpret_cast<const Src*>(r0)[s.ox + t.x2r];
                c = reinterpret_cast<const Src*>(r1)[s.ox + t.x1];
                d = reinterpret_cast<const Src*>(r1)[s.ox + t.x2r];
            }
            value = fk::detail::bilinear_blend(a, b, c, d, t);
        } else {
            value = v.background;
        }
        const OutPixel o = dev::apply_tail(prog.tail, value);
        dev::store_one(job.out, x, y, static_cast<int>(bz), o);
    }
};

// ---- generic -----------------------------------------------------------------------------------------------------
template <typename Sender, typename Receiver>
struct GenericJob {
    static constexpr int LDS_BYTES = 0;
    static constexpr bool READ_IN_PLACE = isBatchOperation<typename Sender::Operation>;
    Sender sender;
    Receiver receiver;
    ActiveThreads active;
    unsigned grid_x, grid_y;

    __device__ static inline void run(const GenericJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char*) {
        const int tid = dev::thread_in_block();
        const int x = static_cast<int>(bx) * 64 + (tid & 63);
        const int y = static_cast<int>(by) * 4 + (tid >> 6);
        if (x >= static_cast<int>(job.active.x) || y >= static_cast<int>(job.active.y)) return;
        const Point thread(x, y, static_cast<int>(bz));
        const auto value = Sender::Operation::exec(thread, job.sender);
        Receiver::Operation::exec(thread, value, job.receiver);
    }
};

// ---- entry points ------------------------------------------------------------------------------------------------
extern __shared__ unsigned char fk_dynamic_lds[];

// The job is the kernel's only argument, so it starts the kernel-argument segment.  It is read in place there
// (uniform, scalar loads) rather than through the by-value parameter: a plane picked with a run-time index would
// otherwise force a private copy of the whole job into scratch memory.
template <typename Job>
__device__ inline const Job& job_in_kernarg() {
    return *(const Job*)__builtin_amdgcn_kernarg_segment_ptr();
}

template <typename Job>
__global__ __attribute__((amdgpu_flat_work_group_size(BLOCK_THREADS, BLOCK_THREADS))) void transform_kernel(const Job job) {
    if constexpr (Job::READ_IN_PLACE) {
        Job::run(job_in_kernarg<Job>(), __builtin_amdgcn_workgroup_id_x(), __builtin_amdgcn_workgroup_id_y(),
                 __builtin_amdgcn_workgroup_id_z(), fk_dynamic_lds);
    } else {
        Job::run(job, __builtin_amdgcn_workgroup_id_x(), __builtin_amdgcn_workgroup_id_y(), __builtin_amdgcn_workgroup_id_z(),
                 fk_dynamic_lds);
    }
}
// Same, with the job read from device memory: for jobs too large for the kernel-argument segment.
template <typename Job>
__global__ __attribute__((amdgpu_flat_work_group_size(BLOCK_THREADS, BLOCK_THREADS))) void transform_kernel_indirect(const Job* __restrict__ job) {
    Job::run(*job, __builtin_amdgcn_workgroup_id_x(), __builtin_amdgcn_workgroup_id_y(), __builtin_amdgcn_workgroup_id_z(),
             fk_dynamic_lds);
}

// Several different jobs in one launch ("divergent horizontal fusion"): the 1-D grid is cut into one contiguous
// range of blocks per job, sized to that job alone, so that a small job does not pay for a large one's grid.
template <typename... Jobs>
struct JobPack;
template <>
struct JobPack<> {
    __device__ static inline void run(const JobPack&, unsigned, unsigned char*) {}
};
template <typename Job, typename... Rest>
struct JobPack<Job, Rest...> {
    Job job;
    unsigned blocks; // blocks of this job: grid_x * grid_y * planes
    JobPack<Rest...> rest;
    __device__ static inline void run(const JobPack& pack, unsigned block, unsigned char* lds) {
        if (block < pack.blocks) {
            const unsigned bx = block % pack.job.grid_x;
            const unsigned q = block / pack.job.grid_x;
            Job::run(pack.job, bx, q % pack.job.grid_y, q / pack.job.grid_y, lds);
        } else {
            JobPack<Rest...>::run(pack.rest, block - pack.blocks, lds);
        }
    }
};
template <typename Pack>
__global__ __attribute__((amdgpu_flat_work_group_size(BLOCK_THREADS, BLOCK_THREADS))) void divergent_kernel(const Pack pack) {
    Pack::run(pack, __builtin_amdgcn_workgroup_id_x(), fk_dynamic_lds);
}
template <typename Pack>
__global__ __attribute__((amdgpu_flat_work_group_size(BLOCK_THREADS, BLOCK_THREADS))) void divergent_kernel_indirect(const Pack* __restrict__ pack) {
    Pack::run(*pack, __builtin_amdgcn_workgroup_id_x(), fk_dynamic_lds);
}

} // namespace exec
} // namespace fk
#endif

// The fused Transform kernels for gfx950 (CDNA4, wave64), hand-written against the views of fk/exec/views.h.
//
// Every launch runs blocks of 256 threads (four wave64).  A "job" is one fused chain over all its planes:
//   PointwiseJob  element-wise chains over a PlainView or a YuvView: each thread owns K consecutive pixels of a row so
//                 that both the source and the destination bytes of a thread are whole 16-byte (or 8/4-byte)
//                 transactions (a YUV thread loads its luma run and the chroma pairs that cover it);
//   ResizeJob     bilinear resize (with optional inner/outer crop and aspect-ratio border): a block owns a 64x16 output
//                 tile, four pixels per thread; it stages the source bounding box of the tile in LDS, one dword-aligned
//                 slot per source pixel (after the operations fused before the resize, e.g. YUV -> RGB, so those run
//                 once per source pixel), and takes the 2x2 taps from there; tiles that gain nothing from it (strong
//                 down-scaling, no tap reuse) read their taps straight from memory; packed outputs leave through LDS
//                 as whole 16-byte pieces;
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

__device__ __attribute__((always_inline)) inline int thread_in_block() { return static_cast<int>(__builtin_amdgcn_workitem_id_x()); }
__device__ __attribute__((always_inline)) inline void block_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Orders a wave's own LDS traffic: the LDS executes one wave's instructions in the order they were issued, so lanes
// see what other lanes of the same wave wrote before this point; only the compiler has to be kept from moving them.
__device__ __attribute__((always_inline)) inline void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int gcd(int a, int b) { return b == 0 ? a : gcd(b, a % b); }
// widest transaction (16, 8 or 4 bytes) that tiles NBYTES
constexpr int chunk_bytes(int nbytes) { return gcd(nbytes, 16); }

// NBYTES (a multiple of 4) from `p`, which is aligned to chunk_bytes(NBYTES)
template <int NBYTES>
__device__ __attribute__((always_inline)) inline void load_words(const void* p, unsigned int* w) {
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
__device__ __attribute__((always_inline)) inline void store_piece(V* p, const V& v) {
    if constexpr (STREAM) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}
template <int NBYTES, bool STREAM = false>
__device__ __attribute__((always_inline)) inline void store_words(void* p, const unsigned int* w) {
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

// x / d with the host's two-float reciprocal r + rl: the short form where every lane of the wave holds an x in
// [2^-40, 2^40], the division instruction sequence elsewhere (the branch is wave-uniform).
template <typename F>
__device__ __attribute__((always_inline)) inline F prepared_divide(const F& x, const F& d, const float* r, const float* rl, const bool fast) {
    if (fast) {
        float lo = __builtin_fabsf(vectorAt(0, x)), hi = lo;
#pragma unroll
        for (int c = 1; c < cn<F>; ++c) {
            const float a = __builtin_fabsf(vectorAt(c, x));
            lo = __builtin_fminf(lo, a);
            hi = __builtin_fmaxf(hi, a);
        }
        // lanes inside the range (a NaN is not); each ballot is one compare, the rest is scalar work
        const unsigned long long inside = __builtin_amdgcn_ballot_w64(lo >= PREPARED_DIV_LO) & __builtin_amdgcn_ballot_w64(hi <= PREPARED_DIV_HI);
        if (inside == __builtin_amdgcn_ballot_w64(true)) {
            float q[cn<F>];
#pragma unroll
            for (int c = 0; c < cn<F>; ++c) {
                const float xc = vectorAt(c, x), dc = vectorAt(c, d), rc = r[c];
                float qc = __builtin_fmaf(xc, rc, xc * rl[c]);
                qc = __builtin_fmaf(__builtin_fmaf(-dc, qc, xc), rc, qc);
                q[c] = qc;
            }
            F out;
            __builtin_memcpy(&out, q, sizeof(F));
            return out;
        }
    }
    return x / d;
}

template <int I, typename V, typename Prepared, typename Op, typename... Rest_>
__device__ __attribute__((always_inline)) inline auto compute_prepared(const V& v, const Prepared& tail, const OperationTuple<Op, Rest_...>& t) {
    using Tuple = OperationTuple<Op, Rest_...>;
    constexpr bool IS_DIV = IsFloatDiv<Op>::value;
    const auto step = [&] {
        if constexpr (IS_DIV && std::is_same_v<V, typename Op::InputType>) {
            return prepared_divide(v, t.instance.params, tail.recip[I], tail.recip_lo[I], (tail.fast >> I & 1u) != 0u);
        } else {
            return fk::detail::chain_step<Op>(Point(), v, t);
        }
    }();
    if constexpr (sizeof...(Rest_) == 0) {
        return step;
    } else if constexpr (Tuple::HAS_NEXT) {
        return compute_prepared<I + (IS_DIV ? 1 : 0)>(step, tail, t.next);
    } else {
        return compute_prepared<I + (IS_DIV ? 1 : 0)>(step, tail, OperationTuple<Rest_...>{});
    }
}

template <typename Tail>
struct IsPreparedTail : std::false_type {};
template <typename Ops, int NDIV>
struct IsPreparedTail<PreparedTail<Ops, NDIV>> : std::true_type {};

template <typename Tail, typename V>
__device__ __attribute__((always_inline)) inline auto apply_tail(const Tail& tail, const V& v) {
    if constexpr (std::is_same_v<Tail, NoTail>) {
        return v;
    } else if constexpr (IsPreparedTail<Tail>::value) {
        return compute_prepared<0>(v, tail, tail.ops);
    } else {
        return fk::detail::tuple_compute(v, tail);
    }
}

template <typename O>
__device__ __attribute__((always_inline)) inline void store_one(const PackedOut<O>& out, int x, int y, int z, const O& v) {
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
    reinterpret_cast<O*>(row)[x] = v;
}
template <typename O>
__device__ __attribute__((always_inline)) inline void store_one(const SplitOut<O>& out, int x, int y, int z, const O& v) {
    using B = VBase<O>;
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
    reinterpret_cast<B*>(row)[x] = v.x;
    reinterpret_cast<B*>(row + out.chan_stride)[x] = v.y;
    if constexpr (cn<O> >= 3) reinterpret_cast<B*>(row + 2 * out.chan_stride)[x] = v.z;
    if constexpr (cn<O> == 4) reinterpret_cast<B*>(row + 3 * out.chan_stride)[x] = v.w;
}

// N elements of a 1- or 2-byte type into whole dwords, in registers (a byte-wise copy would go through scratch memory)
template <int N, typename B>
__device__ __attribute__((always_inline)) inline void pack_elements(const B* e, unsigned int* w) {
    if constexpr (sizeof(B) >= 4) {
        __builtin_memcpy(w, e, N * sizeof(B));
    } else {
        constexpr int PER = 4 / static_cast<int>(sizeof(B));
        static_assert(N % PER == 0, "whole dwords");
#pragma unroll
        for (int i = 0; i < N / PER; ++i) {
            unsigned int word = 0u;
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                using U = std::make_unsigned_t<std::conditional_t<std::is_same_v<B, bool>, unsigned char, B>>;
                word |= static_cast<unsigned int>(static_cast<U>(e[i * PER + j])) << (8 * static_cast<int>(sizeof(B)) * j);
            }
            w[i] = word;
        }
    }
}
// K pixels as the dwords they occupy in memory
template <int K, typename O>
__device__ __attribute__((always_inline)) inline void pack_pixels(const O* v, unsigned int* w) {
    if constexpr (sizeof(O) % 4 == 0) {
        __builtin_memcpy(w, v, K * sizeof(O));
    } else {
        using B = VBase<O>;
        B e[K * cn<O>];
#pragma unroll
        for (int k = 0; k < K; ++k) {
#pragma unroll
            for (int c = 0; c < cn<O>; ++c) e[k * cn<O> + c] = vectorAt(c, v[k]);
        }
        pack_elements<K * cn<O>>(e, w);
    }
}

// K consecutive pixels starting at x0 (caller guarantees the alignment that chunk_bytes asks for)
template <int K, bool STREAM = false, typename O>
__device__ __attribute__((always_inline)) inline void store_group(const PackedOut<O>& out, int x0, int y, int z, const O* v) {
    constexpr int NB = K * static_cast<int>(sizeof(O));
    unsigned int w[NB / 4];
    pack_pixels<K>(v, w);
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
    // a thread's K pixels are one transaction only when they fill exactly one piece
    store_words<NB, STREAM && NB == chunk_bytes(NB)>(row + static_cast<size_t>(x0) * sizeof(O), w);
}
template <int K, bool STREAM = false, typename O>
__device__ __attribute__((always_inline)) inline void store_group(const SplitOut<O>& out, int x0, int y, int z, const O* v) {
    using B = VBase<O>;
    constexpr int NB = K * static_cast<int>(sizeof(B));
    char* const row = reinterpret_cast<char*>(out.data) + static_cast<size_t>(z) * out.z_stride + static_cast<size_t>(y) * out.pitch;
#pragma unroll
    for (int c = 0; c < cn<O>; ++c) {
        B ch[K];
#pragma unroll
        for (int k = 0; k < K; ++k) ch[k] = vectorAt(c, v[k]);
        unsigned int w[NB / 4];
        pack_elements<K>(ch, w);
        store_words<NB, STREAM && NB == chunk_bytes(NB)>(row + c * out.chan_stride + static_cast<size_t>(x0) * sizeof(B), w);
    }
}
// One or the other, chosen at run time (block-uniform).  The empty asm keeps the compiler from merging the two stores
// into one plain store, which it does for stores that differ only in their cache hint.
template <int K, typename Out, typename O>
__device__ __attribute__((always_inline)) inline void store_group_either(const bool stream, const Out& out, int x0, int y, int z, const O* v) {
    if (stream) {
        asm volatile("" ::: "memory");
        store_group<K, true>(out, x0, y, z, v);
        asm volatile("" ::: "memory");
    } else {
        store_group<K>(out, x0, y, z, v);
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

// ---- source access -----------------------------------------------------------------------------------------------
// SourceAccess<View>: one pixel of the window (load_one), K consecutive pixels of a row with vector loads (load_group,
// when the host found the alignment that needs: `aligned`), and the pixels per thread that suit an output pixel type.
template <typename View>
struct SourceAccess;

template <typename T>
struct SourceAccess<PlainView<T>> {
    using View = PlainView<T>;
    static constexpr bool FLATTENS = true; // contiguous rows may be treated as one long row
    static constexpr bool PAIRS_ROWS = false;
    template <typename O, bool SPLIT>
    static constexpr int pixels() { return pixels_per_thread<T, O, SPLIT>(); }
    template <int K>
    static constexpr int group_bytes() { return K * static_cast<int>(sizeof(T)); }
    __device__ __attribute__((always_inline)) static inline const char* row(const View& v, int y) {
        return reinterpret_cast<const char*>(v.data) + static_cast<size_t>(v.oy + y) * v.pitch + static_cast<size_t>(v.ox) * sizeof(T);
    }
    __device__ __attribute__((always_inline)) static inline T load_one(const View& v, int x, int y) {
        return fk::detail::read_element(reinterpret_cast<const T*>(row(v, y)) + x);
    }
    template <int K>
    __device__ __attribute__((always_inline)) static inline void load_group(const View& v, int x0, int y, T* out) {
        constexpr int NB = K * static_cast<int>(sizeof(T));
        unsigned int w[NB / 4];
        dev::load_words<NB>(row(v, y) + static_cast<size_t>(x0) * sizeof(T), w);
        __builtin_memcpy(out, w, NB);
    }
    template <int K>
    static bool aligned(const View& v) {
        constexpr size_t chunk = dev::chunk_bytes(K * static_cast<int>(sizeof(T)));
        const size_t first = reinterpret_cast<size_t>(v.data) + static_cast<size_t>(v.oy) * v.pitch + static_cast<size_t>(v.ox) * sizeof(T);
        return first % chunk == 0 && (v.h == 1 || v.pitch % chunk == 0);
    }
};

template <PixelFormat PF>
struct SourceAccess<YuvView<PF>> {
    using View = YuvView<PF>;
    using Base = typename View::Base;
    using Pixel = typename View::Pixel;
    using Layout = fk::detail::YuvLayout<PF>;
    static constexpr bool FLATTENS = false;
    static constexpr bool pairs_rows() { // 4:2:0: rows 2k and 2k + 1 share a chroma row
        if constexpr (Layout::semi_planar) return Layout::row_shift == 1;
        else return false;
    }
    static constexpr bool PAIRS_ROWS = pairs_rows();
    // smallest power of two >= 4 whose output run is whole 16-byte pieces and whose luma run is whole dwords
    template <typename O, bool SPLIT>
    static constexpr int pixels() {
        const int so = SPLIT ? static_cast<int>(sizeof(VBase<O>)) : static_cast<int>(sizeof(O));
        for (int k = 4; k <= 16; k *= 2) {
            if ((k * so) % 16 == 0 && (k * static_cast<int>(sizeof(Base))) % 4 == 0) return k;
        }
        return 16;
    }
    // bytes of the widest single run a thread loads: K luma samples, or 2K packed samples
    template <int K>
    static constexpr int group_bytes() { return (Layout::semi_planar ? K : 2 * K) * static_cast<int>(sizeof(Base)); }
    __device__ __attribute__((always_inline)) static inline Pixel load_one(const View& v, int x, int y) {
        const RawImage<PF> raw{ RawPtr<ND::_2D, Base>{ const_cast<Base*>(v.data), PtrDims<ND::_2D>(0u, 0u, v.pitch) }, static_cast<uint>(v.img_w),
                                static_cast<uint>(v.img_h) };
        return ReadYUV<PF>::exec(Point(v.ox + x, v.oy + y), raw);
    }
    // x0 and v.ox are even: the K pixels are K/2 whole chroma pairs
    template <int K>
    __device__ __attribute__((always_inline)) static inline void load_group(const View& v, int x0, int y, Pixel* out) {
        const int px = v.ox + x0, py = v.oy + y;
        constexpr int NB = group_bytes<K>();
        if constexpr (Layout::semi_planar) {
            const char* const base = reinterpret_cast<const char*>(v.data);
            unsigned int wl[NB / 4], wc[NB / 4];
            dev::load_words<NB>(base + static_cast<size_t>(py) * v.pitch + static_cast<size_t>(px) * sizeof(Base), wl);
            dev::load_words<NB>(base + (static_cast<size_t>(v.img_h) + (py >> Layout::row_shift)) * v.pitch + static_cast<size_t>(px) * sizeof(Base), wc);
            Base luma[K], chroma[K];
            __builtin_memcpy(luma, wl, NB);
            __builtin_memcpy(chroma, wc, NB);
#pragma unroll
            for (int k = 0; k < K; ++k) out[k] = Pixel{ luma[k], chroma[(k & ~1) + Layout::u], chroma[(k & ~1) + Layout::v] };
        } else {
            unsigned int w[NB / 4];
            dev::load_words<NB>(reinterpret_cast<const char*>(v.data) + static_cast<size_t>(py) * v.pitch + 2 * static_cast<size_t>(px) * sizeof(Base), w);
            Base quad[2 * K];
            __builtin_memcpy(quad, w, NB);
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const int q = 4 * (k >> 1);
                out[k] = Pixel{ quad[q + ((k & 1) ? Layout::y1 : Layout::y0)], quad[q + Layout::u], quad[q + Layout::v] };
            }
        }
    }
    template <int K>
    static bool aligned(const View& v) {
        constexpr size_t chunk = dev::chunk_bytes(group_bytes<K>());
        const size_t first = reinterpret_cast<size_t>(v.data) + (Layout::semi_planar ? 1 : 2) * static_cast<size_t>(v.ox) * sizeof(Base);
        return (v.ox & 1) == 0 && first % chunk == 0 && v.pitch % chunk == 0;
    }
};

// ---- pointwise ---------------------------------------------------------------------------------------------------
enum : unsigned { FLAG_VECTOR_IO = 1u, FLAG_STREAM_STORES = 2u, FLAG_SOURCE_TILE = 4u, FLAG_STAGE_OUT = 8u };

template <typename Prog, size_t N, typename Out>
struct PointwiseJob {
    using View = decltype(Prog::view);
    using Access = SourceAccess<View>;
    using Src = typename View::Source;
    using OutPixel = typename Out::Pixel;
    static constexpr int K = Access::template pixels<OutPixel, Out::IS_SPLIT>();
    static constexpr int IN_BYTES = K * static_cast<int>(sizeof(Src));
    static constexpr int OUT_BYTES = Out::IS_SPLIT ? K * static_cast<int>(sizeof(VBase<OutPixel>)) : K * static_cast<int>(sizeof(OutPixel));
    // A thread's K pixels span more than one 16-byte transaction when pixels are 12 bytes wide (48 bytes per thread).
    // Lanes reading 48-byte runs touch every cache line three times; instead the block moves its contiguous span of up
    // to 256*K pixels with fully coalesced 16-byte accesses and redistributes pixels to threads through LDS.
    static constexpr bool STAGE_IN = Access::FLATTENS && IN_BYTES > 16 && IN_BYTES % 16 == 0;
    static constexpr bool STAGE_OUT = !Out::IS_SPLIT && OUT_BYTES > 16 && OUT_BYTES % 16 == 0;
    static constexpr int STAGE_BYTES = (STAGE_IN && STAGE_OUT) ? (IN_BYTES > OUT_BYTES ? IN_BYTES : OUT_BYTES)
                                       : STAGE_IN              ? IN_BYTES
                                       : STAGE_OUT             ? OUT_BYTES
                                                               : 0;
    static constexpr int LDS_BYTES = BLOCK_THREADS * STAGE_BYTES;
    static constexpr bool READ_IN_PLACE = N > 1 || sizeof(Prog) > 256; // run-time plane index, or a long chain (SGPR pressure)
    struct Plane {
        Prog prog;
        unsigned flags;
    };
    Plane plane[N];
    Out out;
    unsigned tx_shift; // log2 of the thread columns of a block; the other threads cover further rows
    unsigned grid_x, grid_y;
    unsigned pair_limit; // blocks that are re-dealt so that row pairs share an XCD (0: none)
    size_t lds_bytes() const { return LDS_BYTES; }

    // A block that lies on one row and owns `span` pixels of it from pixel bx0 on (a whole number of thread groups, so
    // the span is whole 16-byte pieces on both sides).  FULL: span is the block's whole 256*K pixels, nothing is guarded.
    template <bool FULL>
    __device__ __attribute__((always_inline)) static inline void row_block(const PointwiseJob& job, const Plane& pl, int bx0, int span, int x0, int y,
                                                                          unsigned bz, int tid, unsigned char* lds) {
        const View& v = pl.prog.view;
        // A wave's 64 threads own 64*K consecutive pixels, so a wave moves its own span through its own part of the
        // buffer and never waits for the other waves of the block.
        const int wave = tid >> 6, lane = tid & 63;
        dev::u32x4* const stage = reinterpret_cast<dev::u32x4*>(lds) + wave * (64 * STAGE_BYTES / 16);
        const bool active = FULL || x0 < v.w;
        Src in[K];
        if constexpr (STAGE_IN) {
            constexpr int MINE = IN_BYTES / 16;
            const dev::u32x4* const g =
                reinterpret_cast<const dev::u32x4*>(Access::row(v, y) + static_cast<size_t>(bx0) * sizeof(Src)) + wave * (64 * MINE);
            const int pieces = span * static_cast<int>(sizeof(Src)) / 16 - wave * (64 * MINE); // of this wave's span
#pragma unroll
            for (int j = 0; j < MINE; ++j) {
                if (FULL || j * 64 + lane < pieces) stage[j * 64 + lane] = g[j * 64 + lane];
            }
            dev::wave_sync();
            if (active) {
                dev::u32x4 mine[MINE];
#pragma unroll
                for (int j = 0; j < MINE; ++j) mine[j] = stage[lane * MINE + j];
                __builtin_memcpy(in, mine, IN_BYTES);
            }
        } else {
            if (active) Access::template load_group<K>(v, x0, y, in);
        }
        OutPixel o[K];
        if (active) {
#pragma unroll
            for (int k = 0; k < K; ++k) o[k] = dev::apply_tail(pl.prog.tail, in[k]);
        }
        if constexpr (STAGE_OUT) {
            constexpr int MINE = OUT_BYTES / 16;
            if constexpr (STAGE_IN) dev::wave_sync(); // every lane has taken its input out of the buffer
            if (active) {
                unsigned int w[OUT_BYTES / 4];
                dev::pack_pixels<K>(o, w);
#pragma unroll
                for (int j = 0; j < MINE; ++j) {
                    dev::u32x4 piece;
                    piece.x = w[4 * j]; piece.y = w[4 * j + 1]; piece.z = w[4 * j + 2]; piece.w = w[4 * j + 3];
                    stage[lane * MINE + j] = piece;
                }
            }
            dev::wave_sync();
            dev::u32x4* const g = reinterpret_cast<dev::u32x4*>(
                reinterpret_cast<char*>(job.out.data) + static_cast<size_t>(bz) * job.out.z_stride +
                static_cast<size_t>(y) * job.out.pitch + static_cast<size_t>(bx0) * sizeof(OutPixel)) + wave * (64 * MINE);
            const int pieces = span * static_cast<int>(sizeof(OutPixel)) / 16 - wave * (64 * MINE);
            if ((pl.flags & FLAG_STREAM_STORES) != 0u) {
#pragma unroll
                for (int j = 0; j < MINE; ++j) {
                    if (FULL || j * 64 + lane < pieces) dev::store_piece<true>(g + j * 64 + lane, stage[j * 64 + lane]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < MINE; ++j) {
                    if (FULL || j * 64 + lane < pieces) g[j * 64 + lane] = stage[j * 64 + lane];
                }
            }
        } else if (active) {
            dev::store_group_either<K>((pl.flags & FLAG_STREAM_STORES) != 0u, job.out, x0, y, static_cast<int>(bz), o);
        }
    }

    __device__ __attribute__((always_inline)) static inline void run(const PointwiseJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char* lds) {
        const Plane& pl = job.plane[N == 1 ? 0u : bz];
        const View& v = pl.prog.view;
        const int tid = dev::thread_in_block();
        // pair_limit != 0 (one row per block row, the source shares a chroma row between rows 2k and 2k + 1): workgroups go
        // to the eight XCDs round-robin in launch order, so blocks b and b + 8 run on the same XCD one after the other.
        // Giving them the same columns of rows 2k and 2k + 1 lets the second find the chroma row in that XCD's L2 instead
        // of fetching it from memory again through another one.  The first pair_limit blocks (a multiple of 16 and of two
        // block rows) are dealt out that way among themselves; the few after them keep their places.
        const unsigned launch_index = bx + job.grid_x * by;
        if (launch_index < job.pair_limit) {
            const unsigned xcd = launch_index & 7u, turn = launch_index >> 3;
            const unsigned pair = 8u * (turn >> 1) + xcd; // (columns, row pair) in the order the XCDs take them up
            const unsigned k = pair / job.grid_x;
            bx = pair - k * job.grid_x;
            by = 2u * k + (turn & 1u);
        }
        const int cols = 1 << job.tx_shift;
        const int x0 = (static_cast<int>(bx) * cols + (tid & (cols - 1))) * K;
        const int y = static_cast<int>(by) * (BLOCK_THREADS >> job.tx_shift) + (tid >> job.tx_shift);

        if constexpr (STAGE_IN || STAGE_OUT) {
            // block-uniform decisions
            const int bx0 = static_cast<int>(bx) * BLOCK_THREADS * K; // first pixel of the block
            const int span = v.w - bx0 < BLOCK_THREADS * K ? v.w - bx0 : BLOCK_THREADS * K;
            if ((pl.flags & FLAG_VECTOR_IO) != 0u && job.tx_shift == 8u && y < v.h && span > 0 && span % K == 0) {
                if (span == BLOCK_THREADS * K) row_block<true>(job, pl, bx0, span, x0, y, bz, tid, lds);
                else row_block<false>(job, pl, bx0, span, x0, y, bz, tid, lds);
                return;
            }
        }

        if (y >= v.h || x0 >= v.w) return; // also ends blocks that lie outside a smaller plane of a ragged batch
        if ((pl.flags & FLAG_VECTOR_IO) != 0u && x0 + K <= v.w) {
            Src in[K];
            Access::template load_group<K>(v, x0, y, in);
            OutPixel o[K];
#pragma unroll
            for (int k = 0; k < K; ++k) o[k] = dev::apply_tail(pl.prog.tail, in[k]);
            dev::store_group_either<K>((pl.flags & FLAG_STREAM_STORES) != 0u, job.out, x0, y, static_cast<int>(bz), o);
        } else {
            const int xe = x0 + K < v.w ? x0 + K : v.w;
            for (int x = x0; x < xe; ++x) {
                const OutPixel o = dev::apply_tail(pl.prog.tail, Access::load_one(v, x, y));
                dev::store_one(job.out, x, y, static_cast<int>(bz), o);
            }
        }
    }
};

// ---- resize ------------------------------------------------------------------------------------------------------
// A block owns a 64x16 output tile of one plane; a thread computes four consecutive pixels of one row, so everything
// that depends only on the row (or only on the column) is computed once and shared.
constexpr int RESIZE_TILE_W = 64;
constexpr int RESIZE_TILE_H = 16;
constexpr int RESIZE_PX = 4;                // pixels per thread, along x
constexpr int RESIZE_LDS_DWORDS = 6144;     // source tile capacity (24 KiB)

namespace dev {
// LDS slot of one source pixel: whole dwords, so a tap is one aligned LDS read whatever the pixel's byte size
template <typename T>
constexpr int slot_dwords() { return (static_cast<int>(sizeof(T)) + 3) / 4; }

template <typename T>
struct PixelSlot {
    unsigned int w[slot_dwords<T>()];
};
template <typename T>
__device__ __attribute__((always_inline)) inline T slot_to_pixel(const PixelSlot<T>& s) {
    T out;
    __builtin_memcpy(&out, s.w, sizeof(T));
    return out;
}
// One pixel from memory at any byte alignment, as whole dwords.  `row` points at byte 0 of the window row, `off` is the
// pixel's byte offset in it; [valid_lo, valid_hi) are the byte offsets of that row that belong to the parent image, so
// dwords that would reach past them are assembled from single bytes.
// The dword at byte `voff` from `row - 1`, for a `row` that is the same for the whole wave: the address stays in scalar
// registers and the lane adds its 32-bit offset.
__device__ __attribute__((always_inline)) inline unsigned int load_dword_from_row(const char* row, unsigned voff) {
    struct __attribute__((packed)) UnalignedDword { unsigned int v; };
    using GlobalBytes = const __attribute__((address_space(1))) char*;
    using GlobalDword = const __attribute__((address_space(1))) UnalignedDword*;
    GlobalBytes base = (GlobalBytes)(row - 1);
    asm volatile("" : "+s"(base));
    return ((GlobalDword)(base + voff))->v;
}

template <typename T>
__device__ __attribute__((always_inline)) inline PixelSlot<T> load_pixel_slot(const char* row, int off, int valid_lo, int valid_hi) {
    constexpr int ND = slot_dwords<T>();
    PixelSlot<T> s;
    if constexpr (alignof(T) % 4 == 0) {
        const unsigned int* const p = reinterpret_cast<const unsigned int*>(row + off);
#pragma unroll
        for (int i = 0; i < ND; ++i) s.w[i] = p[i];
    } else if constexpr (sizeof(T) == 3) {
        // one unaligned dword, [p, p + 4) for an aligned p and [p - 1, p + 3) otherwise: its one byte that is not the
        // pixel's lies in an aligned dword that also holds a byte of the pixel, so the load cannot fault and needs no
        // branch (the loads of several rows are in flight together).  `row` is the same for the whole wave: it stays
        // in scalar registers and the lane adds a 32-bit offset, from row - 1 so that the offset is never negative.
        const unsigned aligned = ((static_cast<unsigned>(reinterpret_cast<size_t>(row)) + static_cast<unsigned>(off)) & 3u) == 0u ? 1u : 0u;
        const unsigned int w = load_dword_from_row(row, static_cast<unsigned>(off) + aligned);
        s.w[0] = aligned != 0u ? w : w >> 8u;
    } else {
        const unsigned mis = (static_cast<unsigned>(reinterpret_cast<size_t>(row)) + static_cast<unsigned>(off)) & 3u;
        const int first = off - static_cast<int>(mis); // aligned dword that holds the pixel's first byte
        const bool spills = mis + sizeof(T) > 4u * ND;  // the pixel reaches into one more dword
        if (first >= valid_lo && first + 4 * (ND + (spills ? 1 : 0)) <= valid_hi) {
            const unsigned int* const p = reinterpret_cast<const unsigned int*>(row + first);
            unsigned int lo = p[0];
#pragma unroll
            for (int i = 0; i < ND; ++i) {
                const unsigned int hi = (i + 1 < ND || spills) ? p[i + 1] : 0u;
                s.w[i] = __builtin_amdgcn_alignbyte(hi, lo, mis);
                lo = hi;
            }
        } else { // at the edge of the parent image: byte by byte
#pragma unroll
            for (int i = 0; i < ND; ++i) s.w[i] = 0u;
#pragma unroll
            for (int b = 0; b < static_cast<int>(sizeof(T)); ++b) {
                s.w[b / 4] |= static_cast<unsigned int>(static_cast<unsigned char>(row[off + b])) << (8 * (b % 4));
            }
        }
    }
    return s;
}
} // namespace dev

template <typename Prog, size_t N, typename Out>
struct ResizeJob {
    using View = decltype(Prog::view);
    using SrcView = decltype(View::src);
    using Pre = decltype(View::pre);
    using Access = SourceAccess<SrcView>;
    using Src = typename View::Source; // the pixel that is interpolated: the source view's pixel after Pre
    using Pixel = typename View::Pixel;
    using OutPixel = typename Out::Pixel;
    // packed pixels read as they are: taps and tile slots come straight from memory as dwords
    static constexpr bool RAW_SOURCE = std::is_same_v<SrcView, PlainView<Src>> && std::is_same_v<Pre, NoTail>;
    static constexpr int SLOT = dev::slot_dwords<Src>();
    static constexpr int OUT_ROW_BYTES = RESIZE_TILE_W * static_cast<int>(sizeof(OutPixel));
    // packed outputs whose four pixels per thread are not one 16-byte piece go out through LDS as whole 16-byte pieces
    static constexpr bool STAGE_OUT = !Out::IS_SPLIT && (RESIZE_PX * sizeof(OutPixel)) % 16 == 0 && RESIZE_PX * sizeof(OutPixel) > 16;
    static constexpr int OUT_STAGE_BYTES = STAGE_OUT ? RESIZE_TILE_H * OUT_ROW_BYTES : 0;
    static constexpr bool READ_IN_PLACE = N > 1;
    Prog plane[N];
    Out out;
    unsigned grid_x, grid_y;
    // FLAG_VECTOR_IO: output rows start 16-byte aligned; FLAG_STREAM_STORES: large output; FLAG_SOURCE_TILE: some plane's
    // tiles are worth staging in LDS; FLAG_STAGE_OUT: packed output leaves through LDS.  The last two decide how much
    // LDS the launch asks for (a divergent launch shares one LDS size between all its jobs).
    unsigned flags;
    // The launch asks for as much LDS as the planes' own factors need, not for the capacity: a block's LDS decides how
    // many blocks a CU holds.  tile_dwords is the room for a source tile (a tile that needs more reads its taps
    // directly); the packed output is staged behind it when both fit the capacity (out_stage_offset, in bytes), else in
    // the same place (0), which costs a block barrier between the last tap and the first staged pixel.
    unsigned tile_dwords;
    unsigned out_stage_offset;
    size_t lds_bytes() const {
        size_t n = 0;
        if ((flags & FLAG_SOURCE_TILE) != 0u) n = static_cast<size_t>(tile_dwords) * 4;
        if (STAGE_OUT && (flags & FLAG_STAGE_OUT) != 0u && out_stage_offset + static_cast<size_t>(OUT_STAGE_BYTES) > n) n = out_stage_offset + OUT_STAGE_BYTES;
        return n == 0 ? 0 : n + 16;
    }
    // dwords a tile of a plane with these factors takes when staged, 0 when it is not worth staging (same rule as the
    // kernel applies per tile)
    static unsigned staged_tile_dwords(float fx, float fy) {
        const int cols = static_cast<int>((RESIZE_TILE_W - 1) * fx) + 3, rows = static_cast<int>((RESIZE_TILE_H - 1) * fy) + 3;
        const bool worth = rows * (cols | 1) * SLOT <= RESIZE_LDS_DWORDS && rows * cols <= 3 * RESIZE_TILE_W * RESIZE_TILE_H + 256;
        return worth ? static_cast<unsigned>(rows * (cols | 1) * SLOT) : 0u;
    }
    // fills in the LDS layout from the planes' factors; FLAG_STAGE_OUT has been decided
    void plan_lds() {
        tile_dwords = 0;
        for (size_t i = 0; i < N; ++i) {
            const unsigned need = staged_tile_dwords(plane[i].view.fx, plane[i].view.fy);
            tile_dwords = need > tile_dwords ? need : tile_dwords;
        }
        tile_dwords = (tile_dwords + 3u) & ~3u; // what follows the tile starts at a whole 16 bytes
        if (tile_dwords != 0u) flags |= FLAG_SOURCE_TILE;
        const bool behind = STAGE_OUT && (flags & FLAG_STAGE_OUT) != 0u && tile_dwords * 4u + OUT_STAGE_BYTES <= RESIZE_LDS_DWORDS * 4u;
        out_stage_offset = behind ? tile_dwords * 4u : 0u;
    }

    // source pixel (x, y) of the resampled window, after the operations fused before the resize
    __device__ __attribute__((always_inline)) static inline Src fetch(const View& v, int x, int y) {
        return dev::apply_tail(v.pre, Access::load_one(v.src, x, y));
    }

    // Four consecutive pixels of row y, taps from the staged tile (STAGED) or straight from memory.
    template <bool STAGED, bool INTERIOR>
    __device__ __attribute__((always_inline)) static inline void pixels(const Prog& prog, const unsigned int* tile, const char* window,
                                                                       int sx_lo, int sy_lo, int stride, int x_first, int y, OutPixel* o) {
        const View& v = prog.view;
        const SrcView& s = v.src;
        const int ry = y + v.off_y;
        bool row_inside = INTERIOR || y < v.h;
        if constexpr (View::HAS_ROI && !INTERIOR) row_inside = row_inside && ry >= v.y1 && ry <= v.y2;
        const float src_y = (ry - v.y1) * v.fy;
        // a short tail is taken into registers once, ahead of the pixels (read in place it is fetched where it is used,
        // once per pixel and with the wait in the middle of the arithmetic)
        using Tail = std::decay_t<decltype(prog.tail)>;
        const std::conditional_t<(sizeof(Tail) <= 128), Tail, const Tail&> tail = prog.tail;
        // the float of (rx - x1) for the thread's first pixel; the next ones are that plus 1, 2, 3 (exact: far below 2^24)
        const float rel_x0 = static_cast<float>(x_first + v.off_x - v.x1);
#pragma unroll
        for (int k = 0; k < RESIZE_PX; ++k) {
            const int x = x_first + k;
            const int rx = x + v.off_x;
            bool inside = INTERIOR || (row_inside && x < v.w);
            if constexpr (View::HAS_ROI && !INTERIOR) inside = inside && rx >= v.x1 && rx <= v.x2;
            Pixel value = v.background;
            if (inside) {
                const float src_x = (rel_x0 + static_cast<float>(k)) * v.fx;
                const fk::detail::BilinearTaps t = fk::detail::bilinear_taps(src_x, src_y, Size(s.w, s.h));
                Src a, b, c, d;
                if constexpr (STAGED) {
                    // the tile holds columns sx_lo.. and rows sy_lo.., edge copies included: no clamping here
                    const unsigned int* const row0 = tile + ((t.y1 - sy_lo) * stride - sx_lo) * SLOT; // the same for the thread's four pixels
                    const unsigned int* const p0 = row0 + t.x1 * SLOT;
                    const unsigned int* const p1 = p0 + stride * SLOT;
                    dev::PixelSlot<Src> sa, sb, sc, sd;
#pragma unroll
                    for (int i = 0; i < SLOT; ++i) {
                        sa.w[i] = p0[i];
                        sb.w[i] = p0[SLOT + i];
                        sc.w[i] = p1[i];
                        sd.w[i] = p1[SLOT + i];
                    }
                    a = dev::slot_to_pixel<Src>(sa);
                    b = dev::slot_to_pixel<Src>(sb);
                    c = dev::slot_to_pixel<Src>(sc);
                    d = dev::slot_to_pixel<Src>(sd);
                } else if constexpr (RAW_SOURCE) {
                    const Src* const r0 = reinterpret_cast<const Src*>(window + static_cast<size_t>(t.y1) * s.pitch);
                    const Src* const r1 = reinterpret_cast<const Src*>(window + static_cast<size_t>(t.y2r) * s.pitch);
                    a = fk::detail::read_element(r0 + t.x1);
                    b = fk::detail::read_element(r0 + t.x2r);
                    c = fk::detail::read_element(r1 + t.x1);
                    d = fk::detail::read_element(r1 + t.x2r);
                } else {
                    a = fetch(v, t.x1, t.y1);
                    b = fetch(v, t.x2r, t.y1);
                    c = fetch(v, t.x1, t.y2r);
                    d = fetch(v, t.x2r, t.y2r);
                }
                value = fk::detail::bilinear_blend(a, b, c, d, t);
            }
            o[k] = dev::apply_tail(tail, value);
        }
    }

    __device__ __attribute__((always_inline)) static inline void run(const ResizeJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char* lds_raw) {
        const Prog& prog = job.plane[N == 1 ? 0u : bz];
        const View& v = prog.view;
        const SrcView& s = v.src;
        const int tx0 = static_cast<int>(bx) * RESIZE_TILE_W;
        const int ty0 = static_cast<int>(by) * RESIZE_TILE_H;
        if (tx0 >= v.w || ty0 >= v.h) return; // block outside this plane's own extent
        const int tid = dev::thread_in_block();
        const int x_first = tx0 + (tid & (RESIZE_TILE_W / RESIZE_PX - 1)) * RESIZE_PX;
        const int y = ty0 + tid / (RESIZE_TILE_W / RESIZE_PX);

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
        int stride = 0; // slots per tile row
        // window pixel (0, 0) and the byte range of a window row that belongs to the parent image (raw sources only)
        const char* const window = reinterpret_cast<const char*>(s.data) + static_cast<size_t>(s.oy) * s.pitch +
                                   static_cast<size_t>(s.ox) * sizeof(Src);
        const int valid_lo = -s.ox * static_cast<int>(sizeof(Src));
        const int valid_hi = (s.img_w - s.ox) * static_cast<int>(sizeof(Src));
        if (resamples) {
            // source bounding box of the tile: taps are floor(c) and floor(c) + 1 for c in [lo, hi] * f; the column and
            // row past the source edge are staged as copies of the last one, which is what the clamp of the taps reads
            sx_lo = static_cast<int>(__builtin_floorf((rx_lo - v.x1) * v.fx)); // the floor instruction; same value as floor_to_int
            sy_lo = static_cast<int>(__builtin_floorf((ry_lo - v.y1) * v.fy));
            const int cols = static_cast<int>(__builtin_floorf((rx_hi - v.x1) * v.fx)) + 2 - sx_lo;
            const int rows = static_cast<int>(__builtin_floorf((ry_hi - v.y1) * v.fy)) + 2 - sy_lo;
            stride = cols | 1;
            const int tile_px = (rx_hi - rx_lo + 1) * (ry_hi - ry_lo + 1);
            // staging pays off while a source pixel is used about once or more; strong down-scaling reads taps directly
            staged = (job.flags & FLAG_SOURCE_TILE) != 0u && rows * stride * SLOT <= static_cast<int>(job.tile_dwords) && rows * cols <= 3 * tile_px + 256;
            if (staged) {
                // A wave takes every fourth row, a lane every 64th column; the loads of STAGE_ROWS rows are issued before
                // the first of them is stored, so a tile of up to 4 * STAGE_ROWS rows costs one memory round trip.  A row
                // past the tile's last is the last one again, loaded and stored twice: with a branch around it the
                // compiler moves the load to the store and waits there.
                const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
                constexpr int WAVES = BLOCK_THREADS / 64;
                constexpr int STAGE_ROWS = SLOT == 1 ? 4 : 2;
                bool rows_alike = false;
                if constexpr (RAW_SOURCE && sizeof(Src) == 3) rows_alike = (s.pitch & 3u) == 0u;
                if (rows_alike) {
                    // three-byte pixels, rows a whole number of dwords apart: a column has the same alignment in every
                    // row, so a lane's offset and the shift that takes the pixel out of its dword are found once per column
                    if constexpr (RAW_SOURCE && sizeof(Src) == 3) {
                        for (int c = lane; c < cols; c += 64) {
                            const int sx = sx_lo + c < s.w - 1 ? sx_lo + c : s.w - 1;
                            const unsigned off = static_cast<unsigned>(sx) * 3u;
                            const bool aligned = ((static_cast<unsigned>(reinterpret_cast<size_t>(window)) + off) & 3u) == 0u;
                            const unsigned voff = off + (aligned ? 1u : 0u); // from one byte before the row
                            for (int r0 = wave; r0 < rows; r0 += WAVES * STAGE_ROWS) {
                                unsigned int w[STAGE_ROWS];
#pragma unroll
                                for (int u = 0; u < STAGE_ROWS; ++u) {
                                    const int r = r0 + WAVES * u < rows ? r0 + WAVES * u : rows - 1;
                                    const int sy = sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1;
                                    w[u] = dev::load_dword_from_row(window + static_cast<size_t>(sy) * s.pitch, voff);
                                }
#pragma unroll
                                for (int u = 0; u < STAGE_ROWS; ++u) {
                                    const int r = r0 + WAVES * u < rows ? r0 + WAVES * u : rows - 1;
                                    tile[r * stride + c] = aligned ? w[u] : w[u] >> 8u;
                                }
                            }
                        }
                    }
                } else
                for (int c = lane; c < cols; c += 64) {
                    const int sx = sx_lo + c < s.w - 1 ? sx_lo + c : s.w - 1;
                    for (int r0 = wave; r0 < rows; r0 += WAVES * STAGE_ROWS) {
                        dev::PixelSlot<Src> px[STAGE_ROWS];
#pragma unroll
                        for (int u = 0; u < STAGE_ROWS; ++u) {
                            const int r = r0 + WAVES * u < rows ? r0 + WAVES * u : rows - 1;
                            const int sy = sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1;
                            if constexpr (RAW_SOURCE) {
                                const char* const row = window + static_cast<size_t>(sy) * s.pitch;
                                px[u] = dev::load_pixel_slot<Src>(row, sx * static_cast<int>(sizeof(Src)), valid_lo, valid_hi);
                            } else {
                                const Src value = fetch(v, sx, sy);
#pragma unroll
                                for (int i = 0; i < SLOT; ++i) px[u].w[i] = 0u;
                                __builtin_memcpy(px[u].w, &value, sizeof(Src));
                            }
                        }
#pragma unroll
                        for (int u = 0; u < STAGE_ROWS; ++u) {
                            const int r = r0 + WAVES * u < rows ? r0 + WAVES * u : rows - 1;
#pragma unroll
                            for (int i = 0; i < SLOT; ++i) tile[(r * stride + c) * SLOT + i] = px[u].w[i];
                        }
                    }
                }
            }
        }
        dev::block_sync();

        // ---- this thread's four pixels; the tap source is decided once for the block ----
        OutPixel o[RESIZE_PX];
        // interior tiles (whole tile inside the plane and inside the region that holds the image) need no per-pixel tests
        bool interior = tx0 + RESIZE_TILE_W <= v.w && ty0 + RESIZE_TILE_H <= v.h;
        if constexpr (View::HAS_ROI) {
            interior = interior && tx0 + v.off_x >= v.x1 && tx0 + RESIZE_TILE_W - 1 + v.off_x <= v.x2 && ty0 + v.off_y >= v.y1 &&
                       ty0 + RESIZE_TILE_H - 1 + v.off_y <= v.y2;
        }
        if (!resamples) {
            // a tile that lies wholly beside the image (the bars of a preserved aspect ratio): one value for all of it
            const OutPixel bar = dev::apply_tail(prog.tail, v.background);
#pragma unroll
            for (int k = 0; k < RESIZE_PX; ++k) o[k] = bar;
        } else if (staged) {
            if (interior) pixels<true, true>(prog, tile, window, sx_lo, sy_lo, stride, x_first, y, o);
            else pixels<true, false>(prog, tile, window, sx_lo, sy_lo, stride, x_first, y, o);
        } else {
            if (interior) pixels<false, true>(prog, tile, window, sx_lo, sy_lo, stride, x_first, y, o);
            else pixels<false, false>(prog, tile, window, sx_lo, sy_lo, stride, x_first, y, o);
        }

        // ---- write ----
        const bool whole_width = tx0 + RESIZE_TILE_W <= v.w; // block-uniform
        if constexpr (STAGE_OUT) {
            if (whole_width && (job.flags & FLAG_STAGE_OUT) != 0u) {
                constexpr int PIECES_PER_ROW = OUT_ROW_BYTES / 16;
                constexpr int MINE = RESIZE_PX * static_cast<int>(sizeof(OutPixel)) / 16;
                dev::u32x4* const stage = reinterpret_cast<dev::u32x4*>(lds_raw + job.out_stage_offset);
                // the buffer held the source tile: every thread is done with it
                if (job.out_stage_offset == 0u && (job.flags & FLAG_SOURCE_TILE) != 0u) dev::block_sync();
                // A wave's 64 threads own four whole rows of the tile (64 * MINE pieces), so a wave moves its rows
                // through its own part of the buffer and never waits for the other waves of the block.
                dev::u32x4 mine[MINE];
                __builtin_memcpy(mine, o, sizeof(mine));
#pragma unroll
                for (int j = 0; j < MINE; ++j) stage[tid * MINE + j] = mine[j];
                dev::wave_sync();
                // The wave's four rows start at a row address that is the same for all its lanes: it stays in scalar
                // registers and a lane adds a 32-bit offset.  Instruction j of a lane covers piece j * 64 + lane of the
                // wave's 4 * PIECES_PER_ROW: the end of row R0 for the lanes below THRESHOLD, the start of row R0 + 1
                // for the others, both known at compile time, so no division and no 64-bit arithmetic per lane.
                const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
                const int wave_first = wave * (64 * MINE);
                using GlobalPiece = __attribute__((address_space(1))) dev::u32x4*;
                using GlobalBytes = __attribute__((address_space(1))) char*;
                GlobalBytes wbase = (GlobalBytes)(reinterpret_cast<char*>(job.out.data) + static_cast<size_t>(bz) * job.out.z_stride +
                                                  static_cast<size_t>(ty0 + 4 * wave) * job.out.pitch + static_cast<size_t>(tx0) * sizeof(OutPixel));
                asm volatile("" : "+s"(wbase));
                const int rows_here = (v.h - ty0 < RESIZE_TILE_H ? v.h - ty0 : RESIZE_TILE_H) - 4 * wave; // of this wave's four
                const bool stream = (job.flags & FLAG_STREAM_STORES) != 0u;
                const unsigned pitch = job.out.pitch;
                // the two kinds of store in loops of their own: side by side in one loop body the compiler merges them
                // into a plain store
                const auto store_rows = [&](auto streaming, auto all_rows) { // all_rows: the wave's four rows lie in the plane
#pragma unroll
                    for (int j = 0; j < MINE; ++j) {
                        constexpr int PPR = PIECES_PER_ROW;
                        const int R0 = j * 64 / PPR;                   // row of the instruction's first piece
                        const int THRESHOLD = (R0 + 1) * PPR - j * 64; // lanes from here on are in row R0 + 1
                        const bool next_row = lane >= THRESHOLD;
                        const unsigned row_off = next_row ? static_cast<unsigned>(R0 + 1) * pitch - static_cast<unsigned>(THRESHOLD) * 16u
                                                          : static_cast<unsigned>(R0) * pitch + static_cast<unsigned>(j * 64 - R0 * PPR) * 16u;
                        const int r = R0 + (next_row ? 1 : 0);
                        if (decltype(all_rows)::value || r < rows_here) {
                            const GlobalPiece g = (GlobalPiece)(wbase + (row_off + static_cast<unsigned>(lane) * 16u));
                            const dev::u32x4 piece = stage[wave_first + j * 64 + lane];
                            if constexpr (decltype(streaming)::value) __builtin_nontemporal_store(piece, g);
                            else *g = piece;
                        }
                    }
                };
                if (stream) {
                    asm volatile("" ::: "memory"); // keep the streaming stores from being merged with the plain ones
                    if (rows_here >= 4) store_rows(std::true_type{}, std::true_type{});
                    else store_rows(std::true_type{}, std::false_type{});
                    asm volatile("" ::: "memory");
                } else {
                    store_rows(std::false_type{}, std::false_type{});
                }
                return;
            }
        }
        if (y >= v.h) return;
        if (x_first + RESIZE_PX <= v.w && (job.flags & FLAG_VECTOR_IO) != 0u && (Out::IS_SPLIT || RESIZE_PX * sizeof(OutPixel) == 16)) {
            dev::store_group_either<RESIZE_PX>((job.flags & FLAG_STREAM_STORES) != 0u, job.out, x_first, y, static_cast<int>(bz), o);
        } else {
#pragma unroll
            for (int k = 0; k < RESIZE_PX; ++k) {
                if (x_first + k < v.w) dev::store_one(job.out, x_first + k, y, static_cast<int>(bz), o[k]);
            }
        }
    }
};

// ---- generic -----------------------------------------------------------------------------------------------------
// A block covers 64*K x 4 elements; a thread computes K elements of one row, 64 apart (each of a wave's memory
// instructions still covers 64 neighbours).  A chain that only gathers and stores is bound by the memory round trip, one
// gather in flight per wave; with K = 4 a thread issues the reads of four elements before it uses any of them, provided
// the chain's read is straight-line code (lanes past the end of a row read its last element again instead of branching
// around the read).  K = 1 is kept for small outputs, which need every wave they can get.
constexpr unsigned GENERIC_WIDE_MIN_ELEMS = 1u << 22;
template <typename Sender, typename Receiver>
struct GenericJob {
    static constexpr bool READ_IN_PLACE = isBatchOperation<typename Sender::Operation> || isBatchOperation<typename Receiver::Operation>;
    using Value = std::decay_t<decltype(Sender::Operation::exec(Point(), std::declval<const Sender&>()))>;
    Sender sender;
    Receiver receiver;
    ActiveThreads active;
    unsigned grid_x, grid_y;
    unsigned wide; // 4 elements per thread instead of 1
    // A packed receiver whose pixels are not whole dwords (three bytes, say) would be written with byte stores.  With
    // four elements per thread such a job gives a thread four neighbouring pixels instead of four that are 64 apart:
    // they are sizeof(pixel) whole dwords of the row, packed in registers and stored at once.  (For every other job
    // neighbours are the slower choice: each memory instruction of a wave then covers a quarter of the lines' bytes.)
    using OutView = OutOf<Receiver>;
    template <typename V, typename = void>
    struct PacksRows : std::false_type {};
    template <typename V>
    struct PacksRows<V, std::enable_if_t<V::supported>>
        : std::bool_constant<!V::type::IS_SPLIT && sizeof(typename V::type::Pixel) % 4 != 0 && std::is_same_v<typename V::type::Pixel, Value>> {};
    static constexpr bool PACKS_ROWS = PacksRows<OutView>::value;
    // A packed receiver of whole-dword pixels (float3, float4, uchar4 ...): neighbouring lanes' stores make whole lines,
    // so a large output is written with streaming stores, straight to the receiver's memory.
    template <typename V, typename = void>
    struct StreamsRows : std::false_type {};
    template <typename V>
    struct StreamsRows<V, std::enable_if_t<V::supported>>
        : std::bool_constant<!V::type::IS_SPLIT && sizeof(typename V::type::Pixel) % 4 == 0 && std::is_same_v<typename V::type::Pixel, Value>> {};
    static constexpr bool STREAMS_ROWS = StreamsRows<OutView>::value;
    unsigned stream_rows; // decided by the host: large output, rows and planes at whole dwords (out_data etc. filled in)
    unsigned packs_rows; // the receiver's rows start at whole dwords (decided by the host, which then also fills in:)
    char* out_data;      // element (0, 0, 0) of the receiver, bytes between its rows and between its planes
    unsigned out_pitch;
    size_t out_z_stride;
    size_t lds_bytes() const { return 0; }
    // decides the elements per thread from the size of the output and returns the number of blocks along x
    unsigned plan(const ActiveThreads& extent) {
        const size_t elems = static_cast<size_t>(extent.x) * extent.y * extent.z;
        wide = (elems >= GENERIC_WIDE_MIN_ELEMS && extent.x >= 256u) ? 1u : 0u;
        const unsigned tile_w = wide != 0u ? 256u : 64u;
        return (extent.x + tile_w - 1u) / tile_w;
    }

    // K elements per thread: NEIGHBOURS, or 64 apart (then each of a wave's memory instructions covers 64 neighbours).
    template <int K, bool NEIGHBOURS>
    __device__ __attribute__((always_inline)) static inline void body(const GenericJob& job, unsigned bx, unsigned by, unsigned bz) {
        constexpr int STEP = NEIGHBOURS ? 1 : 64;
        const int tid = dev::thread_in_block();
        const int y = static_cast<int>(by) * 4 + (tid >> 6);
        const int w = static_cast<int>(job.active.x);
        const int x0 = static_cast<int>(bx) * (64 * K) + (tid & 63) * (NEIGHBOURS ? K : 1);
        if (x0 >= w || y >= static_cast<int>(job.active.y)) return;
        Value value[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int x = x0 + STEP * k < w ? x0 + STEP * k : w - 1;
            value[k] = Sender::Operation::exec(Point(x, y, static_cast<int>(bz)), job.sender);
        }
        if constexpr (PACKS_ROWS && NEIGHBOURS && K == 4) {
            if (job.packs_rows != 0u && x0 + K <= w) {
                constexpr int S = static_cast<int>(sizeof(Value)); // bytes per pixel = dwords per thread
                unsigned int words[S];
                dev::pack_pixels<K>(value, words);
                char* const run = job.out_data + static_cast<size_t>(bz) * job.out_z_stride + static_cast<size_t>(y) * job.out_pitch +
                                  static_cast<size_t>(x0) * S;
                if (job.stream_rows != 0u) {
                    asm volatile("" ::: "memory"); // keeps these stores apart from the plain ones (see store_group_either)
                    if constexpr (S == 3) {
                        typedef unsigned int u32x3 __attribute__((ext_vector_type(3)));
                        typedef u32x3 __attribute__((aligned(4))) u32x3_dword_aligned;
                        u32x3 v;
                        v.x = words[0]; v.y = words[1]; v.z = words[2];
                        __builtin_nontemporal_store(v, reinterpret_cast<u32x3_dword_aligned*>(run));
                    } else {
#pragma unroll
                        for (int i = 0; i < S; ++i) __builtin_nontemporal_store(words[i], reinterpret_cast<unsigned int*>(run) + i);
                    }
                    asm volatile("" ::: "memory");
                    return;
                }
                __builtin_memcpy(__builtin_assume_aligned(run, 4), words, 4 * S);
                return;
            }
        }
        if constexpr (STREAMS_ROWS) {
            if (job.stream_rows != 0u) {
                constexpr int S = static_cast<int>(sizeof(Value));
                char* const row = job.out_data + static_cast<size_t>(bz) * job.out_z_stride + static_cast<size_t>(y) * job.out_pitch;
                asm volatile("" ::: "memory"); // keeps these stores apart from the plain ones below (see store_group_either)
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    if (x0 + STEP * k < w) {
                        unsigned int words[S / 4];
                        __builtin_memcpy(words, &value[k], S);
                        char* const at = row + static_cast<size_t>(x0 + STEP * k) * S;
                        if constexpr (S == 12) { // one three-dword store, as the plain form of a float3 is
                            typedef unsigned int u32x3 __attribute__((ext_vector_type(3)));
                            typedef u32x3 __attribute__((aligned(4))) u32x3_dword_aligned;
                            u32x3 v;
                            v.x = words[0]; v.y = words[1]; v.z = words[2];
                            __builtin_nontemporal_store(v, reinterpret_cast<u32x3_dword_aligned*>(at));
                        } else {
                            dev::store_words<S, true>(at, words);
                        }
                    }
                }
                asm volatile("" ::: "memory");
                return;
            }
        }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (x0 + STEP * k < w) Receiver::Operation::exec(Point(x0 + STEP * k, y, static_cast<int>(bz)), value[k], job.receiver);
        }
    }
    __device__ __attribute__((always_inline)) static inline void run(const GenericJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char*) {
        if constexpr (PACKS_ROWS) { // the only jobs that are compiled with the neighbour form
            if (job.wide != 0u && job.packs_rows != 0u) {
                body<4, true>(job, bx, by, bz);
                return;
            }
        }
        if (job.wide != 0u) body<4, false>(job, bx, by, bz);
        else body<1, false>(job, bx, by, bz);
    }
};

// ---- entry points ------------------------------------------------------------------------------------------------
extern __shared__ unsigned char fk_dynamic_lds[];

// The job is the kernel's only argument, so it starts the kernel-argument segment.  It is read in place there
// (uniform, scalar loads) rather than through the by-value parameter: a plane picked with a run-time index would
// otherwise force a private copy of the whole job into scratch memory.
template <typename Job>
__device__ __attribute__((always_inline)) inline const Job& job_in_kernarg() {
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
    __device__ __attribute__((always_inline)) static inline void run(const JobPack&, unsigned, unsigned char*) {}
};
template <typename Job, typename... Rest>
struct JobPack<Job, Rest...> {
    Job job;
    unsigned blocks; // blocks of this job: grid_x * grid_y * planes
    JobPack<Rest...> rest;
    __device__ __attribute__((always_inline)) static inline void run(const JobPack& pack, unsigned block, unsigned char* lds) {
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

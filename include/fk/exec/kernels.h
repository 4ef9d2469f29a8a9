// The fused Transform kernels for gfx950 (CDNA4, wave64), hand-written against the views of fk/exec/views.h.
//
// Every launch runs blocks of 256 threads (four wave64).  A "job" is one fused chain over all its planes:
//   PointwiseJob  element-wise chains over a PlainView or a YuvView: each thread owns K consecutive pixels of a row so
//                 that both the source and the destination bytes of a thread are whole 16-byte (or 8/4-byte)
//                 transactions (a YUV thread loads its luma run and the chroma pairs that cover it);
//   ResizeJob     bilinear resize (with optional inner/outer crop and aspect-ratio border): a block owns an output tile
//                 of 64 columns by 16, 32 or 64 rows, a wave a quarter of its rows, a lane one column of them; the block
//                 stages the source bounding box of the tile in LDS as float taps (after the operations fused before the
//                 resize, e.g. YUV -> RGB, so those and the conversion run once per source pixel) and takes the 2x2 taps
//                 from there; tiles that gain nothing from it (down-scaling, no tap reuse) read their taps straight
//                 from memory; outputs are stored from registers, a row of 64 neighbouring pixels per wave;
//   GenericJob    one thread per output element (or four) through Operation::exec, for any chain the views cannot
//                 describe.
// blockIdx.z selects the plane of a batch; blocks that start outside their plane's own extent return at once.
// What one thread computes per element is the reference's TransformDPP::exec -> read -> compute... -> write
// (core/execution_model/data_parallel_patterns.h:120-181,254-268); the traversal, vector widths and LDS staging
// are this library's.  Build with -ffp-contract=off: results are compared bit for bit with an unfused evaluation.
#ifndef FK_EXEC_KERNELS_H
#define FK_EXEC_KERNELS_H

#include "fk/exec/views.h"

// clang emits a host-side stub for every __global__ function that refers to this runtime entry point; kernels are
// launched through fkrt_launch (which calls it with the stub's address), so only the declaration is needed here.  A
// translation unit that has included the HIP runtime's own header before this one already has it.
#if !defined(HIP_INCLUDE_HIP_HIP_RUNTIME_API_H)
struct fk_launch_dim3 {
    unsigned x, y, z;
};
extern "C" int hipLaunchKernel(const void* function_address, fk_launch_dim3 grid, fk_launch_dim3 block, void** args,
                               size_t lds_bytes, struct ihipStream_t* stream);
#endif

namespace fk {
namespace exec {

constexpr int BLOCK_THREADS = 256;

namespace dev {
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Streaming stores: `nt` keeps the written lines from displacing what the kernel still reads, `sc1` (device scope)
// sends them on to memory at once instead of holding them in the writer's L2; together they measured 3-4 % above `nt`
// alone on a write-only stream (6.06 against 5.79 TB/s in this kernel family's tile pattern).  Only for accesses where
// a wave writes whole cache lines (consecutive lanes, consecutive pieces).  The pair of bits is reachable through the
// buffer form of the store: a descriptor of the memory from an address on that is the same for the whole wave (it
// stays in scalar registers), a per-lane and a per-wave byte offset.
typedef unsigned int u32x3 __attribute__((ext_vector_type(3)));
constexpr int STREAM_POLICY = 0x12;            // nt | sc1
constexpr int WAVE_BUFFER_BYTES = 0x7fffffff;  // offsets are checked against this range; stores beyond it are dropped
__device__ __attribute__((always_inline)) inline __amdgpu_buffer_rsrc_t wave_buffer(void* wave_uniform_base) {
    return __builtin_amdgcn_make_buffer_rsrc(wave_uniform_base, 0, WAVE_BUFFER_BYTES, 0x00020000);
}
template <int ND, typename Words> // ND dwords (a three-element vector is as large as a four-element one)
__device__ __attribute__((always_inline)) inline void stream_store_at(const __amdgpu_buffer_rsrc_t buffer, const unsigned lane_offset,
                                                                    const unsigned wave_offset, const Words v) {
    static_assert(ND >= 1 && ND <= 4, "one to four dwords");
    if constexpr (ND == 1) __builtin_amdgcn_raw_buffer_store_b32(v, buffer, lane_offset, wave_offset, STREAM_POLICY);
    else if constexpr (ND == 2) __builtin_amdgcn_raw_buffer_store_b64(v, buffer, lane_offset, wave_offset, STREAM_POLICY);
    else if constexpr (ND == 3) __builtin_amdgcn_raw_buffer_store_b96(v, buffer, lane_offset, wave_offset, STREAM_POLICY);
    else __builtin_amdgcn_raw_buffer_store_b128(v, buffer, lane_offset, wave_offset, STREAM_POLICY);
}
// Range-checked loads through a buffer descriptor: a lane whose byte offset lies at or past `bytes` receives zero instead
// of faulting.  For boxes of an image that are fetched in aligned pieces, some of which may reach past the image's last
// row or lie past its last column.
__device__ __attribute__((always_inline)) inline __amdgpu_buffer_rsrc_t image_buffer(const void* wave_uniform_base, const unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(wave_uniform_base), 0, static_cast<int>(bytes), 0x00020000);
}
// the same address in every lane, for the compiler to see
__device__ __attribute__((always_inline)) inline char* wave_uniform(char* p) {
    const size_t a = reinterpret_cast<size_t>(p);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(a)));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(a >> 32)));
    return reinterpret_cast<char*>(static_cast<size_t>(hi) << 32 | lo);
}
// a pixel of 1-4 whole dwords as a register vector
template <typename O>
struct WordsOf {
    static constexpr int ND = static_cast<int>(sizeof(O)) / 4;
    typedef unsigned int vec_t __attribute__((ext_vector_type(ND == 1 ? 2 : ND))); // (a one-element vector type does not exist)
    using type = std::conditional_t<ND == 1, unsigned int, vec_t>;
    __device__ __attribute__((always_inline)) static inline type of(const O& v) {
        type w;
        __builtin_memcpy(&w, &v, sizeof(O));
        return w;
    }
};


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
// a pixel of three one-byte channels in the low three bytes of a dword, and back
template <typename P>
__device__ __attribute__((always_inline)) inline P unpack3(const unsigned int w) {
    static_assert(sizeof(P) == 3 && cn<P> == 3, "three one-byte channels");
    using B = VBase<P>;
    return P{ static_cast<B>(static_cast<unsigned char>(w)), static_cast<B>(static_cast<unsigned char>(w >> 8)), static_cast<B>(static_cast<unsigned char>(w >> 16)) };
}
template <typename P>
__device__ __attribute__((always_inline)) inline unsigned int pack3(const P& p) {
    static_assert(sizeof(P) == 3 && cn<P> == 3, "three one-byte channels");
    return static_cast<unsigned int>(static_cast<unsigned char>(p.x)) | static_cast<unsigned int>(static_cast<unsigned char>(p.y)) << 8 |
           static_cast<unsigned int>(static_cast<unsigned char>(p.z)) << 16;
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
    // ---- quads: pixels 4q .. 4q + 3 of a row of the PARENT image, fetched as the whole dwords they occupy ----
    // Three-byte pixels: a quad is twelve bytes, three dwords, when the image starts at a whole dword and its rows are a
    // whole number of dwords apart.
    static constexpr bool HAS_QUADS = sizeof(T) == 3 && alignof(T) == 1;
    using Quad = dev::u32x3;
    // bytes of the parent image from its first pixel to its last, up to the end of the last dword that holds one of them
    static size_t quad_extent(const View& v) {
        return ((static_cast<size_t>(v.img_h) - 1u) * v.pitch + static_cast<size_t>(v.img_w) * sizeof(T) + 3u) & ~static_cast<size_t>(3);
    }
    static bool quads_aligned(const View& v) { return reinterpret_cast<size_t>(v.data) % 4 == 0 && v.pitch % 4 == 0; }
    __device__ __attribute__((always_inline)) static inline __amdgpu_buffer_rsrc_t quad_buffer(const View& v) {
        const unsigned bytes = ((static_cast<unsigned>(v.img_h) - 1u) * v.pitch + static_cast<unsigned>(v.img_w) * static_cast<unsigned>(sizeof(T)) + 3u) & ~3u;
        return dev::image_buffer(v.data, bytes);
    }
    __device__ __attribute__((always_inline)) static inline Quad load_quad(const __amdgpu_buffer_rsrc_t image, const View& v, const int q, const int py) {
        return __builtin_amdgcn_raw_buffer_load_b96(image, static_cast<unsigned>(py) * v.pitch + static_cast<unsigned>(q) * 12u, 0, 0);
    }
    // the four pixels, each in the low three bytes of a dword
    __device__ __attribute__((always_inline)) static inline void quad_dwords(const Quad& w, unsigned int* px) {
        px[0] = w.x;
        px[1] = __builtin_amdgcn_alignbyte(w.y, w.x, 3u);
        px[2] = __builtin_amdgcn_alignbyte(w.z, w.y, 2u);
        px[3] = w.z >> 8u;
    }
    // the four pixels as their type, each channel taken from the byte of the dword that holds it (a conversion to float
    // that follows is then one instruction per channel)
    __device__ __attribute__((always_inline)) static inline void quad_pixels(const Quad& w, T* px) {
        using B = VBase<T>;
        const unsigned int d[3] = { w.x, w.y, w.z };
        const auto channel = [&](const int byte) { return static_cast<B>(static_cast<unsigned char>(d[byte >> 2] >> (8 * (byte & 3)))); };
#pragma unroll
        for (int k = 0; k < 4; ++k) px[k] = T{ channel(3 * k), channel(3 * k + 1), channel(3 * k + 2) };
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
    // ---- quads: pixels 4q .. 4q + 3 of a row of the parent image (8-bit formats) ----
    // 4:2:0 semi-planar: the four luma samples are one dword and the two chroma pairs that cover them another, at the same
    // byte offset of the chroma row; packed 4:2:2: two dwords of one row.
    static constexpr bool quads_supported() {
        if constexpr (sizeof(Base) != 1) return false;
        else if constexpr (Layout::semi_planar) return Layout::row_shift == 1;
        else return true;
    }
    static constexpr bool HAS_QUADS = quads_supported();
    using Quad = dev::u32x2;
    static constexpr unsigned rows_of(const unsigned img_h) { return Layout::semi_planar ? img_h + ((img_h + 1u) >> 1) : img_h; }
    static constexpr unsigned row_bytes_of(const unsigned img_w) { return Layout::semi_planar ? ((img_w + 1u) & ~1u) : 2u * ((img_w + 1u) & ~1u); }
    static size_t quad_extent(const View& v) {
        return ((static_cast<size_t>(rows_of(static_cast<unsigned>(v.img_h))) - 1u) * v.pitch + row_bytes_of(static_cast<unsigned>(v.img_w)) + 3u) & ~static_cast<size_t>(3);
    }
    static bool quads_aligned(const View& v) { return reinterpret_cast<size_t>(v.data) % 4 == 0 && v.pitch % 4 == 0; }
    __device__ __attribute__((always_inline)) static inline __amdgpu_buffer_rsrc_t quad_buffer(const View& v) {
        const unsigned bytes = ((rows_of(static_cast<unsigned>(v.img_h)) - 1u) * v.pitch + row_bytes_of(static_cast<unsigned>(v.img_w)) + 3u) & ~3u;
        return dev::image_buffer(v.data, bytes);
    }
    __device__ __attribute__((always_inline)) static inline Quad load_quad(const __amdgpu_buffer_rsrc_t image, const View& v, const int q, const int py) {
        Quad w;
        if constexpr (Layout::semi_planar) {
            const unsigned at = static_cast<unsigned>(q) * 4u;
            w.x = __builtin_amdgcn_raw_buffer_load_b32(image, static_cast<unsigned>(py) * v.pitch + at, 0, 0);
            w.y = __builtin_amdgcn_raw_buffer_load_b32(image, (static_cast<unsigned>(v.img_h) + (static_cast<unsigned>(py) >> 1)) * v.pitch + at, 0, 0);
        } else {
            w = __builtin_amdgcn_raw_buffer_load_b64(image, static_cast<unsigned>(py) * v.pitch + static_cast<unsigned>(q) * 8u, 0, 0);
        }
        return w;
    }
    // the four {Y, U, V} pixels; the two pixels of a pair receive the very same chroma values, so that what is computed from
    // the chroma alone (centring, products with the matrix) is computed once per pair
    __device__ __attribute__((always_inline)) static inline void quad_pixels(const Quad& w, Pixel* px) {
        if constexpr (Layout::semi_planar) {
            const Base cu[2] = { static_cast<Base>(w.y >> (8 * Layout::u)), static_cast<Base>(w.y >> (16 + 8 * Layout::u)) };
            const Base cv[2] = { static_cast<Base>(w.y >> (8 * Layout::v)), static_cast<Base>(w.y >> (16 + 8 * Layout::v)) };
#pragma unroll
            for (int k = 0; k < 4; ++k) px[k] = Pixel{ static_cast<Base>(w.x >> (8 * k)), cu[k >> 1], cv[k >> 1] };
        } else {
            const unsigned four[2] = { w.x, w.y }; // the samples of pixels 0, 1 and of pixels 2, 3
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const unsigned f = four[k >> 1];
                px[k] = Pixel{ static_cast<Base>(f >> (8 * ((k & 1) ? Layout::y1 : Layout::y0))), static_cast<Base>(f >> (8 * Layout::u)), static_cast<Base>(f >> (8 * Layout::v)) };
            }
        }
    }
};

// ---- planes that only receive a value ----------------------------------------------------------------------------
// A batch read with PlanePolicy::CONDITIONAL_WITH_DEFAULT yields its default value for every element of the planes from
// `used` on (reference batch_operations.h:234-241); those planes have the extent of the batch's thread grid.  A job of
// such a batch carries this, and its blocks of those planes write the value and nothing else.
template <typename O>
struct DefaultPlanes {
    static constexpr bool ENABLED = true;
    unsigned used; // planes that run their program; the rest receive `value`
    int w, h;      // extent of the planes that receive the value
    O value;
};
struct NoDefaultPlanes {
    static constexpr bool ENABLED = false;
};
namespace dev {
// Launch position l of n -> an index of 0 .. n-1 (a permutation) such that positions 8 apart, which run on the same XCD,
// get the indices 2k and 2k + 1: whole runs of sixteen positions are dealt out as eight such pairs, and a last run of
// more than eight positions as the pairs it has, followed by what is left.
__host__ __device__ __attribute__((always_inline)) inline unsigned deal_pairs(const unsigned l, const unsigned n) {
    const unsigned whole = n & ~15u;
    if (l < whole) {
        const unsigned p = l & 15u;
        return (l & ~15u) + 2u * (p & 7u) + (p >> 3);
    }
    const unsigned last = n - whole, k = l - whole;
    if (last <= 8u) return l;
    const unsigned pairs = last - 8u;
    if (k < pairs) return whole + 2u * k;
    if (k >= 8u) return whole + 2u * (k - 8u) + 1u;
    return l + pairs;
}
// the part of such a plane that lies in columns x0 .. x0 + nx - 1 of row y, written by one thread
template <typename Out, typename O>
__device__ __attribute__((always_inline)) inline void fill_default(const Out& out, const DefaultPlanes<O>& d, int x0, int nx, int y, int z) {
    if (y >= d.h) return;
    for (int x = x0; x < x0 + nx && x < d.w; ++x) store_one(out, x, y, z, d.value);
}
} // namespace dev

// ---- pointwise ---------------------------------------------------------------------------------------------------
enum : unsigned { FLAG_VECTOR_IO = 1u, FLAG_STREAM_STORES = 2u, FLAG_SOURCE_TILE = 4u, FLAG_WHOLE_BOX = 8u, FLAG_PACKED_TILE = 16u, FLAG_OFFSETS_32 = 32u, FLAG_PAIR_COLUMNS = 64u, FLAG_PAIR_TILES = 128u, FLAG_QUAD_FILL = 256u };

template <typename Prog, size_t N, typename Out, typename Defaults = NoDefaultPlanes>
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
    Defaults defaults;
    size_t lds_bytes() const { return LDS_BYTES; }

    // A block that lies on one row and owns `span` pixels of it from pixel bx0 on (a whole number of thread groups, so
    // the span is whole 16-byte pieces on both sides).  FULL: span is the block's whole 256*K pixels, nothing is guarded.
    template <bool FULL>
    __device__ __attribute__((always_inline)) static inline void row_block(const Out& job_out, const Plane& pl, const View& v, const unsigned pl_flags, int bx0, int span,
                                                                          int x0, int y, unsigned bz, int tid, unsigned char* lds) {
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
                reinterpret_cast<char*>(job_out.data) + static_cast<size_t>(bz) * job_out.z_stride +
                static_cast<size_t>(y) * job_out.pitch + static_cast<size_t>(bx0) * sizeof(OutPixel)) + wave * (64 * MINE);
            const int pieces = span * static_cast<int>(sizeof(OutPixel)) / 16 - wave * (64 * MINE);
            if ((pl_flags & FLAG_STREAM_STORES) != 0u) {
                // the wave's span starts at the same address for all its lanes
                const __amdgpu_buffer_rsrc_t span_buffer = dev::wave_buffer(dev::wave_uniform(reinterpret_cast<char*>(g)));
#pragma unroll
                for (int j = 0; j < MINE; ++j) {
                    if (FULL || j * 64 + lane < pieces) dev::stream_store_at<4>(span_buffer, static_cast<unsigned>(j * 64 + lane) * 16u, 0u, stage[j * 64 + lane]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < MINE; ++j) {
                    if (FULL || j * 64 + lane < pieces) g[j * 64 + lane] = stage[j * 64 + lane];
                }
            }
        } else if (active) {
            dev::store_group_either<K>((pl_flags & FLAG_STREAM_STORES) != 0u, job_out, x0, y, static_cast<int>(bz), o);
        }
    }

    __device__ __attribute__((always_inline)) static inline void run(const PointwiseJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char* lds) {
        if constexpr (Defaults::ENABLED) {
            if (bz >= job.defaults.used) {
                const int cols = 1 << job.tx_shift, t = dev::thread_in_block();
                dev::fill_default(job.out, job.defaults, (static_cast<int>(bx) * cols + (t & (cols - 1))) * K, K,
                                  static_cast<int>(by) * (BLOCK_THREADS >> job.tx_shift) + (t >> job.tx_shift), static_cast<int>(bz));
                return;
            }
        }
        // What the block needs from the job, read in one batch of scalar loads (a job that lies in the kernel arguments and is
        // read through a reference would otherwise fetch each field where it is first used, one dependent round trip after
        // the other); the tail stays where it is and is read while the pixels are on their way.
        const Plane& pl = job.plane[N == 1 ? 0u : bz];
        const View v = pl.prog.view;
        const unsigned pl_flags = pl.flags, job_grid_x = job.grid_x, job_pair_limit = job.pair_limit, job_tx_shift = job.tx_shift;
        const Out job_out = job.out;
        const int tid = dev::thread_in_block();
        // pair_limit != 0 (one row per block row, the source shares a chroma row between rows 2k and 2k + 1): workgroups go
        // to the eight XCDs round-robin in launch order, so blocks b and b + 8 run on the same XCD one after the other.
        // Giving them the same columns of rows 2k and 2k + 1 lets the second find the chroma row in that XCD's L2 instead
        // of fetching it from memory again through another one.  The first pair_limit blocks (a multiple of 16 and of two
        // block rows) are dealt out that way among themselves; the few after them keep their places.
        const unsigned launch_index = bx + job_grid_x * by;
        if (launch_index < job_pair_limit) {
            const unsigned xcd = launch_index & 7u, turn = launch_index >> 3;
            const unsigned pair = 8u * (turn >> 1) + xcd; // (columns, row pair) in the order the XCDs take them up
            const unsigned k = pair / job_grid_x;
            bx = pair - k * job_grid_x;
            by = 2u * k + (turn & 1u);
        }
        const int cols = 1 << job_tx_shift;
        const int x0 = (static_cast<int>(bx) * cols + (tid & (cols - 1))) * K;
        const int y = static_cast<int>(by) * (BLOCK_THREADS >> job_tx_shift) + (tid >> job_tx_shift);

        // FLAG_WHOLE_BOX (a batch of windows of different sizes): every plane produces the extent of the largest, as the
        // reference's thread grid does (batch_operations.h:153-160), so v.w x v.h is that box and elements beside the
        // plane's own window are the parent image's pixels there; where the box leaves the parent image the source pixel
        // is zero.
        bool whole_box = false;
        if constexpr (std::is_same_v<View, PlainView<Src>>) whole_box = (pl_flags & FLAG_WHOLE_BOX) != 0u;
        if constexpr (STAGE_IN || STAGE_OUT) {
            // block-uniform decisions
            const int bx0 = static_cast<int>(bx) * BLOCK_THREADS * K; // first pixel of the block
            const int span = v.w - bx0 < BLOCK_THREADS * K ? v.w - bx0 : BLOCK_THREADS * K;
            if ((pl_flags & FLAG_VECTOR_IO) != 0u && !whole_box && job_tx_shift == 8u && y < v.h && span > 0 && span % K == 0) {
                if (span == BLOCK_THREADS * K) row_block<true>(job_out, pl, v, pl_flags, bx0, span, x0, y, bz, tid, lds);
                else row_block<false>(job_out, pl, v, pl_flags, bx0, span, x0, y, bz, tid, lds);
                return;
            }
        }

        if (y >= v.h || x0 >= v.w) return;
        bool run_in_parent = true; // the thread's K pixels lie in the parent image
        if constexpr (std::is_same_v<View, PlainView<Src>>) {
            if (whole_box) run_in_parent = v.oy + y < v.img_h && v.ox + x0 + K <= v.img_w;
        }
        if ((pl_flags & FLAG_VECTOR_IO) != 0u && x0 + K <= v.w && run_in_parent) {
            Src in[K];
            Access::template load_group<K>(v, x0, y, in);
            OutPixel o[K];
#pragma unroll
            for (int k = 0; k < K; ++k) o[k] = dev::apply_tail(pl.prog.tail, in[k]);
            dev::store_group_either<K>((pl_flags & FLAG_STREAM_STORES) != 0u, job_out, x0, y, static_cast<int>(bz), o);
        } else {
            const int xe = x0 + K < v.w ? x0 + K : v.w;
            for (int x = x0; x < xe; ++x) {
                Src pixel{};
                bool in_parent = true;
                if constexpr (std::is_same_v<View, PlainView<Src>>) {
                    if (whole_box) in_parent = v.oy + y < v.img_h && v.ox + x < v.img_w;
                }
                if (in_parent) pixel = Access::load_one(v, x, y);
                dev::store_one(job_out, x, y, static_cast<int>(bz), dev::apply_tail(pl.prog.tail, pixel));
            }
        }
    }
};

// ---- resize ------------------------------------------------------------------------------------------------------
// A block owns an output tile of one plane, 64 columns by 4 * wave_rows rows: each of its four waves wave_rows rows of it
// (4, 8 or 16, chosen per launch), each lane one column of those.
constexpr int RESIZE_TILE_W = 64;
constexpr int RESIZE_GROUP_ROWS = 4;      // rows that a wave finishes, and writes, at a time
constexpr int RESIZE_MAX_WAVE_ROWS = 16;
constexpr int RESIZE_LDS_DWORDS = 6144;   // source tile capacity (24 KiB)
// Capacity of a tile of packed three-byte pixels (one dword each), for boxes that hold more source pixels than output
// pixels (down-scaling): 40 KiB, four such blocks per CU.
#ifndef FK_RESIZE_PACKED_DWORDS
#define FK_RESIZE_PACKED_DWORDS 10240
#endif
constexpr int RESIZE_PACKED_DWORDS = FK_RESIZE_PACKED_DWORDS;
// A taller tile is chosen only while the grid keeps this many blocks (measured: five planes of 1920 x 1080 are slower as
// 2550 tiles of 64 x 64 than as 5100 of 64 x 32), and only when every plane's tiles are staged in LDS.
constexpr size_t RESIZE_MIN_BLOCKS_16 = 4096, RESIZE_MIN_BLOCKS_8 = 1024;
static_assert(RESIZE_TILE_W == 64, "a lane per column");

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

template <typename Prog, size_t N, typename Out, typename Defaults = NoDefaultPlanes>
struct ResizeJob {
    using View = decltype(Prog::view);
    using SrcView = decltype(View::src);
    using Pre = decltype(View::pre);
    using Access = SourceAccess<SrcView>;
    using Src = typename View::Source; // the pixel that is interpolated: the source view's pixel after Pre
    using Pixel = typename View::Pixel;
    using OutPixel = typename Out::Pixel;
    // packed pixels read as they are: taps and staged pixels come straight from memory as dwords
    static constexpr bool RAW_SOURCE = std::is_same_v<SrcView, PlainView<Src>> && std::is_same_v<Pre, NoTail>;
    // What is interpolated: the channels of a source pixel as floats, which is what the blend makes of them anyway
    // (a channel times a float weight).  The tile holds them in that form, so a source pixel is converted once, when it
    // is staged, however many output pixels tap it.  Channels of doubles or 64-bit integers stay as they are and are
    // promoted by the blend itself.
    using Tap = std::conditional_t<(sizeof(VBase<Src>) <= 4), Pixel, Src>;
    static_assert(sizeof(Tap) % 4 == 0, "a tap is whole dwords");
    static constexpr int SLOT = static_cast<int>(sizeof(Tap)) / 4; // dwords of a source pixel in the tile
    static constexpr bool READ_IN_PLACE = N > 1;
    // A short tail is taken into registers once, at the start of the block (read in place it is fetched where it is used, once
    // per pixel and with the wait in the middle of the arithmetic); a long one is read in place.
    using Tail = std::decay_t<decltype(Prog::tail)>;
    using TailHeld = std::conditional_t<(sizeof(Tail) <= 128), Tail, const Tail&>;
    // Three-byte pixels (as they lie in memory, or as the operations fused before the resize leave them, e.g. YUV -> RGB)
    // can also be kept in the tile as one dword each.  Such a tile is filled from aligned pieces of the parent image's
    // rows, four pixels per lane and load, all of a box's loads in flight together; it serves the boxes that the tile of
    // float taps does not (down-scaling: more source pixels than output pixels), whose taps would otherwise be gathered
    // from memory one pixel per lane and load, and computed (YUV -> RGB) once per tap instead of once per source pixel.
    static constexpr bool PACKABLE = sizeof(Src) == 3 && alignof(Src) == 1 && sizeof(typename SrcView::Pixel) == 3 && Access::HAS_QUADS;
    // dwords of a pixel in such a tile: pixels as they lie in memory stay one dword (nothing is computed to fill the tile);
    // pixels that are computed are kept as the float taps the blend wants
    static constexpr int PSLOT = RAW_SOURCE ? 1 : SLOT;
    // such a tile is filled only while its box holds at most this many source pixels per output pixel (with more, the taps
    // that are used are a minority of the box: 3x down-scaling of 32 planes of 128x128 took 11.8 us with tiles, 6.2 us with
    // the taps read straight from memory)
    static constexpr int PACKED_MAX_RATIO = 4;
    Prog plane[N];
    Out out;
    unsigned grid_x, grid_y;
    // FLAG_STREAM_STORES: large output whose rows start at whole dwords; FLAG_SOURCE_TILE / FLAG_PACKED_TILE: some plane's
    // tiles are staged in LDS, as float taps / as packed pixels, which decides how much LDS the launch asks for (a
    // divergent launch shares one LDS size between all its jobs).
    unsigned flags;
    // Rows of the tile that each of the block's four waves computes (4, 8 or 16: the tile is 64 x 4 * wave_rows).
    // What a wave does once (the tile's source box, its lanes' columns) is shared by more rows in a taller tile; a
    // launch of few tiles keeps them small so that the grid still fills the device.
    unsigned wave_rows;
    // The launch asks for as much LDS as the planes' own factors need, not for the capacity: a block's LDS decides how
    // many blocks a CU holds.  tile_dwords is the room for a source tile (a tile that needs more reads its taps directly).
    unsigned tile_dwords;
    Defaults defaults;
    size_t lds_bytes() const { return (flags & (FLAG_SOURCE_TILE | FLAG_PACKED_TILE)) != 0u ? static_cast<size_t>(tile_dwords) * 4 + 16 : 0; }
    int tile_h() const { return (BLOCK_THREADS / 64) * static_cast<int>(wave_rows); }
    // dwords a tile of a plane with these factors takes when staged, 0 when it is not worth staging (same rule as the
    // kernel applies per tile)
    static unsigned staged_tile_dwords(float fx, float fy, int tile_h) {
        // strong down-scaling is never staged; this also keeps the factors of a plane whose resized image has no
        // extent at all (infinite: such a plane is all background) out of the integer arithmetic below
        if (!(fx >= 0.f && fx <= 8.f && fy >= 0.f && fy <= 8.f)) return 0u;
        const int cols = static_cast<int>((RESIZE_TILE_W - 1) * fx) + 3, rows = static_cast<int>((tile_h - 1) * fy) + 3;
        const bool worth = rows * (cols | 1) * SLOT <= RESIZE_LDS_DWORDS && rows * cols <= 3 * RESIZE_TILE_W * tile_h + 256;
        return worth ? static_cast<unsigned>(rows * (cols | 1) * SLOT) : 0u;
    }
    // dwords of a tile of float taps that is filled from aligned groups of four pixels (an upper bound of what any tile of
    // a plane with these factors needs), 0 when the plane's tiles are not worth float taps or too wide for it: a row of the
    // tile holds the groups that cover the box's columns and one group more, for the copy of the window's last column
    static unsigned quad_filled_tile_dwords(float fx, float fy, int tile_h) {
        if (staged_tile_dwords(fx, fy, tile_h) == 0u) return 0u;
        const int cols = static_cast<int>((RESIZE_TILE_W - 1) * fx) + 3, rows = static_cast<int>((tile_h - 1) * fy) + 3;
        const int quads = (cols + 6) / 4;
        const unsigned need = static_cast<unsigned>(rows * 4 * (quads + 1) * SLOT);
        // (one group per thread: boxes that need two per thread are filled no faster this way than one pixel per thread: five
        // 1024x768 crops to 1920x1080 with bars, boxes of 47 x 25 pixels, 23.2-24.3 us by machine against 23.1 us)
        return rows * quads <= BLOCK_THREADS && need <= static_cast<unsigned>(RESIZE_PACKED_DWORDS) ? need : 0u;
    }
    // whether the byte offset of every pixel of a window, from the window's first pixel, fits 32 bits (with room for the
    // few bytes that an access adds)
    static bool window_fits_32_bits(const SrcView& s) {
        const size_t rows = s.h > 0 ? static_cast<size_t>(s.h) : 1u, cols = s.w > 0 ? static_cast<size_t>(s.w) : 0u;
        return (rows - 1u) * s.pitch + cols * sizeof(Src) + 16u < (static_cast<size_t>(1) << 32);
    }
    // dwords of a tile of packed pixels for a plane with these factors (an upper bound of what any of its tiles needs), 0
    // when such a tile is not possible: `cols` pixels of a row lie in at most (cols + 6) / 4 aligned groups of four
    static unsigned packed_tile_dwords(float fx, float fy, int tile_h, unsigned capacity) {
        if (!(fx >= 0.f && fx <= 16.f && fy >= 0.f && fy <= 16.f)) return 0u;
        const int cols = static_cast<int>((RESIZE_TILE_W - 1) * fx) + 3, rows = static_cast<int>((tile_h - 1) * fy) + 3;
        const int quads = (cols + 6) / 4;
        const unsigned need = static_cast<unsigned>(rows * quads * 4 * PSLOT);
        return quads <= 64 && need <= capacity && rows * cols <= PACKED_MAX_RATIO * RESIZE_TILE_W * tile_h + 256 ? need : 0u;
    }
    // Chooses the tile height and the LDS size from the factors of the first `count` planes; grid_x has been decided,
    // max_h is the tallest plane.  Returns the number of tile rows (grid_y).
    unsigned plan(size_t count, int max_h, unsigned forced_wave_rows, unsigned packed_capacity = RESIZE_PACKED_DWORDS) {
        // the tallest tile that still leaves the grid enough blocks, and whose source boxes all fit the LDS
        const auto blocks = [&](unsigned wr) { return count * grid_x * ((static_cast<unsigned>(max_h) + 4u * wr - 1u) / (4u * wr)); };
        const auto staged_planes = [&](unsigned wr) {
            unsigned n = 0;
            for (size_t i = 0; i < count; ++i) n += staged_tile_dwords(plane[i].view.fx, plane[i].view.fy, 4 * static_cast<int>(wr)) != 0u ? 1u : 0u;
            return n;
        };
        // (tiles whose taps come straight from memory stay small: measured, eight 1920x1080 planes to 1280x720 take 30.8 us
        // as 64 x 16 tiles and 33.8 us as 64 x 32, although the taller tile executes fewer instructions)
        wave_rows = RESIZE_GROUP_ROWS;
        if (blocks(16) >= RESIZE_MIN_BLOCKS_16 && staged_planes(16) == count) wave_rows = 16;
        else if (blocks(8) >= RESIZE_MIN_BLOCKS_8 && staged_planes(8) == count) wave_rows = 8;
        if (forced_wave_rows == 4u || forced_wave_rows == 8u || forced_wave_rows == 16u) wave_rows = forced_wave_rows;
        // 32-bit byte offsets from a window's first pixel to any of its pixels (the staging loop of three-byte sources and
        // the line touches use them): only when every plane's window spans less than 4 GiB; otherwise nothing is staged
        // or touched, and the taps are read with 64-bit row addresses
        bool narrow = true;
        if constexpr (RAW_SOURCE && sizeof(Src) == 3) {
            for (size_t i = 0; i < count; ++i) narrow = narrow && window_fits_32_bits(plane[i].view.src);
        }
        packed_capacity = packed_capacity < static_cast<unsigned>(RESIZE_PACKED_DWORDS) ? packed_capacity : static_cast<unsigned>(RESIZE_PACKED_DWORDS);
        tile_dwords = 0;
        if (!narrow) return (static_cast<unsigned>(max_h) + static_cast<unsigned>(tile_h()) - 1u) / static_cast<unsigned>(tile_h()); // no tiles: 64-bit addressed taps only
        flags |= FLAG_OFFSETS_32;
        bool packable = PACKABLE && packed_capacity != 0u;
        if constexpr (PACKABLE) {
            // (the kernel addresses a parent image with 32-bit offsets through a descriptor)
            for (size_t i = 0; i < count; ++i) packable = packable && Access::quad_extent(plane[i].view.src) < (static_cast<size_t>(1) << 31);
        }
        for (size_t i = 0; i < count; ++i) {
            const unsigned need = staged_tile_dwords(plane[i].view.fx, plane[i].view.fy, tile_h());
            if (need != 0u) flags |= FLAG_SOURCE_TILE;
            tile_dwords = need > tile_dwords ? need : tile_dwords;
            if constexpr (PACKABLE && RAW_SOURCE) {
                // (launches of 64 x 16 tiles keep the fill of one pixel per thread: the 50-crop batch took 13.35 us this way
                // against 13.05 us, the 16:9 crops in 64 x 32 tiles 22.9 against 23.5 us)
                if (need != 0u && wave_rows >= 8u && packable && Access::quads_aligned(plane[i].view.src)) {
                    const unsigned filled = quad_filled_tile_dwords(plane[i].view.fx, plane[i].view.fy, tile_h());
                    if (filled != 0u) flags |= FLAG_QUAD_FILL;
                    tile_dwords = filled > tile_dwords ? filled : tile_dwords;
                }
            }
            if constexpr (PACKABLE) {
                if (need == 0u && packable && Access::quads_aligned(plane[i].view.src)) {
                    const unsigned packed = packed_tile_dwords(plane[i].view.fx, plane[i].view.fy, tile_h(), packed_capacity);
                    if (packed != 0u) flags |= FLAG_PACKED_TILE;
                    tile_dwords = packed > tile_dwords ? packed : tile_dwords;
                }
            }
        }
        return (static_cast<unsigned>(max_h) + static_cast<unsigned>(tile_h()) - 1u) / static_cast<unsigned>(tile_h());
    }

    // source pixel (x, y) of the resampled window, after the operations fused before the resize
    __device__ __attribute__((always_inline)) static inline Src fetch(const View& v, int x, int y) {
        return dev::apply_tail(v.pre, Access::load_one(v.src, x, y));
    }
    __device__ __attribute__((always_inline)) static inline Tap to_tap(const Src& p) {
        if constexpr (std::is_same_v<Tap, Src>) return p;
        else return fk::detail::cast_channels<Tap>(p);
    }
    __device__ __attribute__((always_inline)) static inline Tap load_tap(const unsigned int* p) {
        unsigned int w[SLOT];
#pragma unroll
        for (int k = 0; k < SLOT; ++k) w[k] = p[k];
        Tap t;
        __builtin_memcpy(&t, w, sizeof(Tap));
        return t;
    }
    __device__ __attribute__((always_inline)) static inline void store_tap(unsigned int* p, const Tap& t) {
        unsigned int w[SLOT];
        __builtin_memcpy(w, &t, sizeof(Tap));
#pragma unroll
        for (int k = 0; k < SLOT; ++k) p[k] = w[k];
    }
    __device__ __attribute__((always_inline)) static inline float lane_float(const float value, const int lane) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, value), lane));
    }

    // The rows of a wave (rows wy0 .. wy0 + wave_rows - 1 of the plane), one column per lane (column x), four rows at a
    // time.  What depends on the column alone is computed once for all the rows.  What depends on the row alone is the
    // same for the whole wave: lane i (i < wave_rows) computes it for row i and it is read from there.
    // `put(g, k, pixel)` takes the finished pixel of row g + k (g the group's first row, k = 0..3 known at compile time).
    // MODE: where the taps come from: TAPS_DIRECT from memory, TAPS_FLOAT_TILE from the tile of float taps (columns from
    // sx_lo, rows from sy_lo, `stride` pixels per row, edge copies included), TAPS_PACKED_TILE from the tile of packed pixels
    // (column 0 is window column tile_x0, rows from sy_lo, `stride` dwords per row, only pixels that exist).
    enum : int { TAPS_DIRECT = 0, TAPS_FLOAT_TILE = 1, TAPS_PACKED_TILE = 2 };
    template <int MODE, bool INTERIOR, typename Put>
    __device__ __attribute__((always_inline)) static inline void sweep(const View& v, const TailHeld& tail, const unsigned int* tile, const char* window, const int sx_lo,
                                                                      const int sy_lo, const int stride, const int tile_x0, const int x, const int wy0,
                                                                      const int lane, const int wave_rows, const Put& put) {
        const SrcView& s = v.src;

        // ---- this lane's column ----
        const int rx = x + v.off_x;
        bool col_in = INTERIOR || x < v.w;
        if constexpr (View::HAS_ROI && !INTERIOR) col_in = col_in && rx >= v.x1 && rx <= v.x2;
        const float src_x = static_cast<float>(rx - v.x1) * v.fx;
        // floor() in float: for |x| < 2^24 the float of x1 is floor(src_x) itself, src_x - x1 is exact, and x2 - src_x,
        // one rounding of 1 - (src_x - x1), is 1.0f minus that difference (fk::detail::bilinear_taps)
        const float x1f = __builtin_floorf(src_x);
        const float wx1 = src_x - x1f, wx0 = 1.0f - wx1;
        const int x1 = col_in ? static_cast<int>(x1f) : sx_lo; // a column beside the image reads (and discards) a valid tap

        // ---- row (lane & 15) of the wave, for the lanes that are asked for it ----
        const int yi = wy0 + (lane & (RESIZE_MAX_WAVE_ROWS - 1));
        const int ry = yi + v.off_y;
        bool row_in = INTERIOR || yi < v.h;
        if constexpr (View::HAS_ROI && !INTERIOR) row_in = row_in && ry >= v.y1 && ry <= v.y2;
        const float src_y = static_cast<float>(ry - v.y1) * v.fy;
        const float y1f = __builtin_floorf(src_y);
        const float wy1 = src_y - y1f, wy0f = 1.0f - wy1;
        const int y1 = row_in ? static_cast<int>(y1f) : sy_lo;
        unsigned rows_in = 0xFFFFu;
        if constexpr (!INTERIOR) rows_in = static_cast<unsigned>(__builtin_amdgcn_ballot_w64(row_in)) & 0xFFFFu;

        const auto emit = [&](const int g, const auto k, const Tap& a, const Tap& b, const Tap& c, const Tap& d) {
            const int i = g + decltype(k)::value;
            const float gy = lane_float(wy0f, i), fy = lane_float(wy1, i);
            fk::detail::BilinearTaps t{};
            t.wa = wx0 * gy;
            t.wb = wx1 * gy;
            t.wc = wx0 * fy;
            t.wd = wx1 * fy;
            Pixel value = fk::detail::bilinear_blend(a, b, c, d, t);
            if constexpr (!INTERIOR) {
                if (!(col_in && (rows_in >> i & 1u) != 0u)) value = v.background;
            }
            put(g, k, dev::apply_tail(tail, value));
        };
        const auto each_of_group = [](const auto& body) {
            body(std::integral_constant<int, 0>{});
            body(std::integral_constant<int, 1>{});
            body(std::integral_constant<int, 2>{});
            body(std::integral_constant<int, 3>{});
        };
        static_assert(RESIZE_GROUP_ROWS == 4, "the group is written out above");

        if constexpr (MODE == TAPS_PACKED_TILE) {
            // the tile holds the pixels of the window as they are: the second taps are clamped to its last column and row
            const int x2 = x1 + 1 < s.w - 1 ? x1 + 1 : s.w - 1;
            const int y2 = y1 + 1 < s.h - 1 ? y1 + 1 : s.h - 1;
            const unsigned int* const column_a = tile + (x1 - tile_x0) * PSLOT;
            const unsigned int* const column_b = tile + (x2 - tile_x0) * PSLOT;
            const int row_a = (y1 - sy_lo) * stride * PSLOT, row_b = (y2 - sy_lo) * stride * PSLOT;
            const auto pixel = [](const unsigned int* p) {
                if constexpr (RAW_SOURCE) return to_tap(dev::unpack3<Src>(*p));
                else return load_tap(p);
            };
            for (int g = 0; g < wave_rows; g += RESIZE_GROUP_ROWS) {
                each_of_group([&](const auto k) {
                    const int ra = __builtin_amdgcn_readlane(row_a, g + decltype(k)::value), rb = __builtin_amdgcn_readlane(row_b, g + decltype(k)::value);
                    emit(g, k, pixel(column_a + ra), pixel(column_b + ra), pixel(column_a + rb), pixel(column_b + rb));
                });
            }
        } else if constexpr (MODE == TAPS_FLOAT_TILE) {
            // the tile holds columns sx_lo.. and rows sy_lo.., edge copies included: no clamping here
            const unsigned int* const column = tile + (x1 - sx_lo) * SLOT;
            const int row_dwords = stride * SLOT;
            const int tile_row = y1 - sy_lo;
            for (int g = 0; g < wave_rows; g += RESIZE_GROUP_ROWS) {
                each_of_group([&](const auto k) {
                    const unsigned int* const p = column + __builtin_amdgcn_readlane(tile_row, g + decltype(k)::value) * row_dwords;
                    emit(g, k, load_tap(p), load_tap(p + SLOT), load_tap(p + row_dwords), load_tap(p + row_dwords + SLOT));
                });
            }
        } else {
            // taps straight from memory, those of a group's four rows requested before the first is used
            const int x2 = x1 + 1 < s.w - 1 ? x1 + 1 : s.w - 1;
            const int y2 = y1 + 1 < s.h - 1 ? y1 + 1 : s.h - 1;
            if constexpr (RAW_SOURCE && sizeof(Src) == 3) {
                if ((s.pitch & 3u) == 0u) {
                    // Three-byte pixels, rows a whole number of dwords apart: a column has the same alignment in every
                    // row, so the offset of the dword that holds the pixel (from one byte before the row, see
                    // load_dword_from_row) and the shift that takes it out are found once per lane; a row's address is
                    // the same for the whole wave.
                    const unsigned base = static_cast<unsigned>(reinterpret_cast<size_t>(window));
                    const unsigned off1 = static_cast<unsigned>(x1) * 3u, off2 = static_cast<unsigned>(x2) * 3u;
                    const bool al1 = ((base + off1) & 3u) == 0u, al2 = ((base + off2) & 3u) == 0u;
                    const unsigned voff1 = off1 + (al1 ? 1u : 0u), voff2 = off2 + (al2 ? 1u : 0u);
                    const unsigned sh1 = al1 ? 0u : 8u, sh2 = al2 ? 0u : 8u;
                    const auto pixel = [](const unsigned int w) {
                        dev::PixelSlot<Src> px;
                        px.w[0] = w;
                        return to_tap(dev::slot_to_pixel<Src>(px));
                    };
                    for (int g = 0; g < wave_rows; g += RESIZE_GROUP_ROWS) {
                        unsigned int a[RESIZE_GROUP_ROWS], b[RESIZE_GROUP_ROWS], c[RESIZE_GROUP_ROWS], d[RESIZE_GROUP_ROWS];
#pragma unroll
                        for (int k = 0; k < RESIZE_GROUP_ROWS; ++k) {
                            const int ya = __builtin_amdgcn_readlane(y1, g + k), yb = __builtin_amdgcn_readlane(y2, g + k);
                            const char* const r0 = window + static_cast<size_t>(ya) * s.pitch;
                            const char* const r1 = window + static_cast<size_t>(yb) * s.pitch;
                            a[k] = dev::load_dword_from_row(r0, voff1);
                            b[k] = dev::load_dword_from_row(r0, voff2);
                            c[k] = dev::load_dword_from_row(r1, voff1);
                            d[k] = dev::load_dword_from_row(r1, voff2);
                        }
                        each_of_group([&](const auto k) {
                            constexpr int K = decltype(k)::value;
                            emit(g, k, pixel(a[K] >> sh1), pixel(b[K] >> sh2), pixel(c[K] >> sh1), pixel(d[K] >> sh2));
                        });
                    }
                    return;
                }
            }
            for (int g = 0; g < wave_rows; g += RESIZE_GROUP_ROWS) {
                Src a[RESIZE_GROUP_ROWS], b[RESIZE_GROUP_ROWS], c[RESIZE_GROUP_ROWS], d[RESIZE_GROUP_ROWS];
#pragma unroll
                for (int k = 0; k < RESIZE_GROUP_ROWS; ++k) {
                    const int ya = __builtin_amdgcn_readlane(y1, g + k), yb = __builtin_amdgcn_readlane(y2, g + k);
                    if constexpr (RAW_SOURCE) {
                        const Src* const r0 = reinterpret_cast<const Src*>(window + static_cast<size_t>(ya) * s.pitch);
                        const Src* const r1 = reinterpret_cast<const Src*>(window + static_cast<size_t>(yb) * s.pitch);
                        a[k] = fk::detail::read_element(r0 + x1);
                        b[k] = fk::detail::read_element(r0 + x2);
                        c[k] = fk::detail::read_element(r1 + x1);
                        d[k] = fk::detail::read_element(r1 + x2);
                    } else {
                        a[k] = fetch(v, x1, ya);
                        b[k] = fetch(v, x2, ya);
                        c[k] = fetch(v, x1, yb);
                        d[k] = fetch(v, x2, yb);
                    }
                }
                each_of_group([&](const auto k) {
                    constexpr int K = decltype(k)::value;
                    emit(g, k, to_tap(a[K]), to_tap(b[K]), to_tap(c[K]), to_tap(d[K]));
                });
            }
        }
    }

    __device__ __attribute__((always_inline)) static inline void run(const ResizeJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char* lds_raw) {
        if constexpr (Defaults::ENABLED) {
            if (bz >= job.defaults.used) {
                const int t = dev::thread_in_block(), rows = static_cast<int>(job.wave_rows);
                const int y0 = (static_cast<int>(by) * (BLOCK_THREADS / 64) + (t >> 6)) * rows;
                for (int i = 0; i < rows; ++i) {
                    dev::fill_default(job.out, job.defaults, static_cast<int>(bx) * RESIZE_TILE_W + (t & 63), 1, y0 + i, static_cast<int>(bz));
                }
                return;
            }
        }
        // Everything the block needs from the job is read here, in one batch of scalar loads with one wait: the job's own
        // fields, the plane's view BY VALUE, and the tail.  Read where they are used (through a reference into the kernel
        // arguments), the same fields arrive one dependent load after the other, ten round trips to the scalar cache between
        // the start of a block and its first memory request.
        const Prog& prog = job.plane[N == 1 ? 0u : bz];
        const View v = prog.view;
        const TailHeld tail = prog.tail;
        const unsigned job_flags = job.flags, job_tile_dwords = job.tile_dwords;
        const Out out = job.out;
        const SrcView& s = v.src;
        const int wave_rows = static_cast<int>(job.wave_rows);
        // FLAG_PAIR_COLUMNS / FLAG_PAIR_TILES: workgroups reach the eight XCDs round-robin in launch order, and each XCD has an
        // L2 of its own.  Two tiles that are neighbours along x read the same cache lines where their source boxes meet (a
        // tile's row of source pixels is often shorter than a line), so the blocks of a row of tiles (of a whole plane, when
        // its rows are a power of two of at most eight tiles) are dealt out such that launch positions p and p + 8, which
        // run on the same XCD at the same time, work on columns 2k and 2k + 1: the second request for a shared line is
        // served by that XCD's L2.
        if ((job_flags & FLAG_PAIR_COLUMNS) != 0u) {
            bx = dev::deal_pairs(bx, job.grid_x);
        } else if ((job_flags & FLAG_PAIR_TILES) != 0u) {
            const unsigned gx = job.grid_x, shift = 31u - static_cast<unsigned>(__builtin_clz(gx));
            const unsigned t = dev::deal_pairs(bx + (by << shift), gx * job.grid_y);
            bx = t & (gx - 1u);
            by = t >> shift;
        }
        const int tile_h = (BLOCK_THREADS / 64) * wave_rows;
        const int tx0 = static_cast<int>(bx) * RESIZE_TILE_W;
        const int ty0 = static_cast<int>(by) * tile_h;
        if (tx0 >= v.w || ty0 >= v.h) return; // block outside this plane's own extent
        const int tid = dev::thread_in_block();

        // part of the tile that resamples the source, in resize coordinates (after the outer crop offset)
        int rx_lo = tx0 + v.off_x, rx_hi = (tx0 + RESIZE_TILE_W < v.w ? tx0 + RESIZE_TILE_W : v.w) - 1 + v.off_x;
        int ry_lo = ty0 + v.off_y, ry_hi = (ty0 + tile_h < v.h ? ty0 + tile_h : v.h) - 1 + v.off_y;
        if constexpr (View::HAS_ROI) {
            rx_lo = rx_lo > v.x1 ? rx_lo : v.x1;
            rx_hi = rx_hi < v.x2 ? rx_hi : v.x2;
            ry_lo = ry_lo > v.y1 ? ry_lo : v.y1;
            ry_hi = ry_hi < v.y2 ? ry_hi : v.y2;
        }
        const bool resamples = rx_lo <= rx_hi && ry_lo <= ry_hi;

        unsigned int* const tile = reinterpret_cast<unsigned int*>(lds_raw);
        bool staged = false; // the tile holds float taps
        bool packed = false; // the tile holds packed pixels
        int sx_lo = 0, sy_lo = 0;
        int stride = 0;  // source pixels per tile row
        int tile_x0 = 0; // window column of the tile's column 0
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
            staged = (job_flags & FLAG_SOURCE_TILE) != 0u && rows * stride * SLOT <= static_cast<int>(job_tile_dwords) && rows * stride * SLOT <= RESIZE_LDS_DWORDS &&
                     rows * cols <= 3 * tile_px + 256;
            tile_x0 = sx_lo;
            if constexpr (PACKABLE) {
                // A box that is not worth a tile of float taps as above (down-scaling: few taps per source pixel), of an image
                // that starts at a whole dword with rows a whole number of dwords apart: the aligned groups of four pixels
                // that cover the box's columns, in the rows of it that exist, each fetched by one thread with one load (two
                // for 4:2:0 sources) through a descriptor of the whole parent image (a group that reaches past the image's
                // last row end reads zeros there and cannot fault).  Pixels as they lie in memory are kept as one dword
                // each; pixels that are computed (operations fused before the resize) are kept as float taps, computed once
                // per source pixel.  Thread t takes groups t, t + 256, ... of the box (rows of `quads` groups); the loads of up
                // to four of them are issued before the first is used, so a box costs one memory round trip.
                const int box_px = rows * cols;
                if (!staged && (job_flags & FLAG_PACKED_TILE) != 0u && box_px <= PACKED_MAX_RATIO * tile_px + 256 &&
                    ((static_cast<unsigned>(reinterpret_cast<size_t>(s.data)) | s.pitch) & 3u) == 0u) {
                    const int last_c = sx_lo + cols - 1 < s.w - 1 ? sx_lo + cols - 1 : s.w - 1; // window columns sx_lo .. last_c
                    const int last_r = sy_lo + rows - 1 < s.h - 1 ? sy_lo + rows - 1 : s.h - 1;
                    const int q_lo = (s.ox + sx_lo) >> 2;
                    const int quads = ((s.ox + last_c) >> 2) - q_lo + 1, box_rows = last_r - sy_lo + 1;
                    const int items = box_rows * quads;
                    if (quads >= 1 && quads <= 64 && box_rows >= 1 && items * 4 * PSLOT <= static_cast<int>(job_tile_dwords)) {
                        packed = true;
                        stride = quads * 4;
                        tile_x0 = 4 * q_lo - s.ox;
                        constexpr int PASSES = 4;
                        const int wave_of_block = __builtin_amdgcn_readfirstlane(tid >> 6);
                        // item / quads as (item * m) >> 20: exact for every item below N when 2^20 / quads <= m < 2^20 / quads *
                        // (1 + 1 / N).  The reciprocal instruction is within 2^-22 of 1 / quads, so its product with 2^20,
                        // truncated, plus 2 lies between 2^20 / quads + 0.7 and 2^20 / quads + 2.3; with quads <= 64 and fewer
                        // than 2560 items (a tile is 10240 dwords at most) the upper limit is 2^20 / quads + 6.4.
                        static_assert(RESIZE_PACKED_DWORDS <= 10240, "the division by multiplication is exact for fewer than 2560 items");
                        const unsigned m = static_cast<unsigned>(1048576.0f * __builtin_amdgcn_rcpf(static_cast<float>(quads))) + 2u;
                        const __amdgpu_buffer_rsrc_t image = Access::quad_buffer(s);
                        const int py0 = s.oy + sy_lo;
                        for (int first = 0; first < items; first += BLOCK_THREADS * PASSES) { // (uniform)
                            typename Access::Quad raw[PASSES];
                            // (no branch between the loads: groups past the box's last repeat it, from the cache)
#pragma unroll
                            for (int u = 0; u < PASSES; ++u) {
                                const int wanted = first + BLOCK_THREADS * u + tid;
                                const int item = wanted < items ? wanted : items - 1;
                                const int r = static_cast<int>((static_cast<unsigned>(item) * m) >> 20);
                                raw[u] = Access::load_quad(image, s, q_lo + (item - r * quads), py0 + r);
                            }
#pragma unroll
                            for (int u = 0; u < PASSES; ++u) {
                                if (first + BLOCK_THREADS * u + 64 * wave_of_block < items) { // (uniform: some group of this wave's pass exists)
                                    const int wanted = first + BLOCK_THREADS * u + tid;
                                    const int item = wanted < items ? wanted : items - 1;
                                    if constexpr (RAW_SOURCE) {
                                        unsigned int px[4];
                                        Access::quad_dwords(raw[u], px);
                                        dev::u32x4 piece;
                                        piece.x = px[0]; piece.y = px[1]; piece.z = px[2]; piece.w = px[3];
                                        *reinterpret_cast<dev::u32x4*>(tile + item * 4) = piece;
                                    } else {
                                        typename SrcView::Pixel px[4];
                                        Access::quad_pixels(raw[u], px);
                                        unsigned int taps[4 * SLOT];
#pragma unroll
                                        for (int k = 0; k < 4; ++k) {
                                            const Tap t = to_tap(dev::apply_tail(v.pre, px[k]));
                                            __builtin_memcpy(taps + k * SLOT, &t, sizeof(Tap));
                                        }
#pragma unroll
                                        for (int k = 0; k < SLOT; ++k) {
                                            dev::u32x4 piece;
                                            piece.x = taps[4 * k]; piece.y = taps[4 * k + 1]; piece.z = taps[4 * k + 2]; piece.w = taps[4 * k + 3];
                                            reinterpret_cast<dev::u32x4*>(tile + item * 4 * SLOT)[k] = piece;
                                        }
                                    }
                                }
                            }
                        }
                    }
                }
            }
            if (packed) {
                // (staged above)
            } else if (staged) {
                // The lanes of a wave cover the box's columns, and where the box is narrow (32 columns or fewer) several
                // of its rows side by side: lane = (row within the wave's pass, column).  The block's waves take the rows
                // of a pass in turn.  Pixels read as they lie in memory (RAW_SOURCE): the loads of STAGE_ROWS passes are
                // issued before the first of them is stored, so a box of up to STAGE_ROWS passes costs one memory round
                // trip, and a row past the box's last is the last one again, loaded and stored twice (with a branch
                // around it the compiler moves the load to the store and waits there).  Pixels that are computed
                // (operations fused before the resize) are computed once each: lanes past the box's last row rest.
                const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
                constexpr int WAVES = BLOCK_THREADS / 64;
                constexpr int STAGE_ROWS = RAW_SOURCE ? (sizeof(Src) <= 4 ? 4 : 2) : 2;
                int lane_cols_log2 = 32 - __builtin_clz(static_cast<unsigned>(cols - 1)); // columns a wave puts side by side: >= cols, at most 64
                lane_cols_log2 = lane_cols_log2 > 6 ? 6 : lane_cols_log2;
                const int lane_cols = 1 << lane_cols_log2;
                const int pass_rows = 64 >> lane_cols_log2;            // rows of a wave's pass
                const int lane_row = wave * pass_rows + (lane >> lane_cols_log2); // this lane's row in the block's first pass
                const int block_rows = WAVES * pass_rows;              // rows of a block's pass
                bool rows_alike = false;
                if constexpr (RAW_SOURCE && sizeof(Src) == 3) rows_alike = (s.pitch & 3u) == 0u;
                bool staged_by_item = false;
                if constexpr (RAW_SOURCE && PACKABLE) {
                    // Three-byte pixels of an image that starts at a whole dword, rows a whole number of dwords apart: the tile
                    // is filled from the aligned groups of four pixels (twelve bytes, one load) that cover the box's columns,
                    // read through a descriptor of the whole parent image, so a thread converts four pixels per load and
                    // address instead of one.  The tile's column 0 is the first group's first pixel, a row holds the groups and
                    // room for one more; rows past the window's last are the last one again, and where the box reaches past
                    // the window's last column, the thread that fetched that column writes its copy behind it.
                    if ((job_flags & FLAG_QUAD_FILL) != 0u && ((static_cast<unsigned>(reinterpret_cast<size_t>(s.data)) | s.pitch) & 3u) == 0u) {
                        const int last_c = sx_lo + cols - 1 < s.w - 1 ? sx_lo + cols - 1 : s.w - 1;
                        const int q_lo = (s.ox + sx_lo) >> 2;
                        const int quads = ((s.ox + last_c) >> 2) - q_lo + 1;
                        const int row_px = 4 * (quads + 1);
                        const int items = rows * quads;
                        const int behind = sx_lo + cols - 1 - last_c; // columns of the box behind the window's last (0 or 1)
                        // (boxes of up to one group per thread, as the host planned for the plane's factors)
                        if (quads >= 1 && items <= BLOCK_THREADS && behind <= 3 && rows * row_px * SLOT <= static_cast<int>(job_tile_dwords)) {
                            staged_by_item = true;
                            stride = row_px;
                            tile_x0 = 4 * q_lo - s.ox;
                            // (item / quads as (item * m) >> 20: see the tiles of packed pixels above; a tile of float taps holds
                            // fewer groups than one of packed pixels)
                            const unsigned m = static_cast<unsigned>(1048576.0f * __builtin_amdgcn_rcpf(static_cast<float>(quads))) + 2u;
                            const __amdgpu_buffer_rsrc_t image = Access::quad_buffer(s);
                            // the window's last column inside its group, and where its copies go from the start of that group
                            const int edge_pixel = (s.ox + s.w - 1) & 3;
                            const int edge_slot = (s.w - tile_x0 - 4 * (quads - 1)) * SLOT;
                            constexpr int PASSES = 1;
                            for (int first = 0; first < items; first += BLOCK_THREADS * PASSES) { // (uniform: one turn)
                                typename Access::Quad raw[PASSES];
                                int at[PASSES];
                                bool last_group[PASSES];
#pragma unroll
                                for (int u = 0; u < PASSES; ++u) {
                                    const int wanted = first + BLOCK_THREADS * u + tid;
                                    const int item = wanted < items ? wanted : items - 1;
                                    const int r = static_cast<int>((static_cast<unsigned>(item) * m) >> 20);
                                    const int q = item - r * quads;
                                    const int sy = sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1;
                                    raw[u] = Access::load_quad(image, s, q_lo + q, s.oy + sy);
                                    at[u] = (r * row_px + 4 * q) * SLOT;
                                    last_group[u] = q == quads - 1;
                                }
#pragma unroll
                                for (int u = 0; u < PASSES; ++u) {
                                    if (first + BLOCK_THREADS * u + 64 * wave < items) { // (uniform: some group of this wave's pass exists)
                                        Src px[4];
                                        Access::quad_pixels(raw[u], px);
                                        unsigned int taps[4 * SLOT];
#pragma unroll
                                        for (int k = 0; k < 4; ++k) {
                                            const Tap t = to_tap(px[k]);
                                            __builtin_memcpy(taps + k * SLOT, &t, sizeof(Tap));
                                        }
#pragma unroll
                                        for (int k = 0; k < SLOT; ++k) {
                                            dev::u32x4 piece;
                                            piece.x = taps[4 * k]; piece.y = taps[4 * k + 1]; piece.z = taps[4 * k + 2]; piece.w = taps[4 * k + 3];
                                            reinterpret_cast<dev::u32x4*>(tile + at[u])[k] = piece;
                                        }
                                        // The copies of the window's last column behind it, by the thread that holds that column (its
                                        // row's last group), after its own stores: the copy lies inside that group or in the room
                                        // behind it, which no other thread writes.
                                        if (behind > 0) { // (uniform)
                                            Src edge = px[0];
                                            if (edge_pixel == 1) edge = px[1];
                                            if (edge_pixel == 2) edge = px[2];
                                            if (edge_pixel == 3) edge = px[3];
                                            if (last_group[u]) {
                                                for (int j = 0; j < behind; ++j) store_tap(tile + at[u] + edge_slot + j * SLOT, to_tap(edge));
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                }
                if constexpr (RAW_SOURCE && sizeof(Src) == 3) {
                    if (rows_alike && !staged_by_item) {
                        // Three-byte pixels, rows a whole number of dwords apart (the common case): the box's pixels in row-major
                        // order, thread t takes pixels t, t + 256, ..., the loads of all of them in flight before the first
                        // is stored, so a box costs one memory round trip with every lane busy (with the lanes
                        // laid over columns, a box of 35 columns leaves 29 lanes of every wave idle and takes five passes of four
                        // rows).  item / cols comes from a multiplication by the reciprocal instruction's result: (item + 0.5) / cols
                        // is at least 0.5 / cols away from a whole number, a tile holds at most 2048 pixels, and the product is off
                        // by less than 2048 / cols * 2^-21, which is below 0.5 / cols.
                        staged_by_item = true;
                        static_assert(RESIZE_LDS_DWORDS / SLOT <= 2048, "the division by multiplication is exact up to 2048 pixels");
                        const int items = rows * cols;
                        const float per_col = __builtin_amdgcn_rcpf(static_cast<float>(cols));
                        const unsigned base = static_cast<unsigned>(reinterpret_cast<size_t>(window));
                        // (as many passes in flight as the box needs, 2, 4 or 8: a pass that no pixel needs still costs its
                        // address arithmetic and a repeated load)
                        const auto stage_passes = [&](const auto passes) {
                            constexpr int PASSES = decltype(passes)::value;
                            for (int first = 0; first < items; first += BLOCK_THREADS * PASSES) { // (uniform; one turn for boxes of up to 256 * PASSES pixels)
                                unsigned int got[PASSES], shift[PASSES];
                                int at[PASSES];
#pragma unroll
                                for (int u = 0; u < PASSES; ++u) {
                                    const int wanted = first + BLOCK_THREADS * u + tid;
                                    const int item = wanted < items ? wanted : items - 1;
                                    const int r = static_cast<int>((static_cast<float>(item) + 0.5f) * per_col);
                                    const int c = item - r * cols;
                                    const int sx = sx_lo + c < s.w - 1 ? sx_lo + c : s.w - 1;
                                    const int sy = sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1;
                                    const unsigned off = static_cast<unsigned>(sx) * 3u;
                                    const bool aligned = ((base + off) & 3u) == 0u;
                                    got[u] = dev::load_dword_from_row(window, static_cast<unsigned>(sy) * s.pitch + off + (aligned ? 1u : 0u));
                                    shift[u] = aligned ? 0u : 8u;
                                    at[u] = (r * stride + c) * SLOT;
                                }
#pragma unroll
                                for (int u = 0; u < PASSES; ++u) {
                                    if (first + BLOCK_THREADS * u + 64 * wave < items) { // (uniform: some pixel of this wave's pass exists)
                                        dev::PixelSlot<Src> px;
                                        px.w[0] = got[u] >> shift[u];
                                        store_tap(tile + at[u], to_tap(dev::slot_to_pixel<Src>(px)));
                                    }
                                }
                            }
                        };
                        if (items <= 2 * BLOCK_THREADS) stage_passes(std::integral_constant<int, 2>{});
                        else if (items <= 4 * BLOCK_THREADS) stage_passes(std::integral_constant<int, 4>{});
                        else stage_passes(std::integral_constant<int, 8>{});
                    }
                }
                for (int c = lane & (lane_cols - 1); c < cols && !staged_by_item; c += lane_cols) {
                    const int sx = sx_lo + c < s.w - 1 ? sx_lo + c : s.w - 1;
                    // three-byte pixels, rows a whole number of dwords apart: a column has the same alignment in every
                    // row, so a lane's offset and the shift that takes the pixel out of its dword are found once per column
                    const unsigned off = static_cast<unsigned>(sx) * static_cast<unsigned>(sizeof(Src));
                    const bool aligned = ((static_cast<unsigned>(reinterpret_cast<size_t>(window)) + off) & 3u) == 0u;
                    const unsigned voff = off + (aligned ? 1u : 0u); // from one byte before the row
                    for (int first = 0; first < rows; first += block_rows * STAGE_ROWS) { // (uniform)
                        if constexpr (RAW_SOURCE) {
                            dev::PixelSlot<Src> px[STAGE_ROWS];
#pragma unroll
                            for (int u = 0; u < STAGE_ROWS; ++u) {
                                const int wanted = first + block_rows * u + lane_row;
                                const int r = wanted < rows ? wanted : rows - 1;
                                const int sy = sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1;
                                if constexpr (sizeof(Src) == 3) {
                                    // (the row's offset from the window's first pixel fits the lane's 32 bits: the host stages
                                    // tiles of three-byte pixels only for windows that span less than 4 GiB, FLAG_OFFSETS_32)
                                    if (rows_alike) {
                                        const unsigned int w = dev::load_dword_from_row(window, static_cast<unsigned>(sy) * s.pitch + voff);
                                        px[u].w[0] = aligned ? w : w >> 8u;
                                    } else {
                                        px[u] = dev::load_pixel_slot<Src>(window, static_cast<int>(static_cast<unsigned>(sy) * s.pitch + off), valid_lo, valid_hi);
                                    }
                                } else {
                                    px[u] = dev::load_pixel_slot<Src>(window + static_cast<size_t>(sy) * s.pitch, static_cast<int>(off), valid_lo, valid_hi);
                                }
                            }
#pragma unroll
                            for (int u = 0; u < STAGE_ROWS; ++u) {
                                const int wanted = first + block_rows * u + lane_row;
                                const int r = wanted < rows ? wanted : rows - 1;
                                store_tap(tile + (r * stride + c) * SLOT, to_tap(dev::slot_to_pixel<Src>(px[u])));
                            }
                        } else {
                            Src px[STAGE_ROWS];
#pragma unroll
                            for (int u = 0; u < STAGE_ROWS; ++u) {
                                const int r = first + block_rows * u + lane_row;
                                if (r < rows) px[u] = fetch(v, sx, sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1);
                            }
#pragma unroll
                            for (int u = 0; u < STAGE_ROWS; ++u) {
                                const int r = first + block_rows * u + lane_row;
                                if (r < rows) store_tap(tile + (r * stride + c) * SLOT, to_tap(px[u]));
                            }
                        }
                    }
                }
            } else if constexpr (RAW_SOURCE) {
                // Taps straight from memory, from a box of moderate size (down-scaling by up to about 1.7): every line of the
                // box is touched once, now, with one load per 128-byte line whose value is not used, so that the gathers,
                // which come after the lanes' set-up and wait for sixteen taps at a time, find the lines on their way
                // (measured: eight 1920x1080 planes to 1280x720 31.3 -> 28.6 us; for larger boxes the touches cost more than
                // they bring, 3x down-scaling 6.3 -> 7.6 us).
                const int last_byte = s.w * static_cast<int>(sizeof(Src)) - 4; // last dword that lies wholly inside a window row
                if (rows * cols <= 3 * tile_px + 256 && last_byte >= 0 && (job_flags & FLAG_OFFSETS_32) != 0u) {
                    const int row_bytes = cols * static_cast<int>(sizeof(Src));
                    const int first_byte = sx_lo * static_cast<int>(sizeof(Src));
                    const int lines = (row_bytes + 127) / 128 + 1;
                    const int total = rows * lines;
                    for (int i = tid; i < total; i += BLOCK_THREADS) {
                        const int r = i / lines, l = i - r * lines;
                        const int sy = sy_lo + r < s.h - 1 ? sy_lo + r : s.h - 1;
                        int at = first_byte + l * 128;
                        at = at < last_byte ? at : last_byte;
                        at = at < 0 ? 0 : at;
                        const unsigned int touched = dev::load_dword_from_row(window, static_cast<unsigned>(sy) * s.pitch + static_cast<unsigned>(at) + 1u);
                        asm volatile("" ::"v"(touched));
                    }
                }
            }
        }
        dev::block_sync();

        // ---- compute: a wave owns wave_rows rows of the tile, a lane one column of them ----
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        const int x = tx0 + lane;
        const int wy0 = ty0 + wave_rows * wave;
        if (wy0 >= v.h) return; // the plane ends above this wave's rows (no barrier follows)
        const bool whole_width = tx0 + RESIZE_TILE_W <= v.w; // block-uniform
        // interior tiles (whole tile inside the plane and inside the region that holds the image) need no per-pixel tests
        bool interior = whole_width && ty0 + tile_h <= v.h;
        if constexpr (View::HAS_ROI) {
            interior = interior && tx0 + v.off_x >= v.x1 && tx0 + RESIZE_TILE_W - 1 + v.off_x <= v.x2 && ty0 + v.off_y >= v.y1 &&
                       ty0 + tile_h - 1 + v.off_y <= v.y2;
        }
        // the whole computation exists once per kind of put
        const auto compute = [&](const auto& put) {
            if (!resamples) {
                // a tile that lies wholly beside the image (the bars of a preserved aspect ratio): one value for all of it
                const OutPixel bar = dev::apply_tail(tail, v.background);
                for (int g = 0; g < wave_rows; g += RESIZE_GROUP_ROWS) {
                    put(g, std::integral_constant<int, 0>{}, bar);
                    put(g, std::integral_constant<int, 1>{}, bar);
                    put(g, std::integral_constant<int, 2>{}, bar);
                    put(g, std::integral_constant<int, 3>{}, bar);
                }
            } else if (staged) {
                // (the tile's column 0 is window column tile_x0: the box's first column, or the first pixel of the group that holds it)
                if (interior) sweep<TAPS_FLOAT_TILE, true>(v, tail, tile, window, tile_x0, sy_lo, stride, tile_x0, x, wy0, lane, wave_rows, put);
                else sweep<TAPS_FLOAT_TILE, false>(v, tail, tile, window, tile_x0, sy_lo, stride, tile_x0, x, wy0, lane, wave_rows, put);
            } else if (PACKABLE && packed) {
                if constexpr (PACKABLE) {
                    if (interior) sweep<TAPS_PACKED_TILE, true>(v, tail, tile, window, sx_lo, sy_lo, stride, tile_x0, x, wy0, lane, wave_rows, put);
                    else sweep<TAPS_PACKED_TILE, false>(v, tail, tile, window, sx_lo, sy_lo, stride, tile_x0, x, wy0, lane, wave_rows, put);
                }
            } else {
                if (interior) sweep<TAPS_DIRECT, true>(v, tail, tile, window, sx_lo, sy_lo, stride, tile_x0, x, wy0, lane, wave_rows, put);
                else sweep<TAPS_DIRECT, false>(v, tail, tile, window, sx_lo, sy_lo, stride, tile_x0, x, wy0, lane, wave_rows, put);
            }
        };
        // One pixel per lane straight from registers: a wave's store covers 64 neighbouring pixels of a row (768
        // consecutive bytes of 12-byte pixels: as fast as 16-byte pieces, measured, and nothing passes through LDS).
        const bool column_here = x < v.w;
        const int rows_here = v.h - wy0; // rows from the wave's first to the plane's last (may exceed the wave's own)
        constexpr bool CAN_STREAM = Out::IS_SPLIT ? sizeof(VBase<OutPixel>) == 4 : (sizeof(OutPixel) % 4 == 0 && sizeof(OutPixel) <= 16);
        if constexpr (CAN_STREAM) {
            if ((job_flags & FLAG_STREAM_STORES) != 0u) {
                // the address of the wave's first row is the same in all its lanes: a descriptor from there on, the row as
                // the wave's offset (in a scalar register) and the column as the lane's
                const __amdgpu_buffer_rsrc_t rows = dev::wave_buffer(dev::wave_uniform(
                    reinterpret_cast<char*>(out.data) + static_cast<size_t>(bz) * out.z_stride + static_cast<size_t>(wy0) * out.pitch));
                const unsigned pitch = out.pitch;
                if constexpr (Out::IS_SPLIT) {
                    const unsigned at = static_cast<unsigned>(x) * 4u;
                    const unsigned chan_stride = static_cast<unsigned>(out.chan_stride); // the host has checked that all offsets fit
                    compute([&](const int g, const auto k, const OutPixel& o) {
                        const int i = g + decltype(k)::value;
                        if (column_here && i < rows_here) {
                            const unsigned row = static_cast<unsigned>(i) * pitch;
                            dev::stream_store_at<1>(rows, at, row, __builtin_bit_cast(unsigned int, o.x));
                            dev::stream_store_at<1>(rows, at, row + chan_stride, __builtin_bit_cast(unsigned int, o.y));
                            if constexpr (cn<OutPixel> >= 3) dev::stream_store_at<1>(rows, at, row + 2u * chan_stride, __builtin_bit_cast(unsigned int, o.z));
                            if constexpr (cn<OutPixel> == 4) dev::stream_store_at<1>(rows, at, row + 3u * chan_stride, __builtin_bit_cast(unsigned int, o.w));
                        }
                    });
                } else {
                    const unsigned at = static_cast<unsigned>(x) * static_cast<unsigned>(sizeof(OutPixel));
                    compute([&](const int g, const auto k, const OutPixel& o) {
                        const int i = g + decltype(k)::value;
                        if (column_here && i < rows_here) {
                            dev::stream_store_at<dev::WordsOf<OutPixel>::ND>(rows, at, static_cast<unsigned>(i) * pitch, dev::WordsOf<OutPixel>::of(o));
                        }
                    });
                }
                return;
            }
        }
        compute([&](const int g, const auto k, const OutPixel& o) {
            const int i = g + decltype(k)::value;
            if (column_here && i < rows_here) dev::store_one(out, x, wy0 + i, static_cast<int>(bz), o);
        });
    }
};

// ---- generic -----------------------------------------------------------------------------------------------------
// A block covers 64*K x 4 elements; a thread computes K elements of one row, 64 apart (each of a wave's memory
// instructions still covers 64 neighbours).  A chain that only gathers and stores is bound by the memory round trip, one
// gather in flight per wave; with K = 4 a thread issues the reads of four elements before it uses any of them, provided
// the chain's read is straight-line code (lanes past the end of a row read its last element again instead of branching
// around the read).  K = 1 is kept for small outputs, which need every wave they can get.
namespace dev {
// Blocks are handed to the eight XCDs in turn, in launch order, and each XCD has its own L2.  Neighbouring tiles read
// source lines in common (the rows and columns where their boxes meet, every line of a slanted row for a warp): with
// the blocks as they come, nearly every such line is fetched by several XCDs.  Here the block with launch number l works
// on tile (l % 8) * total / 8 + l / 8 instead: each XCD covers one contiguous band of the output, and a source line is
// fetched by the one or two XCDs whose bands need it.  For launches whose tiles all cost the same: a band of cheap tiles
// (the planes of a batch that only receive a default value, the bars beside a resized image) would leave its XCD idle
// early; measured on the resize kernel, eight 1920x1080 planes of which five are resized: 31.2 -> 40.8 us.
__device__ __attribute__((always_inline)) inline void xcd_band_block(unsigned& bx, unsigned& by, unsigned& bz, const unsigned gx, const unsigned gy,
                                                                    const unsigned gz) {
    const unsigned total = gx * gy * gz;
    const unsigned l = bx + gx * (by + gy * bz);
    const unsigned share = total >> 3, rest = total & 7u, xcd = l & 7u; // the first `rest` XCDs take one block more
    const unsigned tile = xcd * share + (xcd < rest ? xcd : rest) + (l >> 3);
    const unsigned row = tile / gx;
    bx = tile - row * gx;
    bz = row / gy;
    by = row - bz * gy;
}
} // namespace dev

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
    unsigned xcd_bands; // tiles dealt out in one band per XCD (dev::xcd_band_block)
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
    // the job's own fields as a block holds them (read in one batch at its start; sender and receiver are read in place)
    struct Held {
        ActiveThreads active;
        unsigned stream_rows, packs_rows;
        char* out_data;
        unsigned out_pitch;
        size_t out_z_stride;
    };
    template <int K, bool NEIGHBOURS>
    __device__ __attribute__((always_inline)) static inline void body(const GenericJob& job, const Held& held, unsigned bx, unsigned by, unsigned bz) {
        constexpr int STEP = NEIGHBOURS ? 1 : 64;
        const int tid = dev::thread_in_block();
        const int y = static_cast<int>(by) * 4 + (tid >> 6);
        const int w = static_cast<int>(held.active.x);
        const int x0 = static_cast<int>(bx) * (64 * K) + (tid & 63) * (NEIGHBOURS ? K : 1);
        if (x0 >= w || y >= static_cast<int>(held.active.y)) return;
        Value value[K];
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const int x = x0 + STEP * k < w ? x0 + STEP * k : w - 1;
            value[k] = Sender::Operation::exec(Point(x, y, static_cast<int>(bz)), job.sender);
        }
        if constexpr (PACKS_ROWS && NEIGHBOURS && K == 4) {
            if (held.packs_rows != 0u && x0 + K <= w) {
                constexpr int S = static_cast<int>(sizeof(Value)); // bytes per pixel = dwords per thread
                unsigned int words[S];
                dev::pack_pixels<K>(value, words);
                char* const run = held.out_data + static_cast<size_t>(bz) * held.out_z_stride + static_cast<size_t>(y) * held.out_pitch +
                                  static_cast<size_t>(x0) * S;
                if (held.stream_rows != 0u) {
                    // the row is the same for the whole wave (a wave is one row of the block)
                    const __amdgpu_buffer_rsrc_t row_buffer = dev::wave_buffer(dev::wave_uniform(
                        held.out_data + static_cast<size_t>(bz) * held.out_z_stride + static_cast<size_t>(y) * held.out_pitch));
                    const unsigned at = static_cast<unsigned>(x0) * S;
                    if constexpr (S == 3) {
                        dev::u32x3 v;
                        v.x = words[0]; v.y = words[1]; v.z = words[2];
                        dev::stream_store_at<3>(row_buffer, at, 0u, v);
                    } else {
#pragma unroll
                        for (int i = 0; i < S; ++i) dev::stream_store_at<1>(row_buffer, at + 4u * i, 0u, words[i]);
                    }
                    return;
                }
                __builtin_memcpy(__builtin_assume_aligned(run, 4), words, 4 * S);
                return;
            }
        }
        if constexpr (STREAMS_ROWS) {
            if (held.stream_rows != 0u) {
                constexpr int S = static_cast<int>(sizeof(Value));
                // the row is the same for the whole wave (a wave is one row of the block)
                const __amdgpu_buffer_rsrc_t row_buffer = dev::wave_buffer(dev::wave_uniform(
                    held.out_data + static_cast<size_t>(bz) * held.out_z_stride + static_cast<size_t>(y) * held.out_pitch));
#pragma unroll
                for (int k = 0; k < K; ++k) {
                    if (x0 + STEP * k < w) {
                        const unsigned at = static_cast<unsigned>(x0 + STEP * k) * S;
                        if constexpr (S <= 16) {
                            dev::stream_store_at<S / 4>(row_buffer, at, 0u, dev::WordsOf<Value>::of(value[k]));
                        } else {
                            unsigned int words[S / 4];
                            __builtin_memcpy(words, &value[k], S);
#pragma unroll
                            for (int i = 0; i < S / 16; ++i) {
                                dev::u32x4 piece;
                                piece.x = words[4 * i]; piece.y = words[4 * i + 1]; piece.z = words[4 * i + 2]; piece.w = words[4 * i + 3];
                                dev::stream_store_at<4>(row_buffer, at + 16u * i, 0u, piece);
                            }
                            static_assert(S <= 16 || S % 16 == 0, "larger pixels are whole 16-byte pieces");
                        }
                    }
                }
                return;
            }
        }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (x0 + STEP * k < w) Receiver::Operation::exec(Point(x0 + STEP * k, y, static_cast<int>(bz)), value[k], job.receiver);
        }
    }
    __device__ __attribute__((always_inline)) static inline void run(const GenericJob& job, unsigned bx, unsigned by, unsigned bz, unsigned char*) {
        const Held held{ job.active, job.stream_rows, job.packs_rows, job.out_data, job.out_pitch, job.out_z_stride };
        const unsigned wide = job.wide, bands = job.xcd_bands, gx = job.grid_x, gy = job.grid_y;
        if (bands != 0u) dev::xcd_band_block(bx, by, bz, gx, gy, held.active.z);
        if constexpr (PACKS_ROWS) { // the only jobs that are compiled with the neighbour form
            if (wide != 0u && held.packs_rows != 0u) {
                body<4, true>(job, held, bx, by, bz);
                return;
            }
        }
        if (wide != 0u) body<4, false>(job, held, bx, by, bz);
        else body<1, false>(job, held, bx, by, bz);
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

// Copies a job from the kernel-argument segment to device memory, for a launch that reads it from there (callers that
// bring the memory for the job themselves).  One block.
template <typename Job>
__global__ __attribute__((amdgpu_flat_work_group_size(BLOCK_THREADS, BLOCK_THREADS))) void store_job_kernel(const Job job, Job* __restrict__ at) {
    static_assert(sizeof(Job) % 4 == 0 && alignof(Job) >= 4, "a job is whole dwords");
    const unsigned int* const from = reinterpret_cast<const unsigned int*>(&job_in_kernarg<Job>());
    unsigned int* const to = reinterpret_cast<unsigned int*>(at);
    for (unsigned i = static_cast<unsigned>(dev::thread_in_block()); i < sizeof(Job) / 4; i += BLOCK_THREADS) to[i] = from[i];
}

// Several different jobs in one launch ("divergent horizontal fusion"): the 1-D grid is cut into one contiguous
// range of blocks per job, sized to that job alone, so that a small job does not pay for a large one's grid.
template <typename... Jobs>
struct JobPack;
template <>
struct JobPack<> {
    static constexpr int COUNT = 0;
    __device__ __attribute__((always_inline)) static inline void header(const JobPack&, unsigned*, unsigned*, unsigned*) {}
    template <int I>
    __device__ __attribute__((always_inline)) static inline void dispatch(const JobPack&, unsigned, const unsigned*, const unsigned*, const unsigned*, unsigned char*) {}
};
template <typename Job, typename... Rest>
struct JobPack<Job, Rest...> {
    Job job;
    unsigned blocks; // blocks of this job: grid_x * grid_y * planes
    JobPack<Rest...> rest;
    static constexpr int COUNT = 1 + JobPack<Rest...>::COUNT;
    // The block counts and grids of all the pack's jobs, read in one batch of scalar loads before the block knows which job is
    // its own (found one job after the other, each count would be a dependent load).
    __device__ __attribute__((always_inline)) static inline void header(const JobPack& pack, unsigned* blocks_of, unsigned* grid_x_of, unsigned* grid_y_of) {
        blocks_of[0] = pack.blocks;
        grid_x_of[0] = pack.job.grid_x;
        grid_y_of[0] = pack.job.grid_y;
        JobPack<Rest...>::header(pack.rest, blocks_of + 1, grid_x_of + 1, grid_y_of + 1);
    }
    template <int I>
    __device__ __attribute__((always_inline)) static inline void dispatch(const JobPack& pack, unsigned block, const unsigned* blocks_of, const unsigned* grid_x_of,
                                                                         const unsigned* grid_y_of, unsigned char* lds) {
        if (block < blocks_of[I]) {
            const unsigned bx = block % grid_x_of[I];
            const unsigned q = block / grid_x_of[I];
            Job::run(pack.job, bx, q % grid_y_of[I], q / grid_y_of[I], lds);
        } else {
            JobPack<Rest...>::template dispatch<I + 1>(pack.rest, block - blocks_of[I], blocks_of, grid_x_of, grid_y_of, lds);
        }
    }
    __device__ __attribute__((always_inline)) static inline void run(const JobPack& pack, unsigned block, unsigned char* lds) {
        unsigned blocks_of[COUNT], grid_x_of[COUNT], grid_y_of[COUNT];
        header(pack, blocks_of, grid_x_of, grid_y_of);
        dispatch<0>(pack, block, blocks_of, grid_x_of, grid_y_of, lds);
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

// Host-side analysis of a fused chain: turns the read part of a sender and the receiver into plain descriptors
// ("views") that the hand-written kernels index directly.
//
//   PlainView   out(x, y) = img(x + ox, y + oy)                      PerThreadRead<_2D>, possibly under Crop
//   YuvView     out(x, y) = {Y, U, V} of pixel (x + ox, y + oy)       ReadYUV<PF>, possibly under Crop
//   ResizeView  out(x, y) = bilinear(pre(window), (x + off - roi) * f)  Resize<INTER_LINEAR> over one of the above,
//                                                                    optionally with compute operations fused between
//                                                                    the read and the resize (`pre`, applied to every
//                                                                    source pixel), possibly under an outer Crop
//                                                                    (reads pulled back through it)
// Folding Crop into an origin is what Crop::exec does one element at a time (reference
// algorithms/image_processing/crop.h:35-38); the Resize parameters are the ones Resize::build computed
// (resize.h:105-166).  Chains that do not match keep their generic per-element form.
#ifndef FK_EXEC_VIEWS_H
#define FK_EXEC_VIEWS_H

#include "fk/ops/image_processing.h"
#include "fk/ops/yuv.h"

namespace fk {
namespace exec {

template <typename T>
struct PlainView {
    using Pixel = T;
    using Source = T;
    static constexpr bool IS_RESIZE = false;
    const T* data; // parent image
    uint pitch;    // bytes between parent rows
    int img_w, img_h;
    int ox, oy; // window origin in the parent
    int w, h;   // window size: the extent this plane produces
};

// A window of a raw YUV image, seen as {Y, U, V} pixels of the format's base type.
template <PixelFormat PF>
struct YuvView {
    using Base = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    using Pixel = VectorType_t<Base, 3>;
    using Source = Pixel;
    static constexpr bool IS_RESIZE = false;
    static constexpr PixelFormat FORMAT = PF;
    const Base* data; // first luma (or packed) row of the parent image
    uint pitch;       // bytes between rows, of every plane
    int img_w, img_h; // parent image size in pixels; semi-planar chroma rows follow row img_h - 1
    int ox, oy;       // window origin in the parent
    int w, h;         // window size: the extent this plane produces
};

struct NoTail {};

// SrcView: the window that is resampled (its w, h are the clamp limits); Pre: compute operations applied to each of
// its pixels before interpolation (NoTail for none); T: the pixel type that comes out of Pre.
template <typename SrcView, typename Pre, typename T, AspectRatio AR>
struct ResizeView {
    using Source = T;
    using Pixel = VectorType_t<float, cn<T>>;
    static constexpr bool IS_RESIZE = true;
    static constexpr bool HAS_ROI = AR != AspectRatio::IGNORE_AR;
    SrcView src;
    Pre pre;
    float fx, fy;
    int off_x, off_y;   // added to the output coordinate before resampling (an outer Crop)
    int x1, y1, x2, y2; // destination region that holds the image; the rest is background
    Pixel background;
    int w, h; // the extent this plane produces
};

template <typename View, typename Tail>
struct PlaneProgram {
    View view;
    Tail tail;
};

// ---- divisions by a divisor the host has seen ------------------------------------------------------------------------
// A Div<float..> of a chain's tail divides every pixel by the same values.  IEEE division is eleven instructions on
// this part.  With the reciprocal as two floats from the host, r = RN(1 / d) and rl = RN(1 / d - r), four give the same
// result: q = fma(x, r, x * rl) is x / d to a relative 2^-47 before its one rounding, hence a faithful quotient, and
// the correction q + fma(-d, q, x) * r of a faithful quotient by a correctly rounded reciprocal is the correctly rounded
// quotient (Markstein, "Computation of elementary functions on the IBM RISC System/6000 processor", 1990), as long as
// nothing on the way leaves the normal range.  The host vouches for d (finite, 2^-40 <= |d| <= 2^40), the kernel tests x
// and takes the division instruction sequence where a lane is outside (zeros, subnormals, infinities, huge values).
template <typename Op>
struct IsFloatDiv : std::false_type {};
template <typename F>
struct IsFloatDiv<Div<F, F, F>> : std::bool_constant<std::is_same_v<VBase<F>, float>> {};
template <typename... Ops>
constexpr int float_div_count = (0 + ... + (IsFloatDiv<Ops>::value ? 1 : 0));

constexpr float PREPARED_DIV_LO = 9.09494702e-13f; // 2^-40
constexpr float PREPARED_DIV_HI = 1.09951163e+12f; // 2^40

template <typename Ops, int NDIV>
struct PreparedTail {
    Ops ops;
    float recip[NDIV][4];    // per float division of the tail, in order: r = RN(1 / d) per channel
    float recip_lo[NDIV][4]; // RN(1 / d - r)
    unsigned fast;        // bit i: every divisor of division i is in range, so its reciprocals are valid
};

namespace detail {
inline bool prepared_divisor_ok(const float d) {
    const float a = d < 0.f ? -d : d;
    return a >= PREPARED_DIV_LO && a <= PREPARED_DIV_HI; // false for NaN
}
template <int I, typename Prepared, typename Op, typename... Rest_>
inline void prepare_divisions(Prepared& out, const OperationTuple<Op, Rest_...>& t) {
    constexpr bool IS_DIV = IsFloatDiv<Op>::value;
    if constexpr (IS_DIV) {
        using F = typename Op::ParamsType;
        bool ok = true;
        for (int c = 0; c < 4; ++c) out.recip[I][c] = out.recip_lo[I][c] = 0.f;
        for (int c = 0; c < cn<F>; ++c) {
            const volatile float d = vectorAt(c, t.instance.params); // volatile: divisions at run time, correctly rounded
            ok = ok && prepared_divisor_ok(d);
            if (ok) {
                const volatile float r = 1.0f / d;
                // 1 / d in double is off by 2^-53 relative, far below the last bit of the float it is rounded to here
                const volatile double rest = 1.0 / static_cast<double>(d) - static_cast<double>(r);
                out.recip[I][c] = r;
                out.recip_lo[I][c] = static_cast<float>(rest);
            }
        }
        if (ok) out.fast |= 1u << I;
    }
    if constexpr (sizeof...(Rest_) > 0) {
        prepare_divisions<I + (IS_DIV ? 1 : 0)>(out, fk::detail::tuple_tail(t));
    }
}
} // namespace detail

// ---- read side ---------------------------------------------------------------------------------------------------
template <typename IOp, typename = void>
struct ViewOf {
    static constexpr bool supported = false;
};

template <typename T>
struct ViewOf<Read<PerThreadRead<ND::_2D, T>>> {
    static constexpr bool supported = true;
    using type = PlainView<T>;
    static type make(const Read<PerThreadRead<ND::_2D, T>>& iOp) {
        const auto& d = iOp.params.dims;
        return type{ iOp.params.data, d.pitch, static_cast<int>(d.width), static_cast<int>(d.height), 0, 0,
                     static_cast<int>(d.width), static_cast<int>(d.height) };
    }
};

// a 1-D buffer is one row
template <typename T>
struct ViewOf<Read<PerThreadRead<ND::_1D, T>>> {
    static constexpr bool supported = true;
    using type = PlainView<T>;
    static type make(const Read<PerThreadRead<ND::_1D, T>>& iOp) {
        const int n = static_cast<int>(iOp.params.dims.width);
        return type{ iOp.params.data, 0u, n, 1, 0, 0, n, 1 };
    }
};

template <PixelFormat PF>
struct ViewOf<Read<ReadYUV<PF>>> {
    static constexpr bool supported = true;
    using type = YuvView<PF>;
    static type make(const Read<ReadYUV<PF>>& iOp) {
        const RawImage<PF>& raw = iOp.params;
        return type{ raw.data.data, raw.data.dims.pitch, static_cast<int>(raw.width), static_cast<int>(raw.height), 0, 0,
                     static_cast<int>(raw.width), static_cast<int>(raw.height) };
    }
};

template <typename Back>
struct ViewOf<ReadBack<Crop<Back>>, std::enable_if_t<ViewOf<Back>::supported>> {
    static constexpr bool supported = true;
    using type = typename ViewOf<Back>::type;
    static type make(const ReadBack<Crop<Back>>& iOp) {
        type v = ViewOf<Back>::make(iOp.backIOp);
        const Rect& r = iOp.params;
        if constexpr (type::IS_RESIZE) {
            v.off_x += static_cast<int>(r.x);
            v.off_y += static_cast<int>(r.y);
        } else {
            v.ox += static_cast<int>(r.x);
            v.oy += static_cast<int>(r.y);
        }
        v.w = r.width;
        v.h = r.height;
        return v;
    }
};

// What a resize resamples: a window view plus the compute operations fused between the read and the resize.
template <typename IOp, typename = void>
struct SourceOf {
    static constexpr bool supported = false;
};
template <typename IOp>
struct SourceOf<IOp, std::enable_if_t<ViewOf<IOp>::supported && !ViewOf<IOp>::type::IS_RESIZE>> {
    static constexpr bool supported = true;
    using View = typename ViewOf<IOp>::type;
    using Pre = NoTail;
    using Pixel = typename View::Pixel;
    static View view(const IOp& iOp) { return ViewOf<IOp>::make(iOp); }
    static Pre pre(const IOp&) { return Pre{}; }
};
template <typename Head, typename... ComputeOps>
struct SourceOf<Read<FusedOperation<Head, ComputeOps...>>,
                std::enable_if_t<isAnyReadType<Head> && ViewOf<Instantiable<Head>>::supported && !ViewOf<Instantiable<Head>>::type::IS_RESIZE &&
                                 (sizeof...(ComputeOps) > 0) && noneAnyWriteType<ComputeOps...>>> {
    static constexpr bool supported = true;
    using IOp = Read<FusedOperation<Head, ComputeOps...>>;
    using View = typename ViewOf<Instantiable<Head>>::type;
    using Pre = OperationTuple<ComputeOps...>;
    using Pixel = typename IOp::Operation::OutputType;
    static View view(const IOp& iOp) { return ViewOf<Instantiable<Head>>::make(toIOp<Head>(iOp.params.instance)); }
    static Pre pre(const IOp& iOp) { return fk::detail::tuple_tail(iOp.params); }
};
// a crop of a read that is fused with compute operations: the operations commute with the window
template <typename Back>
struct SourceOf<ReadBack<Crop<Back>>, std::enable_if_t<!ViewOf<Back>::supported && SourceOf<Back>::supported>> {
    static constexpr bool supported = true;
    using View = typename SourceOf<Back>::View;
    using Pre = typename SourceOf<Back>::Pre;
    using Pixel = typename SourceOf<Back>::Pixel;
    static View view(const ReadBack<Crop<Back>>& iOp) {
        View v = SourceOf<Back>::view(iOp.backIOp);
        const Rect& r = iOp.params;
        v.ox += static_cast<int>(r.x);
        v.oy += static_cast<int>(r.y);
        v.w = r.width;
        v.h = r.height;
        return v;
    }
    static Pre pre(const ReadBack<Crop<Back>>& iOp) { return SourceOf<Back>::pre(iOp.backIOp); }
};

template <AspectRatio AR, typename Back>
struct ViewOf<ReadBack<Resize<InterpolationType::INTER_LINEAR, AR, Back>>, std::enable_if_t<SourceOf<Back>::supported>> {
    static constexpr bool supported = true;
    using Src = SourceOf<Back>;
    using Source = typename Src::Pixel;
    using type = ResizeView<typename Src::View, typename Src::Pre, Source, AR>;
    static type make(const ReadBack<Resize<InterpolationType::INTER_LINEAR, AR, Back>>& iOp) {
        type v{};
        v.src = Src::view(iOp.backIOp);
        v.pre = Src::pre(iOp.backIOp);
        const auto& p = iOp.params;
        v.fx = p.src_conv_factors.x;
        v.fy = p.src_conv_factors.y;
        v.off_x = 0;
        v.off_y = 0;
        if constexpr (AR == AspectRatio::IGNORE_AR) {
            v.x1 = 0;
            v.y1 = 0;
            v.x2 = p.dstSize.width - 1;
            v.y2 = p.dstSize.height - 1;
            v.background = typename type::Pixel{};
        } else {
            v.x1 = p.x1;
            v.y1 = p.y1;
            v.x2 = p.x2;
            v.y2 = p.y2;
            v.background = p.defaultValue;
        }
        v.w = p.dstSize.width;
        v.h = p.dstSize.height;
        return v;
    }
};

// One plane of a sender as {view, tail of compute operations}.
template <typename IOp, typename = void>
struct ProgramOf {
    static constexpr bool supported = false;
};
template <typename IOp>
struct ProgramOf<IOp, std::enable_if_t<ViewOf<IOp>::supported>> {
    static constexpr bool supported = true;
    using View = typename ViewOf<IOp>::type;
    using type = PlaneProgram<View, NoTail>;
    using OutputType = typename View::Pixel;
    static type make(const IOp& iOp) { return type{ ViewOf<IOp>::make(iOp), NoTail{} }; }
};
template <typename Head, typename... ComputeOps>
struct ProgramOf<Read<FusedOperation<Head, ComputeOps...>>,
                 std::enable_if_t<isAnyReadType<Head> && ViewOf<Instantiable<Head>>::supported && (sizeof...(ComputeOps) > 0) &&
                                  noneAnyWriteType<ComputeOps...>>> { // a chain that writes on its way runs as a generic job
    static constexpr bool supported = true;
    using IOp = Read<FusedOperation<Head, ComputeOps...>>;
    using View = typename ViewOf<Instantiable<Head>>::type;
    using Ops = OperationTuple<ComputeOps...>;
    static constexpr int NDIV = float_div_count<ComputeOps...>;
    using Tail = std::conditional_t<(NDIV > 0 && NDIV <= 32), PreparedTail<Ops, NDIV>, Ops>;
    using type = PlaneProgram<View, Tail>;
    using OutputType = typename IOp::Operation::OutputType;
    static type make(const IOp& iOp) {
        if constexpr (std::is_same_v<Tail, Ops>) {
            return type{ ViewOf<Instantiable<Head>>::make(toIOp<Head>(iOp.params.instance)), fk::detail::tuple_tail(iOp.params) };
        } else {
            type prog{ ViewOf<Instantiable<Head>>::make(toIOp<Head>(iOp.params.instance)), Tail{ fk::detail::tuple_tail(iOp.params), {}, {}, 0u } };
            detail::prepare_divisions<0>(prog.tail, prog.tail.ops);
            return prog;
        }
    }
};

// ---- write side --------------------------------------------------------------------------------------------------
// Packed pixels: element (x, y, z) at data + z*z_stride + y*pitch + x*sizeof(O).
template <typename O>
struct PackedOut {
    using Pixel = O;
    static constexpr bool IS_SPLIT = false;
    O* data;
    uint pitch;
    size_t z_stride; // bytes between planes
};
// Channel c of element (x, y, z) at data + z*z_stride + c*chan_stride + y*pitch + x*sizeof(base).
template <typename O>
struct SplitOut {
    using Pixel = O;
    static constexpr bool IS_SPLIT = true;
    VBase<O>* data;
    uint pitch;
    size_t z_stride;
    size_t chan_stride; // bytes between channel planes
};

template <typename IOp>
struct OutOf {
    static constexpr bool supported = false;
};
template <typename O>
struct OutOf<Write<PerThreadWrite<ND::_2D, O>>> {
    static constexpr bool supported = true;
    using type = PackedOut<O>;
    static type make(const Write<PerThreadWrite<ND::_2D, O>>& iOp) { return type{ iOp.params.data, iOp.params.dims.pitch, 0 }; }
};
template <typename O>
struct OutOf<Write<PerThreadWrite<ND::_1D, O>>> {
    static constexpr bool supported = true;
    using type = PackedOut<O>;
    static type make(const Write<PerThreadWrite<ND::_1D, O>>& iOp) { return type{ iOp.params.data, 0u, 0 }; }
};
template <typename O>
struct OutOf<Write<PerThreadWrite<ND::_3D, O>>> {
    static constexpr bool supported = true;
    using type = PackedOut<O>;
    static type make(const Write<PerThreadWrite<ND::_3D, O>>& iOp) {
        const auto& d = iOp.params.dims;
        return type{ iOp.params.data, d.pitch, static_cast<size_t>(d.plane_pitch) * d.color_planes };
    }
};
template <typename O>
struct OutOf<Write<TensorWrite<O>>> {
    static constexpr bool supported = true;
    using type = PackedOut<O>;
    static type make(const Write<TensorWrite<O>>& iOp) {
        const auto& d = iOp.params.dims;
        return type{ iOp.params.data, d.pitch, static_cast<size_t>(d.plane_pitch) * d.color_planes };
    }
};
template <typename O>
struct OutOf<Write<TensorSplit<O>>> {
    static constexpr bool supported = true;
    using type = SplitOut<O>;
    static type make(const Write<TensorSplit<O>>& iOp) {
        const auto& d = iOp.params.dims;
        // TensorSplit steps channels by width*height elements (memory_operations.h:203-219)
        return type{ iOp.params.data, d.pitch, static_cast<size_t>(d.plane_pitch) * d.color_planes,
                     static_cast<size_t>(d.width) * d.height * sizeof(VBase<O>) };
    }
};

} // namespace exec
} // namespace fk
#endif

// Host-side analysis of a fused chain: turns the read part of a sender and the receiver into plain descriptors
// ("views") that the hand-written kernels index directly.
//
//   PlainView   out(x, y) = img(x + ox, y + oy)                      PerThreadRead<_2D>, possibly under Crop
//   ResizeView  out(x, y) = bilinear(window, (x + off - roi) * f)     Resize<INTER_LINEAR> over a PlainView, possibly
//                                                                    under an outer Crop (reads pulled back through it)
// Folding Crop into an origin is what Crop::exec does one element at a time (reference
// algorithms/image_processing/crop.h:35-38); the Resize parameters are the ones Resize::build computed
// (resize.h:105-166).  Chains that do not match keep their generic per-element form.
#ifndef FK_EXEC_VIEWS_H
#define FK_EXEC_VIEWS_H

#include "fk/ops/image_processing.h"

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

template <typename T, AspectRatio AR>
struct ResizeView {
    using Source = T;
    using Pixel = VectorType_t<float, cn<T>>;
    static constexpr bool IS_RESIZE = true;
    static constexpr bool HAS_ROI = AR != AspectRatio::IGNORE_AR;
    PlainView<T> src; // the window that is resampled; its w, h are the clamp limits
    float fx, fy;
    int off_x, off_y;   // added to the output coordinate before resampling (an outer Crop)
    int x1, y1, x2, y2; // destination region that holds the image; the rest is background
    Pixel background;
    int w, h; // the extent this plane produces
};

struct NoTail {};

template <typename View, typename Tail>
struct PlaneProgram {
    View view;
    Tail tail;
};

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

namespace detail {
template <typename Back, typename = void>
struct BackIsPlain : std::false_type {};
template <typename Back>
struct BackIsPlain<Back, std::enable_if_t<ViewOf<Back>::supported && !ViewOf<Back>::type::IS_RESIZE>> : std::true_type {};
} // namespace detail

template <AspectRatio AR, typename Back>
struct ViewOf<ReadBack<Resize<InterpolationType::INTER_LINEAR, AR, Back>>, std::enable_if_t<detail::BackIsPlain<Back>::value>> {
    static constexpr bool supported = true;
    using Source = typename ViewOf<Back>::type::Source;
    using type = ResizeView<Source, AR>;
    static type make(const ReadBack<Resize<InterpolationType::INTER_LINEAR, AR, Back>>& iOp) {
        type v{};
        v.src = ViewOf<Back>::make(iOp.backIOp);
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
                 std::enable_if_t<isAnyReadType<Head> && ViewOf<Instantiable<Head>>::supported && (sizeof...(ComputeOps) > 0)>> {
    static constexpr bool supported = true;
    using IOp = Read<FusedOperation<Head, ComputeOps...>>;
    using View = typename ViewOf<Instantiable<Head>>::type;
    using Tail = OperationTuple<ComputeOps...>;
    using type = PlaneProgram<View, Tail>;
    using OutputType = typename IOp::Operation::OutputType;
    static type make(const IOp& iOp) {
        return type{ ViewOf<Instantiable<Head>>::make(toIOp<Head>(iOp.params.instance)), fk::detail::tuple_tail(iOp.params) };
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

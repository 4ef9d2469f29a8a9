// Warping: affine and perspective resampling of a back read with bilinear interpolation.
// Same names, parameters and arithmetic as the reference's algorithms/image_processing/warping.h:25-139
// (WarpType, WarpingParameters with the matrix by value, WarpingCoords, Warping complete and builder forms).  The
// matrix maps destination coordinates to source coordinates; destinations whose source point lies outside
// [0, width) x [0, height) are zero.
#ifndef FK_OPS_WARPING_H
#define FK_OPS_WARPING_H

#include "fk/ops/image_processing.h"

namespace fk {

enum class WarpType { Affine = 0, Perspective = 1 };

template <WarpType WType>
struct WarpingParameters;
template <>
struct WarpingParameters<WarpType::Affine> {
    StaticRawPtr<StaticPtrDims2D<3, 2>, float> transformMatrix; // data[2][3]
    Size dstSize;
};
template <>
struct WarpingParameters<WarpType::Perspective> {
    StaticRawPtr<StaticPtrDims2D<3, 3>, float> transformMatrix; // data[3][3]
    Size dstSize;
};

namespace detail {
// (r0 * x + r1 * y) + r2, every product and sum rounded to float: one row of the matrix applied to a pixel position
FK_HD_CNST float warp_row(const float (&row)[3], const int x, const int y) {
    return row[0] * x + row[1] * y + row[2];
}
} // namespace detail

// Source coordinate of a destination pixel; for the perspective case the first two rows are multiplied by the reciprocal
// of the third (a float division, then two multiplications).
template <WarpType WT>
struct WarpingCoords {
private:
    using SelfType = WarpingCoords<WT>;

public:
    FK_BINARY_OPERATION(WarpingCoords, Point, WarpingParameters<WT>, float2)
    FK_HD_STATIC OutputType exec(const InputType& thread, const ParamsType& params) {
        const auto& matrix = params.transformMatrix.data;
        float2 source{ detail::warp_row(matrix[0], thread.x, thread.y), detail::warp_row(matrix[1], thread.x, thread.y) };
        if constexpr (WT == WarpType::Perspective) {
            const float scale = 1.0f / detail::warp_row(matrix[2], thread.x, thread.y);
            source = float2{ scale * source.x, scale * source.y };
        }
        return source;
    }
};

template <WarpType WT, typename BackIOp_ = void>
struct Warping {
private:
    using SelfType = Warping<WT, BackIOp_>;

public:
    FK_STATIC_STRUCT(Warping, SelfType)
    using ReadDataType = typename BackIOp_::Operation::OutputType;
    using OutputType = VectorType_t<float, cn<ReadDataType>>;
    using ParamsType = WarpingParameters<WT>;
    using BackIOp = BackIOp_;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;
    static constexpr WarpType WARP = WT;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params, const BackIOp& backIOp) {
        const float2 coord = WarpingCoords<WT>::exec(thread, params);
        const Size sourceSize(static_cast<int>(BackIOp::Operation::num_elems_x(thread, backIOp)),
                              static_cast<int>(BackIOp::Operation::num_elems_y(thread, backIOp)));
        const bool inside = coord.x >= 0.f && coord.x < sourceSize.width && coord.y >= 0.f && coord.y < sourceSize.height;
        // A position outside the source samples nothing and yields zero.  It is moved to the origin so that the sample
        // can be taken without a branch: straight-line code lets the reads of neighbouring work overlap on a GPU.
        const float2 position = inside ? coord : float2{ 0.f, 0.f };
        const OutputType sample = Interpolate<InterpolationType::INTER_LINEAR, BackIOp>::exec(position, { sourceSize }, backIOp);
        return inside ? sample : make_set<OutputType>(0.f);
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params, opData.backIOp); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.dstSize.width); }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.dstSize.height); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), 1u };
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
};

// Builder form: Warping<WT>::build(params) waits for the read that precedes it in a .then() chain.
template <WarpType WT>
struct Warping<WT, void> {
private:
    using SelfType = Warping<WT, void>;

public:
    FK_STATIC_STRUCT(Warping, SelfType)
    static constexpr bool BUILDER_ONLY = true;
    using ReadDataType = NullType;
    using OutputType = NullType;
    using ParamsType = WarpingParameters<WT>;
    using BackIOp = NullType;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params, {} } }; }
    template <typename RealBackIOp, std::enable_if_t<isAnyReadType<RealBackIOp>, int> = 0>
    FK_HD_STATIC auto build(const RealBackIOp& backIOp, const InstantiableType& self) {
        return Warping<WT, RealBackIOp>::build(self.params, backIOp);
    }
};

} // namespace fk
#endif

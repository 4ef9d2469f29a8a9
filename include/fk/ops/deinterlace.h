// Deinterlace: BLEND (each line averaged with the one above) and INTER_LINEAR (the lines of one field kept, the others
// rebuilt as the average of their neighbours).  Same names, parameters and arithmetic as the reference's
// algorithms/image_processing/deinterlace.h:25-176: sums are taken in the integer type the pixel promotes to, one is
// added, and the result is multiplied by 0.5f.
#ifndef FK_OPS_DEINTERLACE_H
#define FK_OPS_DEINTERLACE_H

#include "fk/ops/arithmetic.h"
#include "fk/ops/memory_operations.h"

namespace fk {

enum class DeinterlaceType { BLEND, INTER_LINEAR };

template <DeinterlaceType DType>
struct DeinterlaceParameters {};
template <>
struct DeinterlaceParameters<DeinterlaceType::INTER_LINEAR> {
    bool useEvenLines{ true };
};

enum class DeinterlaceLinear : bool { USE_EVEN = true, USE_ODD = false };

template <DeinterlaceType DType, typename BackIOp_ = void>
struct Deinterlace {
private:
    using SelfType = Deinterlace<DType, BackIOp_>;
    using ReadOperation = typename BackIOp_::Operation;

public:
    FK_STATIC_STRUCT(Deinterlace, SelfType)
    using ReadDataType = typename ReadOperation::OutputType;
    using OutputType = VectorType_t<float, cn<ReadDataType>>;
    using ParamsType = DeinterlaceParameters<DType>;
    using BackIOp = BackIOp_;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params, const BackIOp& backIOp) {
        const Point above(thread.x, thread.y - 1, thread.z), below(thread.x, thread.y + 1, thread.z);
        if constexpr (DType == DeinterlaceType::BLEND) {
            const auto current = ReadOperation::exec(thread, backIOp);
            if (thread.y > 0) return (current + ReadOperation::exec(above, backIOp) + 1) * 0.5f;
            return current * 1.f;
        } else {
            // the kept field's lines pass through; the first / last line has only one neighbour and passes through too
            // (the reference assumes an even number of lines: with an odd one its USE_ODD case reads one line past the
            // image for the last line, which passes through here)
            const bool odd = (thread.y & 1) != 0;
            const int last = static_cast<int>(ReadOperation::num_elems_y(Point(), backIOp)) - 1;
            const bool interpolate = thread.y != last && (params.useEvenLines ? odd : (!odd && thread.y != 0));
            if (interpolate) return (ReadOperation::exec(above, backIOp) + ReadOperation::exec(below, backIOp) + 1) * 0.5f;
            return ReadOperation::exec(thread, backIOp) * 1.f;
        }
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params, opData.backIOp); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return ReadOperation::num_elems_x(thread, opData.backIOp); }
    FK_HD_STATIC uint num_elems_y(const Point& thread, const OperationDataType& opData) { return ReadOperation::num_elems_y(thread, opData.backIOp); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), 1u };
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
    template <DeinterlaceType D = DType, std::enable_if_t<D == DeinterlaceType::BLEND, int> = 0>
    FK_HD_STATIC InstantiableType build(const BackIOp& backIOp) {
        return InstantiableType{ { ParamsType{}, backIOp } };
    }
    template <DeinterlaceType D = DType, std::enable_if_t<D == DeinterlaceType::INTER_LINEAR, int> = 0>
    FK_HD_STATIC InstantiableType build(const DeinterlaceLinear& lin, const BackIOp& backIOp) {
        return InstantiableType{ { ParamsType{ static_cast<bool>(lin) }, backIOp } };
    }
};

// Builder / entry form: waits for the read that precedes it in a .then() chain, or names it in build().
template <DeinterlaceType DType>
struct Deinterlace<DType, void> {
private:
    using SelfType = Deinterlace<DType, void>;

public:
    FK_STATIC_STRUCT(Deinterlace, SelfType)
    static constexpr bool BUILDER_ONLY = true;
    using ReadDataType = NullType;
    using OutputType = NullType;
    using ParamsType = DeinterlaceParameters<DType>;
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
    template <DeinterlaceType D = DType, std::enable_if_t<D == DeinterlaceType::BLEND, int> = 0>
    FK_HD_STATIC InstantiableType build() {
        return InstantiableType{ { ParamsType{}, {} } };
    }
    template <typename RealBackIOp, std::enable_if_t<isAnyReadType<RealBackIOp>, int> = 0>
    FK_HD_STATIC auto build(const RealBackIOp& backIOp, const InstantiableType& self) {
        return Deinterlace<DType, RealBackIOp>::build(self.params, backIOp);
    }
    template <typename RealBackIOp, DeinterlaceType D = DType, std::enable_if_t<D == DeinterlaceType::BLEND && isAnyReadType<RealBackIOp>, int> = 0>
    FK_HD_STATIC auto build(const RealBackIOp& backIOp) {
        return Deinterlace<DeinterlaceType::BLEND, RealBackIOp>::build(backIOp);
    }
    template <typename RealBackIOp, DeinterlaceType D = DType, std::enable_if_t<D == DeinterlaceType::INTER_LINEAR && isAnyReadType<RealBackIOp>, int> = 0>
    FK_HD_STATIC auto build(const DeinterlaceLinear& lin, const RealBackIOp& backIOp) {
        return Deinterlace<DeinterlaceType::INTER_LINEAR, RealBackIOp>::build(lin, backIOp);
    }
};

} // namespace fk
#endif

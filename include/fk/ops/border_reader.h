// BorderReader: a ReadBack that gives every coordinate, inside or outside its back read, a value.
// Same names, template parameters, build() overloads and index arithmetic as the reference's
// algorithms/image_processing/border_reader.h:24-277 (BorderType, BorderReaderParameters, BorderReader for CONSTANT,
// REPLICATE, REFLECT, WRAP and REFLECT_101; TRANSPARENT_ and ISOLATED are declared there without an implementation).
// Its extent is its back read's: on its own it is the identity; under a Crop whose rectangle leaves the image, a
// Warping or a Resize it supplies the pixels beyond the edge.
#ifndef FK_OPS_BORDER_READER_H
#define FK_OPS_BORDER_READER_H

#include "fk/ops/arithmetic.h"
#include "fk/ops/memory_operations.h"

namespace fk {

// Image boundaries are written `|`.
enum class BorderType : int {
    CONSTANT = 0,     // iiiiii|abcdefgh|iiiiiii with a given i
    REPLICATE = 1,    // aaaaaa|abcdefgh|hhhhhhh
    REFLECT = 2,      // fedcba|abcdefgh|hgfedcb
    WRAP = 3,         // cdefgh|abcdefgh|abcdefg
    REFLECT_101 = 4,  // gfedcb|abcdefgh|gfedcba
    TRANSPARENT_ = 5, // declared only
    DEFAULT = REFLECT_101,
    ISOLATED = 16     // declared only
};

template <BorderType BT, typename ReadType>
struct BorderReaderParameters {};
template <typename ReadType>
struct BorderReaderParameters<BorderType::CONSTANT, ReadType> {
    ReadType value;
};

namespace detail {
FK_HD_CNST int border_abs(const int v) { return v < 0 ? -v : v; }
// v % n for v >= 0.  A value already below n is its own remainder, which is every coordinate within one image size of
// the image; only the rest pay for the integer division (the GPU has no divide instruction: ~40 instructions each).
FK_HD_CNST int border_mod(const int v, const int n) { return v < n ? v : v % n; }
// Source index for coordinate `i` of an axis with `n` elements: high side first, then low side, as the reference
// composes them (border_reader.h:159-277), with the same results for every int.  CONSTANT is handled by its own exec.
template <BorderType BT>
FK_HD_CNST int border_index(const int i, const int n) {
    const int last = n - 1;
    if constexpr (BT == BorderType::REPLICATE) {
        const int high = i < last ? i : last;
        return high > 0 ? high : 0;
    } else if constexpr (BT == BorderType::REFLECT) {
        const int high = last - border_abs(last - i) + (i > last ? 1 : 0);
        return border_mod(border_abs(high) - (high < 0 ? 1 : 0), n);
    } else if constexpr (BT == BorderType::WRAP) {
        const int high = i < n ? i : (i - n < n ? i - n : i % n);
        if (high >= 0) return high;
        return high >= -n ? high + n : high - ((high - n + 1) / n) * n;
    } else {
        static_assert(BT == BorderType::REFLECT_101, "border type without an implementation");
        // |last - |last - i|| is not negative, so its remainder lies in [0, n) and the reference's second
        // `abs(...) % n` leaves it as it is
        return border_mod(border_abs(last - border_abs(last - i)), n);
    }
}
} // namespace detail

template <BorderType BT, typename BackIOp_ = void, typename Enabler = void>
struct BorderReader;

// Complete form: reads `BackIOp_` at the remapped coordinate (or returns the constant).
template <BorderType BT, typename BackIOp_>
struct BorderReader<BT, BackIOp_, std::enable_if_t<isAnyReadType<BackIOp_>>> {
private:
    using SelfType = BorderReader<BT, BackIOp_>;
    using IOType = typename BackIOp_::Operation::OutputType;

public:
    FK_STATIC_STRUCT(BorderReader, SelfType)
    using ReadDataType = IOType;
    using OutputType = IOType;
    using ParamsType = BorderReaderParameters<BT, IOType>;
    using BackIOp = BackIOp_;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;
    static constexpr BorderType BORDER = BT;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params, const BackIOp& backIOp) {
        const int width = static_cast<int>(BackIOp::Operation::num_elems_x(thread, backIOp));
        const int height = static_cast<int>(BackIOp::Operation::num_elems_y(thread, backIOp));
        if constexpr (BT == BorderType::CONSTANT) {
            // No branch around the read: a coordinate outside reads element (0, 0) and drops it.  A thread that handles
            // several elements can then have all its reads in flight at once instead of waiting for each in turn.
            const bool inside = thread.x >= 0 && thread.x < width && thread.y >= 0 && thread.y < height;
            const Point source(inside ? thread.x : 0, inside ? thread.y : 0, thread.z);
            const OutputType sample = BackIOp::Operation::exec(source, backIOp);
            return inside ? sample : params.value;
        } else {
            const Point source(detail::border_index<BT>(thread.x, width), detail::border_index<BT>(thread.y, height), thread.z);
            return BackIOp::Operation::exec(source, backIOp);
        }
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params, opData.backIOp); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return BackIOp::Operation::num_elems_x(thread, opData.backIOp); }
    FK_HD_STATIC uint num_elems_y(const Point& thread, const OperationDataType& opData) { return BackIOp::Operation::num_elems_y(thread, opData.backIOp); }
    FK_HD_STATIC uint num_elems_z(const Point& thread, const OperationDataType& opData) { return BackIOp::Operation::num_elems_z(thread, opData.backIOp); }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), num_elems_z(Point(), opData) };
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
    template <BorderType BT_ = BT, std::enable_if_t<BT_ != BorderType::CONSTANT, int> = 0>
    FK_HD_STATIC InstantiableType build(const BackIOp& backIOp) {
        return InstantiableType{ { {}, backIOp } };
    }
    template <BorderType BT_ = BT, std::enable_if_t<BT_ == BorderType::CONSTANT, int> = 0>
    FK_HD_STATIC InstantiableType build(const BackIOp& backIOp, const ReadDataType& defaultValue) {
        return InstantiableType{ { { defaultValue }, backIOp } };
    }
};

// Builder form with its parameters, waiting for the read that precedes it in a .then() chain.
template <BorderType BT, typename T>
struct BorderReader<BT, TypeList<void, T>, void> {
private:
    using SelfType = BorderReader<BT, TypeList<void, T>, void>;

public:
    FK_STATIC_STRUCT(BorderReader, SelfType)
    static constexpr bool BUILDER_ONLY = true;
    using ReadDataType = T;
    using OutputType = T;
    using ParamsType = BorderReaderParameters<BT, T>;
    using BackIOp = NullType;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    template <typename ReadIOp, std::enable_if_t<isAnyReadType<ReadIOp>, int> = 0>
    FK_HD_STATIC auto build(const ReadIOp& readIOp, const InstantiableType& self) {
        using Complete = BorderReader<BT, ReadIOp>;
        if constexpr (BT == BorderType::CONSTANT) {
            return Complete::build(readIOp, detail::cast_channels<typename Complete::ReadDataType>(self.params.value));
        } else {
            return Complete::build(readIOp);
        }
    }
};

// Entry form: BorderReader<BT>::build(...) with no back read named in the type.
template <BorderType BT>
struct BorderReader<BT, void, void> {
private:
    using SelfType = BorderReader<BT, void, void>;

public:
    FK_STATIC_STRUCT(BorderReader, SelfType)
    using InstanceType = ReadBackType;
    static constexpr bool BUILDER_ONLY = true;

    template <typename T, BorderType BT_ = BT, std::enable_if_t<BT_ == BorderType::CONSTANT && !isAnyReadType<T>, int> = 0>
    FK_HD_STATIC auto build(const T& defaultValue) {
        return BorderReader<BT, TypeList<void, T>>::build({ { defaultValue }, {} });
    }
    template <typename T, BorderType BT_ = BT, std::enable_if_t<BT_ != BorderType::CONSTANT, int> = 0>
    FK_HD_STATIC auto build() {
        return BorderReader<BT, TypeList<void, T>>::build({});
    }
    template <typename BF, BorderType BT_ = BT, std::enable_if_t<BT_ != BorderType::CONSTANT && isAnyReadType<BF>, int> = 0>
    FK_HD_STATIC auto build(const BF& backIOp) {
        return BorderReader<BT, BF>::build(backIOp);
    }
    template <typename BF, BorderType BT_ = BT, std::enable_if_t<BT_ == BorderType::CONSTANT && isAnyReadType<BF>, int> = 0>
    FK_HD_STATIC auto build(const BF& backIOp, const typename BF::Operation::OutputType& defaultValue) {
        return BorderReader<BT, BF>::build(backIOp, defaultValue);
    }
};

} // namespace fk
#endif

// Compile-time description of reading several small elements as one wider vector ("thread fusion" in the vocabulary of
// the Fused Kernel Library): which wider type carries how many elements, and how to take them apart and put them together.
//
// Follows the reference's core/execution_model/thread_fusion.h:27-152.  The wider type of an element type with base B:
//   1-byte B:  1 or 2 channels -> B4 (4 or 2 elements); 3 and 4 channels stay as they are
//   2-/4-byte B: 1 channel -> B2 (2 elements); more channels stay as they are
//   8-byte B:  stays as it is
// The transform kernels of this library choose their own grouping (whole dwords per lane, staged through LDS), so this
// type is a utility for user code, not what the executors consult.
#ifndef FK_CORE_THREAD_FUSION_INFO_H
#define FK_CORE_THREAD_FUSION_INFO_H

#include "fk/core/type_utils.h"
#include "fk/core/vector_types.h"

namespace fk {
namespace detail {
template <typename Source>
constexpr int widened_channels() {
    constexpr int c = cn<Source>;
    constexpr size_t bytes = sizeof(VBase<Source>);
    if (bytes == 1) return c <= 2 ? 4 : c;
    if (bytes <= 4) return c == 1 ? 2 : c;
    return c;
}
template <typename Source, int CHANNELS = widened_channels<Source>()>
struct Widened {
    using type = VectorType_t<VBase<Source>, CHANNELS>;
};
template <typename Source>
struct Widened<Source, 1> { // 8-byte scalars and one-channel vectors of them: unchanged
    using type = Source;
};
} // namespace detail

template <typename SourceType>
using TFBiggerType_t = typename detail::Widened<SourceType>::type;

template <uint CHANNELS>
constexpr bool isValidChannelNumber = CHANNELS >= 1 && CHANNELS <= 4;

template <typename ReadType, typename WriteType, bool ENABLED_>
struct ThreadFusionInfo {
    static constexpr bool ENABLED = ENABLED_ && isValidChannelNumber<static_cast<uint>((cn<TFBiggerType_t<ReadType>> / cn<ReadType>) * cn<WriteType>)>;
    using BiggerReadType = std::conditional_t<ENABLED, TFBiggerType_t<ReadType>, ReadType>;
    static constexpr uint elems_per_thread = static_cast<uint>(cn<BiggerReadType> / cn<ReadType>);
    using BiggerWriteType = VectorType_t<VBase<WriteType>, static_cast<int>(elems_per_thread) * cn<WriteType>>;

    // element IDX of a wide value
    template <int IDX>
    FK_HD_STATIC ReadType get(const BiggerReadType& data) {
        static_assert(IDX >= 0 && IDX < static_cast<int>(elems_per_thread), "Index out of range for this ThreadFusionInfo");
        return take<IDX * cn<ReadType>>(data, std::make_integer_sequence<int, cn<ReadType>>{});
    }
    // the wide value made of elems_per_thread elements
    template <typename... OriginalTypes>
    FK_HD_STATIC BiggerWriteType make(const OriginalTypes&... data) {
        static_assert(and_v<std::is_same_v<WriteType, OriginalTypes>...>, "Not all types are the same when making the ThreadFusion BiggerType value");
        static_assert(sizeof...(OriginalTypes) == elems_per_thread, "One value per fused element");
        if constexpr (sizeof...(OriginalTypes) == 1) {
            return first(data...);
        } else if constexpr (cn<WriteType> == 1) {
            return make_<BiggerWriteType>(vget<0>(data)...);
        } else {
            static_assert(cn<WriteType> == 2 && sizeof...(OriginalTypes) == 2, "Only pairs of two-channel elements fuse");
            return join(data...);
        }
    }

private:
    template <int FIRST, int... K>
    FK_HD_STATIC ReadType take(const BiggerReadType& data, std::integer_sequence<int, K...>) {
        if constexpr (validCUDAVec<BiggerReadType>) {
            return make_<ReadType>(vget<FIRST + K>(data)...);
        } else {
            return data;
        }
    }
    FK_HD_STATIC BiggerWriteType first(const WriteType& data) { return data; }
    FK_HD_STATIC BiggerWriteType join(const WriteType& a, const WriteType& b) { return make_<BiggerWriteType>(a.x, a.y, b.x, b.y); }
};

// What an operation that handles ELEMS_PER_THREAD elements of SourceType at once takes or returns: the vector of that many
// elements when the operation passes its data through unchanged, otherwise its declared OutputType.
namespace detail {
template <typename SourceType, uint ELEMS_PER_THREAD, typename OutputType, typename = void>
struct FusedElements {
    using Wide = VectorType<VBase<SourceType>, cn<SourceType> * static_cast<int>(ELEMS_PER_THREAD)>;
    using type = std::conditional_t<validCUDAVec<SourceType>, typename Wide::type_v, typename Wide::type>;
};
template <typename SourceType, uint ELEMS_PER_THREAD, typename OutputType>
struct FusedElements<SourceType, ELEMS_PER_THREAD, OutputType,
                     std::enable_if_t<!std::is_same_v<SourceType, OutputType> || std::is_same_v<SourceType, NullType>>> {
    using type = OutputType;
};
} // namespace detail
template <typename SourceType, uint ELEMS_PER_THREAD, typename OutputType = SourceType>
using ThreadFusionType = typename detail::FusedElements<SourceType, ELEMS_PER_THREAD, OutputType>::type;

template <bool THREAD_FUSION_ENABLED, typename... IOpTypes>
FK_HD_CNST bool isThreadFusionEnabled() {
    using ReadOperation = typename TypeAt_t<0, TypeList<IOpTypes...>>::Operation;
    using WriteOperation = typename TypeAt_t<-1, TypeList<IOpTypes...>>::Operation;
    return ReadOperation::THREAD_FUSION && WriteOperation::THREAD_FUSION && THREAD_FUSION_ENABLED;
}
} // namespace fk
#endif

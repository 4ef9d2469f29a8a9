// Planar / transposed tensor layouts, circular (ring) memory operations and CircularTensor.
//
// Same names, template parameters and addressing as the reference's core/execution_model/memory_operations.h:228-255
// (TensorTSplit), :257-348 (TensorPack, TensorTPack), :350-407 (SplitWrite), :425-590 (CircularDirection,
// CircularMemoryParams, CircularBatchRead/Write, CircularTensorRead/Write) and core/data/circular_tensor.h:24-161
// (CircularTensorOrder, SequenceSelectorType, ColorPlanes, CircularTensor).
//
// CircularTensor::update runs here: the reference builds its two operation sequences but ships no executor for the
// divergent launch they need (circular_tensor.h:136-150).  One launch does what that code describes: the new frame's
// chain writes the newest plane of the tensor and the ring slot `next`, every other plane is copied from the ring slot
// that holds the frame of its age.
#ifndef FK_OPS_CIRCULAR_H
#define FK_OPS_CIRCULAR_H

#include <vector>

#include "fk/exec/executor.h"

namespace fk {

// ---- layouts ---------------------------------------------------------------------------------------------------
// Channels of the pixel into the channel planes of a transposed tensor: C x N x H x W.
template <typename T>
struct TensorTSplit {
private:
    using SelfType = TensorTSplit<T>;

public:
    FK_STATIC_STRUCT(TensorTSplit, SelfType)
    static_assert(cn<T> >= 2, "Wrong type for split tensor write. It must be one of <type>2, <type>3 or <type>4.");
    using ParamsType = RawPtr<ND::T3D, VBase<T>>;
    using InputType = T;
    using WriteDataType = VBase<T>;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        *PtrAccessor<ND::T3D>::point(thread, params, 0) = input.x;
        *PtrAccessor<ND::T3D>::point(thread, params, 1) = input.y;
        if constexpr (cn<T> >= 3) *PtrAccessor<ND::T3D>::point(thread, params, 2) = input.z;
        if constexpr (cn<T> == 4) *PtrAccessor<ND::T3D>::point(thread, params, 3) = input.w;
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Ptr<ND::T3D, VBase<T>>& ptr) { return build(ptr.ptr()); }
};

#define FK_TENSOR_READ_COMMON(SELF, PARAMS)                                                                            \
    FK_STATIC_STRUCT(SELF, SelfType)                                                                                   \
    static_assert(cn<T> >= 2, "Wrong type for split tensor read. It must be one of <type>2, <type>3 or <type>4.");      \
    using ParamsType = PARAMS;                                                                                         \
    using ReadDataType = VBase<T>;                                                                                     \
    using OutputType = T;                                                                                              \
    using InstanceType = ReadType;                                                                                     \
    using OperationDataType = OperationData<SelfType>;                                                                 \
    using InstantiableType = Read<SelfType>;                                                                           \
    static constexpr bool IS_FUSED_OP = false;                                                                         \
    static constexpr bool THREAD_FUSION = false;                                                                       \
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); } \
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }  \
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return opData.params.dims.height; } \
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType& opData) { return opData.params.dims.planes; } \
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }        \
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {                                     \
        return { opData.params.dims.width, opData.params.dims.height, opData.params.dims.planes };                     \
    }                                                                                                                  \
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }           \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }

// The inverse of TensorSplit: channel planes of image z (N x C x H x W) into one pixel.
template <typename T>
struct TensorPack {
private:
    using SelfType = TensorPack<T>;
    using PtrType = RawPtr<ND::_3D, VBase<T>>;

public:
    FK_TENSOR_READ_COMMON(TensorPack, PtrType)
    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        const int planePixels = static_cast<int>(params.dims.width * params.dims.height);
        const ReadDataType* const work_plane = PtrAccessor<ND::_3D>::cr_point(thread, params);
        if constexpr (cn<T> == 2) return T{ work_plane[0], work_plane[planePixels] };
        else if constexpr (cn<T> == 3) return T{ work_plane[0], work_plane[planePixels], work_plane[planePixels * 2] };
        else return T{ work_plane[0], work_plane[planePixels], work_plane[planePixels * 2], work_plane[planePixels * 3] };
    }
    static inline InstantiableType build(const Ptr<ND::_3D, VBase<T>>& ptr) { return build(ptr.ptr()); }
};

// The inverse of TensorTSplit.
template <typename T>
struct TensorTPack {
private:
    using SelfType = TensorTPack<T>;
    using PtrType = RawPtr<ND::T3D, VBase<T>>;

public:
    FK_TENSOR_READ_COMMON(TensorTPack, PtrType)
    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        const ReadDataType x = *PtrAccessor<ND::T3D>::cr_point(thread, params, 0);
        const ReadDataType y = *PtrAccessor<ND::T3D>::cr_point(thread, params, 1);
        if constexpr (cn<T> == 2) {
            return T{ x, y };
        } else if constexpr (cn<T> == 3) {
            return T{ x, y, *PtrAccessor<ND::T3D>::cr_point(thread, params, 2) };
        } else {
            return T{ x, y, *PtrAccessor<ND::T3D>::cr_point(thread, params, 2), *PtrAccessor<ND::T3D>::cr_point(thread, params, 3) };
        }
    }
    static inline InstantiableType build(const Ptr<ND::T3D, VBase<T>>& ptr) { return build(ptr.ptr()); }
};
#undef FK_TENSOR_READ_COMMON

// One buffer per channel.
template <ND D, typename T, typename Enabler = void>
struct SplitWriteParams {};
template <ND D, typename T>
struct SplitWriteParams<D, T, std::enable_if_t<cn<T> == 2>> {
    RawPtr<D, VBase<T>> x, y;
};
template <ND D, typename T>
struct SplitWriteParams<D, T, std::enable_if_t<cn<T> == 3>> {
    RawPtr<D, VBase<T>> x, y, z;
};
template <ND D, typename T>
struct SplitWriteParams<D, T, std::enable_if_t<cn<T> == 4>> {
    RawPtr<D, VBase<T>> x, y, z, w;
};
template <ND D, typename T>
struct SplitWrite {
private:
    using SelfType = SplitWrite<D, T>;

public:
    FK_STATIC_STRUCT(SplitWrite, SelfType)
    static_assert(cn<T> >= 2, "Wrong type for split write. It must be one of <type>2, <type>3 or <type>4.");
    using ParamsType = SplitWriteParams<D, T>;
    using InputType = T;
    using WriteDataType = VBase<T>;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        *PtrAccessor<D>::point(thread, params.x) = input.x;
        *PtrAccessor<D>::point(thread, params.y) = input.y;
        if constexpr (cn<T> >= 3) *PtrAccessor<D>::point(thread, params.z) = input.z;
        if constexpr (cn<T> == 4) *PtrAccessor<D>::point(thread, params.w) = input.w;
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.x.dims.width; }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.x.dims.pitch; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const std::vector<Ptr2D<VBase<T>>>& output) {
        static_assert(D == ND::_2D, "one 2D buffer per channel");
        if constexpr (cn<T> == 2) return InstantiableType{ { { output.at(0).ptr(), output.at(1).ptr() } } };
        else if constexpr (cn<T> == 3) return InstantiableType{ { { output.at(0).ptr(), output.at(1).ptr(), output.at(2).ptr() } } };
        else return InstantiableType{ { { output.at(0).ptr(), output.at(1).ptr(), output.at(2).ptr(), output.at(3).ptr() } } };
    }
};

// ---- circular memory operations ------------------------------------------------------------------------------
enum class CircularDirection { Ascendent, Descendent };

template <typename OperationDataTypeArray>
struct CircularMemoryParams {
    int first;
    OperationDataTypeArray opData;
};

namespace circular_batch_internal {
// Plane z of the logical order is ring slot first + z (Ascendent) or first - z (Descendent), modulo BATCH.
template <CircularDirection direction, int BATCH>
FK_HD_CNST Point computeCircularThreadIdx(const Point& currentIdx, const int& fst) {
    if constexpr (direction == CircularDirection::Ascendent) {
        const int z = currentIdx.z + fst;
        return Point(currentIdx.x, currentIdx.y, z >= BATCH ? z - BATCH : z);
    } else {
        const int z = fst - currentIdx.z;
        return Point(currentIdx.x, currentIdx.y, z < 0 ? BATCH + z : z);
    }
}
} // namespace circular_batch_internal

#define FK_CIRCULAR_COMMON(SELF)                                                                                       \
    FK_STATIC_STRUCT(SELF, SelfType)                                                                                   \
    using OperationDataType = OperationData<SelfType>;                                                                 \
    static constexpr bool IS_FUSED_OP = false;                                                                         \
    static constexpr bool THREAD_FUSION = false;                                                                       \
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }           \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }

// BATCH separate buffers read as a ring.
template <CircularDirection direction, typename Operation, int BATCH>
struct CircularBatchRead {
private:
    using SelfType = CircularBatchRead<direction, Operation, BATCH>;

public:
    using ParamsType = CircularMemoryParams<OperationData<Operation>[BATCH]>;
    using ReadDataType = typename Operation::ReadDataType;
    using OutputType = typename Operation::OutputType;
    using InstanceType = ReadType;
    using InstantiableType = Read<SelfType>;
    FK_CIRCULAR_COMMON(CircularBatchRead)
    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        const Point slot = circular_batch_internal::computeCircularThreadIdx<direction, BATCH>(thread, params.first);
        return Operation::exec(slot, params.opData[slot.z]);
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData[thread.z]); }
    FK_HD_STATIC uint num_elems_y(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_y(thread, opData.params.opData[thread.z]); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return BATCH; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), static_cast<uint>(BATCH) };
    }
};
template <CircularDirection direction, typename Operation, int BATCH>
struct CircularBatchWrite {
private:
    using SelfType = CircularBatchWrite<direction, Operation, BATCH>;

public:
    using ParamsType = CircularMemoryParams<OperationData<Operation>[BATCH]>;
    using InputType = typename Operation::InputType;
    using WriteDataType = typename Operation::WriteDataType;
    using InstanceType = WriteType;
    using InstantiableType = Write<SelfType>;
    FK_CIRCULAR_COMMON(CircularBatchWrite)
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        const Point slot = circular_batch_internal::computeCircularThreadIdx<direction, BATCH>(thread, params.first);
        Operation::exec(slot, input, params.opData[slot.z]);
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData[thread.z]); }
};

// One tensor whose planes are read / written as a ring.
template <CircularDirection direction, typename Operation, int BATCH>
struct CircularTensorRead {
private:
    using SelfType = CircularTensorRead<direction, Operation, BATCH>;

public:
    using ParamsType = CircularMemoryParams<OperationData<Operation>>;
    using ReadDataType = typename Operation::ReadDataType;
    using OutputType = typename Operation::OutputType;
    using InstanceType = ReadType;
    using InstantiableType = Read<SelfType>;
    FK_CIRCULAR_COMMON(CircularTensorRead)
    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        return Operation::exec(circular_batch_internal::computeCircularThreadIdx<direction, BATCH>(thread, params.first), params.opData);
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData); }
    FK_HD_STATIC uint num_elems_y(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_y(thread, opData.params.opData); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return BATCH; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), static_cast<uint>(BATCH) };
    }
};
template <CircularDirection direction, typename Operation, int BATCH>
struct CircularTensorWrite {
private:
    using SelfType = CircularTensorWrite<direction, Operation, BATCH>;

public:
    using ParamsType = CircularMemoryParams<OperationData<Operation>>;
    using InputType = typename Operation::InputType;
    using WriteDataType = typename Operation::WriteDataType;
    using InstanceType = WriteType;
    using InstantiableType = Write<SelfType>;
    FK_CIRCULAR_COMMON(CircularTensorWrite)
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        Operation::exec(circular_batch_internal::computeCircularThreadIdx<direction, BATCH>(thread, params.first), input, params.opData);
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData); }
};
#undef FK_CIRCULAR_COMMON

// ---- CircularTensor ----------------------------------------------------------------------------------------------
enum class CircularTensorOrder { NewestFirst, OldestFirst };

// Which of the two sequences of an update plane `index` runs: 1 = the new frame's chain, 2 = copy from the ring.
template <CircularTensorOrder CTO, int BATCH>
struct SequenceSelectorType {
    FK_HD_STATIC uint at(const uint& index) {
        if constexpr (CTO == CircularTensorOrder::NewestFirst) return index > 0 ? 2u : 1u;
        else return index != BATCH - 1 ? 2u : 1u;
    }
};

// the struct forms behind CTReadDirection_v and CoreType_t (circular_tensor.h:37-66)
template <CircularTensorOrder CT_ORDER>
struct CTReadDirection {
    static constexpr CircularDirection dir = CT_ORDER == CircularTensorOrder::NewestFirst ? CircularDirection::Descendent : CircularDirection::Ascendent;
};
template <CircularTensorOrder CT_ORDER>
constexpr CircularDirection CTReadDirection_v = CT_ORDER == CircularTensorOrder::NewestFirst ? CircularDirection::Descendent : CircularDirection::Ascendent;

enum class ColorPlanes { Standard, Transposed };
template <typename T, ColorPlanes CP_MODE>
using CoreType_t = std::conditional_t<CP_MODE == ColorPlanes::Standard, Tensor<T>, TensorT<T>>;
template <typename T, ColorPlanes CP_MODE>
struct CoreType {
    using type = CoreType_t<T, CP_MODE>;
};

template <typename T, int COLOR_PLANES, typename Enabler = void>
struct CircularTensorStoreType {};
template <typename T, int COLOR_PLANES>
struct CircularTensorStoreType<T, COLOR_PLANES, std::enable_if_t<std::is_aggregate_v<T> && COLOR_PLANES == 1>> {
    using type = T;
};
template <typename T, int COLOR_PLANES>
struct CircularTensorStoreType<T, COLOR_PLANES, std::enable_if_t<!std::is_aggregate_v<T> && (COLOR_PLANES > 1)>> {
    using type = VectorType_t<T, COLOR_PLANES>;
};

namespace detail {
// Shifts thread.z by `offset` before `Op` sees it and reports `planes` planes: lets one job of a divergent launch
// cover a sub-range of the planes of an operation.
template <typename Op>
struct PlaneOffsetRead {
private:
    using SelfType = PlaneOffsetRead<Op>;

public:
    FK_STATIC_STRUCT(PlaneOffsetRead, SelfType)
    struct ParamsType {
        OperationData<Op> inner;
        int offset;
        uint planes;
    };
    using ReadDataType = typename Op::ReadDataType;
    using OutputType = typename Op::OutputType;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;
    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        return Op::exec(Point(thread.x, thread.y, thread.z + params.offset), params.inner);
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return Op::num_elems_x(Point(0, 0, opData.params.offset), opData.params.inner); }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return Op::num_elems_y(Point(0, 0, opData.params.offset), opData.params.inner); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType& opData) { return opData.params.planes; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), opData.params.planes };
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
};
template <typename Op>
struct PlaneOffsetWrite {
private:
    using SelfType = PlaneOffsetWrite<Op>;

public:
    FK_STATIC_STRUCT(PlaneOffsetWrite, SelfType)
    struct ParamsType {
        OperationData<Op> inner;
        int offset;
    };
    using InputType = typename Op::InputType;
    using WriteDataType = typename Op::WriteDataType;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        Op::exec(Point(thread.x, thread.y, thread.z + params.offset), input, params.inner);
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
};
// Two writes of the same value.
template <typename First, typename Second>
struct TeeWrite {
private:
    using SelfType = TeeWrite<First, Second>;

public:
    FK_STATIC_STRUCT(TeeWrite, SelfType)
    static_assert(std::is_same_v<typename First::InputType, typename Second::InputType>, "both writes take the same pixel");
    struct ParamsType {
        OperationData<First> first;
        OperationData<Second> second;
    };
    using InputType = typename First::InputType;
    using WriteDataType = typename First::WriteDataType;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        First::exec(thread, input, params.first);
        Second::exec(thread, input, params.second);
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
};

template <typename WriteOp, typename StoreT>
struct RingReadFor;
template <typename StoreT>
struct RingReadFor<TensorWrite<StoreT>, StoreT> { using type = TensorRead<StoreT>; };
template <typename StoreT>
struct RingReadFor<TensorSplit<StoreT>, StoreT> { using type = TensorPack<StoreT>; };
template <typename StoreT>
struct RingReadFor<TensorTSplit<StoreT>, StoreT> { using type = TensorTPack<StoreT>; };
} // namespace detail

// The last BATCH results of a chain, kept in age order: after every update plane 0 (NewestFirst) or plane BATCH - 1
// (OldestFirst) is the newest result and the others follow by age.  T with COLOR_PLANES > 1 is a base type whose pixels
// (VectorType_t<T, COLOR_PLANES>) are stored as channel planes; an aggregate T with COLOR_PLANES == 1 is stored packed.
template <typename T, int COLOR_PLANES, int BATCH, CircularTensorOrder CT_ORDER, ColorPlanes CP_MODE>
class CircularTensor : public CoreType_t<T, CP_MODE> {
    using ParentType = CoreType_t<T, CP_MODE>;
    using StoreT = typename CircularTensorStoreType<T, COLOR_PLANES>::type;

public:
    CircularTensor() {}
    CircularTensor(const uint& width_, const uint& height_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : ParentType(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_), m_tempTensor(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_) {}
    // Views over device memory the caller owns: the tensor and its ring of the same size; `nextUpdateIdx` is the ring
    // slot the next update fills.
    CircularTensor(T* tensor, T* ring, const uint& width_, const uint& height_, const int& nextUpdateIdx, const int& deviceID_ = 0)
        : ParentType(tensor, width_, height_, BATCH, COLOR_PLANES, MemType::Device, deviceID_),
          m_tempTensor(ring, width_, height_, BATCH, COLOR_PLANES, MemType::Device, deviceID_), m_nextUpdateIdx(nextUpdateIdx) {}

    void Alloc(const uint& width_, const uint& height_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->allocTensor(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_);
        m_tempTensor.allocTensor(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_);
    }
    int nextUpdateIdx() const { return m_nextUpdateIdx; }

    // update(stream, read, compute..., write): `write` is TensorWrite / TensorSplit / TensorTSplit of StoreT built on
    // this tensor.
    template <typename... IOpTypes>
    void update(Stream& stream, const IOpTypes&... iOps) {
        const auto& userWrite = exec::last_of(iOps...);
        using WriteIOp = std::decay_t<decltype(userWrite)>;
        using WriteOp = typename WriteIOp::Operation;
        static_assert(std::is_same_v<WriteOp, TensorWrite<StoreT>> || std::is_same_v<WriteOp, TensorSplit<StoreT>> ||
                          std::is_same_v<WriteOp, TensorTSplit<StoreT>>,
                      "The write of a CircularTensor update must be TensorWrite, TensorSplit or TensorTSplit of its stored pixel type.");
        static_assert(CP_MODE != ColorPlanes::Transposed || std::is_same_v<WriteOp, TensorTSplit<StoreT>>,
                      "Need to use TensorTSplit as write function because you are using a transposed CircularTensor (CP_MODE = Transposed)");
        using RingRead = CircularTensorRead<CTReadDirection_v<CT_ORDER>, typename detail::RingReadFor<WriteOp, StoreT>::type, BATCH>;
        using RingWrite = CircularTensorWrite<CircularDirection::Ascendent, WriteOp, BATCH>;
        constexpr int NEW_PLANE = CT_ORDER == CircularTensorOrder::NewestFirst ? 0 : BATCH - 1;
        constexpr int FIRST_COPIED = CT_ORDER == CircularTensorOrder::NewestFirst ? 1 : 0;
        static_assert(SequenceSelectorType<CT_ORDER, BATCH>::at(NEW_PLANE) == 1u, "the selector's plane for the new frame");

        // sequence 1: the chain of the new frame, into its plane of the tensor and into ring slot next (+ that plane)
        const auto chain = exec::sender_of(iOps...);
        using ChainOp = typename std::decay_t<decltype(chain)>::Operation;
        const Read<detail::PlaneOffsetRead<ChainOp>> newSender{ { { static_cast<const OperationData<ChainOp>&>(chain), NEW_PLANE, 1u } } };
        OperationData<RingWrite> toRing{};
        toRing.params.first = m_nextUpdateIdx;
        toRing.params.opData.params = m_tempTensor.ptr();
        using Tee = detail::TeeWrite<RingWrite, WriteOp>;
        const OperationData<Tee> tee{ { toRing, static_cast<const OperationData<WriteOp>&>(userWrite) } };
        const Write<detail::PlaneOffsetWrite<Tee>> newReceiver{ { { tee, NEW_PLANE } } };

        // sequence 2: every other plane from the ring slot that holds the frame of its age
        OperationData<RingRead> fromRing{};
        fromRing.params.first = m_nextUpdateIdx;
        fromRing.params.opData.params = m_tempTensor.ptr();
        const Read<detail::PlaneOffsetRead<RingRead>> copySender{ { { fromRing, FIRST_COPIED, static_cast<uint>(BATCH - 1) } } };
        const Write<detail::PlaneOffsetWrite<WriteOp>> copyReceiver{ { { static_cast<const OperationData<WriteOp>&>(userWrite), FIRST_COPIED } } };

        using NewSeq = InstantiableOperationSequence<std::decay_t<decltype(newSender)>, std::decay_t<decltype(newReceiver)>>;
        using CopySeq = InstantiableOperationSequence<std::decay_t<decltype(copySender)>, std::decay_t<decltype(copyReceiver)>>;
        if constexpr (BATCH > 1 && (std::is_same_v<WriteOp, TensorSplit<StoreT>> || std::is_same_v<WriteOp, TensorWrite<StoreT>>)) {
            // In these two layouts a frame is one run of rows in the tensor and in the ring alike (its channel planes
            // follow each other), so sequence 2 moves whole frames: the same copy as a batch of BATCH - 1 images read
            // and written as they lie, which the executor runs with 16-byte accesses instead of one element at a time.
            using E = std::remove_pointer_t<decltype(userWrite.params.data)>;
            const auto& dst = userWrite.params;
            const RawPtr<ND::_3D, E> ring = m_tempTensor.ptr();
            const bool tight = dst.dims.plane_pitch == dst.dims.pitch * dst.dims.height && ring.dims.plane_pitch == ring.dims.pitch * ring.dims.height &&
                               ring.dims.pitch == dst.dims.pitch && ring.dims.color_planes == dst.dims.color_planes;
            if (tight) {
                const uint rows = dst.dims.height * dst.dims.color_planes;
                const size_t frame_bytes = static_cast<size_t>(dst.dims.pitch) * rows;
                std::array<RawPtr<ND::_2D, E>, BATCH - 1> frames;
                for (int i = 0; i < BATCH - 1; ++i) {
                    const Point slot = circular_batch_internal::computeCircularThreadIdx<CTReadDirection_v<CT_ORDER>, BATCH>(Point(0, 0, FIRST_COPIED + i), m_nextUpdateIdx);
                    frames[i] = RawPtr<ND::_2D, E>{ reinterpret_cast<E*>(reinterpret_cast<char*>(ring.data) + slot.z * frame_bytes),
                                                   PtrDims<ND::_2D>(dst.dims.width, rows, dst.dims.pitch) };
                }
                const RawPtr<ND::_3D, E> copied{ reinterpret_cast<E*>(reinterpret_cast<char*>(dst.data) + FIRST_COPIED * frame_bytes),
                                                 PtrDims<ND::_3D>(dst.dims.width, rows, BATCH - 1, 1, dst.dims.pitch) };
                const auto framesSender = PerThreadRead<ND::_2D, E>::build(frames);
                const auto framesReceiver = TensorWrite<E>::build(copied);
                using FramesSeq = InstantiableOperationSequence<std::decay_t<decltype(framesSender)>, std::decay_t<decltype(framesReceiver)>>;
                Executor<DivergentBatchTransformDPP<ParArch::GPU_AMD>>::executeOperations(stream, NewSeq{ newSender, newReceiver }, FramesSeq{ framesSender, framesReceiver });
                m_nextUpdateIdx = (m_nextUpdateIdx + 1) % BATCH;
                return;
            }
        }
        Executor<DivergentBatchTransformDPP<ParArch::GPU_AMD>>::executeOperations(stream, NewSeq{ newSender, newReceiver }, CopySeq{ copySender, copyReceiver });
        m_nextUpdateIdx = (m_nextUpdateIdx + 1) % BATCH;
    }

private:
    CoreType_t<T, CP_MODE> m_tempTensor;
    int m_nextUpdateIdx{ 0 };
};

} // namespace fk
#endif

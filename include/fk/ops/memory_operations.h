// Memory operations: PerThreadRead/Write, TensorRead/Write, TensorSplit, ReadSet.
// Same names, template parameters, build() overloads and addressing as the reference's
// core/execution_model/memory_operations.h:71-226 and algorithms/basic_ops/set.h:23-77.
#ifndef FK_OPS_MEMORY_OPERATIONS_H
#define FK_OPS_MEMORY_OPERATIONS_H

#include "fk/core/operation_model.h"
#include "fk/core/ptr.h"

namespace fk {

// Size (x, y) that a read IOp spans (memory_operations.h:35-69).
template <typename IOp>
struct Num_elems {
    FK_HD_STATIC uint x(const Point& thread, const IOp& iOp) { return IOp::Operation::num_elems_x(thread, iOp); }
    FK_HD_STATIC uint y(const Point& thread, const IOp& iOp) { return IOp::Operation::num_elems_y(thread, iOp); }
    FK_HD_STATIC uint z(const Point& thread, const IOp& iOp) { return IOp::Operation::num_elems_z(thread, iOp); }
    FK_HD_STATIC Size size(const Point& thread, const IOp& iOp) {
        return Size(static_cast<int>(x(thread, iOp)), static_cast<int>(y(thread, iOp)));
    }
};

template <ND D, typename T>
struct PerThreadRead : BatchBuilders<PerThreadRead<D, T>> {
private:
    using SelfType = PerThreadRead<D, T>;

public:
    FK_STATIC_STRUCT(PerThreadRead, SelfType)
    using ParamsType = RawPtr<D, T>;
    using ReadDataType = T;
    using OutputType = T;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = true;
    static constexpr ND DIMS = D;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        return fk::detail::read_element(PtrAccessor<D>::cr_point(thread, params));
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) {
        if constexpr (D == ND::_1D) return 1;
        else return opData.params.dims.height;
    }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType& opData) {
        if constexpr (D == ND::_1D || D == ND::_2D) return 1;
        else return opData.params.dims.planes;
    }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), num_elems_z(Point(), opData) };
    }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Ptr<D, T>& ptr) { return build(ptr.ptr()); }
    using BatchBuilders<SelfType>::build;
};

template <ND D, typename T>
struct PerThreadWrite {
private:
    using SelfType = PerThreadWrite<D, T>;

public:
    FK_STATIC_STRUCT(PerThreadWrite, SelfType)
    using ParamsType = RawPtr<D, T>;
    using InputType = T;
    using WriteDataType = T;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = true;
    static constexpr ND DIMS = D;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) { *PtrAccessor<D>::point(thread, params) = input; }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
    // one write per buffer (memory_operations.h:113-152: the batch builders of a write return the array itself)
    template <size_t BATCH_N, typename Buffer>
    static inline constexpr std::array<InstantiableType, BATCH_N> build_batch(const std::array<Buffer, BATCH_N>& buffers) {
        std::array<InstantiableType, BATCH_N> out{};
        for (size_t i = 0; i < BATCH_N; ++i) out[i] = build(buffers[i]);
        return out;
    }
    // all of them behind one Write operation: plane z of the launch goes to buffer z
    template <size_t BATCH_N, typename Buffer>
    static inline constexpr auto build(const std::array<Buffer, BATCH_N>& buffers) {
        return BatchWrite<BATCH_N, SelfType>::build(build_batch(buffers));
    }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Ptr<D, T>& ptr) { return build(ptr.ptr()); }
};

template <typename T>
struct TensorRead : BatchBuilders<TensorRead<T>> {
private:
    using SelfType = TensorRead<T>;

public:
    FK_STATIC_STRUCT(TensorRead, SelfType)
    using ParamsType = RawPtr<ND::_3D, T>;
    using ReadDataType = T;
    using OutputType = T;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = true;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        return fk::detail::read_element(PtrAccessor<ND::_3D>::cr_point(thread, params));
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return opData.params.dims.height; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType& opData) { return opData.params.dims.planes; }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), num_elems_z(Point(), opData) };
    }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Ptr<ND::_3D, T>& ptr) { return build(ptr.ptr()); }
};

// Packed pixels into plane z of a tensor.
template <typename T>
struct TensorWrite {
private:
    using SelfType = TensorWrite<T>;

public:
    FK_STATIC_STRUCT(TensorWrite, SelfType)
    using ParamsType = RawPtr<ND::_3D, T>;
    using InputType = T;
    using WriteDataType = T;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = true;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) { *PtrAccessor<ND::_3D>::point(thread, params) = input; }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Ptr<ND::_3D, T>& ptr) { return build(ptr.ptr()); }
};

// Channels of the pixel into separate planes of image z: N x C x H x W (memory_operations.h:195-226).
template <typename T>
struct TensorSplit {
private:
    using SelfType = TensorSplit<T>;

public:
    FK_STATIC_STRUCT(TensorSplit, SelfType)
    static_assert(cn<T> >= 2, "Wrong type for split tensor write. It must be one of <type>2, <type>3 or <type>4.");
    using ParamsType = RawPtr<ND::_3D, VBase<T>>;
    using InputType = T;
    using WriteDataType = VBase<T>;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        const int planePixels = static_cast<int>(params.dims.width * params.dims.height);
        WriteDataType* const work_plane = PtrAccessor<ND::_3D>::point(thread, params);
        *work_plane = input.x;
        *(work_plane + planePixels) = input.y;
        if constexpr (cn<T> >= 3) *(work_plane + planePixels * 2) = input.z;
        if constexpr (cn<T> == 4) *(work_plane + planePixels * 3) = input.w;
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HD_STATIC uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Ptr<ND::_3D, VBase<T>>& ptr) { return build(ptr.ptr()); }
};

// A read that yields the same value for every element of a given extent (algorithms/basic_ops/set.h:23-77).
template <typename T>
struct ReadSetParams {
    T value;
    ActiveThreads size;
};
template <typename T>
struct ReadSet {
private:
    using SelfType = ReadSet<T>;

public:
    FK_STATIC_STRUCT(ReadSet, SelfType)
    using ParamsType = ReadSetParams<T>;
    using ReadDataType = T;
    using OutputType = T;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC OutputType exec(const Point&, const ParamsType& params) { return params.value; }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.size.x; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return opData.params.size.y; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType& opData) { return opData.params.size.z; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) { return opData.params.size; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const T& value, const ActiveThreads& size) { return InstantiableType{ { { value, size } } }; }
};

} // namespace fk
#endif

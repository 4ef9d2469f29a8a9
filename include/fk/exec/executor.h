// Host dispatch: TransformDPP / DivergentBatchTransformDPP tags, Executor and job construction.
//
// API counterpart of the reference's core/execution_model/data_parallel_patterns.h:65-67,194-235,301-353 (the DPP
// types named in executeOperations<...>) and core/execution_model/executors.h:44-128,245-293 (Executor, the overload
// set of executeOperations, grid computation and launch).  A chain is analysed at compile time into one of the
// kernel families of fk/exec/kernels.h; the launch itself goes through the C runtime ABI (fkrt_launch).
#ifndef FK_EXEC_EXECUTOR_H
#define FK_EXEC_EXECUTOR_H

#include <cstdlib>
#include <cstring>
#include <tuple>
#include <memory>

#include "fk/core/stream.h"
#include "fk/exec/kernels.h"

namespace fk {

template <ParArch PA = defaultParArch, TF TFEN = TF::DISABLED>
struct TransformDPP {
    static constexpr ParArch PAR_ARCH = PA;
    static_assert(PA == ParArch::GPU_AMD || PA == ParArch::CPU, "Only ParArch::GPU_AMD and ParArch::CPU are implemented by this library.");
};

// One fused chain per group of thread planes, all in one launch.
template <ParArch PA = defaultParArch>
struct DivergentBatchTransformDPP {
    static constexpr ParArch PAR_ARCH = PA;
    static_assert(PA == ParArch::GPU_AMD,
                  "Only ParArch::GPU_AMD is implemented by this library; there is no host fallback executor.");
};

// A (sender..., receiver) chain kept as a value, for divergent launches (core/data/tuple.h:199-215).
template <typename Sender, typename Receiver>
struct InstantiableOperationSequence {
    Sender sender;
    Receiver receiver;
};
template <typename First, typename... Rest>
inline constexpr auto buildOperationSequence(const First& first, const Rest&... rest);

namespace exec {

inline unsigned ceil_div(unsigned a, unsigned b) { return (a + b - 1u) / b; }
// Outputs of this size and more are written with streaming stores.  One XCD's L2 is 4 MiB and the L2s do not share:
// what one XCD wrote, a later kernel's blocks on the other seven read from memory (or the Infinity Cache) anyway, so
// keeping a large output in the writer's L2 buys nothing and costs the lines of the source that it displaces
// (measured from 4 MiB up: 50 crops -> 224x224 planar, 30 MB, 13.3 -> 11.9 us; NV12 4K -> RGB, 25 MB, 10.4 -> 8.9 us).
#ifndef FK_STREAM_STORE_MIN_MIB
#define FK_STREAM_STORE_MIN_MIB 4
#endif
constexpr size_t STREAM_STORE_MIN_BYTES = static_cast<size_t>(FK_STREAM_STORE_MIN_MIB) << 20;
inline bool aligned_to(const void* p, size_t a) { return reinterpret_cast<size_t>(p) % a == 0; }
// FK_RESIZE_WAVE_ROWS=4|8|16 fixes the resize kernel's tile height (64 x 4 * rows) instead of the choice made per launch:
// for measurements.
inline unsigned resize_wave_rows_override() {
    static const unsigned rows = [] {
        const char* env = std::getenv("FK_RESIZE_WAVE_ROWS");
        return env != nullptr ? static_cast<unsigned>(std::strtoul(env, nullptr, 10)) : 0u;
    }();
    return rows;
}

// FK_RESIZE_PACKED_DWORDS=n sets the capacity of the resize kernel's tile of packed pixels (0: no such tiles): for
// measurements.
inline unsigned resize_packed_capacity() {
    static const unsigned dwords = [] {
        const char* env = std::getenv("FK_RESIZE_PACKED_DWORDS");
        return env != nullptr ? static_cast<unsigned>(std::strtoul(env, nullptr, 10)) : static_cast<unsigned>(RESIZE_PACKED_DWORDS);
    }();
    return dwords;
}

// Switches for measurements, read once: FK_RESIZE_NO_QUAD_FILL (tiles of float taps filled one pixel per thread),
// FK_RESIZE_NO_PAIRS (tiles in launch order), FK_RESIZE_LDS_DWORDS=n (a launch that uses LDS asks for at least n dwords per block).
struct ResizeSwitches {
    bool no_quad_fill, no_pairs;
    unsigned lds_dwords;
};
inline const ResizeSwitches& resize_switches() {
    static const ResizeSwitches switches = [] {
        const char* lds = std::getenv("FK_RESIZE_LDS_DWORDS");
        return ResizeSwitches{ std::getenv("FK_RESIZE_NO_QUAD_FILL") != nullptr, std::getenv("FK_RESIZE_NO_PAIRS") != nullptr,
                               lds != nullptr ? static_cast<unsigned>(std::strtoul(lds, nullptr, 10)) : 0u };
    }();
    return switches;
}

// ---- job construction ----------------------------------------------------------------------------------------
namespace detail {
// operations that resample through a matrix (Warping): their taps wander over the source rows
template <typename Op, typename = void>
struct IsWarp : std::false_type {};
template <typename Op>
struct IsWarp<Op, std::void_t<decltype(Op::WARP)>> : std::true_type {};
// The planes of a sender: `capacity` is the size of its plane table (known at compile time), `count` the planes of the
// thread grid (a batch filled in at run time holds fewer than its capacity), `used` the planes that run their program
// (the others receive the default value of a CONDITIONAL_WITH_DEFAULT batch).
template <typename Sender, typename = void>
struct PlaneIOpOf {
    using type = Sender;
    static constexpr size_t capacity = 1;
    static constexpr bool conditional = false;
    static const type& get(const Sender& s, size_t) { return s; }
    static size_t count(const Sender&) { return 1; }
    static size_t used(const Sender&) { return 1; }
};
template <typename Sender>
struct PlaneIOpOf<Sender, std::enable_if_t<isBatchOperation<typename Sender::Operation>>> {
    using Batch = typename Sender::Operation;
    using type = Instantiable<typename Batch::Operation>;
    static constexpr size_t capacity = Batch::BATCH;
    static constexpr bool conditional = Batch::PP == PlanePolicy::CONDITIONAL_WITH_DEFAULT;
    static type get(const Sender& s, size_t i) { return toIOp<typename Batch::Operation>(s.params.opData[i]); }
    static size_t count(const Sender& s) {
        const size_t z = s.params.activeThreads.z;
        return z < capacity ? z : capacity;
    }
    static size_t used(const Sender& s) {
        if constexpr (conditional) {
            const size_t n = count(s), u = s.params.usedPlanes < 0 ? 0 : static_cast<size_t>(s.params.usedPlanes);
            return u < n ? u : n;
        } else {
            return count(s);
        }
    }
};
template <typename PlaneIOp, typename = void>
struct IsResizeProgram : std::false_type {};
template <typename PlaneIOp>
struct IsResizeProgram<PlaneIOp, std::enable_if_t<ProgramOf<PlaneIOp>::supported>>
    : std::bool_constant<ProgramOf<PlaneIOp>::View::IS_RESIZE> {};
template <typename PlaneIOp, typename Receiver, typename = void>
struct Matches : std::false_type {};
template <typename PlaneIOp, typename Receiver>
struct Matches<PlaneIOp, Receiver, std::enable_if_t<ProgramOf<PlaneIOp>::supported && OutOf<Receiver>::supported>>
    : std::is_same<typename ProgramOf<PlaneIOp>::OutputType, typename OutOf<Receiver>::type::Pixel> {};
} // namespace detail

template <typename Sender, typename Receiver>
struct JobOf {
    using Planes = detail::PlaneIOpOf<Sender>;
    using PlaneIOp = typename Planes::type;
    static constexpr size_t N = Planes::capacity;
#ifdef FK_INTERPOLATE_Y1_FROM_X
    // the reference's host-branch interpolation takes the tap row from the x coordinate: rows and columns are no longer
    // separable, so resize chains run on the generic per-element kernel in such a build
    static constexpr bool separable = !detail::IsResizeProgram<PlaneIOp>::value;
#else
    static constexpr bool separable = true;
#endif
    static constexpr bool viewable = separable && detail::Matches<PlaneIOp, Receiver>::value;

    // what the planes from `used` on receive (a CONDITIONAL_WITH_DEFAULT batch), with the extent of the batch's grid
    template <typename Defaults>
    static Defaults defaults_of(const Sender& sender) {
        if constexpr (Defaults::ENABLED) {
            const ActiveThreads grid = sender.getActiveThreads();
            return Defaults{ static_cast<unsigned>(Planes::used(sender)), static_cast<int>(grid.x), static_cast<int>(grid.y), sender.params.default_value };
        } else {
            return Defaults{};
        }
    }

    static auto make(const Sender& sender, const Receiver& receiver) {
        if constexpr (viewable) {
            using Prog = typename ProgramOf<PlaneIOp>::type;
            using Out = typename OutOf<Receiver>::type;
            using View = decltype(Prog::view);
            using Defaults = std::conditional_t<Planes::conditional, DefaultPlanes<typename Out::Pixel>, NoDefaultPlanes>;
            const Out out = OutOf<Receiver>::make(receiver);
            const size_t count = Planes::count(sender), used = Planes::used(sender);
            const Defaults defaults = defaults_of<Defaults>(sender);
            int max_w = 0, max_h = 0;
            if constexpr (Defaults::ENABLED) {
                if (used < count) {
                    max_w = defaults.w;
                    max_h = defaults.h;
                }
            }
            if constexpr (View::IS_RESIZE) {
                ResizeJob<Prog, N, Out, Defaults> job{};
                job.defaults = defaults;
                for (size_t i = 0; i < used; ++i) {
                    job.plane[i] = ProgramOf<PlaneIOp>::make(Planes::get(sender, i));
                    max_w = job.plane[i].view.w > max_w ? job.plane[i].view.w : max_w;
                    max_h = job.plane[i].view.h > max_h ? job.plane[i].view.h : max_h;
                }
                job.out = out;
                job.grid_x = ceil_div(static_cast<unsigned>(max_w), RESIZE_TILE_W);
                // streaming stores for large outputs whose rows, planes and channel planes start at whole dwords
                bool dwords = aligned_to(out.data, 4) && out.pitch % 4 == 0 && out.z_stride % 4 == 0;
                // (the kernel addresses a wave's rows, and their channel planes, with 32-bit offsets from its first row)
                if constexpr (Out::IS_SPLIT) dwords = dwords && out.chan_stride % 4 == 0 && out.chan_stride * 4 + static_cast<size_t>(out.pitch) * 64 < (1u << 30);
                dwords = dwords && static_cast<size_t>(out.pitch) * 64 < (1u << 30);
                const bool large = static_cast<size_t>(max_w) * max_h * count * sizeof(typename Out::Pixel) >= STREAM_STORE_MIN_BYTES;
                job.flags = dwords && large ? FLAG_STREAM_STORES : 0u;
                // tile height, grid rows and LDS layout; sets FLAG_SOURCE_TILE when some plane's tiles are worth staging
                job.grid_y = job.plan(used, max_h, resize_wave_rows_override(), resize_packed_capacity());
                // x-neighbouring tiles in pairs on one XCD (FK_RESIZE_NO_PAIRS switches it off: for measurements)
                const ResizeSwitches& switches = resize_switches();
                if (switches.no_quad_fill) job.flags &= ~FLAG_QUAD_FILL;
                if (job.tile_dwords != 0u && switches.lds_dwords > job.tile_dwords) job.tile_dwords = switches.lds_dwords;
                if (!switches.no_pairs) {
                    const unsigned gx = job.grid_x;
                    if (gx > 9u) job.flags |= FLAG_PAIR_COLUMNS;
                    else if (gx > 1u && (gx & (gx - 1u)) == 0u && gx * job.grid_y > 9u) job.flags |= FLAG_PAIR_TILES;
                }
                return job;
            } else {
                using Job = PointwiseJob<Prog, N, Out, Defaults>;
                using Src = typename Job::Src;
                using Access = typename Job::Access;
                Job job{};
                job.defaults = defaults;
                job.out = out;
                constexpr size_t out_elem = Out::IS_SPLIT ? sizeof(VBase<typename Out::Pixel>) : sizeof(typename Out::Pixel);
                constexpr size_t out_chunk = dev::chunk_bytes(Job::K * static_cast<int>(out_elem));
                for (size_t i = 0; i < used; ++i) {
                    job.plane[i].prog = ProgramOf<PlaneIOp>::make(Planes::get(sender, i));
                    const auto& v = job.plane[i].prog.view;
                    max_w = v.w > max_w ? v.w : max_w;
                    max_h = v.h > max_h ? v.h : max_h;
                }
                // Windows of different sizes: every plane produces the extent of the batch's thread grid, as in the
                // reference (batch_operations.h:153-160: max width x max height for every plane; a batch that is launched in
                // parts carries the extent of the whole batch in its grid); beside its own window a plane then holds the
                // parent image's pixels there (zero where the parent ends).  Decided before anything that depends on a
                // plane's extent: the alignment tests below must see the rows the plane will really produce.
                bool ragged = false;
                if constexpr (std::is_same_v<View, PlainView<Src>>) {
                    if constexpr (isBatchOperation<typename Sender::Operation>) {
                        const ActiveThreads grid = sender.getActiveThreads();
                        max_w = static_cast<int>(grid.x) > max_w ? static_cast<int>(grid.x) : max_w;
                        max_h = static_cast<int>(grid.y) > max_h ? static_cast<int>(grid.y) : max_h;
                    }
                    for (size_t i = 0; i < used; ++i) ragged = ragged || job.plane[i].prog.view.w != max_w || job.plane[i].prog.view.h != max_h;
                    if (ragged) {
                        for (size_t i = 0; i < used; ++i) {
                            job.plane[i].prog.view.w = max_w;
                            job.plane[i].prog.view.h = max_h;
                        }
                    }
                }
                bool flatten = Access::FLATTENS && used == count && !ragged;
                if constexpr (Access::FLATTENS) {
                    for (size_t i = 0; i < used; ++i) {
                        const auto& v = job.plane[i].prog.view;
                        flatten = flatten && v.ox == 0 && v.oy == 0 && v.w == v.img_w && v.h > 1 &&
                                  v.pitch == static_cast<uint>(v.w) * sizeof(Src) && out.pitch == static_cast<uint>(v.w) * out_elem &&
                                  static_cast<size_t>(v.w) * v.h < (1u << 30);
                    }
                }
                if (flatten) max_w = max_h = 0; // found again below, from the flattened planes
                for (size_t i = 0; i < used; ++i) {
                    auto& v = job.plane[i].prog.view;
                    if constexpr (Access::FLATTENS) {
                        if (flatten) {
                            // rows are contiguous on both sides, in every plane: treat each image as one long row, so no
                            // block is cut short at a row end
                            v.w = v.img_w = v.w * v.h;
                            v.h = v.img_h = 1;
                        }
                    }
                    bool vec = Access::template aligned<Job::K>(v);
                    const char* const ofirst = reinterpret_cast<const char*>(out.data) + i * out.z_stride;
                    vec = vec && aligned_to(ofirst, out_chunk) && (v.h == 1 || out.pitch % out_chunk == 0);
                    if constexpr (Out::IS_SPLIT) vec = vec && out.chan_stride % out_chunk == 0;
                    // outputs larger than the caches are written with streaming stores
                    const bool stream = static_cast<size_t>(v.w) * v.h * count * sizeof(typename Out::Pixel) >= STREAM_STORE_MIN_BYTES;
                    job.plane[i].flags = (vec ? FLAG_VECTOR_IO : 0u) | (vec && stream ? FLAG_STREAM_STORES : 0u) | (ragged ? FLAG_WHOLE_BOX : 0u);
                    max_w = v.w > max_w ? v.w : max_w;
                    max_h = v.h > max_h ? v.h : max_h;
                }
                // thread columns per block: enough to span the widest row, at most the whole block
                const unsigned groups = ceil_div(static_cast<unsigned>(max_w), Job::K);
                unsigned shift = 0;
                while ((1u << shift) < groups && shift < 8u) ++shift;
                if (shift < 4u) shift = 4u; // keep a wave's accesses within a few rows
                job.tx_shift = shift;
                job.grid_x = ceil_div(groups, 1u << shift);
                job.grid_y = ceil_div(static_cast<unsigned>(max_h), BLOCK_THREADS >> shift);
                job.pair_limit = 0u;
                if constexpr (N == 1 && Access::PAIRS_ROWS) {
                    // one row per block row: rows that share a chroma row are handed to the same XCD
                    if (shift == 8u) {
                        const unsigned total = job.grid_x * job.grid_y, unit = 16u * job.grid_x; // whole turns of all XCDs, whole row pairs
                        job.pair_limit = total / unit * unit;
                    }
                }
                return job;
            }
        } else {
            GenericJob<Sender, Receiver> job{};
            job.sender = sender;
            job.receiver = receiver;
            job.active = sender.getActiveThreads();
            job.grid_x = job.plan(job.active);
            job.grid_y = ceil_div(job.active.y, 4u);
            // Bands per XCD for warps, once every XCD has a few hundred tiles of its own (measured on 3840x2160 uchar3: the
            // perspective warp to 1920x1080 10.1 -> 9.2 us and 33 -> 23.5 MB fetched, the 5 degree rotation 56 -> 24.3 MB
            // fetched at the same 26.5 us; a reflected border 10.2 -> 10.5 us, so other chains keep the plain order).
            job.xcd_bands = detail::IsWarp<typename Sender::Operation>::value && static_cast<size_t>(job.grid_x) * job.grid_y * job.active.z >= 4096u ? 1u : 0u;
            job.stream_rows = 0u;
            if constexpr (decltype(job)::STREAMS_ROWS) {
                const auto out = OutOf<Receiver>::make(receiver);
                const size_t bytes = static_cast<size_t>(job.active.x) * job.active.y * job.active.z * sizeof(typename decltype(job)::Value);
                const size_t piece = dev::chunk_bytes(static_cast<int>(sizeof(typename decltype(job)::Value)));
                job.stream_rows = (bytes >= STREAM_STORE_MIN_BYTES && aligned_to(out.data, piece) && out.pitch % piece == 0u && out.z_stride % piece == 0u) ? 1u : 0u;
                job.out_data = reinterpret_cast<char*>(out.data);
                job.out_pitch = out.pitch;
                job.out_z_stride = out.z_stride;
            }
            job.packs_rows = 0u;
            if constexpr (decltype(job)::PACKS_ROWS) {
                const auto out = OutOf<Receiver>::make(receiver);
                job.packs_rows = (aligned_to(out.data, 4) && out.pitch % 4u == 0u && out.z_stride % 4u == 0u) ? 1u : 0u;
                const size_t bytes = static_cast<size_t>(job.active.x) * job.active.y * job.active.z * sizeof(typename decltype(job)::Value);
                job.stream_rows = (job.packs_rows != 0u && bytes >= STREAM_STORE_MIN_BYTES) ? 1u : 0u;
                job.out_data = reinterpret_cast<char*>(out.data);
                job.out_pitch = out.pitch;
                job.out_z_stride = out.z_stride;
            }
            return job;
        }
    }
    static unsigned planes(const Sender& sender) {
        if constexpr (viewable) return static_cast<unsigned>(Planes::count(sender));
        else return sender.getActiveThreads().z;
    }
};

// Launch `kernel(args)` by value, or through a staged copy when `Args` exceeds the kernel-argument limit.
template <typename Args>
inline void launch_args(const void* by_value, const void* indirect, const Args& args, unsigned gx, unsigned gy, unsigned gz,
                        size_t lds_bytes, fkrt_stream stream) {
    if (gx == 0 || gy == 0 || gz == 0) return; // nothing to do
    if (sizeof(Args) <= fkrt_max_kernarg_bytes()) {
        void* argv[] = { const_cast<Args*>(&args) };
        gpuErrchk(fkrt_launch(by_value, gx, gy, gz, BLOCK_THREADS, 1, 1, argv, lds_bytes, stream));
    } else {
        void* device_args = nullptr;
        gpuErrchk(fkrt_params_upload(&device_args, &args, sizeof(Args), stream));
        void* argv[] = { &device_args };
        const int status = fkrt_launch(indirect, gx, gy, gz, BLOCK_THREADS, 1, 1, argv, lds_bytes, stream);
        gpuErrchk(fkrt_params_release(device_args, stream));
        gpuErrchk(status);
    }
}

template <typename Job>
inline void launch_job(const Job& job, unsigned planes, fkrt_stream stream) {
    launch_args(reinterpret_cast<const void*>(&transform_kernel<Job>), reinterpret_cast<const void*>(&transform_kernel_indirect<Job>),
                job, job.grid_x, job.grid_y, planes, job.lds_bytes(), stream);
}

// The same launch with the job read from `device_block`, device memory of `block_bytes` bytes that the caller brings (and
// that no other launch in flight uses): one small kernel copies the job there from its kernel arguments, the chain's
// kernel then reads it from there.  Nothing is allocated.  False when the job does not fit the block or the kernel
// arguments.
template <typename Job>
inline bool launch_job_from(void* device_block, size_t block_bytes, const Job& job, unsigned planes, fkrt_stream stream) {
    if (sizeof(Job) > block_bytes || sizeof(Job) > fkrt_max_kernarg_bytes()) return false;
    if (job.grid_x == 0 || job.grid_y == 0 || planes == 0) return true; // nothing to do
    Job* at = static_cast<Job*>(device_block);
    void* store_argv[] = { const_cast<Job*>(&job), &at };
    gpuErrchk(fkrt_launch(reinterpret_cast<const void*>(&store_job_kernel<Job>), 1, 1, 1, BLOCK_THREADS, 1, 1, store_argv, 0, stream));
    void* argv[] = { &at };
    gpuErrchk(fkrt_launch(reinterpret_cast<const void*>(&transform_kernel_indirect<Job>), job.grid_x, job.grid_y, planes, BLOCK_THREADS, 1, 1, argv,
                          job.lds_bytes(), stream));
    return true;
}

// (read, compute..., write) as (sender, receiver)
template <typename Receiver>
inline constexpr const Receiver& last_of(const Receiver& r) { return r; }
template <typename First, typename... Rest>
inline constexpr const auto& last_of(const First&, const Rest&... rest) { return last_of(rest...); }

template <size_t... Idx, typename Tuple>
inline constexpr auto fuse_front(std::index_sequence<Idx...>, const Tuple& t) {
    if constexpr (sizeof...(Idx) == 1) {
        return std::get<0>(t);
    } else {
        return Fuser::fuse(std::get<Idx>(t)...);
    }
}
template <typename... IOps>
inline constexpr auto sender_of(const IOps&... iOps) {
    static_assert(sizeof...(IOps) >= 2, "A chain needs at least a read and a write operation.");
    return fuse_front(std::make_index_sequence<sizeof...(IOps) - 1>{}, std::forward_as_tuple(iOps...));
}

} // namespace exec

template <typename First, typename... Rest>
inline constexpr auto buildOperationSequence(const First& first, const Rest&... rest) {
    const auto sender = exec::sender_of(first, rest...);
    const auto& receiver = exec::last_of(rest...);
    static_assert(isAnyReadType<std::decay_t<decltype(sender)>>, "The first operation of a chain must be a read.");
    static_assert(isWriteType<std::decay_t<decltype(receiver)>>, "The last operation of a chain must be a write.");
    return InstantiableOperationSequence<std::decay_t<decltype(sender)>, std::decay_t<decltype(receiver)>>{ sender, receiver };
}

template <typename DPP>
struct Executor;

template <TF TFEN>
struct Executor<TransformDPP<ParArch::GPU_AMD, TFEN>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::GPU_AMD; }

    // executeOperations(stream, read, [compute...], write): one kernel for the whole chain
    template <typename... IOps>
    static inline void executeOperations(Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        const auto seq = buildOperationSequence(iOps...);
        using Sender = std::decay_t<decltype(seq.sender)>;
        using Receiver = std::decay_t<decltype(seq.receiver)>;
        using Plan = exec::JobOf<Sender, Receiver>;
        const auto job = Plan::make(seq.sender, seq.receiver);
        exec::launch_job(job, Plan::planes(seq.sender), stream.getHIPStream());
    }
    // The same with the chain's job kept in device memory that the caller brings instead of in the kernel arguments
    // (this library's extension, for callers that must not allocate and hold such a block anyway; see
    // exec::launch_job_from).  False when the job does not fit.
    template <typename... IOps>
    static inline bool executeOperationsFrom(void* device_block, size_t block_bytes, Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        const auto seq = buildOperationSequence(iOps...);
        using Plan = exec::JobOf<std::decay_t<decltype(seq.sender)>, std::decay_t<decltype(seq.receiver)>>;
        const auto job = Plan::make(seq.sender, seq.receiver);
        return exec::launch_job_from(device_block, block_bytes, job, Plan::planes(seq.sender), stream.getHIPStream());
    }
    // Convenience forms over buffers (executors.h:52-93).
    template <ND D, typename I, typename... IOps>
    static inline void executeOperations(const Ptr<D, I>& input, Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<D, I>::build(input), iOps...);
    }
    template <ND D, typename I, typename O, typename... IOps>
    static inline void executeOperations(const Ptr<D, I>& input, const Ptr<D, O>& output, Stream_<ParArch::GPU_AMD>& stream,
                                         const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<D, I>::build(input), iOps..., PerThreadWrite<D, O>::build(output));
    }
    template <typename I, size_t BATCH, typename... IOps>
    static inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                                         Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(activeBatch, defaultValue, input), iOps...);
    }
    template <typename I, size_t BATCH, typename... IOps>
    static inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, Stream_<ParArch::GPU_AMD>& stream,
                                         const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(input), iOps...);
    }
    template <typename I, typename O, size_t BATCH, typename... IOps>
    static inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const int& activeBatch, const I& defaultValue,
                                         const Tensor<O>& output, Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(activeBatch, defaultValue, input), iOps...,
                          PerThreadWrite<ND::_3D, O>::build(output));
    }
    template <typename I, typename O, size_t BATCH, typename... IOps>
    static inline void executeOperations(const std::array<Ptr2D<I>, BATCH>& input, const Tensor<O>& output,
                                         Stream_<ParArch::GPU_AMD>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<ND::_2D, I>::build(input), iOps..., PerThreadWrite<ND::_3D, O>::build(output));
    }
};

// The same chains on the host, for user code that asks for them by name (executors.h:147-173): one element after the other
// in the reference's order, planes outermost then rows then columns (data_parallel_patterns.h:285-298), each through the
// operations' own exec functions, which are the ones the generic kernel calls per element.  Memory must be host memory
// (MemType::Host, HostPinned, or the pinned side of a buffer).  Nothing here is used by the GPU path, and the GPU path
// never falls back to it: the executor is chosen by the ParArch that the caller names.
template <TF TFEN>
struct Executor<TransformDPP<ParArch::CPU, TFEN>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::CPU; }

    template <typename... IOps>
    static inline void executeOperations(Stream_<ParArch::CPU>&, const IOps&... iOps) {
        const auto seq = buildOperationSequence(iOps...);
        using Sender = std::decay_t<decltype(seq.sender)>;
        using Receiver = std::decay_t<decltype(seq.receiver)>;
        const ActiveThreads grid = seq.sender.getActiveThreads();
        for (int z = 0; z < static_cast<int>(grid.z); ++z) {
            for (int y = 0; y < static_cast<int>(grid.y); ++y) {
                for (int x = 0; x < static_cast<int>(grid.x); ++x) {
                    const Point thread(x, y, z);
                    Receiver::Operation::exec(thread, Sender::Operation::exec(thread, seq.sender), seq.receiver);
                }
            }
        }
    }
    // Convenience forms over buffers (executors.h:52-93); the buffers' host side is what is read and written.
    template <ND D, typename I, typename... IOps>
    static inline void executeOperations(const Ptr<D, I>& input, Stream_<ParArch::CPU>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<D, I>::build(host_side(input)), iOps...);
    }
    template <ND D, typename I, typename O, typename... IOps>
    static inline void executeOperations(const Ptr<D, I>& input, const Ptr<D, O>& output, Stream_<ParArch::CPU>& stream, const IOps&... iOps) {
        executeOperations(stream, PerThreadRead<D, I>::build(host_side(input)), iOps..., PerThreadWrite<D, O>::build(host_side(output)));
    }

private:
    template <ND D, typename T>
    static RawPtr<D, T> host_side(const Ptr<D, T>& p) {
        return p.getMemType() == MemType::DeviceAndPinned ? p.ptrPinned() : p.ptr();
    }
};

template <>
struct Executor<DivergentBatchTransformDPP<ParArch::GPU_AMD>> {
    FK_STATIC_STRUCT(Executor, Executor)
    static constexpr ParArch parArch() { return ParArch::GPU_AMD; }

    // executeOperations(stream, sequence0, sequence1, ...): every sequence is a chain built with
    // buildOperationSequence; all of them run in one launch, each over its own planes.
    template <typename... Senders, typename... Receivers>
    static inline void executeOperations(Stream_<ParArch::GPU_AMD>& stream,
                                         const InstantiableOperationSequence<Senders, Receivers>&... sequences) {
        static_assert(sizeof...(Senders) >= 1, "A divergent launch needs at least one sequence.");
        using Pack = exec::JobPack<std::decay_t<decltype(exec::JobOf<Senders, Receivers>::make(sequences.sender, sequences.receiver))>...>;
        // the pack holds every job by value; build it on the heap, it can be several KiB
        auto pack = std::make_unique<Pack>();
        unsigned total = 0;
        size_t lds = 0;
        fill(*pack, total, lds, sequences...);
        exec::launch_args(reinterpret_cast<const void*>(&exec::divergent_kernel<Pack>),
                          reinterpret_cast<const void*>(&exec::divergent_kernel_indirect<Pack>), *pack, total, 1, 1, lds,
                          stream.getHIPStream());
    }

private:
    template <typename Pack>
    static inline void fill(Pack&, unsigned&, size_t&) {}
    template <typename Pack, typename Seq, typename... Rest>
    static inline void fill(Pack& pack, unsigned& total, size_t& lds, const Seq& seq, const Rest&... rest) {
        using Plan = exec::JobOf<std::decay_t<decltype(seq.sender)>, std::decay_t<decltype(seq.receiver)>>;
        pack.job = Plan::make(seq.sender, seq.receiver);
        pack.blocks = pack.job.grid_x * pack.job.grid_y * Plan::planes(seq.sender);
        total += pack.blocks;
        lds = lds > pack.job.lds_bytes() ? lds : pack.job.lds_bytes();
        fill(pack.rest, total, lds, rest...);
    }
};

} // namespace fk
#endif

// reference_sweeps.cpp — the four benchmark sweeps of the Fused Kernel Library, written as user code against this
// library's operator API, so that results can be set beside the reference's own figures:
//   horizontal fusion   benchmarks/fusion/benchmark_horizontal_fusion.h   iterated vs fused batch of 60x120 crops, batch 1..46
//   instructions per op benchmarks/numinstructions/benchmark_numinstructions_x_operation.h   50 additions as 50/n launches of n vs 1 launch
//   vertical fusion     benchmarks/latencyhiding/benchmark_latency_hiding.h   one launch of StaticLoop<StaticLoop<Mul,20>,n/20>
//   thread fusion       benchmarks/fusion/benchmark_thread_fusion.h   TF::DISABLED vs TF::ENABLED copies and casts, 1024..5120 (+1) pixels per side
// Same chains, element counts, crop sizes and sweep values as there; each variant is timed ITERS times with an event
// pair around it (launch overhead of iterated variants included, as in the reference).  Every sweep point checks its
// outputs, all of their elements, against the chain evaluated on the host.  Prints one JSON object per sweep point.
#include <fused_kernel/fused_kernel.h>
#include <fused_kernel/algorithms/basic_ops/static_loop.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>
#include <fused_kernel/core/data/ptr_utils.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

using namespace fk;

static int ITERS = 100; // as in the reference (benchmarks/fkBenchmarksCommon.h:31)
static bool all_passed = true;

struct Timer {
    void *a = nullptr, *b = nullptr;
    Timer() {
        gpuErrchk(fkrt_event_create(&a));
        gpuErrchk(fkrt_event_create(&b));
    }
    ~Timer() {
        (void)fkrt_event_destroy(a);
        (void)fkrt_event_destroy(b);
    }
    template <typename F>
    float time_ms(Stream& stream, F&& body) {
        gpuErrchk(fkrt_event_record(a, stream.getHIPStream()));
        body();
        gpuErrchk(fkrt_event_record(b, stream.getHIPStream()));
        gpuErrchk(fkrt_event_sync(b));
        float ms = 0.f;
        gpuErrchk(fkrt_event_elapsed_ms(&ms, a, b));
        return ms;
    }
};

struct Stats {
    double mean, stddev, min;
};
static Stats stats_of(const std::vector<float>& v) {
    double s = 0, mn = v[0];
    for (float x : v) {
        s += x;
        mn = x < mn ? x : mn;
    }
    const double mean = s / v.size();
    double var = 0;
    for (float x : v) var += (x - mean) * (x - mean);
    return { mean, std::sqrt(var / v.size()), mn };
}

template <typename First, typename Second>
static void two_variants(const char* sweep, const char* dimension, size_t value, const char* first_label, const char* second_label, Stream& stream,
                         First&& first, Second&& second, bool passed, const std::string& extra = "") {
    Timer timer;
    first();
    second(); // warm-up
    stream.sync();
    std::vector<float> t1(ITERS), t2(ITERS);
    for (int i = 0; i < ITERS; ++i) {
        t1[i] = timer.time_ms(stream, first);
        t2[i] = timer.time_ms(stream, second);
    }
    const Stats a = stats_of(t1), b = stats_of(t2);
    double speedup = 0;
    for (int i = 0; i < ITERS; ++i) speedup += t1[i] / t2[i];
    std::printf("{\"sweep\": \"%s\", \"%s\": %zu, \"%s_ms\": %.6f, \"%s_ms\": %.6f, \"%s_std\": %.6f, \"%s_std\": %.6f, \"%s_min_ms\": %.6f, "
                "\"%s_min_ms\": %.6f, \"mean_speedup\": %.3f, \"passed\": %s%s}\n",
                sweep, dimension, value, first_label, a.mean, second_label, b.mean, first_label, a.stddev, second_label, b.stddev, first_label, a.min,
                second_label, b.min, speedup / ITERS, passed ? "true" : "false", extra.c_str());
    std::fflush(stdout);
    all_passed = all_passed && passed;
}

template <size_t FIRST, size_t INCREMENT, size_t... Is>
constexpr std::array<size_t, sizeof...(Is)> sweep_values(std::index_sequence<Is...>) {
    return { (FIRST + INCREMENT * Is)... };
}

// ---- horizontal fusion -----------------------------------------------------------------------------------------------
template <size_t BATCH>
static void horizontal_fusion(Stream& stream) {
    using I = uchar;
    using O = float;
    const Size cropSize(60, 120);
    Ptr2D<I> d_input(3840, 2160);
    setTo(static_cast<I>(10u), d_input, stream);
    std::array<Ptr2D<O>, BATCH> d_outputs;
    Tensor<O> d_tensor(cropSize.width, cropSize.height, BATCH);
    std::array<Ptr2D<I>, BATCH> crops;
    for (size_t i = 0; i < BATCH; ++i) {
        crops[i] = d_input.crop(Point(static_cast<int>(i), static_cast<int>(i)),
                                PtrDims<ND::_2D>{ static_cast<uint>(cropSize.width), static_cast<uint>(cropSize.height), d_input.dims().pitch });
        d_outputs[i].Alloc(cropSize);
    }
    const auto read_array = PerThreadRead<ND::_2D, I>::build_batch(crops);
    const auto read = PerThreadRead<ND::_2D, I>::build(crops);
    const auto saturate = SaturateCast<I, O>::build();
    const auto mul = Mul<O>::build(1.0f);
    const auto sub = Sub<O>::build(1.f);
    const auto div = Div<O>::build(3.2f);
    const auto write_array = PerThreadWrite<ND::_2D, O>::build_batch(d_outputs);
    const auto write = TensorWrite<O>::build(d_tensor);
    const auto iterated = [&]() {
        for (size_t i = 0; i < BATCH; ++i) executeOperations<TransformDPP<>>(stream, read_array[i], saturate, mul, sub, div, write_array[i]);
    };
    const auto fused = [&]() { executeOperations<TransformDPP<>>(stream, read, saturate, mul, sub, div, write); };
    iterated();
    fused();
    d_tensor.download(stream);
    for (size_t i = 0; i < BATCH; ++i) d_outputs[i].download(stream);
    stream.sync();
    bool passed = true;
    for (size_t i = 0; i < BATCH; ++i) {
        Ptr2D<O> plane = d_tensor.getPlane(static_cast<uint>(i));
        for (uint y = 0; y < 120; ++y)
            for (uint x = 0; x < 60; ++x) passed = passed && plane.at(x, y) == d_outputs[i].at(x, y) && plane.at(x, y) == (10.f * 1.0f - 1.f) / 3.2f;
    }
    two_variants("horizontal_fusion", "batch", BATCH, "iterated", "fused", stream, iterated, fused, passed);
}
template <size_t... Is>
static void horizontal_fusion_sweep(Stream& stream, std::index_sequence<Is...>) {
    constexpr auto values = sweep_values<1, 5>(std::make_index_sequence<10>{});
    (horizontal_fusion<values[Is]>(stream), ...);
}

// ---- instructions per operation --------------------------------------------------------------------------------------
constexpr int NUM_ELEMENTS = 3840 * 2160 * 8;
constexpr int TOTAL_INSTRUCTIONS = 50;

template <size_t PER_OP>
static void instructions_per_operation(Stream& stream, Ptr1D<float>& input, Ptr1D<float>& output) {
    using AddOp = Add<float>;
    const auto manyInst = StaticLoop<AddOp, static_cast<int>(PER_OP)>::build(1.f);
    const auto allInstr = StaticLoop<AddOp, TOTAL_INSTRUCTIONS>::build(1.f);
    constexpr int remaining = TOTAL_INSTRUCTIONS % static_cast<int>(PER_OP);
    const auto readDF = PerThreadRead<ND::_1D, float>::build(input);
    const auto writeDF = PerThreadWrite<ND::_1D, float>::build(output);
    const auto separated = [&]() {
        for (int i = 0; i < TOTAL_INSTRUCTIONS / static_cast<int>(PER_OP); ++i) executeOperations<TransformDPP<>>(stream, readDF, manyInst, writeDF);
        if constexpr (remaining != 0) executeOperations<TransformDPP<>>(stream, readDF, StaticLoop<AddOp, remaining>::build(1.f), writeDF);
    };
    const auto all = [&]() { executeOperations<TransformDPP<>>(stream, readDF, allInstr, writeDF); };
    // input element i holds i mod 1000 (small integers: every sum below is exact), so a result that lands on the wrong
    // element shows; every element of both launches is compared with its closed form
    for (uint i = 0; i < static_cast<uint>(NUM_ELEMENTS); ++i) input.at(i) = static_cast<float>(i % 1000u);
    input.upload(stream);
    setTo(0.f, output, stream);
    all();
    output.download(stream);
    stream.sync();
    bool passed = true;
    for (uint i = 0; i < static_cast<uint>(NUM_ELEMENTS); ++i) passed = passed && output.at(i) == static_cast<float>(i % 1000u) + static_cast<float>(TOTAL_INSTRUCTIONS);
    executeOperations<TransformDPP<>>(stream, readDF, manyInst, writeDF);
    output.download(stream);
    stream.sync();
    for (uint i = 0; i < static_cast<uint>(NUM_ELEMENTS); ++i) passed = passed && output.at(i) == static_cast<float>(i % 1000u) + static_cast<float>(PER_OP);
    two_variants("instructions_per_operation", "instructions_per_op", PER_OP, "separated", "all", stream, separated, all, passed);
}
template <size_t... Is>
static void instructions_sweep(Stream& stream, std::index_sequence<Is...>) {
    constexpr auto values = sweep_values<1, 5>(std::make_index_sequence<10>{});
    Ptr1D<float> input(NUM_ELEMENTS), output(NUM_ELEMENTS);
    (instructions_per_operation<values[Is]>(stream, input, output), ...);
}

// ---- vertical fusion (latency hiding) ----------------------------------------------------------------------------------
template <size_t NUM_OPS>
static void vertical_fusion(Stream& stream, Ptr1D<float>& input, Ptr1D<float>& output) {
    constexpr int INCREMENT = 20;
    using Loop = StaticLoop<StaticLoop<Mul<float>, INCREMENT>, static_cast<int>(NUM_OPS) / INCREMENT>;
    // multiplications actually applied: the inner loop runs 20, the outer at least once
    constexpr int applied = INCREMENT * (static_cast<int>(NUM_OPS) / INCREMENT > 1 ? static_cast<int>(NUM_OPS) / INCREMENT : 1);
    const auto readDF = PerThreadRead<ND::_1D, float>::build(input);
    const auto writeDF = PerThreadWrite<ND::_1D, float>::build(output);
    const auto launch = [&]() { executeOperations<TransformDPP<>>(stream, readDF, Loop::build(2.f), writeDF); };
    // (the reference fills the input with 1; seven different values here, so that an element written from the wrong input
    // shows: a multiplication by two is exact until it overflows, so every output is known)
    for (uint i = 0; i < static_cast<uint>(NUM_ELEMENTS); ++i) input.at(i) = 1.f + static_cast<float>(i % 7u) * 0.125f;
    input.upload(stream);
    launch();
    output.download(stream);
    stream.sync();
    bool passed = true;
    for (uint i = 0; i < static_cast<uint>(NUM_ELEMENTS); ++i) passed = passed && output.at(i) == std::ldexp(input.at(i), applied);
    Timer timer;
    std::vector<float> t(ITERS);
    for (int i = 0; i < ITERS; ++i) t[i] = timer.time_ms(stream, launch);
    const Stats s = stats_of(t);
    std::printf("{\"sweep\": \"vertical_fusion\", \"operations\": %zu, \"multiplications_applied\": %d, \"ms\": %.6f, \"std\": %.6f, \"min_ms\": %.6f, "
                "\"gb_s\": %.1f, \"passed\": %s}\n",
                NUM_OPS, applied, s.mean, s.stddev, s.min, 2.0 * NUM_ELEMENTS * 4 / (s.mean * 1e-3) / 1e9, passed ? "true" : "false");
    std::fflush(stdout);
    all_passed = all_passed && passed;
}
template <size_t... Is>
static void vertical_sweep(Stream& stream, std::index_sequence<Is...>) {
    constexpr auto values = sweep_values<1, 20>(std::make_index_sequence<5>{});
    Ptr1D<float> input(NUM_ELEMENTS), output(NUM_ELEMENTS);
    (vertical_fusion<values[Is]>(stream, input, output), ...);
}

// ---- thread fusion -------------------------------------------------------------------------------------------------------
template <typename T>
static bool same_pixel(const T& a, const T& b) { return std::memcmp(&a, &b, sizeof(T)) == 0; }

// the chain's operations (all unary here) applied on the host, one after the other
template <typename V>
static V on_host(const V& v) { return v; }
template <typename V, typename Op, typename... Rest>
static auto on_host(const V& v, const Op&, const Rest&... rest) { return on_host(Op::Operation::exec(v), rest...); }
// a value that depends on the position and on the channel, different in neighbouring pixels, rows and channels, within the
// range of every pixel type of the sweep
template <typename T>
static T pattern_pixel(uint x, uint y) {
    using B = VBase<T>;
    const auto channel = [&](uint c) { return static_cast<B>((x * 7u + y * 13u + c * 29u) % 251u); };
    if constexpr (cn<T> == 1) return T{ channel(0) };
    else if constexpr (cn<T> == 2) return T{ channel(0), channel(1) };
    else if constexpr (cn<T> == 3) return T{ channel(0), channel(1), channel(2) };
    else return T{ channel(0), channel(1), channel(2), channel(3) };
}

template <typename I, typename O, size_t RESOLUTION, typename... Ops>
static void thread_fusion_case(Stream& stream, const char* name, const Ops&... ops) {
    Ptr2D<I> d_input(RESOLUTION, RESOLUTION);
    for (uint y = 0; y < RESOLUTION; ++y)
        for (uint x = 0; x < RESOLUTION; ++x) d_input.at(x, y) = pattern_pixel<I>(x, y);
    d_input.upload(stream);
    Ptr2D<O> d_plain(RESOLUTION, RESOLUTION), d_fused(RESOLUTION, RESOLUTION);
    const auto read = PerThreadRead<ND::_2D, I>::build(d_input);
    const auto plain = [&]() { executeOperations<TransformDPP<defaultParArch, TF::DISABLED>>(stream, read, ops..., PerThreadWrite<ND::_2D, O>::build(d_plain)); };
    const auto fused = [&]() { executeOperations<TransformDPP<defaultParArch, TF::ENABLED>>(stream, read, ops..., PerThreadWrite<ND::_2D, O>::build(d_fused)); };
    plain();
    fused();
    d_plain.download(stream);
    d_fused.download(stream);
    stream.sync();
    // the two tags give the same launch in this library (the kernels vectorise by themselves), so comparing them with each
    // other proves nothing: every pixel of both outputs is compared with the chain evaluated on the host
    bool passed = true;
    for (uint y = 0; y < RESOLUTION; ++y) {
        for (uint x = 0; x < RESOLUTION; ++x) {
            const O expected = on_host(pattern_pixel<I>(x, y), ops...);
            passed = passed && same_pixel(d_plain.at(x, y), expected) && same_pixel(d_fused.at(x, y), expected);
        }
    }
    const double bytes = static_cast<double>(RESOLUTION) * RESOLUTION * (sizeof(I) + sizeof(O));
    char extra[160];
    std::snprintf(extra, sizeof(extra), ", \"case\": \"%s\", \"bytes\": %.0f", name, bytes);
    two_variants("thread_fusion", "pixels_per_side", RESOLUTION, "tf_disabled", "tf_enabled", stream, plain, fused, passed, extra);
}
template <size_t RESOLUTION>
static void thread_fusion_resolution(Stream& stream) {
    thread_fusion_case<uchar, uchar, RESOLUTION>(stream, "uchar copy");
    thread_fusion_case<uchar3, uchar3, RESOLUTION>(stream, "uchar3 copy");
    thread_fusion_case<uchar4, uchar4, RESOLUTION>(stream, "uchar4 copy");
    thread_fusion_case<ushort2, ushort2, RESOLUTION>(stream, "ushort2 copy");
    thread_fusion_case<float, float, RESOLUTION>(stream, "float copy");
    thread_fusion_case<float3, float3, RESOLUTION>(stream, "float3 copy");
    thread_fusion_case<float4, float4, RESOLUTION>(stream, "float4 copy");
    thread_fusion_case<uchar, float, RESOLUTION>(stream, "uchar -> float", SaturateCast<uchar, float>::build());
    thread_fusion_case<uchar3, float3, RESOLUTION>(stream, "uchar3 -> float3", SaturateCast<uchar3, float3>::build());
    thread_fusion_case<uchar4, float4, RESOLUTION>(stream, "uchar4 -> float4", SaturateCast<uchar4, float4>::build());
    thread_fusion_case<ushort3, float3, RESOLUTION>(stream, "ushort3 -> float3", SaturateCast<ushort3, float3>::build());
    thread_fusion_case<uchar3, float4, RESOLUTION>(stream, "uchar3 -> float3 -> RGB2RGBA float4", SaturateCast<uchar3, float3>::build(),
                                                   ColorConversion<ColorConversionCodes::COLOR_RGB2RGBA, float3, float4>::build());
    thread_fusion_case<float4, uchar, RESOLUTION>(stream, "float4 -> uchar4 -> RGBA2GRAY uchar", SaturateCast<float4, uchar4>::build(),
                                                  ColorConversion<ColorConversionCodes::COLOR_RGBA2GRAY, uchar4, uchar>::build());
}
template <size_t... Is>
static void thread_fusion_sweep(Stream& stream, std::index_sequence<Is...>) {
    constexpr auto values = sweep_values<1024, 1024>(std::make_index_sequence<5>{});
    ((thread_fusion_resolution<values[Is]>(stream), thread_fusion_resolution<values[Is] + 1>(stream)), ...);
}

int main(int argc, char** argv) {
    std::string only = argc > 1 ? argv[1] : "all";
    if (argc > 2) ITERS = std::atoi(argv[2]);
    if (ITERS < 1) ITERS = 1;
    Stream stream;
    if (only == "all" || only == "horizontal") horizontal_fusion_sweep(stream, std::make_index_sequence<10>{});
    if (only == "all" || only == "instructions") instructions_sweep(stream, std::make_index_sequence<10>{});
    if (only == "all" || only == "vertical") vertical_sweep(stream, std::make_index_sequence<5>{});
    if (only == "all" || only == "thread") thread_fusion_sweep(stream, std::make_index_sequence<5>{});
    stream.sync();
    return all_passed ? 0 : 1;
}

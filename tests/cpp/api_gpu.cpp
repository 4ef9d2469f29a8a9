// The rest of the executeOperations surface on the GPU, as user code: buffer overloads (fused_kernel.h:26-54 of the
// reference), conditional batches with a default value (batch_operations.h:234-241), 1-D reads (one long row of the pointwise kernel) with StaticLoop, 3-D reads (generic kernel),
// cropped buffer views, the thread-fusion tag, setTo, stream sharing and error reporting.  Self-checking: exit code 0.
#include <fused_kernel/fused_kernel.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>

using namespace fk;

static int failures = 0;
#define EXPECT(cond)                                                                                                   \
    do {                                                                                                               \
        if (!(cond)) {                                                                                                 \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                                              \
            ++failures;                                                                                                \
        }                                                                                                              \
    } while (0)

template <typename T>
static void fill_ramp(Ptr2D<T>& img, Stream& stream, int scale) {
    const auto d = img.dims();
    for (uint y = 0; y < d.height; ++y)
        for (uint x = 0; x < d.width; ++x) img.at(x, y) = make_set<T>((x * 3 + y * 7) * scale % 251);
    img.upload(stream);
}

// Operations written by a user in the style of the Fused Kernel Library: a Parent names the member types, the DECLARE
// macro imports them (parent_operations.h of the reference).  One of each kind that a chain can hold.
template <typename T>
struct UserMirrorRead { // reads the row back to front
private:
    using SelfType = UserMirrorRead<T>;

public:
    FK_STATIC_STRUCT(UserMirrorRead, SelfType)
    using Parent = ReadOperation<T, RawPtr<ND::_2D, T>, T, TF::DISABLED, UserMirrorRead<T>>;
    DECLARE_READ_PARENT
    FK_HOST_DEVICE_FUSE OutputType exec(const Point& thread, const ParamsType& params) {
        return *PtrAccessor<ND::_2D>::cr_point(Point(static_cast<int>(params.dims.width) - 1 - thread.x, thread.y), params);
    }
    FK_HOST_DEVICE_FUSE uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HOST_DEVICE_FUSE uint num_elems_y(const Point&, const OperationDataType& opData) { return opData.params.dims.height; }
    FK_HOST_DEVICE_FUSE uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HOST_DEVICE_FUSE ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return ActiveThreads(opData.params.dims.width, opData.params.dims.height, 1);
    }
};
template <typename T>
struct UserSquare {
private:
    using SelfType = UserSquare<T>;

public:
    FK_STATIC_STRUCT(UserSquare, SelfType)
    using Parent = UnaryOperation<T, T, UserSquare<T>>;
    DECLARE_UNARY_PARENT
    FK_HOST_DEVICE_FUSE OutputType exec(const InputType& input) { return input * input; }
};
template <typename T>
struct UserAxpy { // a * x + b with { a, b } as parameters
private:
    using SelfType = UserAxpy<T>;

public:
    FK_STATIC_STRUCT(UserAxpy, SelfType)
    using Parent = BinaryOperation<T, Tuple<T, T>, T, UserAxpy<T>>;
    DECLARE_BINARY_PARENT
    FK_HOST_DEVICE_FUSE OutputType exec(const InputType& input, const ParamsType& params) { return get<0>(params) * input + get<1>(params); }
};
template <typename T>
struct UserTransposedWrite {
private:
    using SelfType = UserTransposedWrite<T>;

public:
    FK_STATIC_STRUCT(UserTransposedWrite, SelfType)
    using Parent = WriteOperation<T, RawPtr<ND::_2D, T>, T, TF::DISABLED, UserTransposedWrite<T>>;
    DECLARE_WRITE_PARENT
    FK_HOST_DEVICE_FUSE void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        *PtrAccessor<ND::_2D>::point(Point(thread.y, thread.x), params) = input;
    }
    FK_HOST_DEVICE_FUSE uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.dims.width; }
    FK_HOST_DEVICE_FUSE uint pitch(const Point&, const OperationDataType& opData) { return opData.params.dims.pitch; }
};

int main() {
    Stream stream;
    Stream alias = stream; // copies share the native stream
    EXPECT(alias.getHIPStream() == stream.getHIPStream() && stream.getRefCount() == 2);

    // 1. conditional batch: planes >= activeBatch take the default value, then run through the same compute operations
    {
        constexpr size_t BATCH = 3;
        std::array<Ptr2D<uchar3>, BATCH> inputs{ Ptr2D<uchar3>(16, 8), Ptr2D<uchar3>(16, 8), Ptr2D<uchar3>(16, 8) };
        for (size_t i = 0; i < BATCH; ++i) setTo(uchar3{ static_cast<uchar>(10 * (i + 1)), 1, 2 }, inputs[i], stream);
        Tensor<float3> out(16, 8, BATCH);
        executeOperations<TransformDPP<>>(inputs, 2, uchar3{ 9, 9, 9 }, out, stream, Cast<uchar3, float3>::build(),
                                          Mul<float3>::build(make_set<float3>(2.f)));
        out.download(stream);
        stream.sync();
        bool ok = true;
        for (uint y = 0; y < 8; ++y)
            for (uint x = 0; x < 16; ++x) {
                ok = ok && out.at(x, y, 0).x == 20.f && out.at(x, y, 0).z == 4.f && out.at(x, y, 1).x == 40.f && out.at(x, y, 2).x == 18.f &&
                     out.at(x, y, 2).y == 18.f;
            }
        EXPECT(ok);
    }
    // 2. input / output buffer overload, scalar pixels (16 per thread), odd size and the runtime's padded pitch
    {
        Ptr2D<uchar> in(1237, 19);
        Ptr2D<float> out(1237, 19);
        fill_ramp(in, stream, 1);
        executeOperations<TransformDPP<>>(in, out, stream, Cast<uchar, float>::build(), Add<float>::build(0.5f));
        out.download(stream);
        stream.sync();
        bool ok = true;
        for (uint y = 0; y < 19; ++y)
            for (uint x = 0; x < 1237; ++x) ok = ok && out.at(x, y) == static_cast<float>(in.at(x, y)) + 0.5f;
        EXPECT(ok);
    }
    // 3. 1-D buffers under the thread-fusion tag; lengths that are and are not whole thread groups; StaticLoop
    for (const uint n : { 1000u, 1003u, 1u, 262144u + 7u }) {
        Ptr1D<float> in(n), out(n);
        for (uint i = 0; i < n; ++i) in.at(i) = 0.25f * static_cast<float>(i % 4096u);
        Stream s2;
        in.upload(s2);
        executeOperations<TransformDPP<ParArch::GPU_AMD, TF::ENABLED>>(in, out, s2, Mul<float>::build(3.f), Sub<float>::build(1.f));
        out.download(s2);
        s2.sync();
        bool ok = true;
        for (uint i = 0; i < n; ++i) ok = ok && out.at(i) == 0.25f * static_cast<float>(i % 4096u) * 3.f - 1.f;
        EXPECT(ok);
        // five additions in one operation; a loop of zero iterations still applies its operation once, as in the reference
        executeOperations<TransformDPP<>>(s2, PerThreadRead<ND::_1D, float>::build(in), StaticLoop<Add<float>, 5>::build(0.5f),
                                          StaticLoop<StaticLoop<Mul<float>, 2>, 0>::build(2.f), PerThreadWrite<ND::_1D, float>::build(out));
        out.download(s2);
        s2.sync();
        ok = true;
        for (uint i = 0; i < n; ++i) ok = ok && out.at(i) == (0.25f * static_cast<float>(i % 4096u) + 2.5f) * 4.f;
        EXPECT(ok);
    }
    // 4. 3-D read into a 3-D write, every plane (generic kernel), and getPlane views
    {
        Tensor<float> in(33, 5, 4), out(33, 5, 4);
        for (uint z = 0; z < 4; ++z)
            for (uint y = 0; y < 5; ++y)
                for (uint x = 0; x < 33; ++x) in.at(x, y, z) = static_cast<float>(z * 1000 + y * 100 + x);
        in.upload(stream);
        executeOperations<TransformDPP<>>(stream, TensorRead<float>::build(in), Add<float>::build(1.f), TensorWrite<float>::build(out));
        out.download(stream);
        stream.sync();
        bool ok = true;
        for (uint z = 0; z < 4; ++z)
            for (uint y = 0; y < 5; ++y)
                for (uint x = 0; x < 33; ++x) ok = ok && out.at(x, y, z) == static_cast<float>(z * 1000 + y * 100 + x) + 1.f;
        EXPECT(ok);
        EXPECT(out.getPlane(2).at(7, 3) == 2000.f + 300.f + 7.f + 1.f);
    }
    // 5. a cropped view of a buffer as the source (unaligned base), SaturateCast and RGB2Gray
    {
        Ptr2D<float4> in(100, 40);
        for (uint y = 0; y < 40; ++y)
            for (uint x = 0; x < 100; ++x) in.at(x, y) = float4{ x * 3.f - 20.f, y * 7.f + 0.5f, 127.5f, 300.f };
        in.upload(stream);
        Ptr2D<float4> view = in.crop2D(Point(3, 2), PtrDims<ND::_2D>(61, 33));
        Ptr2D<uchar4> out(61, 33);
        executeOperations<TransformDPP<>>(view, out, stream, SaturateCast<float4, uchar4>::build());
        out.download(stream);
        stream.sync();
        bool ok = true;
        for (uint y = 0; y < 33; ++y)
            for (uint x = 0; x < 61; ++x) {
                const float fx = (x + 3) * 3.f - 20.f, fy = (y + 2) * 7.f + 0.5f;
                const uchar4 v = out.at(x, y);
                ok = ok && v.x == (fx < 0.f ? 0 : fx > 255.f ? 255 : static_cast<uchar>(fx)) &&
                     v.y == (fy > 255.f ? 255 : static_cast<uchar>(fy + 0.5f)) && v.z == 128 && v.w == 255;
            }
        EXPECT(ok);
        Ptr2D<uchar3> rgb(77, 9);
        Ptr2D<uchar> gray(77, 9);
        fill_ramp(rgb, stream, 5);
        executeOperations<TransformDPP<>>(rgb, gray, stream, ColorConversion<ColorConversionCodes::COLOR_RGB2GRAY, uchar3, uchar>::build());
        gray.download(stream);
        stream.sync();
        ok = true;
        for (uint y = 0; y < 9; ++y)
            for (uint x = 0; x < 77; ++x) {
                const uchar3 p = rgb.at(x, y);
                ok = ok && gray.at(x, y) == static_cast<uchar>(std::nearbyint((p.x * 0.299f + p.y * 0.587f) + p.z * 0.114f));
            }
        EXPECT(ok);
    }
    // 6. YUV images: an NV12 frame allocated by Image<PF>, read as {Y, U, V}, converted, and written back as UYVY
    {
        constexpr uint W = 64, H = 48;
        Image<PixelFormat::NV12> nv12(W, H);
        EXPECT(nv12.getData().dims().width == W && nv12.getData().dims().height == H + H / 2 && nv12.imageHeight() == H);
        auto bytes = nv12.getData();
        for (uint y = 0; y < H; ++y)
            for (uint x = 0; x < W; ++x) bytes.at(x, y) = static_cast<uchar>((x + 2 * y) % 220 + 16);
        for (uint y = 0; y < H / 2; ++y)
            for (uint x = 0; x < W; x += 2) {
                bytes.at(x, H + y) = static_cast<uchar>(100 + x / 2 + y);     // U
                bytes.at(x + 1, H + y) = static_cast<uchar>(200 - x / 2 - y); // V
            }
        nv12.upload(stream);
        EXPECT(nv12.readAt(Point(5, 7)).x == (5 + 14) % 220 + 16 && nv12.readAt(Point(5, 7)).y == 100 + 2 + 3 && nv12.readAt(Point(5, 7)).z == 200 - 2 - 3);

        Ptr2D<uchar3> yuv(W, H);
        Ptr2D<uchar4> rgba(W, H);
        Image<PixelFormat::UYVY> uyvy(W, H);
        const auto read = ReadYUV<PixelFormat::NV12>::build(nv12);
        executeOperations<TransformDPP<>>(stream, read, PerThreadWrite<ND::_2D, uchar3>::build(yuv));
        executeOperations<TransformDPP<>>(stream, read, ConvertYUVToRGB<PixelFormat::NV12, ColorRange::Full, ColorPrimitives::bt709, true>::build(),
                                          PerThreadWrite<ND::_2D, uchar4>::build(rgba));
        executeOperations<TransformDPP<>>(stream, read, WriteYUV<PixelFormat::UYVY>::build(uyvy));
        yuv.download(stream);
        rgba.download(stream);
        uyvy.download(stream);
        stream.sync();
        bool ok = true;
        for (uint y = 0; y < H; ++y)
            for (uint x = 0; x < W; ++x) {
                const uchar3 want = nv12.readAt(Point(static_cast<int>(x), static_cast<int>(y)));
                const uchar3 got = yuv.at(x, y);
                ok = ok && got.x == want.x && got.y == want.y && got.z == want.z;
                const uchar4 host_rgba = ConvertYUVToRGB<PixelFormat::NV12, ColorRange::Full, ColorPrimitives::bt709, true>::exec(want);
                const uchar4 dev_rgba = rgba.at(x, y);
                ok = ok && dev_rgba.x == host_rgba.x && dev_rgba.y == host_rgba.y && dev_rgba.z == host_rgba.z && dev_rgba.w == 255;
                // 4:2:2 keeps the chroma of even rows and of odd rows apart; NV12 gives both rows the same pair
                const uchar3 back = uyvy.readAt(Point(static_cast<int>(x), static_cast<int>(y)));
                ok = ok && back.x == want.x && back.y == want.y && back.z == want.z;
            }
        EXPECT(ok);
    }
    // 7. CircularTensor (owning its memory): the last four results of a chain in age order, in the three layouts
    {
        constexpr int B = 4;
        constexpr uint W = 40, H = 12;
        CircularTensor<float, 3, B, CircularTensorOrder::NewestFirst, ColorPlanes::Standard> newest_first(W, H);
        CircularTensor<float, 3, B, CircularTensorOrder::OldestFirst, ColorPlanes::Transposed> transposed(W, H);
        CircularTensor<float3, 1, B, CircularTensorOrder::OldestFirst, ColorPlanes::Standard> packed(W, H);
        Ptr2D<uchar3> frame(W, H);
        const auto read = PerThreadRead<ND::_2D, uchar3>::build(frame);
        bool ok = true;
        for (int k = 0; k < 7; ++k) {
            setTo(uchar3{ static_cast<uchar>(k + 1), static_cast<uchar>(10 + k), static_cast<uchar>(100 + k) }, frame, stream);
            newest_first.update(stream, read, Cast<uchar3, float3>::build(), Mul<float3>::build(make_set<float3>(2.f)), TensorSplit<float3>::build(newest_first.ptr()));
            transposed.update(stream, read, Cast<uchar3, float3>::build(), TensorTSplit<float3>::build(transposed.ptr()));
            packed.update(stream, read, Cast<uchar3, float3>::build(), TensorWrite<float3>::build(packed.ptr()));
            newest_first.download(stream);
            transposed.download(stream);
            packed.download(stream);
            stream.sync();
            for (int age = 0; age <= (k < B - 1 ? k : B - 1); ++age) {
                const float r = static_cast<float>(k - age + 1), g = static_cast<float>(10 + k - age), b = static_cast<float>(100 + k - age);
                // split: channel planes of image `age` follow each other; at() addresses channel 0, the others are W*H further
                const float* p = &newest_first.at(5, 3, static_cast<uint>(age));
                ok = ok && p[0] == 2.f * r && p[W * H] == 2.f * g && p[2 * W * H] == 2.f * b;
                const uint z = static_cast<uint>(B - 1 - age);
                const float* t = &transposed.at(7, 2, z); // transposed: channel planes are outermost, B*W*H apart
                ok = ok && t[0] == r && t[B * W * H] == g && t[2 * B * W * H] == b;
                const float3 q = packed.at(W - 1, H - 1, z);
                ok = ok && q.x == r && q.y == g && q.z == b;
            }
        }
        EXPECT(ok && newest_first.nextUpdateIdx() == 7 % B);
    }
    // 9. BatchRead -> BatchWrite: plane z of one launch is read from image z and written to its own output image
    {
        constexpr size_t BATCH = 3;
        std::array<Ptr2D<uchar3>, BATCH> inputs{ Ptr2D<uchar3>(70, 9), Ptr2D<uchar3>(70, 9), Ptr2D<uchar3>(70, 9) };
        std::array<Ptr2D<float3>, BATCH> outputs{ Ptr2D<float3>(70, 9), Ptr2D<float3>(70, 9), Ptr2D<float3>(70, 9) };
        std::array<RawPtr<ND::_2D, float3>, BATCH> raw{};
        for (size_t i = 0; i < BATCH; ++i) {
            fill_ramp(inputs[i], stream, static_cast<int>(i) + 1);
            raw[i] = outputs[i].ptr();
        }
        const auto writeAll = PerThreadWrite<ND::_2D, float3>::build(raw);
        static_assert(isWriteType<std::decay_t<decltype(writeAll)>> && isBatchOperation<typename std::decay_t<decltype(writeAll)>::Operation>, "BatchWrite");
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, uchar3>::build(inputs), Cast<uchar3, float3>::build(),
                                          Mul<float3>::build(make_set<float3>(0.5f)), writeAll);
        bool ok = true;
        for (size_t i = 0; i < BATCH; ++i) {
            outputs[i].download(stream);
            stream.sync();
            for (uint y = 0; y < 9; ++y)
                for (uint x = 0; x < 70; ++x) ok = ok && outputs[i].at(x, y).y == 0.5f * inputs[i].at(x, y).y;
        }
        EXPECT(ok);
    }
    // 10. a write in the middle of a chain stores the value at that point and hands it on; a chain that starts with a
    //     write is one MidWrite operation
    {
        Ptr2D<uchar> in(130, 7);
        Ptr2D<float> mid(130, 7), mid2(130, 7), last(130, 7);
        fill_ramp(in, stream, 1);
        const auto tee = fuse(PerThreadWrite<ND::_2D, float>::build(mid2), Add<float>::build(1.f)); // write, then add
        static_assert(isMidWriteType<std::decay_t<decltype(tee)>>, "a write-first chain is a MidWrite operation");
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, uchar>::build(in), Cast<uchar, float>::build(),
                                          MidWrite<PerThreadWrite<ND::_2D, float>>{ { mid.ptr() } }, Mul<float>::build(3.f), tee,
                                          PerThreadWrite<ND::_2D, float>::build(last));
        mid.download(stream);
        mid2.download(stream);
        last.download(stream);
        stream.sync();
        bool ok = true;
        for (uint y = 0; y < 7; ++y)
            for (uint x = 0; x < 130; ++x) {
                const float v = static_cast<float>(in.at(x, y));
                ok = ok && mid.at(x, y) == v && mid2.at(x, y) == 3.f * v && last.at(x, y) == 3.f * v + 1.f;
            }
        EXPECT(ok);
    }
    // 11. user-defined operations of every kind in one chain, between library operations
    {
        constexpr uint W = 77, H = 13;
        Ptr2D<float> in(W, H), out(H, W);
        for (uint y = 0; y < H; ++y)
            for (uint x = 0; x < W; ++x) in.at(x, y) = static_cast<float>(x) - 0.25f * static_cast<float>(y);
        in.upload(stream);
        executeOperations<TransformDPP<>>(stream, UserMirrorRead<float>::build(in.ptr()), UserSquare<float>::build(), Add<float>::build(1.f),
                                          UserAxpy<float>::build(Tuple<float, float>{ 2.f, -3.f }), UserTransposedWrite<float>::build(out.ptr()));
        out.download(stream);
        stream.sync();
        bool ok = true;
        for (uint y = 0; y < H; ++y)
            for (uint x = 0; x < W; ++x) {
                const float v = in.at(W - 1 - x, y);
                ok = ok && out.at(y, x) == 2.f * (v * v + 1.f) + -3.f;
            }
        EXPECT(ok);
    }
    // 12. Div on the GPU gives the results of the IEEE division for every float (the kernels are built without fast-math
    //     and keep subnormals): random bit patterns, subnormal operands and results, exact ties among subnormal results
    //     (x = k * 2^-149 * d), infinities, NaNs and signed zeros
    {
        const uint N = 1u << 20;
        Ptr1D<float> in(N), out(N);
        unsigned long long state = 42;
        const auto next = [&state]() {
            state += 0x9E3779B97F4A7C15ull;
            unsigned long long z = state;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
            z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
            return static_cast<unsigned>(z ^ (z >> 31));
        };
        int mismatches = 0;
        // second pass per divisor: every operand within [2^-40, 2^40], where whole waves take the kernels' short division
        // by the host's reciprocal instead of the division instruction sequence
        for (const bool moderate : { false, true })
        for (const float d : { 255.f, 6.f, 0.229f, 1e-30f, 3e38f, -7.f, 5e-39f, 1.f / 3.f, 1.99999988f, 1.00000012f, 57.375f, 9.5e-13f, 1.0e12f }) {
            for (uint i = 0; i < N; ++i) {
                unsigned bits = next();
                if (moderate) {
                    bits = (bits & 0x807fffffu) | ((87u + next() % 80u) << 23);
                } else {
                    if (i % 4 == 1) bits &= 0x807fffffu;                        // subnormal operands
                    if (i % 4 == 2) bits = (bits & 0x80ffffffu) | 0x00800000u; // smallest normal operands
                    if (i % 64 == 3) bits = (i / 64 % 4 == 0) ? 0x7f800000u : (i / 64 % 4 == 1) ? 0xff800000u : (i / 64 % 4 == 2) ? 0x7fc00000u : 0x80000000u;
                }
                float v;
                std::memcpy(&v, &bits, 4);
                if (!moderate && i % 4 == 3 && i < 4096) v = static_cast<float>(i / 4) * 1.40129846e-45f * d;
                in.at(i) = v;
            }
            in.upload(stream);
            executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_1D, float>::build(in), Div<float>::build(d), PerThreadWrite<ND::_1D, float>::build(out));
            out.download(stream);
            stream.sync();
            for (uint i = 0; i < N; ++i) {
                const volatile float x = in.at(i), divisor = d; // volatile: the host compiler must divide, not fold
                const float want = x / divisor, got = out.at(i);
                if (std::memcmp(&want, &got, 4) != 0 && !(std::isnan(want) && std::isnan(got))) ++mismatches;
            }
        }
        EXPECT(mismatches == 0);
    }
    // 13. executeOperations keeps no state of its own: host threads on streams of their own, each with its own buffers,
    // launch the same chains at the same time (one small enough for by-value parameters, one batch large enough for the
    // staged parameter block) and get what a single thread gets
    {
        constexpr int THREADS = 4, ROUNDS = 12;
        constexpr size_t BATCH = 50;
        Ptr2D<uchar3> source(640, 360);
        fill_ramp(source, stream, 3);
        std::array<Rect, BATCH> rects;
        for (size_t i = 0; i < BATCH; ++i) rects[i] = Rect(static_cast<uint>(7 * i), static_cast<uint>(3 * i), 40 + 5 * static_cast<int>(i), 30 + 4 * static_cast<int>(i));
        const auto run_batch = [&](Stream& s, Tensor<float>& out) {
            executeOperations<TransformDPP<>>(s,
                PerThreadRead<ND::_2D, uchar3>::build(source).then(Crop<>::build(rects)).then(Resize<InterpolationType::INTER_LINEAR>::build(Size(64, 48))),
                Mul<float3>::build(make_set<float3>(1.f / 255.f)), TensorSplit<float3>::build(out));
        };
        const auto run_plain = [&](Stream& s, Ptr2D<float3>& out) {
            executeOperations<TransformDPP<>>(s, PerThreadRead<ND::_2D, uchar3>::build(source), Cast<uchar3, float3>::build(),
                                              Add<float3>::build(make_set<float3>(0.25f)), PerThreadWrite<ND::_2D, float3>::build(out));
        };
        Tensor<float> want_batch(64, 48, BATCH, 3);
        Ptr2D<float3> want_plain(640, 360);
        run_batch(stream, want_batch);
        run_plain(stream, want_plain);
        want_batch.download(stream);
        want_plain.download(stream);
        stream.sync();
        int bad[THREADS] = {};
        std::vector<std::thread> workers;
        for (int t = 0; t < THREADS; ++t) {
            workers.emplace_back([&, t]() {
                try {
                    Stream mine;
                    Tensor<float> got_batch(64, 48, BATCH, 3);
                    Ptr2D<float3> got_plain(640, 360);
                    for (int round = 0; round < ROUNDS; ++round) {
                        setTo(-1.f, got_batch, mine);
                        run_batch(mine, got_batch);
                        run_plain(mine, got_plain);
                        got_batch.download(mine);
                        got_plain.download(mine);
                        mine.sync();
                        if (std::memcmp(got_batch.ptrPinned().data, want_batch.ptrPinned().data, got_batch.sizeInBytes()) != 0) ++bad[t];
                        for (uint y = 0; y < 360; y += 7)
                            for (uint x = 0; x < 640; ++x)
                                if (std::memcmp(&got_plain.at(x, y), &want_plain.at(x, y), sizeof(float3)) != 0) ++bad[t];
                    }
                } catch (const std::exception& e) {
                    std::printf("thread %d: %s\n", t, e.what());
                    bad[t] = -1;
                }
            });
        }
        for (auto& w : workers) w.join();
        for (int t = 0; t < THREADS; ++t) EXPECT(bad[t] == 0);
        EXPECT(source.getRefCount() == 1);
    }
    // 14. a batch whose parameter block is far beyond 4 KiB and still travels by value: 200 crops in one launch against
    // 200 launches of one crop each
    {
        constexpr size_t BATCH = 200;
        Ptr2D<uchar3> source(512, 256);
        fill_ramp(source, stream, 5);
        std::array<Rect, BATCH> rects;
        for (size_t i = 0; i < BATCH; ++i) rects[i] = Rect(static_cast<uint>(2 * i), static_cast<uint>(i), 20 + static_cast<int>(i % 90), 12 + static_cast<int>(i % 40));
        Tensor<float3> together(32, 24, BATCH), one_by_one(32, 24, BATCH);
        executeOperations<TransformDPP<>>(stream,
            PerThreadRead<ND::_2D, uchar3>::build(source).then(Crop<>::build(rects)).then(Resize<InterpolationType::INTER_LINEAR>::build(Size(32, 24))),
            Mul<float3>::build(make_set<float3>(0.5f)), TensorWrite<float3>::build(together));
        for (size_t i = 0; i < BATCH; ++i) {
            executeOperations<TransformDPP<>>(stream,
                PerThreadRead<ND::_2D, uchar3>::build(source).then(Crop<>::build(rects[i])).then(Resize<InterpolationType::INTER_LINEAR>::build(Size(32, 24))),
                Mul<float3>::build(make_set<float3>(0.5f)), PerThreadWrite<ND::_2D, float3>::build(one_by_one.getPlane(static_cast<uint>(i))));
        }
        together.download(stream);
        one_by_one.download(stream);
        stream.sync();
        EXPECT(std::memcmp(together.ptrPinned().data, one_by_one.ptrPinned().data, together.sizeInBytes()) == 0);
        bool varied = false;
        for (uint x = 1; x < 32; ++x) varied = varied || together.at(x, 3, 150).x != together.at(0, 3, 150).x;
        EXPECT(varied);
    }
    // 15. the README chain through the host executor (TransformDPP<ParArch::CPU>, host memory) and through the GPU executor:
    // the same bits, on the README's own crops (up- and down-scaling, bars on either side) and on a small frame
    {
        constexpr size_t BATCH = 5;
        Ptr2D<uchar3> frame(320, 200);
        fill_ramp(frame, stream, 7);
        Ptr2D<uchar3> host_frame(320, 200, 0, MemType::Host);
        for (uint y = 0; y < 200; ++y)
            for (uint x = 0; x < 320; ++x) host_frame.at(x, y) = frame.at(x, y);
        const std::array<Rect, BATCH> crops{ Rect(0, 0, 34, 25), Rect(10, 10, 70, 15), Rect(20, 20, 60, 59), Rect(30, 30, 20, 23), Rect(40, 40, 12, 11) };
        const auto chain = [&](const auto& image) {
            return PerThreadRead<ND::_2D, uchar3>::build(image)
                .then(Crop<>::build(crops))
                .then(Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(Size(60, 60), float3{ 0.f, 0.f, 0.f }))
                .then(Mul<float3>::build(make_set<float3>(1.4f)))
                .then(Sub<float3>::build(make_set<float3>(0.5f)))
                .then(Div<float3>::build(make_set<float3>(255.f)))
                .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
        };
        Tensor<float3> on_gpu(60, 60, BATCH);
        Tensor<float3> on_host(60, 60, BATCH, 1, MemType::Host);
        executeOperations<TransformDPP<>>(stream, chain(frame), TensorWrite<float3>::build(on_gpu));
        on_gpu.download(stream);
        stream.sync();
        Stream_<ParArch::CPU> host_stream;
        executeOperations<TransformDPP<ParArch::CPU>>(host_stream, chain(host_frame), TensorWrite<float3>::build(on_host));
        host_stream.sync();
        EXPECT(std::memcmp(on_gpu.ptrPinned().data, on_host.ptr().data, on_host.sizeInBytes()) == 0);
        bool varied = false;
        for (uint x = 1; x < 60; ++x) varied = varied || on_host.at(x, 30, 2).x != on_host.at(0, 30, 2).x;
        EXPECT(varied);
    }
    // 8. a launch the runtime rejects surfaces as the reference's exception text
    {
        bool threw = false;
        try {
            gpuErrchk(fkrt_launch(nullptr, 1, 1, 1, 256, 1, 1, nullptr, 0, stream));
        } catch (const std::runtime_error& e) {
            threw = std::string(e.what()).rfind("GPU Error: ", 0) == 0;
        }
        EXPECT(threw);
    }
    if (failures == 0) std::printf("api_gpu ok\n");
    return failures == 0 ? 0 : 1;
}

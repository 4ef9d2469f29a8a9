// The README example of the Fused Kernel Library as a user would write it (same includes, same calls; the reference's
// own copy is tests/examples/readme_test_code.h:26-72), compiled against this library and run on the GPU.
// usage: readme_dropin <input.bin: 3840x2160 uchar3, tight rows> <output.bin: 60x60x5 float3>
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/algorithms/image_processing/resize.h>
#include <fused_kernel/fused_kernel.h>

#include <cstdio>
#include <vector>

using namespace fk;

int main(int argc, char** argv) {
    if (argc != 3) return 2;
    Stream stream;

    const Size outputSize(60, 60);
    constexpr int BATCH = 5;
    Ptr2D<uchar3> inputImage(3840, 2160);
    Tensor<float3> output(outputSize.width, outputSize.height, BATCH);

    std::array<Rect, BATCH> crops{ Rect(0, 0, 34, 25), Rect(10, 10, 70, 15), Rect(20, 20, 60, 59), Rect(30, 30, 20, 23), Rect(40, 40, 12, 11) };

    // initImageValues(inputImage): seeded bytes handed over by the test
    {
        std::FILE* f = std::fopen(argv[1], "rb");
        if (f == nullptr) return 3;
        const RawPtr<ND::_2D, uchar3> host = inputImage.ptrPinned();
        for (uint y = 0; y < host.dims.height; ++y) {
            if (std::fread(reinterpret_cast<char*>(host.data) + static_cast<size_t>(y) * host.dims.pitch, sizeof(uchar3), host.dims.width, f) != host.dims.width) return 4;
        }
        std::fclose(f);
        inputImage.upload(stream);
    }
    const float3 backgroundColor{ 0.f, 0.f, 0.f };
    const float3 mulValue = make_set<float3>(1.4f);
    const float3 subValue = make_set<float3>(0.5f);
    const float3 divValue = make_set<float3>(255.f);

    const auto mySender = PerThreadRead<ND::_2D, uchar3>::build(inputImage)
        .then(Crop<>::build(crops))
        .then(Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(outputSize, backgroundColor))
        .then(Mul<float3>::build(mulValue))
        .then(Sub<float3>::build(subValue))
        .then(Div<float3>::build(divValue))
        .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
    const auto myReceiver = TensorWrite<float3>::build(output);

    executeOperations<fk::TransformDPP<>>(stream, mySender, myReceiver);
    output.download(stream);
    stream.sync();

    std::FILE* f = std::fopen(argv[2], "wb");
    if (f == nullptr) return 5;
    for (int z = 0; z < BATCH; ++z)
        for (int y = 0; y < outputSize.height; ++y)
            for (int x = 0; x < outputSize.width; ++x) {
                const float3 v = output.at(x, y, z);
                std::fwrite(&v, sizeof(float3), 1, f);
            }
    std::fclose(f);

    // setTo through the same executor, device and host mirror alike (core/data/ptr_utils.h:23-45 of the reference)
    Ptr2D<uchar3> filled(33, 7);
    setTo(uchar3{ 1, 2, 3 }, filled, stream);
    stream.sync();
    Ptr2D<uchar3> back(33, 7, 0, MemType::HostPinned);
    filled.downloadTo(back, stream);
    stream.sync();
    for (uint y = 0; y < 7; ++y)
        for (uint x = 0; x < 33; ++x) {
            const uchar3 d = back.at(x, y), h = filled.at(x, y);
            if (d.x != 1 || d.y != 2 || d.z != 3 || h.x != 1 || h.y != 2 || h.z != 3) return 6;
        }
    std::printf("readme_dropin ok\n");
    return 0;
}

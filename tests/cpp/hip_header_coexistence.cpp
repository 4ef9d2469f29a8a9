// User code that includes the HIP runtime's own header BEFORE the library's (for its streams, events or interop calls).
// The library's vector types live in namespace fk and HIP's at global scope, so such a translation unit qualifies them;
// the chain itself is written as always.  Runs a fused chain on a stream that the HIP API created, brackets it with HIP
// events, and checks the result.
#include <hip/hip_runtime.h>

#include <fused_kernel/fused_kernel.h>

#include <cstdio>
#include <vector>

int main() {
    hipStream_t raw = nullptr;
    if (hipStreamCreate(&raw) != hipSuccess) return 2;
    hipEvent_t begin = nullptr, end = nullptr;
    if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) return 2;
    {
        fk::Stream stream(raw); // borrowed
        constexpr int W = 257, H = 33;
        fk::Ptr2D<fk::float3> in(W, H), out(W, H);
        for (int y = 0; y < H; ++y) {
            for (int x = 0; x < W; ++x) in.at(fk::Point(x, y)) = fk::float3{ float(x), float(y), float(x + y) };
        }
        in.upload(stream);
        if (hipEventRecord(begin, raw) != hipSuccess) return 2;
        fk::executeOperations<fk::TransformDPP<>>(stream, fk::PerThreadRead<fk::ND::_2D, fk::float3>::build(in),
                                                  fk::Mul<fk::float3>::build(fk::float3{ 2.f, 3.f, 4.f }),
                                                  fk::Add<fk::float3>::build(fk::float3{ 1.f, 1.f, 1.f }),
                                                  fk::PerThreadWrite<fk::ND::_2D, fk::float3>::build(out));
        if (hipEventRecord(end, raw) != hipSuccess) return 2;
        out.download(stream);
        stream.sync();
        float ms = -1.f;
        if (hipEventElapsedTime(&ms, begin, end) != hipSuccess || !(ms >= 0.f)) return 3;
        for (int y = 0; y < H; ++y) {
            for (int x = 0; x < W; ++x) {
                const fk::float3 got = out.at(fk::Point(x, y));
                if (got.x != 2.f * x + 1.f || got.y != 3.f * y + 1.f || got.z != 4.f * (x + y) + 1.f) {
                    std::printf("mismatch at %d %d\n", x, y);
                    return 1;
                }
            }
        }
        // HIP's own vector types are still there beside the library's (by their template name: the plain names are
        // the library's at global scope as well once its forwarding headers are included)
        const HIP_vector_type<float, 3> theirs(1.f, 2.f, 3.f);
        if (theirs.y != 2.f) return 4;
    }
    (void)hipEventDestroy(begin);
    (void)hipEventDestroy(end);
    (void)hipStreamDestroy(raw);
    std::printf("hip_header_coexistence ok\n");
    return 0;
}

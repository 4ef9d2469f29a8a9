// store_patterns.hip — how fast one MI355X writes the headline's output (five 1920x1080 planes of float3, 124.4 MB), by
// the pattern of the stores alone: kernels that compute nothing and read nothing.  The resize kernel's own pattern (a block
// writes a 64 x 32 pixel tile, a wave eight rows of 768 bytes) is one of them, so its time here is what that kernel could
// reach if its reads and arithmetic were free.
//
// Every kernel is timed over rotating buffers (six of 124.4 MB: more than the 256 MB Infinity Cache holds), as the median of
// nine blocks of 100 launches, each block behind 20 untimed launches, with HIP events on the launch stream.
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops store_patterns.hip -o store_patterns
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <vector>

#define CHECK(call)                                                                                   \
    do {                                                                                              \
        const hipError_t status_ = (call);                                                            \
        if (status_ != hipSuccess) {                                                                  \
            std::printf("%s failed: %s (line %d)\n", #call, hipGetErrorString(status_), __LINE__);    \
            return 1;                                                                                 \
        }                                                                                             \
    } while (0)

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f3 __attribute__((ext_vector_type(3)));
constexpr int W = 1920, H = 1080, PLANES = 5;
constexpr size_t FLOATS = static_cast<size_t>(W) * H * PLANES * 3;

template <bool STREAM, typename V>
__device__ inline void put(V* p, const V v) {
    if (STREAM) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// one 16-byte store per thread, the buffer as one long row: a block writes 4 KiB
template <bool STREAM>
__global__ __launch_bounds__(256) void linear_f4(float* out, float v) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i + 3 < FLOATS) put<STREAM>(reinterpret_cast<f4*>(out + i), f4{v, v, v, v});
}
// one 12-byte store per thread (a float3 pixel), the buffer as one long row
__global__ __launch_bounds__(256) void linear_f3(float* out, float v) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 3;
    if (i + 2 < FLOATS) put<true>(reinterpret_cast<f3*>(out + i), f3{v, v, v});
}
// PER_WAVE 12-byte stores per thread, a wave's pieces of 768 bytes next to each other (same addresses in the same order
// as linear_f3, fewer and longer-lived waves)
template <int PER_WAVE>
__global__ __launch_bounds__(256) void linear_f3_per_wave(float* out, float v) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t block0 = static_cast<size_t>(blockIdx.x) * 256 * PER_WAVE * 3;
#pragma unroll
    for (int u = 0; u < PER_WAVE; ++u) {
        const size_t i = block0 + (static_cast<size_t>(wave * PER_WAVE + u) * 64 + lane) * 3;
        if (i + 2 < FLOATS) put<true>(reinterpret_cast<f3*>(out + i), f3{v, v, v});
    }
}
// the resize kernel's pattern: a block of WAVES waves writes a tile of 64 x (WAVES * ROWS) pixels, a lane one column, a
// wave ROWS rows (768 bytes per row)
template <bool STREAM, int ROWS, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void tiles_f3(float* out, float v) {
    const int x = blockIdx.x * 64 + (threadIdx.x & 63);
    const int y0 = (blockIdx.y * WAVES + (threadIdx.x >> 6)) * ROWS;
    if (x >= W) return;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int y = y0 + r;
        if (y < H) put<STREAM>(reinterpret_cast<f3*>(out + ((static_cast<size_t>(blockIdx.z) * H + y) * W + x) * 3), f3{v, v + 1, v + 2});
    }
}
// the same 64 x 32 tile with 16-byte stores: a wave's eight rows as six stores of 1 KiB (four rows = three stores)
__global__ __launch_bounds__(256) void tiles_f4(float* out, float v) {
    const int lane = threadIdx.x & 63;
    const int y0 = (blockIdx.y * 4 + (threadIdx.x >> 6)) * 8;
    const int x0 = blockIdx.x * 64;
#pragma unroll
    for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int q = 64 * k + lane; // 16-byte piece of the four rows
            const int y = y0 + 4 * g + q / 48;
            if (y < H) put<true>(reinterpret_cast<f4*>(out + ((static_cast<size_t>(blockIdx.z) * H + y) * W + x0) * 3) + q % 48, f4{v, v + 1, v + 2, v});
        }
    }
}
// three float planes per image (a split write), 64 x 32 tiles: one dword per lane and channel ...
__global__ __launch_bounds__(256) void planar_b32(float* out, float v) {
    const int x = blockIdx.x * 64 + (threadIdx.x & 63);
    const int y0 = (blockIdx.y * 4 + (threadIdx.x >> 6)) * 8;
    if (x >= W) return;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int y = y0 + r;
        if (y < H) {
#pragma unroll
            for (int c = 0; c < 3; ++c) put<true>(out + ((static_cast<size_t>(blockIdx.z) * 3 + c) * H + y) * W + x, v);
        }
    }
}
// ... and four rows per 16-byte store: lane = (row of four, four neighbouring pixels)
__global__ __launch_bounds__(256) void planar_b128(float* out, float v) {
    const int lane = threadIdx.x & 63;
    const int x = blockIdx.x * 64 + 4 * (lane & 15);
    const int y0 = (blockIdx.y * 4 + (threadIdx.x >> 6)) * 8;
    if (x >= W) return;
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        const int y = y0 + 4 * g + (lane >> 4);
        if (y < H) {
#pragma unroll
            for (int c = 0; c < 3; ++c) put<true>(reinterpret_cast<f4*>(out + ((static_cast<size_t>(blockIdx.z) * 3 + c) * H + y) * W + x), f4{v, v, v, v});
        }
    }
}
// as many blocks as the device holds at once, each striding over the buffer
__global__ __launch_bounds__(256) void persistent_f4(float* out, float v) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < FLOATS / 4; i += static_cast<size_t>(gridDim.x) * 256) {
        put<true>(reinterpret_cast<f4*>(out) + i, f4{v, v, v, v});
    }
}

template <typename Launch>
float median_us(const Launch& launch, hipStream_t stream) {
    hipEvent_t begin, end;
    if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) return -1.f;
    for (int i = 0; i < 60; ++i) launch(i);
    (void)hipStreamSynchronize(stream);
    std::vector<float> per_launch;
    for (int block = 0; block < 9; ++block) {
        for (int i = 0; i < 20; ++i) launch(i);
        (void)hipEventRecord(begin, stream);
        for (int i = 0; i < 100; ++i) launch(i);
        (void)hipEventRecord(end, stream);
        (void)hipEventSynchronize(end);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, begin, end);
        per_launch.push_back(ms * 10.f);
    }
    (void)hipEventDestroy(begin);
    (void)hipEventDestroy(end);
    std::sort(per_launch.begin(), per_launch.end());
    return per_launch[per_launch.size() / 2];
}

int main() {
    constexpr int BUFFERS = 6;
    float* buffer[BUFFERS];
    for (int i = 0; i < BUFFERS; ++i) CHECK(hipMalloc(&buffer[i], FLOATS * 4));
    hipStream_t stream;
    CHECK(hipStreamCreate(&stream));
    const double megabytes = FLOATS * 4 / 1e6;
    std::printf("%.1f MB per launch, %d rotating buffers\n", megabytes, BUFFERS);
#define RUN(name, kernel, grid, threads)                                                                                                    \
    {                                                                                                                                       \
        const float us = median_us([&](int i) { hipLaunchKernelGGL(kernel, grid, dim3(threads), 0, stream, buffer[i % BUFFERS], 1.5f); }, stream); \
        std::printf("%-58s %6.2f us  %5.2f TB/s\n", name, us, megabytes / us);                                                             \
        std::fflush(stdout);                                                                                                                \
    }
    const unsigned pieces = static_cast<unsigned>((FLOATS / 4 + 255) / 256), pixels = static_cast<unsigned>((FLOATS / 3 + 255) / 256);
    RUN("linear, 16 B per thread, plain stores", (linear_f4<false>), dim3(pieces), 256);
    RUN("linear, 16 B per thread, streaming stores", (linear_f4<true>), dim3(pieces), 256);
    RUN("linear, 12 B per thread", linear_f3, dim3(pixels), 256);
    RUN("linear, 12 B per thread, 2 stores per wave", (linear_f3_per_wave<2>), dim3((pixels + 1) / 2), 256);
    RUN("linear, 12 B per thread, 8 stores per wave", (linear_f3_per_wave<8>), dim3((pixels + 7) / 8), 256);
    RUN("tiles 64 x 4 (1 row per wave)", (tiles_f3<true, 1, 4>), dim3(30, 270, PLANES), 256);
    RUN("tiles 64 x 16 (4 rows per wave)", (tiles_f3<true, 4, 4>), dim3(30, 68, PLANES), 256);
    RUN("tiles 64 x 32 (8 rows per wave): the resize kernel's", (tiles_f3<true, 8, 4>), dim3(30, 34, PLANES), 256);
    RUN("tiles 64 x 32, plain stores", (tiles_f3<false, 8, 4>), dim3(30, 34, PLANES), 256);
    RUN("tiles 64 x 32 by 8 waves of 4 rows", (tiles_f3<true, 4, 8>), dim3(30, 34, PLANES), 512);
    RUN("tiles 64 x 32, six 16-byte stores per wave", tiles_f4, dim3(30, 34, PLANES), 256);
    RUN("tiles 64 x 64 (16 rows per wave)", (tiles_f3<true, 16, 4>), dim3(30, 17, PLANES), 256);
    RUN("three planes, tiles 64 x 32, 4 B per lane and channel", planar_b32, dim3(30, 34, PLANES), 256);
    RUN("three planes, tiles 64 x 32, 16 B per lane and channel", planar_b128, dim3(30, 34, PLANES), 256);
    RUN("2048 resident blocks striding over the buffer", persistent_f4, dim3(2048), 256);
    CHECK(hipDeviceSynchronize());
    for (int i = 0; i < BUFFERS; ++i) CHECK(hipFree(buffer[i]));
    return 0;
}

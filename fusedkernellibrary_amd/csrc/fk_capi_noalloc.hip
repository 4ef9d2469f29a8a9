// fk_capi_noalloc.hip — fk_crop_resize_muls_bgr_tensor_noalloc: the README pipeline for callers that must not allocate.
//
// The chain's job (its plane table and parameters) normally travels in the kernel arguments, or, above the runtime's
// limit for those, in a block that the library allocates per launch.  Here it lies in a fixed array in device memory
// that belongs to the library: `scratch` below, one copy per GPU, held until the process ends.  A call copies the job
// there with a one-block kernel and launches the chain's kernel with the array's address; it allocates and frees
// nothing.  Every call on a GPU uses that GPU's one array, which keeps the last call's job: a call overwrites all of
// its own job before the chain's kernel reads it, in stream order, so nothing has to be cleared, but two calls that
// overlap on one GPU (different streams, or different host threads) race for the array.
#include "fk_capi_readme.h"

#include <mutex>
#include <stdexcept>
#include <string>

using namespace fk;
using namespace fk_capi;

// No header of the HIP runtime is included in a translation unit with this library's kernels (it declares the vector
// types and the launch entry point itself): the one runtime function used here is declared by hand.
extern "C" int hipGetSymbolAddress(void** device_pointer, const void* symbol);
#define HIP_SYMBOL(X) X
#ifndef __align__
#define __align__(n) __attribute__((aligned(n)))
#endif

namespace {
constexpr size_t SCRATCH_BYTES = FK_NOALLOC_MAX_JOB_BYTES;
constexpr int MAX_DEVICES = 64;

static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

// The array's address on the current device.  In host code `scratch` names a host-side stand-in, not device memory:
// the address is asked for once per device, with that device current, and kept.
int scratch_of_current_device(void** out) {
    static std::mutex lock;
    static void* address[MAX_DEVICES] = {};
    int device = 0;
    if (const int rc = fkrt_get_device(&device)) return rc;
    if (device < 0 || device >= MAX_DEVICES) return -1;
    std::lock_guard<std::mutex> hold(lock);
    if (address[device] == nullptr) {
        void* ptr = nullptr;
        if (const int rc = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch))) return rc;
        if (ptr == nullptr) return -1;
        address[device] = ptr;
    }
    *out = address[device];
    return 0;
}

constexpr size_t PLANES = FK_NOALLOC_MAX_PLANES;

template <AspectRatio AR>
int run(Stream& stream, void* block, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, int dw, int dh, const float* bg,
        const float* mul, const float* sub, const float* div, float* out) {
    using PlaneIOp = decltype(readme_plane<AR>(src, w, h, pitch, rects[0], dw, dh, bg, mul, sub, div));
    PlaneIOp planes[PLANES];
    for (int i = 0; i < n; ++i) planes[i] = readme_plane<AR>(src, w, h, pitch, rects[i], dw, dh, bg, mul, sub, div);
    const auto sender = BatchRead<PLANES>::build_first(planes, static_cast<size_t>(n));
    const auto receiver = TensorWrite<float3>::build(view3d<float3>(out, dw, dh, n, 1));
    // a job that outgrows the block must fail the build, not the call
    using Job = decltype(exec::JobOf<std::decay_t<decltype(sender)>, std::decay_t<decltype(receiver)>>::make(sender, receiver));
    static_assert(sizeof(Job) <= SCRATCH_BYTES, "the job of a full batch no longer fits FK_NOALLOC_MAX_JOB_BYTES");
    const bool fits = Executor<TransformDPP<>>::executeOperationsFrom(block, SCRATCH_BYTES, stream, sender, receiver);
    return fits ? FK_OK : unsupported("the chain's parameters exceed the library's fixed device block (or the kernel-argument limit)");
}
} // namespace

extern "C" {

int fk_crop_resize_muls_bgr_tensor_noalloc(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n, int dst_w,
                                           int dst_h, int aspect, const float background[3], const float mul[3], const float sub[3],
                                           const float div[3], float* out, void* stream) {
    if (const int rc = check_readme_arguments(src, src_w, src_h, rects, n, dst_w, dst_h, out)) return rc;
    if (n > static_cast<int>(PLANES)) return unsupported("at most 64 planes per call: the plane table lies in a fixed block of device memory");
    return guarded([&]() -> int {
        void* block = nullptr;
        if (const int rc = scratch_of_current_device(&block)) {
            throw std::runtime_error("the address of the library's device block is not available (hipGetSymbolAddress: " +
                                     std::string(rc > 0 ? fkrt_error_string(rc) : "no address") + ")");
        }
        Stream s(stream);
        switch (aspect) {
        case FK_PRESERVE_AR: return run<AspectRatio::PRESERVE_AR>(s, block, src, src_w, src_h, src_pitch, rects, n, dst_w, dst_h, background, mul, sub, div, out);
        case FK_IGNORE_AR: return run<AspectRatio::IGNORE_AR>(s, block, src, src_w, src_h, src_pitch, rects, n, dst_w, dst_h, background, mul, sub, div, out);
        case FK_PRESERVE_AR_RN_EVEN: return run<AspectRatio::PRESERVE_AR_RN_EVEN>(s, block, src, src_w, src_h, src_pitch, rects, n, dst_w, dst_h, background, mul, sub, div, out);
        case FK_PRESERVE_AR_LEFT: return run<AspectRatio::PRESERVE_AR_LEFT>(s, block, src, src_w, src_h, src_pitch, rects, n, dst_w, dst_h, background, mul, sub, div, out);
        default: return unsupported("unknown aspect-ratio mode");
        }
    });
}

} // extern "C"

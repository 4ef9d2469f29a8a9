// fk_hip_rt.cpp — implementation of the C ABI in include/fk_hip_rt.h on the HIP runtime.
// The only translation unit of the library that includes the HIP runtime's headers (compiled as HIP: it holds one small
// kernel of its own, the kernel-argument probe).
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>

#include "fk_hip_rt.h"
#include "fk_staging_ring.h"

namespace {
inline hipStream_t as_stream(fkrt_stream s) { return static_cast<hipStream_t>(s); }

inline hipMemcpyKind as_kind(int kind) {
    switch (kind) {
    case FKRT_H2D: return hipMemcpyHostToDevice;
    case FKRT_D2H: return hipMemcpyDeviceToHost;
    case FKRT_D2D: return hipMemcpyDeviceToDevice;
    default: return hipMemcpyHostToHost;
    }
}
} // namespace

extern "C" {

int fkrt_device_count(int* count) { return static_cast<int>(hipGetDeviceCount(count)); }
int fkrt_set_device(int device) { return static_cast<int>(hipSetDevice(device)); }
int fkrt_get_device(int* device) { return static_cast<int>(hipGetDevice(device)); }

int fkrt_stream_create(fkrt_stream* out) {
    hipStream_t s = nullptr;
    const hipError_t e = hipStreamCreate(&s); // default priority only
    *out = s;
    return static_cast<int>(e);
}
int fkrt_stream_destroy(fkrt_stream s) { return static_cast<int>(hipStreamDestroy(as_stream(s))); }
int fkrt_stream_sync(fkrt_stream s) { return static_cast<int>(hipStreamSynchronize(as_stream(s))); }

int fkrt_malloc(void** out, size_t bytes) { return static_cast<int>(hipMalloc(out, bytes)); }
int fkrt_malloc_pitch(void** out, size_t* pitch, size_t width_bytes, size_t height) {
    return static_cast<int>(hipMallocPitch(out, pitch, width_bytes, height));
}
int fkrt_free(void* p) { return static_cast<int>(hipFree(p)); }
int fkrt_malloc_host(void** out, size_t bytes) { return static_cast<int>(hipHostMalloc(out, bytes, hipHostMallocDefault)); }
int fkrt_free_host(void* p) { return static_cast<int>(hipHostFree(p)); }

int fkrt_memcpy_async(void* dst, const void* src, size_t bytes, int kind, fkrt_stream s) {
    return static_cast<int>(hipMemcpyAsync(dst, src, bytes, as_kind(kind), as_stream(s)));
}
int fkrt_memcpy2d_async(void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t width_bytes,
                        size_t height, int kind, fkrt_stream s) {
    return static_cast<int>(
        hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width_bytes, height, as_kind(kind), as_stream(s)));
}
int fkrt_memset_async(void* dst, int value, size_t bytes, fkrt_stream s) {
    return static_cast<int>(hipMemsetAsync(dst, value, bytes, as_stream(s)));
}

int fkrt_launch(const void* kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block_x,
                unsigned block_y, unsigned block_z, void** args, size_t lds_bytes, fkrt_stream s) {
    if (kernel == nullptr || grid_x == 0 || grid_y == 0 || grid_z == 0 || block_x == 0 || block_y == 0 ||
        block_z == 0 || static_cast<size_t>(block_x) * block_y * block_z > 1024) {
        return static_cast<int>(hipErrorInvalidConfiguration);
    }
    const hipError_t e =
        hipLaunchKernel(kernel, dim3(grid_x, grid_y, grid_z), dim3(block_x, block_y, block_z), args, lds_bytes, as_stream(s));
    if (e != hipSuccess) return static_cast<int>(e);
    return static_cast<int>(hipGetLastError());
}

// Staged parameter blocks go through a small ring of slots that this layer owns, each a pinned host buffer and a device
// buffer of the same size (64 KiB, grown when a larger block comes).  The caller's block is copied into the slot's host
// buffer on the spot (so it may go out of scope at once), and from there to the slot's device buffer with a true
// asynchronous copy from pinned memory, ordered in the stream like the kernel that reads it.  The slot is leased to the
// caller until fkrt_params_release, which the caller issues after enqueueing that kernel and which records the slot's
// event behind it; a slot is taken again only after that event has completed (fk_staging_ring.h has the state machine).
// Nothing is allocated per launch (a stream-ordered allocation and its release cost more than the copy).  Slots belong
// to the device that was current when their buffers were made.
namespace {
int ring_current_device(int* device) { return static_cast<int>(hipGetDevice(device)); }
int ring_alloc_slot(void** host, void** device, void** event, size_t bytes) {
    hipEvent_t ev = nullptr;
    hipError_t e = hipHostMalloc(host, bytes, hipHostMallocPortable);
    if (e == hipSuccess) e = hipMalloc(device, bytes);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    *event = ev;
    return static_cast<int>(e);
}
void ring_free_slot(void* host, void* device, void* event) {
    if (host != nullptr) (void)hipHostFree(host);
    if (device != nullptr) (void)hipFree(device);
    if (event != nullptr) (void)hipEventDestroy(static_cast<hipEvent_t>(event));
}
int ring_copy_to_device(void* device, const void* host, size_t bytes, void* stream) {
    return static_cast<int>(hipMemcpyAsync(device, host, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
}
int ring_event_record(void* event, void* stream) {
    return static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}
int ring_event_sync(void* event) { return static_cast<int>(hipEventSynchronize(static_cast<hipEvent_t>(event))); }
int ring_event_done(void* event, bool* done) {
    const hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
    *done = e == hipSuccess;
    return e == hipSuccess || e == hipErrorNotReady ? 0 : static_cast<int>(e);
}
fkrt::StagingRing& staging_ring() {
    // lives until the process ends; its buffers are released with the process
    static fkrt::StagingRing ring(fkrt::RingBackend{ ring_current_device, ring_alloc_slot, ring_free_slot, ring_copy_to_device, ring_event_record,
                                                     ring_event_sync, ring_event_done });
    return ring;
}
int ring_status(int status) {
    if (status == fkrt::StagingRing::RING_FULL) return static_cast<int>(hipErrorNotReady); // eight blocks leased and none released in time
    if (status == fkrt::StagingRing::NOT_A_LEASED_SLOT) return static_cast<int>(hipErrorInvalidValue);
    return status;
}
} // namespace

int fkrt_params_upload(void** device_out, const void* host_src, size_t bytes, fkrt_stream s) {
    if (device_out == nullptr || host_src == nullptr) return static_cast<int>(hipErrorInvalidValue);
    return ring_status(staging_ring().upload(device_out, host_src, bytes, s));
}
int fkrt_params_release(void* device_params, fkrt_stream s) { return ring_status(staging_ring().release(device_params, s)); }

// ---- how large a by-value kernel argument may be ---------------------------------------------------------------------
// The HIP documentation promises 4 KiB of kernel arguments.  This runtime passes far more (64 KiB arrived intact, also with
// thousands of launches in flight on two streams), and the library's jobs of up to 32 KiB rely on it.  Rather than trust a
// version, the first call asks the device: one block receives a 32 KiB argument filled with a known pattern and sums it up
// with position weights; anything but the expected sum (or a launch that fails) makes the limit the documented 4 KiB, and
// larger jobs then go through fkrt_params_upload.  The result lands in a device variable of this library and is read back
// with a synchronous copy: nothing is allocated, but the first call must not be made while a stream is being captured.
namespace {
constexpr unsigned PROBE_DWORDS = 32768 / 4;
struct ProbeBlock {
    unsigned int w[PROBE_DWORDS];
};
__device__ unsigned int fkrt_probe_sum;
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void fkrt_probe_kernarg(const ProbeBlock block) {
    unsigned int sum = 0u;
    for (unsigned i = __builtin_amdgcn_workitem_id_x(); i < PROBE_DWORDS; i += 256u) sum += block.w[i] * (i + 1u);
    atomicAdd(&fkrt_probe_sum, sum);
}
bool large_kernel_arguments_arrive() {
    static ProbeBlock block; // (32 KiB: not on the stack)
    unsigned int expected = 0u;
    for (unsigned i = 0; i < PROBE_DWORDS; ++i) {
        block.w[i] = (i * 2654435761u) ^ 0x9E3779B9u;
        expected += block.w[i] * (i + 1u);
    }
    const unsigned int zero = 0u;
    if (hipMemcpyToSymbol(HIP_SYMBOL(fkrt_probe_sum), &zero, sizeof(zero)) != hipSuccess) return false;
    void* argv[] = { &block };
    if (hipLaunchKernel(reinterpret_cast<const void*>(&fkrt_probe_kernarg), dim3(1, 1, 1), dim3(256, 1, 1), argv, 0, nullptr) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    unsigned int got = 0u;
    if (hipMemcpyFromSymbol(&got, HIP_SYMBOL(fkrt_probe_sum), sizeof(got)) != hipSuccess) return false; // (waits for the kernel)
    return got == expected;
}
} // namespace

size_t fkrt_max_kernarg_bytes(void) {
    static const size_t limit = [] {
        const char* env = std::getenv("FK_MAX_KERNARG_BYTES");
        if (env != nullptr) {
            const long v = std::strtol(env, nullptr, 10);
            if (v >= 256) return static_cast<size_t>(v);
        }
        return large_kernel_arguments_arrive() ? static_cast<size_t>(32768) : static_cast<size_t>(4096);
    }();
    return limit;
}

int fkrt_last_error(void) { return static_cast<int>(hipGetLastError()); }
const char* fkrt_error_string(int status) { return hipGetErrorString(static_cast<hipError_t>(status)); }

int fkrt_event_create(void** out) {
    hipEvent_t ev = nullptr;
    const hipError_t e = hipEventCreate(&ev);
    *out = ev;
    return static_cast<int>(e);
}
int fkrt_event_destroy(void* ev) { return static_cast<int>(hipEventDestroy(static_cast<hipEvent_t>(ev))); }
int fkrt_event_record(void* ev, fkrt_stream s) {
    return static_cast<int>(hipEventRecord(static_cast<hipEvent_t>(ev), as_stream(s)));
}
int fkrt_event_sync(void* ev) { return static_cast<int>(hipEventSynchronize(static_cast<hipEvent_t>(ev))); }
int fkrt_event_elapsed_ms(float* ms, void* start, void* stop) {
    return static_cast<int>(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}

} // extern "C"

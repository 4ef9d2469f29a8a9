// fk_hip_rt.cpp — implementation of the C ABI in include/fk_hip_rt.h on the HIP runtime.
// The only translation unit of the library that includes the HIP host API.
#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <cstring>
#include <mutex>

#include "fk_hip_rt.h"

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
// asynchronous copy from pinned memory, ordered in the stream like the kernel that reads it.  fkrt_params_release, which
// the caller issues after enqueueing that kernel, records the slot's event behind it; a slot is taken again only after
// that event has completed.  Nothing is allocated per launch (a stream-ordered allocation and its release cost more
// than the copy).  Slots belong to the device that was current when their buffers were made.
namespace {
struct StagingRing {
    static constexpr int SLOTS = 8;
    static constexpr size_t MIN_BYTES = 64 * 1024;
    std::mutex lock;
    void* host[SLOTS] = {};
    void* device[SLOTS] = {};
    size_t bytes[SLOTS] = {};
    int owner[SLOTS] = {}; // device of the slot's buffers
    hipEvent_t done[SLOTS] = {};
    bool in_flight[SLOTS] = {};
    int next = 0;
};
StagingRing& staging_ring() {
    static StagingRing ring; // lives until the process ends; its buffers are released with the process
    return ring;
}
} // namespace

int fkrt_params_upload(void** device_out, const void* host_src, size_t bytes, fkrt_stream s) {
    StagingRing& ring = staging_ring();
    std::lock_guard<std::mutex> hold(ring.lock);
    const int slot = ring.next;
    ring.next = (ring.next + 1) % StagingRing::SLOTS;
    int current = 0;
    hipError_t e = hipGetDevice(&current);
    if (e != hipSuccess) return static_cast<int>(e);
    if (ring.in_flight[slot]) { // the kernel that last read this slot must have finished
        e = hipEventSynchronize(ring.done[slot]);
        if (e != hipSuccess) return static_cast<int>(e);
        ring.in_flight[slot] = false;
    }
    if (ring.bytes[slot] < bytes || ring.owner[slot] != current || ring.done[slot] == nullptr) {
        if (ring.host[slot] != nullptr) (void)hipHostFree(ring.host[slot]);
        if (ring.device[slot] != nullptr) (void)hipFree(ring.device[slot]);
        if (ring.done[slot] != nullptr) (void)hipEventDestroy(ring.done[slot]);
        ring.host[slot] = ring.device[slot] = nullptr;
        ring.done[slot] = nullptr;
        ring.bytes[slot] = 0;
        const size_t wanted = bytes > StagingRing::MIN_BYTES ? bytes : StagingRing::MIN_BYTES;
        e = hipHostMalloc(&ring.host[slot], wanted, hipHostMallocPortable);
        if (e == hipSuccess) e = hipMalloc(&ring.device[slot], wanted);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&ring.done[slot], hipEventDisableTiming);
        if (e != hipSuccess) return static_cast<int>(e);
        ring.bytes[slot] = wanted;
        ring.owner[slot] = current;
    }
    std::memcpy(ring.host[slot], host_src, bytes);
    e = hipMemcpyAsync(ring.device[slot], ring.host[slot], bytes, hipMemcpyHostToDevice, as_stream(s));
    if (e != hipSuccess) return static_cast<int>(e);
    // (should the caller never release it, the slot still waits for this copy before it is used again)
    e = hipEventRecord(ring.done[slot], as_stream(s));
    if (e != hipSuccess) return static_cast<int>(e);
    ring.in_flight[slot] = true;
    *device_out = ring.device[slot];
    return 0;
}
int fkrt_params_release(void* device_params, fkrt_stream s) {
    StagingRing& ring = staging_ring();
    std::lock_guard<std::mutex> hold(ring.lock);
    for (int slot = 0; slot < StagingRing::SLOTS; ++slot) {
        if (ring.device[slot] == device_params && device_params != nullptr) {
            return static_cast<int>(hipEventRecord(ring.done[slot], as_stream(s))); // behind the kernel that reads the slot
        }
    }
    return static_cast<int>(hipErrorInvalidValue);
}

size_t fkrt_max_kernarg_bytes(void) {
    static const size_t limit = [] {
        const char* env = std::getenv("FK_MAX_KERNARG_BYTES");
        if (env != nullptr) {
            const long v = std::strtol(env, nullptr, 10);
            if (v >= 256) return static_cast<size_t>(v);
        }
        // Arguments of up to 64 KiB were verified to arrive intact on ROCm 7.2 / gfx950, also with thousands of launches
        // in flight on two streams; half of that is used.
        return static_cast<size_t>(32768);
    }();
    return limit;
}

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

/* fk_hip_rt.h — the thin C ABI between the fk:: C++17 template layer and the HIP runtime.
 *
 * Everything the templates need from the GPU runtime goes through these entry points: streams, device and
 * pinned-host allocation, asynchronous copies, and the kernel launch.  They stand where the reference calls the
 * CUDA runtime directly:
 *   stream create/sync/destroy      core/execution_model/stream.h:52-109      (cudaStreamCreate/Synchronize/Destroy)
 *   device / pitched / pinned alloc core/data/ptr_nd.h:47-126,153-201         (cudaMalloc, cudaMallocPitch, cudaMallocHost)
 *   free                            core/data/ptr_nd.h:203-249                (cudaFree, cudaFreeHost)
 *   async 1D / 2D copies            core/data/ptr_nd.h:252-268                (cudaMemcpyAsync, cudaMemcpy2DAsync)
 *   kernel launch + error check     core/execution_model/executors.h:262-287  (<<<grid, block, 0, stream>>>, cudaGetLastError)
 *   error text                      core/utils/utils.h:95-147                 (gpuErrchk / cudaGetErrorString)
 *
 * All functions return 0 on success or the HIP error code; fkrt_error_string() gives its text.  Pointers and
 * sizes only: no C++ types cross this boundary.  Implemented in fusedkernellibrary_amd/csrc/fk_hip_rt.cpp
 * (libfk_hip_rt.so).
 */
#ifndef FK_HIP_RT_H
#define FK_HIP_RT_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* fkrt_stream; /* a hipStream_t; NULL is the default stream */

enum { FKRT_H2D = 1, FKRT_D2H = 2, FKRT_D2D = 3, FKRT_H2H = 0 };

int fkrt_device_count(int* count);
int fkrt_set_device(int device);
int fkrt_get_device(int* device);

int fkrt_stream_create(fkrt_stream* out);
int fkrt_stream_destroy(fkrt_stream s);
int fkrt_stream_sync(fkrt_stream s);

int fkrt_malloc(void** out, size_t bytes);
/* rows of `width_bytes` padded to the runtime's preferred pitch, returned in *pitch */
int fkrt_malloc_pitch(void** out, size_t* pitch, size_t width_bytes, size_t height);
int fkrt_free(void* p);
int fkrt_malloc_host(void** out, size_t bytes); /* pinned */
int fkrt_free_host(void* p);

int fkrt_memcpy_async(void* dst, const void* src, size_t bytes, int kind, fkrt_stream s);
int fkrt_memcpy2d_async(void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t width_bytes,
                        size_t height, int kind, fkrt_stream s);
int fkrt_memset_async(void* dst, int value, size_t bytes, fkrt_stream s);

/* Launch the kernel whose host-side handle is `kernel` (the address of a __global__ function taken in host code).
 * `args` holds one pointer per kernel parameter.  Returns the launch status (hipGetLastError after the launch). */
int fkrt_launch(const void* kernel, unsigned grid_x, unsigned grid_y, unsigned grid_z, unsigned block_x,
                unsigned block_y, unsigned block_z, void** args, size_t lds_bytes, fkrt_stream s);

/* Stream-ordered staging of a parameter block that is too large for the kernel-argument segment: copies `bytes`
 * from host memory into a device buffer that stays valid until the work enqueued on `s` up to the matching
 * fkrt_params_release has run; call that after enqueueing the kernel that reads the block.  `host_src` is copied before
 * the call returns and may be released at once.  The buffers come from a ring of eight slots that this layer owns (a
 * pinned host buffer and a device buffer each): nothing is allocated per call.  A slot is leased to its caller from the
 * upload to the release and is handed out again only when the kernel behind the release has finished: an upload that
 * finds no slot free waits for that kernel on the host (without blocking other callers of this layer), and an upload
 * that finds all eight slots leased waits up to two seconds for a release and then fails with the runtime's "not ready"
 * status rather than overwrite a block whose kernel has not run.  A block that is never released keeps its slot. */
int fkrt_params_upload(void** device_out, const void* host_src, size_t bytes, fkrt_stream s);
int fkrt_params_release(void* device_params, fkrt_stream s);

/* Largest by-value kernel-argument block, in bytes, that launches are allowed to use: 32768 where the device is seen to
 * receive such a block intact (the first call launches a one-block probe kernel whose 32 KiB argument it sums up; it
 * allocates nothing but synchronises, so it must not be made during stream capture), else the 4096 that HIP documents.
 * The environment variable FK_MAX_KERNARG_BYTES (>= 256) overrides both. */
size_t fkrt_max_kernarg_bytes(void);

/* Status of the last runtime call of this thread, cleared by the call (hipGetLastError; CUDA: cudaGetLastError, used by the
 * reference's gpuErrchk after every launch, core/utils/utils.h:95-147). */
int fkrt_last_error(void);

const char* fkrt_error_string(int status);

/* Event pair timing on a stream, for benchmarks: returns elapsed milliseconds between two recorded events. */
int fkrt_event_create(void** out);
int fkrt_event_destroy(void* ev);
int fkrt_event_record(void* ev, fkrt_stream s);
int fkrt_event_sync(void* ev);
int fkrt_event_elapsed_ms(float* ms, void* start, void* stop);

#ifdef __cplusplus
}
#endif
#endif

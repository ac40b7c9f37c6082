/*
 * rafhip_device.h -- C ABI over the HIP runtime calls that a `rocm` DeviceAPI for awslabs/raf needs:
 * the ROCm counterpart of CUDADeviceAPI (src/device_api/cuda/cuda.cc:25-248), whose virtual
 * interface is include/raf/device_api.h:19-177.  Plain C, pointers and sizes only; streams and
 * events cross as void*.  Every function returns a rafhip_status (rafhip_optim.h; 0 = success) and
 * leaves its message in rafhip_last_error().  None of them launches a kernel.
 */
#ifndef RAFHIP_DEVICE_H_
#define RAFHIP_DEVICE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* cuda.cc:49-52: make `device_id` current for the calling thread. */
int rafhip_dev_set(int32_t device_id);

/* cuda.cc:37-47: synchronous allocation on the current device / free.  nbytes == 0 gives NULL. */
int rafhip_dev_alloc(int64_t nbytes, void** out);
int rafhip_dev_free(void* ptr);

/* cuda.cc:54-95: stream-ordered allocation from the device's default memory pool, whose release
 * threshold is raised to "never give memory back" on first use; if the pool is exhausted the call
 * synchronises the stream once and retries.  Free is stream-ordered too. */
int rafhip_dev_alloc_async(int32_t device_id, int64_t nbytes, void* stream, void** out);
int rafhip_dev_free_async(void* ptr, void* stream);

/* cuda.cc:64-73: bytes handed out by, and bytes reserved in, the device's default memory pool. */
int rafhip_dev_pool_size(int32_t device_id, int64_t* used_out, int64_t* reserved_out);

/* cuda.cc:112-157, :236-245: contiguous copies.  stream == NULL makes the copy synchronous;
 * host<->device copies are only truly asynchronous from pinned host memory. */
typedef enum rafhip_copy_kind {
  RAFHIP_COPY_H2H = 0,
  RAFHIP_COPY_H2D = 1,
  RAFHIP_COPY_D2H = 2,
  RAFHIP_COPY_D2D = 3
} rafhip_copy_kind;
int rafhip_dev_memcpy(void* dst, const void* src, int64_t nbytes, int32_t kind, void* stream);
int rafhip_dev_memcpy_peer(void* dst, int32_t dst_device, const void* src, int32_t src_device,
                           int64_t nbytes, void* stream);

/* cuda.cc:159-171: streams (default priority). */
int rafhip_dev_stream_create(int32_t device_id, void** stream_out);
int rafhip_dev_stream_destroy(int32_t device_id, void* stream);

/* cuda.cc:183-207: events.  flags are hipEventDefault (0), hipEventBlockingSync (1),
 * hipEventDisableTiming (2), numerically the CUDA values the reference's callers pass. */
int rafhip_dev_event_create(int32_t device_id, uint32_t flags, void** event_out);
int rafhip_dev_event_destroy(int32_t device_id, void* event);
int rafhip_dev_event_elapsed_ms(void* start_event, void* end_event, float* ms_out);
int rafhip_dev_event_record(void* event, void* stream);

/* cuda.cc:209-232: ordering and host-side waits. */
int rafhip_dev_stream_wait_event(void* stream, void* event);
int rafhip_dev_sync_device(int32_t device_id);
int rafhip_dev_sync_stream(void* stream);
int rafhip_dev_sync_event(void* event);

#ifdef __cplusplus
}
#endif
#endif /* RAFHIP_DEVICE_H_ */

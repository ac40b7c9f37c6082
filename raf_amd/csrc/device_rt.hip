// HIP runtime calls behind a `rocm` DeviceAPI: the C ABI of rafhip_device.h.  Counterpart of the
// reference's CUDADeviceAPI (src/device_api/cuda/cuda.cc:25-248); host code only, no kernels.
#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>

#include "rafhip_device.h"
#include "status.h"

using namespace rafhip;

namespace {

// The device's default memory pool with its release threshold raised once, so that freed blocks
// stay cached for later stream-ordered allocations (cuda.cc:54-62).
int default_pool(int32_t device_id, hipMemPool_t* pool) {
  RAFHIP_HIP_TRY(hipDeviceGetDefaultMemPool(pool, device_id));
  static std::mutex mu;
  static uint64_t raised = 0;  // bit per device
  std::lock_guard<std::mutex> lock(mu);
  if (device_id < 64 && !(raised & (1ull << device_id))) {
    uint64_t keep = UINT64_MAX;
    RAFHIP_HIP_TRY(hipMemPoolSetAttribute(*pool, hipMemPoolAttrReleaseThreshold, &keep));
    raised |= 1ull << device_id;
  }
  return RAFHIP_OK;
}

}  // namespace

extern "C" {

int rafhip_dev_set(int32_t device_id) {
  clear_error();
  RAFHIP_HIP_TRY(hipSetDevice(device_id));
  return RAFHIP_OK;
}

int rafhip_dev_alloc(int64_t nbytes, void** out) {
  clear_error();
  if (!out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_alloc: out is NULL");
  *out = nullptr;
  if (nbytes < 0) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_alloc: nbytes = %lld < 0", (long long)nbytes);
  if (nbytes == 0) return RAFHIP_OK;
  RAFHIP_HIP_TRY(hipMalloc(out, (size_t)nbytes));
  return RAFHIP_OK;
}

int rafhip_dev_free(void* ptr) {
  clear_error();
  if (!ptr) return RAFHIP_OK;
  RAFHIP_HIP_TRY(hipFree(ptr));
  return RAFHIP_OK;
}

int rafhip_dev_alloc_async(int32_t device_id, int64_t nbytes, void* stream, void** out) {
  clear_error();
  if (!out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_alloc_async: out is NULL");
  *out = nullptr;
  if (nbytes < 0)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_alloc_async: nbytes = %lld < 0", (long long)nbytes);
  if (nbytes == 0) return RAFHIP_OK;
  hipMemPool_t pool;
  if (int st = default_pool(device_id, &pool)) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipMallocFromPoolAsync(out, (size_t)nbytes, pool, s);
  if (e != hipSuccess) {  // let pending frees on the stream land, then try once more (cuda.cc:80-88)
    (void)hipGetLastError();
    RAFHIP_HIP_TRY(hipStreamSynchronize(s));
    RAFHIP_HIP_TRY(hipMallocFromPoolAsync(out, (size_t)nbytes, pool, s));
  }
  return RAFHIP_OK;
}

int rafhip_dev_free_async(void* ptr, void* stream) {
  clear_error();
  if (!ptr) return RAFHIP_OK;
  RAFHIP_HIP_TRY(hipFreeAsync(ptr, static_cast<hipStream_t>(stream)));
  return RAFHIP_OK;
}

int rafhip_dev_pool_size(int32_t device_id, int64_t* used_out, int64_t* reserved_out) {
  clear_error();
  if (!used_out || !reserved_out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_pool_size: null output");
  hipMemPool_t pool;
  RAFHIP_HIP_TRY(hipDeviceGetDefaultMemPool(&pool, device_id));
  uint64_t used = 0, reserved = 0;
  RAFHIP_HIP_TRY(hipMemPoolGetAttribute(pool, hipMemPoolAttrReservedMemCurrent, &reserved));
  RAFHIP_HIP_TRY(hipMemPoolGetAttribute(pool, hipMemPoolAttrUsedMemCurrent, &used));
  *used_out = (int64_t)used;
  *reserved_out = (int64_t)reserved;
  return RAFHIP_OK;
}

int rafhip_dev_memcpy(void* dst, const void* src, int64_t nbytes, int32_t kind, void* stream) {
  clear_error();
  if (nbytes < 0) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_memcpy: nbytes = %lld < 0", (long long)nbytes);
  if (nbytes == 0) return RAFHIP_OK;
  if (!dst || !src) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_memcpy: null pointer");
  hipMemcpyKind k;
  switch (kind) {
    case RAFHIP_COPY_H2H:
      std::memcpy(dst, src, (size_t)nbytes);  // cuda.cc:126-129
      return RAFHIP_OK;
    case RAFHIP_COPY_H2D:
      k = hipMemcpyHostToDevice;
      break;
    case RAFHIP_COPY_D2H:
      k = hipMemcpyDeviceToHost;
      break;
    case RAFHIP_COPY_D2D:
      k = hipMemcpyDeviceToDevice;
      break;
    default:
      return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_memcpy: kind = %d", kind);
  }
  if (stream)
    RAFHIP_HIP_TRY(hipMemcpyAsync(dst, src, (size_t)nbytes, k, static_cast<hipStream_t>(stream)));
  else
    RAFHIP_HIP_TRY(hipMemcpy(dst, src, (size_t)nbytes, k));
  return RAFHIP_OK;
}

int rafhip_dev_memcpy_peer(void* dst, int32_t dst_device, const void* src, int32_t src_device,
                           int64_t nbytes, void* stream) {
  clear_error();
  if (nbytes < 0) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_memcpy_peer: nbytes < 0");
  if (nbytes == 0) return RAFHIP_OK;
  if (!dst || !src) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_memcpy_peer: null pointer");
  RAFHIP_HIP_TRY(hipMemcpyPeerAsync(dst, dst_device, src, src_device, (size_t)nbytes,
                                    static_cast<hipStream_t>(stream)));
  return RAFHIP_OK;
}

int rafhip_dev_stream_create(int32_t device_id, void** stream_out) {
  clear_error();
  if (!stream_out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_stream_create: stream_out is NULL");
  *stream_out = nullptr;
  RAFHIP_HIP_TRY(hipSetDevice(device_id));
  hipStream_t s = nullptr;
  RAFHIP_HIP_TRY(hipStreamCreate(&s));
  *stream_out = s;
  return RAFHIP_OK;
}

int rafhip_dev_stream_destroy(int32_t device_id, void* stream) {
  clear_error();
  if (!stream) return RAFHIP_OK;
  RAFHIP_HIP_TRY(hipSetDevice(device_id));
  RAFHIP_HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return RAFHIP_OK;
}

int rafhip_dev_event_create(int32_t device_id, uint32_t flags, void** event_out) {
  clear_error();
  if (!event_out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_event_create: event_out is NULL");
  *event_out = nullptr;
  RAFHIP_HIP_TRY(hipSetDevice(device_id));
  hipEvent_t e = nullptr;
  RAFHIP_HIP_TRY(hipEventCreateWithFlags(&e, flags));
  *event_out = e;
  return RAFHIP_OK;
}

int rafhip_dev_event_destroy(int32_t device_id, void* event) {
  clear_error();
  if (!event) return RAFHIP_OK;
  RAFHIP_HIP_TRY(hipSetDevice(device_id));
  RAFHIP_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return RAFHIP_OK;
}

int rafhip_dev_event_elapsed_ms(void* start_event, void* end_event, float* ms_out) {
  clear_error();
  if (!start_event || !end_event || !ms_out)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_event_elapsed_ms: null argument");
  RAFHIP_HIP_TRY(hipEventElapsedTime(ms_out, static_cast<hipEvent_t>(start_event),
                                     static_cast<hipEvent_t>(end_event)));
  return RAFHIP_OK;
}

int rafhip_dev_event_record(void* event, void* stream) {
  clear_error();
  if (!event) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_event_record: event is NULL");
  RAFHIP_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return RAFHIP_OK;
}

int rafhip_dev_stream_wait_event(void* stream, void* event) {
  clear_error();
  if (!event) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_dev_stream_wait_event: event is NULL");
  RAFHIP_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
  return RAFHIP_OK;
}

int rafhip_dev_sync_device(int32_t device_id) {
  clear_error();
  RAFHIP_HIP_TRY(hipSetDevice(device_id));
  RAFHIP_HIP_TRY(hipDeviceSynchronize());
  return RAFHIP_OK;
}

int rafhip_dev_sync_stream(void* stream) {
  clear_error();
  RAFHIP_HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return RAFHIP_OK;
}

int rafhip_dev_sync_event(void* event) {
  clear_error();
  if (!event) return fail(RAFHIP_ERR_INVALID_ARG, "Cannot sync a null event");  // cuda.cc:229
  RAFHIP_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
  return RAFHIP_OK;
}

}  // extern "C"

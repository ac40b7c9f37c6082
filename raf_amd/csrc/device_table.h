// A table of per-tensor records (pointers, sizes) that lives in device memory and has to follow
// the pointers the caller passes with every call.  Shared by the multi-tensor plans (LANS, SGD,
// fuse/defuse): the records go through a pinned staging buffer and an asynchronous copy on the
// call's stream, and a call whose records equal the ones sent last time sends nothing -- a
// training loop updates the same buffers every step.
//
// Rec must be trivially copyable with every byte initialised (records are compared with memcmp).
#pragma once
#include <hip/hip_runtime.h>

#include <cstring>
#include <type_traits>
#include <vector>

namespace rafhip {

template <typename Rec>
class RecordUploader {
  static_assert(std::is_trivially_copyable<Rec>::value, "records are copied and compared bytewise");

 public:
  RecordUploader() = default;
  RecordUploader(const RecordUploader&) = delete;
  RecordUploader& operator=(const RecordUploader&) = delete;
  ~RecordUploader() { release(); }

  // `device_table` must hold `count` records and outlive this object.
  hipError_t init(Rec* device_table, size_t count) {
    release();
    device_ = device_table;
    count_ = count;
    if (count == 0) return hipSuccess;
    hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&staging_), sizeof(Rec) * count,
                                 hipHostMallocDefault);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&staging_free_, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&handover_, hipEventDisableTiming);
    if (e != hipSuccess) release();
    // Its final size from the start: sync() swaps it with the caller's vector, so neither side
    // ever has to grow (a step allocates nothing, host memory included).
    if (e == hipSuccess) last_sent_.assign(count, Rec{});
    return e;
  }

  void release() {
    // An upload that is still reading the staging buffer must finish before the buffer goes away.
    if (staging_free_ && sent_once_) (void)hipEventSynchronize(staging_free_);
    if (staging_free_) (void)hipEventDestroy(staging_free_);
    if (handover_) (void)hipEventDestroy(handover_);
    if (staging_) (void)hipHostFree(staging_);
    staging_free_ = nullptr;
    handover_ = nullptr;
    staging_ = nullptr;
    sent_once_ = false;
    last_sent_.clear();
  }

  // Makes the device table equal to `recs` for work enqueued on `s` after this call.  Takes the
  // vector's contents (swap) when it uploads.
  hipError_t sync(std::vector<Rec>& recs, hipStream_t s) {
    if (count_ == 0) return hipSuccess;
    if (sent_once_ && std::memcmp(last_sent_.data(), recs.data(), sizeof(Rec) * count_) == 0)
      return follow(s);
    return upload(recs, s);
  }

  // The records are the ones sent last time (the caller knows, or sync() compared them) and the
  // next reader of the table runs on `s`.  When that is another stream than the last one, `s` is
  // ordered behind everything enqueued there so far: behind the upload, and behind the kernels
  // that read the table, so that the table has a single line of readers and writers however the
  // caller moves between streams.  A stream under graph capture is left alone (events of other
  // streams cannot be recorded into it): capture after a warm-up call on that stream has completed.
  hipError_t follow(hipStream_t s) {
    if (count_ == 0 || !sent_once_ || s == last_stream_) return hipSuccess;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone) return hipSuccess;
    hipError_t e = order_behind_last_stream(s);
    if (e != hipSuccess) return e;
    last_stream_ = s;
    return hipSuccess;
  }

 private:
  // Everything enqueued on last_stream_ so far happens before what is enqueued on `s` from now on.
  // If the old stream no longer exists its work has completed or is completed by the fallback.
  hipError_t order_behind_last_stream(hipStream_t s) {
    hipError_t e = hipEventRecord(handover_, last_stream_);
    if (e == hipSuccess) return hipStreamWaitEvent(s, handover_, 0);
    (void)hipGetLastError();
    return hipDeviceSynchronize();
  }

  hipError_t upload(std::vector<Rec>& recs, hipStream_t s) {
    const size_t bytes = sizeof(Rec) * count_;
    if (sent_once_) {
      // The previous upload may still be reading the staging buffer ...
      hipError_t e = hipEventSynchronize(staging_free_);
      if (e != hipSuccess) return e;
      // ... and kernels launched earlier on another stream may still be reading the device table.
      if (s != last_stream_) {
        e = order_behind_last_stream(s);
        if (e != hipSuccess) return e;
      }
    }
    std::memcpy(staging_, recs.data(), bytes);
    hipError_t e = hipMemcpyAsync(device_, staging_, bytes, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipEventRecord(staging_free_, s);
    if (e != hipSuccess) return e;
    last_sent_.swap(recs);
    sent_once_ = true;
    last_stream_ = s;
    return hipSuccess;
  }

  Rec* device_ = nullptr;
  size_t count_ = 0;
  Rec* staging_ = nullptr;  // pinned
  hipEvent_t staging_free_ = nullptr;  // recorded after the last upload was enqueued
  hipEvent_t handover_ = nullptr;      // orders a new stream behind the previous one
  hipStream_t last_stream_ = nullptr;  // the stream of the last upload or reader
  std::vector<Rec> last_sent_;
  bool sent_once_ = false;
};

// CUs x 8 workgroups: enough resident wavefronts to cover HBM latency on every CU; grid-stride
// loops do the rest.
inline int streaming_grid_cap() {
  static int cap = [] {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
          v > 0)
        cus = v;
    }
    return cus * 8;
  }();
  return cap;
}

}  // namespace rafhip

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
    if (staging_) (void)hipHostFree(staging_);
    staging_free_ = nullptr;
    staging_ = nullptr;
    sent_once_ = false;
    last_sent_.clear();
  }

  // Makes the device table equal to `recs` for work enqueued on `s` after this call.  Takes the
  // vector's contents (swap) when it uploads.
  hipError_t sync(std::vector<Rec>& recs, hipStream_t s) {
    if (count_ == 0) return hipSuccess;
    const size_t bytes = sizeof(Rec) * count_;
    if (sent_once_ && std::memcmp(last_sent_.data(), recs.data(), bytes) == 0) {
      // Same records, but a different stream than the one that carried them: order this stream
      // behind the upload unless it has landed already.  A stream under graph capture is left
      // alone (event queries are not allowed there): capture after a warm-up call has completed.
      if (s != last_stream_) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capturing) != hipSuccess) (void)hipGetLastError();
        if (capturing == hipStreamCaptureStatusNone) {
          if (hipEventQuery(staging_free_) == hipErrorNotReady) {
            (void)hipGetLastError();  // "not ready" is an answer, not a failure
            hipError_t e = hipStreamWaitEvent(s, staging_free_, 0);
            if (e != hipSuccess) return e;
          }
          last_stream_ = s;
        }
      }
      return hipSuccess;
    }
    // The previous upload may still be reading the staging buffer.
    if (sent_once_) {
      hipError_t e = hipEventSynchronize(staging_free_);
      if (e != hipSuccess) return e;
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

 private:
  Rec* device_ = nullptr;
  size_t count_ = 0;
  Rec* staging_ = nullptr;  // pinned
  hipEvent_t staging_free_ = nullptr;  // recorded after the last upload was enqueued
  hipStream_t last_stream_ = nullptr;  // the stream that upload went to
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

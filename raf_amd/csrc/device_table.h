// Tables of per-tensor records (pointers, sizes) that live in device memory and have to follow the
// pointers the caller passes with every call.  Shared by the multi-tensor plans (LANS, SGD,
// fuse/defuse).
//
// A plan keeps a few device tables ("slots"), each with the records it was last sent.  A call
// whose records equal those of a slot uses that slot and sends nothing: a training loop that
// updates the same buffers every step, an executor whose gradient list alternates between two
// allocations, two models of one architecture stepped in turn -- all settle on one slot per
// distinct pointer set.  Other records replace the least recently used slot: they go through that
// slot's own pinned staging buffer and an asynchronous copy on the call's stream, so the host
// waits only for the upload that used the same slot kSlots uploads ago, i.e. in practice never
// (it can run kSlots - 1 steps ahead of the device even when the pointers change at every call).
//
// Stream capture: a call made while its stream is being captured into a graph leaves kernel nodes
// that read a slot's device table (and, if the records were new, a copy node that reads the slot's
// staging buffer) at every replay.  Such a slot is held from then on: it is never chosen for other
// records, so a graph keeps finding the pointers it was captured with for as long as the plan
// lives.  When every slot is held a call with yet other records is refused.
//
// Rec must be trivially copyable with every byte initialised (records are compared with memcmp).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <type_traits>
#include <vector>

#include "status.h"

namespace rafhip {

template <typename Rec>
class RecordTables {
  static_assert(std::is_trivially_copyable<Rec>::value, "records are copied and compared bytewise");

 public:
  static constexpr int kSlots = 4;

  RecordTables() = default;
  RecordTables(const RecordTables&) = delete;
  RecordTables& operator=(const RecordTables&) = delete;
  ~RecordTables() { release(); }

  // Device and pinned host memory for kSlots tables of `count` records each.
  hipError_t init(size_t count) {
    release();
    count_ = count;
    if (count == 0) return hipSuccess;
    stride_ = (sizeof(Rec) * count + 255) / 256 * 256;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&device_), stride_ * kSlots);
    if (e == hipSuccess)
      e = hipHostMalloc(reinterpret_cast<void**>(&staging_), stride_ * kSlots, hipHostMallocDefault);
    for (int k = 0; e == hipSuccess && k < kSlots; ++k) {
      Slot& sl = slots_[k];
      sl.device = reinterpret_cast<Rec*>(device_ + stride_ * (size_t)k);
      sl.staging = reinterpret_cast<Rec*>(staging_ + stride_ * (size_t)k);
      e = hipEventCreateWithFlags(&sl.staging_free, hipEventDisableTiming);
      // Its final size from the start: sync() swaps it with the caller's vector, so neither side
      // ever has to grow (a step allocates nothing, host memory included).
      if (e == hipSuccess) sl.sent.assign(count, Rec{});
    }
    if (e == hipSuccess) e = hipEventCreateWithFlags(&handover_, hipEventDisableTiming);
    if (e != hipSuccess) release();
    return e;
  }

  void release() {
    for (Slot& sl : slots_) {
      // An upload that is still reading the staging buffer must finish before the buffer goes away.
      if (sl.staging_free && sl.valid) (void)hipEventSynchronize(sl.staging_free);
      if (sl.staging_free) (void)hipEventDestroy(sl.staging_free);
      sl = Slot{};
    }
    if (handover_) (void)hipEventDestroy(handover_);
    if (staging_) (void)hipHostFree(staging_);
    if (device_) (void)hipFree(device_);
    handover_ = nullptr;
    staging_ = nullptr;
    device_ = nullptr;
    current_ = -1;
    refused_ = false;
    used_once_ = false;
    last_stream_ = nullptr;
    clock_ = 0;
    uploads_ = 0;
  }

  // The device table that equals `recs` for work enqueued on `s` after this call.  Takes the
  // vector's contents (swap) when it uploads.
  hipError_t sync(std::vector<Rec>& recs, hipStream_t s, const Rec** table_out) {
    *table_out = nullptr;
    if (count_ == 0) return hipSuccess;
    const size_t bytes = sizeof(Rec) * count_;
    int hit = -1;
    // The slot used last first: nearly every call finds its records there.  A slot with other
    // pointers differs within its first record, so a miss costs next to nothing.
    if (current_ >= 0 && std::memcmp(slots_[current_].sent.data(), recs.data(), bytes) == 0) hit = current_;
    for (int k = 0; hit < 0 && k < kSlots; ++k)
      if (k != current_ && slots_[k].valid && std::memcmp(slots_[k].sent.data(), recs.data(), bytes) == 0)
        hit = k;
    if (hit >= 0) {
      current_ = hit;
      return use(slots_[hit], s, table_out);
    }
    int victim = -1;
    for (int k = 0; k < kSlots; ++k) {
      if (slots_[k].held) continue;
      if (!slots_[k].valid) {
        victim = k;
        break;
      }
      if (victim < 0 || slots_[k].last_use < slots_[victim].last_use) victim = k;
    }
    refused_ = victim < 0;
    if (refused_) return hipErrorNotSupported;
    Slot& sl = slots_[victim];
    if (sl.valid) {
      // The slot's previous upload may still be reading its staging buffer.
      hipError_t e = hipEventSynchronize(sl.staging_free);
      if (e != hipSuccess) return e;
    }
    // Kernels launched earlier on another stream may still be reading the slot's device table.
    hipError_t e = use(sl, s, table_out);
    if (e != hipSuccess) return e;
    std::memcpy(sl.staging, recs.data(), bytes);
    e = hipMemcpyAsync(sl.device, sl.staging, bytes, hipMemcpyHostToDevice, s);
    // Under capture the copy is a graph node, not an upload in flight: there is nothing to wait
    // for, and the slot (held now) is not written again.
    if (e == hipSuccess && !sl.held) e = hipEventRecord(sl.staging_free, s);
    if (e != hipSuccess) return e;
    sl.sent.swap(recs);
    sl.valid = true;
    ++uploads_;
    current_ = victim;
    return hipSuccess;
  }

  // The table of the last sync() again (the caller knows that its records are the ones it passed
  // then), its next reader running on `s`.
  hipError_t follow(hipStream_t s, const Rec** table_out) {
    *table_out = nullptr;
    if (count_ == 0) return hipSuccess;
    if (current_ < 0) return hipErrorInvalidValue;
    return use(slots_[current_], s, table_out);
  }

  // Uploads made so far (what a caller with steady pointers expects to stop growing).
  int64_t uploads() const { return uploads_; }
  // Whether the last sync() failed because every slot is held by a captured graph.
  bool refused() const { return refused_; }

 private:
  struct Slot {
    Rec* device = nullptr;
    Rec* staging = nullptr;              // pinned
    hipEvent_t staging_free = nullptr;   // recorded after the slot's last upload was enqueued
    std::vector<Rec> sent;               // what the device table holds
    bool valid = false;
    bool held = false;                   // read by a captured graph: keeps its records for good
    uint64_t last_use = 0;
  };

  // The next writer or reader of a table runs on `s`.  When that is another stream than the one
  // of the plan's previous call, `s` is ordered behind everything enqueued there so far: behind
  // the uploads, and behind the kernels that read a table or wrote the caller's workspace.  The
  // calls of one plan thus form a single line however the caller moves between streams (one step
  // at a time per plan is the contract; this makes it hold on the device too).  A stream under
  // graph capture is left alone (events of other streams cannot be recorded into it; the graph's
  // launches are ordered by whoever replays it) and the slot it reads becomes a held one.
  hipError_t use(Slot& sl, hipStream_t s, const Rec** table_out) {
    sl.last_use = ++clock_;
    *table_out = sl.device;
    if (capturing(s)) {
      sl.held = true;
      return hipSuccess;
    }
    if (!used_once_) {
      used_once_ = true;
      last_stream_ = s;
      return hipSuccess;
    }
    if (s == last_stream_) return hipSuccess;
    hipError_t e = order_behind(last_stream_, s);
    if (e != hipSuccess) return e;
    last_stream_ = s;
    return hipSuccess;
  }

  static bool capturing(hipStream_t s) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &status) != hipSuccess) {
      (void)hipGetLastError();  // e.g. the legacy default stream while another stream captures
      return false;
    }
    return status != hipStreamCaptureStatusNone;
  }

  // Everything enqueued on `before` so far happens before what is enqueued on `s` from now on.
  // If the old stream no longer exists its work has completed or is completed by the fallback.
  hipError_t order_behind(hipStream_t before, hipStream_t s) {
    hipError_t e = hipEventRecord(handover_, before);
    if (e == hipSuccess) return hipStreamWaitEvent(s, handover_, 0);
    (void)hipGetLastError();
    return hipDeviceSynchronize();
  }

  size_t count_ = 0;
  size_t stride_ = 0;       // bytes from one slot's table to the next (256-byte multiple)
  char* device_ = nullptr;  // kSlots tables
  char* staging_ = nullptr;
  Slot slots_[kSlots];
  hipEvent_t handover_ = nullptr;  // orders a new stream behind a slot's previous one
  hipStream_t last_stream_ = nullptr;  // the stream of the plan's last call
  bool used_once_ = false;
  int current_ = -1;               // the slot of the last sync()
  bool refused_ = false;
  uint64_t clock_ = 0;
  int64_t uploads_ = 0;
};

// sync() for the entry points: a HIP failure or a refusal becomes a status code with a message.
template <typename Rec>
int sync_tables(const char* who, RecordTables<Rec>& tables, std::vector<Rec>& recs, hipStream_t s,
                const Rec** table_out) {
  const hipError_t e = tables.sync(recs, s, table_out);
  if (e == hipSuccess) return RAFHIP_OK;
  if (tables.refused())
    return fail(RAFHIP_ERR_UNSUPPORTED,
                "%s: all %d pointer tables of the plan are held by captured graphs; these pointers are "
                "new to it (use another plan for them)",
                who, RecordTables<Rec>::kSlots);
  return fail(RAFHIP_ERR_HIP, "%s: sending the pointer table failed: %s", who, hipGetErrorString(e));
}

// HIP refuses a launch of 2^32 threads or more; with the 256-thread workgroups used throughout
// that is a grid of 2^24.  One-workgroup-per-item launches are capped here and stride over the rest.
constexpr int64_t kMaxGridBlocks = (1 << 24) - 1;

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

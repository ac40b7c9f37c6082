// Host side of the multi-tensor LANS step: the plan (tensor table, work lists, timing events) and
// the C-ABI entry points.  The plan plays the part of the reference's LansImpl constructor
// (src/op/dialect/cuda/lans.cc:27-83) and rafhip_lans_step that of LansImpl::Execute (:92-131),
// without its blocking copy of `step` to the host and without its per-element scratch buffer.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <array>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <memory>
#include <mutex>
#include <new>
#include <vector>

#include "device_table.h"
#include "lans_kernels.h"
#include "status.h"

using namespace rafhip;

static_assert(RecordTables<TensorRec>::kSlots == RAFHIP_TABLE_SLOTS, "header and table cache disagree");

// Scratch memory of rafhip_lans_step_noalloc, the step for callers that cannot allocate: the
// step scalars, per-tensor statistics, chunk partial sums and ticket words that the other step
// entry points find in the caller's workspace.  Every GPU the library runs on holds its own copy
// of the array, at its own address, until the process ends.  In host code the name below is only
// a handle for hipGetSymbolAddress; the kernels receive the resolved address as an argument.
static __device__ __align__(256) unsigned char scratch[RAFHIP_LANS_STATIC_SCRATCH_BYTES];

namespace {

constexpr int64_t kAlign = 256;
inline int64_t align_up(int64_t x) { return (x + kAlign - 1) / kAlign * kAlign; }

struct WorkspaceLayout {
  int64_t scalars_off, stats_off, partials_off, sync_off, total;
};

WorkspaceLayout make_layout(int32_t n_tensors, int64_t n_chunks) {
  WorkspaceLayout l;
  l.scalars_off = 0;
  l.stats_off = align_up((int64_t)sizeof(StepScalars));
  l.partials_off = l.stats_off + align_up((int64_t)sizeof(TensorStats) * n_tensors);
  l.sync_off = l.partials_off + align_up((int64_t)sizeof(double) * kPartialSlots * n_chunks);
  l.total = l.sync_off + align_up((int64_t)sizeof(SyncHeader));
  return l;
}

inline int64_t chunks_of(int64_t numel) {
  const int64_t c = chunk_elems_for(numel);
  return (numel + c - 1) / c;
}
inline int64_t units_a_of(int64_t numel) {
  const int64_t u = (int64_t)kChunksPerA * chunk_elems_for(numel);
  return (numel + u - 1) / u;
}

// Default size of a cache group in elements (measured optimum on MI355X for BERT-large and
// GPT-2-1.5B lists): pass C of a group finds the 12 bytes per element of w, m, v that pass B of the
// same group left in the 256 MB Infinity Cache one round earlier.
constexpr int64_t kDefaultGroupElems = 13 * 1000 * 1000;
// Lists at least this long run pipelined by default; shorter ones are launch- and latency-bound
// and do better with one launch per pass (measured on prefixes of the BERT-large list: phased 9 %
// faster at 26 M elements, 2 % at 51 M, pipelined 1-3 % faster at 65 M, 4 % at 80 M).
constexpr int64_t kPipelinedFromElems = 64 * 1024 * 1024;
// Lists whose g, w, m, v together stay under this many bytes fit in the cache: temporal accesses.
constexpr int64_t kResidentBytes = 192LL << 20;

// From this many elements on a tensor counts as long when the persistent kernel's occupancy is chosen.
constexpr int64_t kLongTensorElems = 6 * 1000 * 1000;

// Slices per round in which passes B and C alternate (measured on MI355X: 4 to 16 are within
// 0.1 % of each other on the BERT-large list, 1 is 3 % slower).
constexpr int kDefaultRoundSlices = 8;

inline WorkItem make_item(int32_t tensor, uint32_t phase, int64_t chunk, uint32_t flags = 0) {
  return WorkItem{tensor, (phase << kPhaseShift) | flags | (uint32_t)chunk};
}

// A tensor whose w, m, v alone exceed the 256 MB Infinity Cache cannot keep anything there between
// its passes; handled like the others it would only flush the groups that can.
constexpr int64_t kStreamedTensorFromElems = (256LL << 20) / 12;

// Resident workgroups of the persistent kernel on a 256-CU device, for the host-only queries.
constexpr int kDefaultPipelineGrid = 256 * 3;

// The pipelined work list.
//
// Cached groups.  Tensors are packed, in list order, into groups of at most group_elems elements.
// "Round" r holds pass A of group r, then pass B of group r-1 and pass C of group r-2 in
// alternating slices, so that a group's gradient survives in the cache from pass A to pass B and
// its w, m, v from pass B to pass C.  (Merging all three so that they advance together was
// measured too: items then sit right behind the ones they depend on and the kernel waits more.)
//
// Streamed tensors.  A tensor too large for the cache forms no group.  Its three passes depend on
// each other as a whole, so on its own it would run them one after the other, each bound by HBM
// alone while the cache and the rest of the fabric idle -- at the head of a BERT list (the word
// embedding comes first) that was a tenth of the step.  Its items are marked streaming and spread
// over the whole list of rounds in proportion to the bytes they move: the tensor then trickles
// through HBM underneath the cached groups' traffic.
//
// Invariant the kernel's waits rely on, per tensor: pass-A units, then its finish-A item, then
// pass-B chunks, then its finish-B item, then pass-C chunks.
struct PipelineCut {
  int64_t group_elems;
  int64_t stream_from;  // tensors from this many elements on are streamed
  int round_slices;
  int hold_items;       // < 0: 4 x grid
};

std::vector<WorkItem> build_pipeline(int32_t n, const int64_t* numel, const PipelineCut& cut,
                                     int grid = kDefaultPipelineGrid) {
  const int64_t group_elems = cut.group_elems;
  struct Group {
    std::vector<WorkItem> a, b, c;
  };
  std::vector<Group> groups;
  std::vector<WorkItem> streamed;  // every streamed tensor: A units, finish A, B chunks, finish B, C chunks
  std::vector<int64_t> streamed_bytes;  // what each of those items moves (for the proportional merge)
  const int64_t stream_from = cut.stream_from;
  std::vector<int32_t> cached_tensors;
  for (int32_t t = 0; t < n; ++t) {
    if (numel[t] == 0) continue;
    const int64_t nc = chunks_of(numel[t]);
    const int64_t ce = chunk_elems_for(numel[t]);
    if (numel[t] >= stream_from) {
      auto len_of = [&](int64_t idx, int64_t unit) { return std::min(unit, numel[t] - idx * unit); };
      for (int64_t u = 0; u < units_a_of(numel[t]); ++u) {
        streamed.push_back(make_item(t, kPhaseA, u, kStreamBit));
        streamed_bytes.push_back(4 * len_of(u, ce * kChunksPerA));
      }
      streamed.push_back(make_item(t, kPhaseFinishA, 0));
      streamed_bytes.push_back(0);
      for (int64_t c = 0; c < nc; ++c) {
        streamed.push_back(make_item(t, kPhaseB, c, kStreamBit));
        streamed_bytes.push_back(16 * len_of(c, ce));
      }
      streamed.push_back(make_item(t, kPhaseFinishB, 0));
      streamed_bytes.push_back(0);
      for (int64_t c = 0; c < nc; ++c) {
        streamed.push_back(make_item(t, kPhaseC, c, kStreamBit));
        streamed_bytes.push_back(28 * len_of(c, ce));
      }
      continue;
    }
    cached_tensors.push_back(t);
  }

  // (Small groups at either end, to fill and drain the pipeline faster, were measured and are
  // slower: a short round puts pass-B items right behind the finish items they wait for.)
  int64_t in_group = 0;
  for (const int32_t t : cached_tensors) {
    const int64_t nc = chunks_of(numel[t]);
    if (groups.empty() || (in_group > 0 && in_group + numel[t] > group_elems)) {
      groups.emplace_back();
      in_group = 0;
    }
    in_group += numel[t];
    Group& g = groups.back();
    if (nc == 1) {
      g.a.push_back(make_item(t, kPhaseWhole, 0));  // one workgroup does all three passes
      continue;
    }
    for (int64_t u = 0; u < units_a_of(numel[t]); ++u) g.a.push_back(make_item(t, kPhaseA, u));
    for (int64_t c = 0; c < nc; ++c) {
      g.b.push_back(make_item(t, kPhaseB, c));
      g.c.push_back(make_item(t, kPhaseC, c));
    }
    g.a.push_back(make_item(t, kPhaseFinishA, 0));  // after the tensor's chunks of the pass
    g.b.push_back(make_item(t, kPhaseFinishB, 0));
  }
  std::vector<WorkItem> cached;
  const int64_t ng = (int64_t)groups.size();
  // Within a round, passes B and C alternate in slices: pass C then follows more closely behind
  // the pass B that loaded its group one round earlier, which shortens the time a group has to
  // survive in the cache (3 % on the BERT-large list; a dependency never crosses: the C items of
  // a round belong to an earlier group than its B items).
  static const std::vector<WorkItem> none;
  const size_t slices = (size_t)cut.round_slices;
  for (int64_t r = 0; r < ng + 2; ++r) {
    const std::vector<WorkItem>& b = (r >= 1 && r - 1 < ng) ? groups[r - 1].b : none;
    const std::vector<WorkItem>& c = (r >= 2 && r - 2 < ng) ? groups[r - 2].c : none;
    if (r < ng) cached.insert(cached.end(), groups[r].a.begin(), groups[r].a.end());
    for (size_t k = 0; k < slices; ++k) {
      cached.insert(cached.end(), b.begin() + b.size() * k / slices, b.begin() + b.size() * (k + 1) / slices);
      cached.insert(cached.end(), c.begin() + c.size() * k / slices, c.begin() + c.size() * (k + 1) / slices);
    }
  }

  // Merge the two streams so that each has moved the same share of its bytes at every point.
  std::vector<WorkItem> out;
  if (streamed.empty()) {
    out.swap(cached);
  } else if (cached.empty()) {
    out.swap(streamed);
  } else {
    auto bytes_of = [&](const WorkItem& it) -> int64_t {
      const int64_t ne = numel[it.tensor];
      const int64_t ce = chunk_elems_for(ne);
      const int64_t c = it.chunk_phase & kChunkMask;
      switch (it.chunk_phase >> kPhaseShift) {
        case kPhaseA: return 4 * std::min(ce * kChunksPerA, ne - c * ce * kChunksPerA);
        case kPhaseB: return 16 * std::min(ce, ne - c * ce);
        case kPhaseC: return 28 * std::min(ce, ne - c * ce);
        case kPhaseWhole: return 48 * ne;
        default: return 0;
      }
    };
    const int hold_items = cut.hold_items >= 0 ? cut.hold_items : 4 * grid;
    double total_c = 0, total_s = 0;
    for (const WorkItem& it : cached) total_c += (double)bytes_of(it);
    for (int64_t b : streamed_bytes) total_s += (double)b;
    if (total_c <= 0) total_c = 1;
    if (total_s <= 0) total_s = 1;
    out.reserve(cached.size() + streamed.size());
    size_t i = 0, j = 0;
    double left_c = total_c, left_s = total_s;  // bytes still to be placed
    double base_c = total_c, base_s = total_s;  // ... when the pacing was last set
    // What follows a finish item of the streamed tensor waits for it, and it waits for the last
    // items of the pass before it, which have only just been drawn: the streamed stream pauses for
    // a few items per workgroup of cached work, or most workgroups would sit in that wait.  After
    // the pause the two streams are paced by what each has left, so that the streamed one does
    // not catch up in one burst (which would be a stretch of pure HBM traffic again).
    int64_t hold = 0;
    while (i < cached.size() || j < streamed.size()) {
      if (hold == 0) {
        base_c = left_c > 0 ? left_c : 1;
        base_s = left_s > 0 ? left_s : 1;
        hold = -1;
      }
      const bool take_streamed =
          j < streamed.size() &&
          (i >= cached.size() || (hold < 0 && (base_s - left_s) / base_s <= (base_c - left_c) / base_c));
      if (take_streamed) {
        left_s -= (double)streamed_bytes[j];
        const uint32_t kind = streamed[j].chunk_phase >> kPhaseShift;
        if (kind == kPhaseFinishA || kind == kPhaseFinishB) hold = hold_items > 0 ? (int64_t)hold_items : 0;
        out.push_back(streamed[j++]);
      } else {
        left_c -= (double)bytes_of(cached[i]);
        if (hold > 0) --hold;
        out.push_back(cached[i++]);
      }
    }
  }
  return out;
}

// The settings in force for a plan: the built-in defaults, overridden by the three user-facing
// environment variables, overridden by what the caller set in rafhip_lans_plan_options.
struct ResolvedOptions {
  int schedule;  // -1: by list length
  PipelineCut cut;
  int blocks_per_cu;  // 0: by the list
  int64_t resident_bytes;
  int apply_slice_shift;
  uint32_t spin_limit;
};

ResolvedOptions resolve_options(const rafhip_lans_plan_options* o) {
  ResolvedOptions r;
  r.schedule = -1;
  r.cut = PipelineCut{kDefaultGroupElems, kStreamedTensorFromElems, kDefaultRoundSlices, -1};
  r.blocks_per_cu = 0;
  r.resident_bytes = kResidentBytes;
  r.apply_slice_shift = 10;
  // Polls a wait of the pipelined kernel may take before it gives up and raises the error word:
  // with a sleep of a few hundred cycles per poll the default is seconds, far beyond any real
  // dependency latency.
  r.spin_limit = 1u << 22;
  if (const char* e = std::getenv("RAFHIP_LANS_SCHEDULE")) {
    if (!std::strcmp(e, "phased")) r.schedule = RAFHIP_LANS_PHASED;
    if (!std::strcmp(e, "pipelined")) r.schedule = RAFHIP_LANS_PIPELINED;
  }
  if (const char* e = std::getenv("RAFHIP_LANS_GROUP_ELEMS")) {
    const long long v = std::atoll(e);
    if (v > 0) r.cut.group_elems = v;
  }
  if (const char* e = std::getenv("RAFHIP_LANS_SPIN_LIMIT")) {
    const long long v = std::atoll(e);
    if (v >= 0 && v <= 0xFFFFFFFFll) r.spin_limit = (uint32_t)v;
  }
  if (!o) return r;
  if (o->schedule == RAFHIP_LANS_PHASED || o->schedule == RAFHIP_LANS_PIPELINED) r.schedule = o->schedule;
  if (o->group_elements > 0) r.cut.group_elems = o->group_elements;
  if (o->round_slices > 0) r.cut.round_slices = o->round_slices < 4096 ? o->round_slices : 4096;
  if (o->stream_from_elements > 0) r.cut.stream_from = o->stream_from_elements;
  if (o->stream_hold_items >= 0) r.cut.hold_items = o->stream_hold_items;
  if (o->blocks_per_cu > 0) r.blocks_per_cu = o->blocks_per_cu;
  if (o->resident_mib >= 0) r.resident_bytes = (int64_t)o->resident_mib << 20;
  if (o->apply_slice_shift == 0 || (o->apply_slice_shift >= 10 && o->apply_slice_shift < kChunkShift))
    r.apply_slice_shift = o->apply_slice_shift;
  if (o->spin_limit >= 0 && o->spin_limit <= 0xFFFFFFFFll) r.spin_limit = (uint32_t)o->spin_limit;
  return r;
}

// The address of `scratch` on a device, resolved once per device with that device current.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// `device` must be the current device.  Returns nullptr (and leaves the reason in *err) on failure.
void* static_scratch_of(int device, hipError_t* err) {
  *err = hipSuccess;
  if (device < 0 || device >= kMaxDevices) {
    *err = hipErrorInvalidDevice;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      *err = e != hipSuccess ? e : hipErrorInvalidSymbol;
      return nullptr;
    }
    g_scratch_ptr[device] = ptr;
  }
  return g_scratch_ptr[device];
}

}  // namespace

struct rafhip_lans_plan {
  int device = 0;
  int n_cus = 256;
  int32_t n_tensors = 0;
  int32_t grad_dtype = RAFHIP_F32;
  int32_t schedule = RAFHIP_LANS_PHASED;
  int64_t n_chunks = 0;
  int64_t total_elements = 0;
  uint32_t spin_limit = 1u << 22;
  int64_t resident_bytes = kResidentBytes;  // lists up to this size use temporal accesses throughout
  int apply_slice_shift = 10;  // phased schedule, streaming lists: log2 of the last pass's slice
  bool short_tensors_only = false;  // no tensor has more than kInlineFinishChunks chunks
  uint32_t n_pipeline_items = 0;
  unsigned pipeline_grid = 0;
  std::vector<int64_t> numel;
  std::vector<int32_t> first_chunk;
  WorkspaceLayout ws{};

  // Work lists in one allocation: [chunk items][pipeline items][pass-A items].
  void* d_tables = nullptr;
  WorkItem* d_items = nullptr;
  WorkItem* d_items_a = nullptr;
  int64_t n_items_a = 0;
  WorkItem* d_pipeline = nullptr;
  uint64_t* d_trace = nullptr;  // diagnostics, only with RAFHIP_LANS_TRACE=1
  // One word of pinned, device-visible host memory: the persistent kernel raises it when a bounded
  // wait runs out, and the next call on the plan reports it without any copy or synchronisation.
  uint32_t* host_error = nullptr;
  uint32_t* host_error_dev = nullptr;  // the device's address of the same word

  RecordTables<TensorRec> tensors;  // device tensor tables; a step whose pointers are known sends nothing
  std::vector<TensorRec> recs;        // this call's records, built in place: a step allocates nothing
  // rafhip_lans_plan_bind: records of tensors that stay where they are, built and checked once.
  std::vector<TensorRec> bound;
  bool bound_valid = false;
  bool bound_on_device = false;  // the table used last holds `bound` (no other step intervened)
  int32_t bound_p_dtype = RAFHIP_F16;
  // rafhip_lans_plan_set_dynamic_scale: optional device words read by every kernel of a step.
  const float* unscale_dev = nullptr;
  const float* found_inf_dev = nullptr;

  // This device's address of the static scratch array (rafhip_lans_step_noalloc), resolved when the
  // plan is made; nullptr with the reason in static_scratch_error if that failed.
  void* static_scratch = nullptr;
  hipError_t static_scratch_error = hipSuccess;

  // Optional per-kernel timing: slots x 6 events.
  std::vector<std::array<hipEvent_t, 6>> timing;
  std::vector<int> timing_marks;  // which events the slot's last step recorded (each costs microseconds)
  int64_t steps_done = 0;
};

namespace {

void destroy_timing(rafhip_lans_plan* p) {
  for (auto& slot : p->timing)
    for (auto& e : slot)
      if (e) (void)hipEventDestroy(e);
  p->timing.clear();
  p->timing_marks.clear();
}

void free_plan(rafhip_lans_plan* p) {
  if (!p) return;
  destroy_timing(p);
  p->tensors.release();
  if (p->d_tables) (void)hipFree(p->d_tables);
  if (p->d_trace) (void)hipFree(p->d_trace);
  if (p->host_error) (void)hipHostFree(p->host_error);
  delete p;
}

inline bool aligned_to(const void* p, uintptr_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

int validate_list(const char* who, int32_t n_tensors, const int64_t* numel) {
  if (n_tensors < 0) return fail(RAFHIP_ERR_INVALID_ARG, "%s: n_tensors = %d < 0", who, n_tensors);
  if (n_tensors > 0 && !numel) return fail(RAFHIP_ERR_INVALID_ARG, "%s: numel is NULL", who);
  int64_t chunks = 0;
  for (int32_t t = 0; t < n_tensors; ++t) {
    if (numel[t] < 0)
      return fail(RAFHIP_ERR_INVALID_ARG, "%s: numel[%d] = %lld < 0", who, t, (long long)numel[t]);
    chunks += chunks_of(numel[t]);
    if (chunks >= (int64_t)kChunkMask)
      return fail(RAFHIP_ERR_UNSUPPORTED, "%s: too many chunks (more than 2^28)", who);
  }
  return RAFHIP_OK;
}

int lans_step_impl(rafhip_lans_plan* plan, const void* const* g, float* const* w, float* const* m,
                   float* const* v, void* const* p, int32_t p_dtype, const float* step_dev,
                   int32_t step_host, const rafhip_lans_hparams* hp, void* workspace,
                   int64_t workspace_bytes, void* stream);

}  // namespace

extern "C" {

void rafhip_lans_default_hparams(rafhip_lans_hparams* hp) {
  if (!hp) return;
  // python/raf/optim/lans.py:44-55; True -> 1 as the schema's int fields receive them
  hp->learning_rate = 1e-3f;
  hp->beta1 = 0.9f;
  hp->beta2 = 0.999f;
  hp->eps = 1e-6f;
  hp->bias_correction = 1;
  hp->weight_decay = 0.01f;
  hp->grad_averaging = 1;
  hp->mode = 1;
  hp->normalize_grad = 1;
  hp->grad_unscale = 1.0f;
}

int32_t rafhip_lans_chunk_elements(int64_t numel) { return chunk_elems_for(numel); }
int32_t rafhip_lans_pass_a_unit_elements(int64_t numel) { return kChunksPerA * chunk_elems_for(numel); }

int rafhip_lans_query_layout(int32_t n_tensors, const int64_t* numel, int64_t* n_chunks_out,
                             int64_t* workspace_bytes_out) {
  clear_error();
  if (int st = validate_list("rafhip_lans_query_layout", n_tensors, numel)) return st;
  int64_t chunks = 0;
  for (int32_t t = 0; t < n_tensors; ++t) chunks += chunks_of(numel[t]);
  if (n_chunks_out) *n_chunks_out = chunks;
  if (workspace_bytes_out) *workspace_bytes_out = make_layout(n_tensors, chunks).total;
  return RAFHIP_OK;
}

void rafhip_lans_default_plan_options(rafhip_lans_plan_options* o) {
  if (!o) return;
  o->schedule = -1;
  o->round_slices = 0;
  o->group_elements = 0;
  o->stream_from_elements = 0;
  o->stream_hold_items = -1;
  o->blocks_per_cu = 0;
  o->resident_mib = -1;
  o->apply_slice_shift = -1;
  o->spin_limit = -1;
}

int rafhip_lans_pipeline_order_with(int32_t n_tensors, const int64_t* numel,
                                    const rafhip_lans_plan_options* options, int32_t* triples_out,
                                    int64_t capacity, int64_t* n_items_out) {
  clear_error();
  const char* who = "rafhip_lans_pipeline_order";
  if (int st = validate_list(who, n_tensors, numel)) return st;
  if (!n_items_out) return fail(RAFHIP_ERR_INVALID_ARG, "%s: n_items_out is NULL", who);
  return guarded(who, [&]() -> int {
    const std::vector<WorkItem> items = build_pipeline(n_tensors, numel, resolve_options(options).cut);
    *n_items_out = (int64_t)items.size();
    if (triples_out) {
      if (capacity < (int64_t)items.size())
        return fail(RAFHIP_ERR_INVALID_ARG, "%s: capacity %lld < %zu items", who, (long long)capacity,
                    items.size());
      for (size_t i = 0; i < items.size(); ++i) {
        const uint32_t cp = items[i].chunk_phase;
        triples_out[3 * i + 0] = (int32_t)(cp >> kPhaseShift) + ((cp & kStreamBit) ? 8 : 0);
        triples_out[3 * i + 1] = items[i].tensor;
        triples_out[3 * i + 2] = (int32_t)(cp & kChunkMask);
      }
    }
    return RAFHIP_OK;
  });
}

int rafhip_lans_pipeline_order(int32_t n_tensors, const int64_t* numel, int64_t group_elements,
                               int32_t* triples_out, int64_t capacity, int64_t* n_items_out) {
  rafhip_lans_plan_options o;
  rafhip_lans_default_plan_options(&o);
  o.group_elements = group_elements > 0 ? group_elements : kDefaultGroupElems;
  return rafhip_lans_pipeline_order_with(n_tensors, numel, &o, triples_out, capacity, n_items_out);
}

int rafhip_lans_plan_create(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                            rafhip_lans_plan** out_plan) {
  return rafhip_lans_plan_create_with(n_tensors, numel, grad_dtype, nullptr, out_plan);
}

int rafhip_lans_plan_create_with(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                                 const rafhip_lans_plan_options* options,
                                 rafhip_lans_plan** out_plan) {
  clear_error();
  if (!out_plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_create: out_plan is NULL");
  *out_plan = nullptr;
  if (int st = validate_list("rafhip_lans_plan_create", n_tensors, numel)) return st;
  if (grad_dtype != RAFHIP_F32 && grad_dtype != RAFHIP_F16 && grad_dtype != RAFHIP_BF16)
    return fail(RAFHIP_ERR_UNSUPPORTED,
                "rafhip_lans_plan_create: gradient dtype %d (LANS takes fp32 weights and state; "
                "gradients may be fp32, fp16 or bf16)",
                grad_dtype);

  return guarded("rafhip_lans_plan_create", [&]() -> int {
    std::unique_ptr<rafhip_lans_plan, void (*)(rafhip_lans_plan*)> p(new rafhip_lans_plan(), free_plan);
    p->n_tensors = n_tensors;
    p->grad_dtype = grad_dtype;
    p->numel.assign(numel, numel + n_tensors);
    p->first_chunk.resize(n_tensors);
    int64_t chunks = 0, total = 0, longest = 0;
    for (int32_t t = 0; t < n_tensors; ++t) {
      p->first_chunk[t] = (int32_t)chunks;
      chunks += chunks_of(numel[t]);
      longest = std::max(longest, chunks_of(numel[t]));
      total += numel[t];
    }
    const ResolvedOptions opt = resolve_options(options);
    p->short_tensors_only = longest <= kInlineFinishChunks;
    p->resident_bytes = opt.resident_bytes;
    p->apply_slice_shift = opt.apply_slice_shift;
    p->n_chunks = chunks;
    p->total_elements = total;
    p->schedule = opt.schedule >= 0 ? opt.schedule
                                    : (total >= kPipelinedFromElems ? RAFHIP_LANS_PIPELINED : RAFHIP_LANS_PHASED);
    p->spin_limit = opt.spin_limit;
    p->ws = make_layout(n_tensors, chunks);

    if (hipGetDevice(&p->device) != hipSuccess) {
      (void)hipGetLastError();
      return fail(RAFHIP_ERR_NO_DEVICE, "rafhip_lans_plan_create: no HIP device available");
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, p->device) == hipSuccess &&
        cus > 0)
      p->n_cus = cus;
    p->static_scratch = static_scratch_of(p->device, &p->static_scratch_error);
    p->recs.resize((size_t)n_tensors);
    p->bound.resize((size_t)n_tensors);

    if (n_tensors > 0) {
      std::vector<WorkItem> phased((size_t)chunks);
      size_t k = 0;
      for (int32_t t = 0; t < n_tensors; ++t)
        for (int64_t c = 0; c < chunks_of(numel[t]); ++c) phased[k++] = make_item(t, kPhaseA, c);
      std::vector<WorkItem> phased_a;
      for (int32_t t = 0; t < n_tensors; ++t)
        for (int64_t u = 0; u < units_a_of(numel[t]); ++u) phased_a.push_back(make_item(t, kPhaseA, u));
      p->n_items_a = (int64_t)phased_a.size();
      // Resident workgroups per CU: never more than fit (every workgroup must be running), and by
      // default three; a larger window of in-flight items measured slower on MI355X (it crowds the
      // Infinity Cache).  Lists whose bulk is in long tensors (GPT-2's 8-10 M element matrices)
      // measured 3 % faster with two, lists of shorter tensors (BERT: up to 4 M) 1-2 % slower.
      // rafhip_lans_plan_options.blocks_per_cu overrides the choice downwards or up to the fit.
      const int fit = pipelined_blocks_per_cu(grad_dtype);
      int64_t in_long_tensors = 0;
      for (int32_t t = 0; t < n_tensors; ++t)
        if (numel[t] >= kLongTensorElems) in_long_tensors += numel[t];
      const int wanted = 2 * in_long_tensors > total ? 2 : 3;
      int per_cu = fit > 0 ? (fit < wanted ? fit : wanted) : 2;
      if (opt.blocks_per_cu > 0) per_cu = (fit > 0 && opt.blocks_per_cu > fit) ? fit : opt.blocks_per_cu;
      p->pipeline_grid = (unsigned)(p->n_cus * per_cu);
      const std::vector<WorkItem> pipeline =
          build_pipeline(n_tensors, numel, opt.cut, (int)p->pipeline_grid);
      p->n_pipeline_items = (uint32_t)pipeline.size();
      if (p->pipeline_grid > p->n_pipeline_items) p->pipeline_grid = p->n_pipeline_items;

      const size_t phased_bytes = (size_t)align_up((int64_t)sizeof(WorkItem) * (int64_t)phased.size());
      const size_t pipe_bytes = (size_t)align_up((int64_t)sizeof(WorkItem) * (int64_t)pipeline.size());
      const size_t a_bytes = (size_t)align_up((int64_t)sizeof(WorkItem) * (int64_t)phased_a.size());
      hipError_t e = hipMalloc(&p->d_tables, phased_bytes + pipe_bytes + a_bytes + kAlign);
      if (e == hipSuccess) e = p->tensors.init((size_t)n_tensors);
      if (e != hipSuccess)
        return fail(RAFHIP_ERR_HIP, "rafhip_lans_plan_create: allocation failed: %s",
                    hipGetErrorString(e));
      char* base = static_cast<char*>(p->d_tables);
      p->d_items = reinterpret_cast<WorkItem*>(base);
      p->d_pipeline = reinterpret_cast<WorkItem*>(base + phased_bytes);
      p->d_items_a = reinterpret_cast<WorkItem*>(base + phased_bytes + pipe_bytes);
      if (!phased_a.empty())
        e = hipMemcpy(p->d_items_a, phased_a.data(), sizeof(WorkItem) * phased_a.size(),
                      hipMemcpyHostToDevice);
      if (e == hipSuccess && !phased.empty())
        e = hipMemcpy(p->d_items, phased.data(), sizeof(WorkItem) * phased.size(),
                      hipMemcpyHostToDevice);
      if (e == hipSuccess && !pipeline.empty())
        e = hipMemcpy(p->d_pipeline, pipeline.data(), sizeof(WorkItem) * pipeline.size(),
                      hipMemcpyHostToDevice);
      if (e == hipSuccess)
        e = hipHostMalloc(reinterpret_cast<void**>(&p->host_error), 64, hipHostMallocMapped);
      if (e == hipSuccess) {
        *p->host_error = 0u;
        e = hipHostGetDevicePointer(reinterpret_cast<void**>(&p->host_error_dev), p->host_error, 0);
      }
      if (e == hipSuccess && std::getenv("RAFHIP_LANS_TRACE") && !pipeline.empty())
        e = hipMalloc(reinterpret_cast<void**>(&p->d_trace), 32 * pipeline.size());
      if (e != hipSuccess)
        return fail(RAFHIP_ERR_HIP, "rafhip_lans_plan_create: work list upload failed: %s",
                    hipGetErrorString(e));
    }
    *out_plan = p.release();
    return RAFHIP_OK;
  });
}

int rafhip_lans_plan_destroy(rafhip_lans_plan* plan) {
  clear_error();
  free_plan(plan);
  return RAFHIP_OK;
}

int rafhip_lans_plan_set_schedule(rafhip_lans_plan* plan, int32_t schedule) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_set_schedule: plan is NULL");
  if (schedule != RAFHIP_LANS_PHASED && schedule != RAFHIP_LANS_PIPELINED)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_set_schedule: schedule = %d", schedule);
  plan->schedule = schedule;
  return RAFHIP_OK;
}

int32_t rafhip_lans_plan_schedule(const rafhip_lans_plan* plan) { return plan ? plan->schedule : -1; }

int64_t rafhip_lans_workspace_bytes(const rafhip_lans_plan* plan) {
  return plan ? plan->ws.total : -1;
}
int32_t rafhip_lans_plan_num_tensors(const rafhip_lans_plan* plan) {
  return plan ? plan->n_tensors : -1;
}
int64_t rafhip_lans_plan_num_chunks(const rafhip_lans_plan* plan) {
  return plan ? plan->n_chunks : -1;
}
int64_t rafhip_lans_plan_total_elements(const rafhip_lans_plan* plan) {
  return plan ? plan->total_elements : -1;
}

int64_t rafhip_lans_plan_table_uploads(const rafhip_lans_plan* plan) {
  return plan ? plan->tensors.uploads() : -1;
}

int rafhip_lans_step(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                     float* const* m, float* const* v, const float* step_dev, int32_t step_host,
                     const rafhip_lans_hparams* hp, void* workspace, int64_t workspace_bytes,
                     void* stream) {
  return rafhip_lans_step_mixed(plan, g, w, m, v, nullptr, RAFHIP_F16, step_dev, step_host, hp,
                                workspace, workspace_bytes, stream);
}

int rafhip_lans_step_mixed(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                           float* const* m, float* const* v, void* const* p, int32_t p_dtype,
                           const float* step_dev, int32_t step_host,
                           const rafhip_lans_hparams* hp, void* workspace,
                           int64_t workspace_bytes, void* stream) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: plan is NULL");
  return lans_step_impl(plan, g, w, m, v, p, p_dtype, step_dev, step_host, hp, workspace,
                        workspace_bytes, stream);
}

int rafhip_lans_step_noalloc(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                             float* const* m, float* const* v, void* const* p, int32_t p_dtype,
                             const float* step_dev, int32_t step_host,
                             const rafhip_lans_hparams* hp, void* stream) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step_noalloc: plan is NULL");
  if (plan->ws.total > (int64_t)RAFHIP_LANS_STATIC_SCRATCH_BYTES)
    return fail(RAFHIP_ERR_WORKSPACE,
                "rafhip_lans_step_noalloc: this tensor list needs %lld bytes of scratch, the static "
                "buffer holds %lld; use rafhip_lans_step with a workspace of your own",
                (long long)plan->ws.total, (long long)RAFHIP_LANS_STATIC_SCRATCH_BYTES);
  if (plan->n_tensors > 0 && plan->n_chunks > 0 && !plan->static_scratch)
    return fail(RAFHIP_ERR_HIP,
                "rafhip_lans_step_noalloc: the static scratch array could not be located on device "
                "%d when the plan was made: %s",
                plan->device, hipGetErrorString(plan->static_scratch_error));
  return lans_step_impl(plan, g, w, m, v, p, p_dtype, step_dev, step_host, hp, plan->static_scratch,
                        (int64_t)RAFHIP_LANS_STATIC_SCRATCH_BYTES, stream);
}

}  // extern "C"

namespace {

constexpr uintptr_t kWorkspaceAlign = 16;  // what the kernels' 8- and 16-byte accesses need

// Checks that are the same for every kind of step; *nothing_to_do is set for an empty list.
int check_step_args(const char* who, rafhip_lans_plan* plan, const rafhip_lans_hparams* hp,
                    bool* nothing_to_do) {
  *nothing_to_do = false;
  if (!hp) return fail(RAFHIP_ERR_INVALID_ARG, "%s: hparams is NULL", who);
  if (hp->mode != 0 && hp->mode != 1)
    return fail(RAFHIP_ERR_INVALID_ARG, "%s: mode = %d (0 = L2, 1 = decoupled)", who, hp->mode);
  if (plan->n_tensors == 0 || plan->n_chunks == 0) {
    *nothing_to_do = true;
    return RAFHIP_OK;
  }
  if (int st = check_plan_device(who, plan->device)) return st;
  if (plan->host_error && __atomic_load_n(plan->host_error, __ATOMIC_RELAXED) != 0) {
    // Raised by the persistent kernel of an earlier step; reported once, then the plan works on.
    __atomic_store_n(plan->host_error, 0u, __ATOMIC_RELAXED);
    return fail(RAFHIP_ERR_HIP,
                "%s: an earlier pipelined step on this plan ran out of a bounded wait; its results are "
                "invalid (this call did nothing)",
                who);
  }
  return RAFHIP_OK;
}

// The tensor table of a call, built into `recs` (already n long: no allocation); 4-byte (fp16 g:
// 2-byte) alignment is the hard requirement, 16-byte alignment of all four selects the vector path.
int build_records(const char* who, const rafhip_lans_plan* plan, const void* const* g,
                  float* const* w, float* const* m, float* const* v, void* const* p, int32_t p_dtype,
                  std::vector<TensorRec>& recs) {
  if (p && p_dtype != RAFHIP_F16 && p_dtype != RAFHIP_BF16)
    return fail(RAFHIP_ERR_UNSUPPORTED, "%s: weight-copy dtype %d (binary16 or bfloat16)", who, p_dtype);
  if (!g || !w || !m || !v) return fail(RAFHIP_ERR_INVALID_ARG, "%s: null pointer list", who);
  const int32_t n = plan->n_tensors;
  const uintptr_t g_elem = plan->grad_dtype == RAFHIP_F32 ? 4 : 2;
  const uintptr_t g_vec = 16;  // pass A reads the gradient with 16-byte lane accesses
  recs.resize((size_t)n);
  for (int32_t t = 0; t < n; ++t) {
    TensorRec& r = recs[t];
    r.g = g[t];
    r.w = w[t];
    r.m = m[t];
    r.v = v[t];
    r.p = p ? p[t] : nullptr;
    r.numel = plan->numel[t];
    r.first_chunk = plan->first_chunk[t];
    r.vec_ok = 0;
    r.chunk_shift = chunk_shift_for(r.numel);
    r.reserved = 0;
    if (r.numel == 0) continue;
    if (!r.g || !r.w || !r.m || !r.v)
      return fail(RAFHIP_ERR_INVALID_ARG, "%s: tensor %d has a null data pointer", who, t);
    if (!aligned_to(r.g, g_elem) || !aligned_to(r.w, 4) || !aligned_to(r.m, 4) ||
        !aligned_to(r.v, 4) || !aligned_to(r.p, 2))
      return fail(RAFHIP_ERR_INVALID_ARG, "%s: tensor %d is not element-aligned", who, t);
    r.vec_ok = aligned_to(r.g, g_vec) && aligned_to(r.w, 16) && aligned_to(r.m, 16) &&
               aligned_to(r.v, 16) && aligned_to(r.p, 8);
  }
  return RAFHIP_OK;
}

// Enqueues the kernels of one step on `s`; `table` is the device tensor table to read, up to date
// for that stream.
int launch_step(const char* who, rafhip_lans_plan* plan, const TensorRec* table, int32_t p_dtype,
                const float* step_dev, int32_t step_host, const rafhip_lans_hparams* hp,
                void* workspace, int64_t workspace_bytes, hipStream_t s) {
  (void)who;
  char* ws = static_cast<char*>(workspace);
  LansDeviceArgs a;
  a.tensors = table;
  a.n_tensors = plan->n_tensors;
  a.items = plan->d_items;
  a.n_chunks = plan->n_chunks;
  a.items_a = plan->d_items_a;
  a.n_items_a = plan->n_items_a;
  a.n_items = plan->n_pipeline_items;
  a.pipeline_items = plan->d_pipeline;
  a.unscale = hp->grad_unscale;
  a.unscale_dev = plan->unscale_dev;
  a.found_inf_dev = plan->found_inf_dev;
  a.spin_limit = plan->spin_limit;
  a.host_error = plan->host_error_dev;
  a.p_is_bf16 = p_dtype == RAFHIP_BF16 ? 1 : 0;
  a.scalars = reinterpret_cast<StepScalars*>(ws + plan->ws.scalars_off);
  a.stats = reinterpret_cast<TensorStats*>(ws + plan->ws.stats_off);
  a.partials = reinterpret_cast<double*>(ws + plan->ws.partials_off);
  a.sync = reinterpret_cast<SyncHeader*>(ws + plan->ws.sync_off);
  a.trace = plan->d_trace;

  HParamsPod pod;
  pod.learning_rate = hp->learning_rate;
  pod.beta1 = hp->beta1;
  pod.beta2 = hp->beta2;
  pod.eps = hp->eps;
  pod.weight_decay = hp->weight_decay;
  pod.bias_correction = hp->bias_correction;
  pod.grad_averaging = hp->grad_averaging;
  pod.mode = hp->mode;
  pod.normalize_grad = hp->normalize_grad ? 1 : 0;

  hipEvent_t* marks = nullptr;
  if (!plan->timing.empty()) {
    const size_t slot = (size_t)(plan->steps_done % (int64_t)plan->timing.size());
    marks = plan->timing[slot].data();
    // bit j: event j is recorded in this step (a launch that is skipped needs no event after it)
    const int64_t bytes_per_elt = plan->grad_dtype == RAFHIP_F32 ? 16 : 14;
    const bool inline_finish =
        plan->short_tensors_only && plan->total_elements * bytes_per_elt <= plan->resident_bytes;
    plan->timing_marks[slot] = plan->schedule == RAFHIP_LANS_PIPELINED ? 0x07 : inline_finish ? 0x2B : 0x3F;
  }

  if (plan->schedule == RAFHIP_LANS_PIPELINED) {
    if (marks) RAFHIP_HIP_TRY(hipEventRecord(marks[0], s));
    launch_prepare(s, a, step_dev, step_host, pod);
    if (marks) RAFHIP_HIP_TRY(hipEventRecord(marks[1], s));
    launch_pipelined(plan->grad_dtype, plan->pipeline_grid, s, a);
    if (marks) RAFHIP_HIP_TRY(hipEventRecord(marks[2], s));
  } else {
    const int64_t bytes_per_elt = plan->grad_dtype == RAFHIP_F32 ? 16 : 14;
    launch_phased(plan->grad_dtype, plan->total_elements * bytes_per_elt > plan->resident_bytes,
                  plan->short_tensors_only, s, a, step_dev, step_host, pod, marks,
                  plan->apply_slice_shift);
  }
  RAFHIP_HIP_TRY(hipGetLastError());
  plan->steps_done++;
  return RAFHIP_OK;
}

int check_workspace(const char* who, const rafhip_lans_plan* plan, const void* workspace,
                    int64_t workspace_bytes) {
  if (!workspace || workspace_bytes < plan->ws.total)
    return fail(RAFHIP_ERR_WORKSPACE, "%s: workspace %p of %lld bytes, need %lld", who, workspace,
                (long long)workspace_bytes, (long long)plan->ws.total);
  if (!aligned_to(workspace, kWorkspaceAlign))
    return fail(RAFHIP_ERR_WORKSPACE, "%s: workspace %p is not %d-byte aligned", who, workspace,
                (int)kWorkspaceAlign);
  return RAFHIP_OK;
}

// The step behind rafhip_lans_step, _mixed and _noalloc.  Allocates neither device nor host memory.
int lans_step_impl(rafhip_lans_plan* plan, const void* const* g, float* const* w, float* const* m,
                   float* const* v, void* const* p, int32_t p_dtype, const float* step_dev,
                   int32_t step_host, const rafhip_lans_hparams* hp, void* workspace,
                   int64_t workspace_bytes, void* stream) {
  const char* who = "rafhip_lans_step";
  bool nothing = false;
  if (int st = check_step_args(who, plan, hp, &nothing)) return st;
  if (nothing) return RAFHIP_OK;
  return guarded(who, [&]() -> int {
    if (int st = check_workspace(who, plan, workspace, workspace_bytes)) return st;
    if (int st = build_records(who, plan, g, w, m, v, p, p_dtype, plan->recs)) return st;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const TensorRec* table = nullptr;
    if (int st = sync_tables(who, plan->tensors, plan->recs, s, &table)) return st;
    plan->bound_on_device = false;  // whatever was bound, the table used last now follows this call
    return launch_step(who, plan, table, p_dtype, step_dev, step_host, hp, workspace, workspace_bytes, s);
  });
}

}  // namespace

extern "C" {

int rafhip_lans_plan_bind(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                          float* const* m, float* const* v, void* const* p, int32_t p_dtype) {
  clear_error();
  const char* who = "rafhip_lans_plan_bind";
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "%s: plan is NULL", who);
  return guarded(who, [&]() -> int {
    plan->bound_valid = false;
    if (int st = build_records(who, plan, g, w, m, v, p, p_dtype, plan->bound)) return st;
    plan->bound_p_dtype = p ? p_dtype : RAFHIP_F16;
    plan->bound_valid = true;
    plan->bound_on_device = false;
    return RAFHIP_OK;
  });
}

int rafhip_lans_step_bound(rafhip_lans_plan* plan, const float* step_dev, int32_t step_host,
                           const rafhip_lans_hparams* hp, void* workspace, int64_t workspace_bytes,
                           void* stream) {
  clear_error();
  const char* who = "rafhip_lans_step_bound";
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "%s: plan is NULL", who);
  bool nothing = false;
  if (int st = check_step_args(who, plan, hp, &nothing)) return st;
  if (nothing) return RAFHIP_OK;
  if (!plan->bound_valid)
    return fail(RAFHIP_ERR_INVALID_ARG, "%s: no tensors are bound (rafhip_lans_plan_bind first)", who);
  return guarded(who, [&]() -> int {
    if (int st = check_workspace(who, plan, workspace, workspace_bytes)) return st;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const TensorRec* table = nullptr;
    if (plan->bound_on_device) {
      RAFHIP_HIP_TRY(plan->tensors.follow(s, &table));  // nothing to build, compare or send
    } else {
      plan->recs = plan->bound;  // same size: a copy, no allocation
      if (int st = sync_tables(who, plan->tensors, plan->recs, s, &table)) return st;
      plan->bound_on_device = true;
    }
    return launch_step(who, plan, table, plan->bound_p_dtype, step_dev, step_host, hp, workspace,
                       workspace_bytes, s);
  });
}

int rafhip_lans_plan_set_dynamic_scale(rafhip_lans_plan* plan, const float* grad_unscale_dev,
                                       const float* found_inf_dev) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_set_dynamic_scale: plan is NULL");
  if (!aligned_to(grad_unscale_dev, 4) || !aligned_to(found_inf_dev, 4))
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_set_dynamic_scale: pointers must be 4-byte aligned");
  plan->unscale_dev = grad_unscale_dev;
  plan->found_inf_dev = found_inf_dev;
  return RAFHIP_OK;
}

}  // extern "C"

extern "C" {

int rafhip_lans_read_norms(const rafhip_lans_plan* plan, const void* workspace, double* host_out,
                           void* stream) {
  clear_error();
  if (!plan || !workspace || !host_out)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_read_norms: null argument");
  const int32_t n = plan->n_tensors;
  if (n == 0) return RAFHIP_OK;
  return guarded("rafhip_lans_read_norms", [&]() -> int {
    std::vector<TensorStats> st((size_t)n);
    SyncHeader sync{};
    hipStream_t s = static_cast<hipStream_t>(stream);
    const char* ws = static_cast<const char*>(workspace);
    RAFHIP_HIP_TRY(hipMemcpyAsync(st.data(), ws + plan->ws.stats_off, sizeof(TensorStats) * (size_t)n,
                                  hipMemcpyDeviceToHost, s));
    RAFHIP_HIP_TRY(hipMemcpyAsync(&sync, ws + plan->ws.sync_off, sizeof(sync), hipMemcpyDeviceToHost, s));
    RAFHIP_HIP_TRY(hipStreamSynchronize(s));
    for (int32_t t = 0; t < n; ++t) {
      if (plan->numel[t] == 0) {  // no chunks, nothing was computed: an empty tensor has zero norms
        for (int q = 0; q < 4; ++q) host_out[4 * t + q] = 0.0;
        continue;
      }
      host_out[4 * t + 0] = st[t].grad_norm;
      host_out[4 * t + 1] = st[t].param_norm;
      host_out[4 * t + 2] = st[t].um_norm;
      host_out[4 * t + 3] = st[t].ug_norm;
    }
    if (plan->n_chunks > 0 && sync.error != 0) {
      if (plan->host_error) __atomic_store_n(plan->host_error, 0u, __ATOMIC_RELAXED);  // reported here
      return fail(RAFHIP_ERR_HIP,
                  "rafhip_lans_read_norms: the last pipelined step ran out of a bounded wait; its "
                  "results are invalid");
    }
    return RAFHIP_OK;
  });
}

int rafhip_lans_debug_trace(rafhip_lans_plan* plan, uint64_t* words_out, int64_t capacity_items,
                            int64_t* n_items_out) {
  clear_error();
  if (!plan || !n_items_out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_debug_trace: null argument");
  *n_items_out = plan->d_trace ? (int64_t)plan->n_pipeline_items : 0;
  if (!plan->d_trace || !words_out) return RAFHIP_OK;
  if (capacity_items < (int64_t)plan->n_pipeline_items)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_debug_trace: capacity too small");
  RAFHIP_HIP_TRY(hipDeviceSynchronize());
  RAFHIP_HIP_TRY(hipMemcpy(words_out, plan->d_trace, 32 * (size_t)plan->n_pipeline_items,
                           hipMemcpyDeviceToHost));
  return RAFHIP_OK;
}

int rafhip_lans_timing_enable(rafhip_lans_plan* plan, int32_t slots) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_enable: plan is NULL");
  if (slots < 0 || slots > 4096)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_enable: slots = %d", slots);
  return guarded("rafhip_lans_timing_enable", [&]() -> int {
    destroy_timing(plan);
    plan->steps_done = 0;
    plan->timing.resize((size_t)slots);
    plan->timing_marks.assign((size_t)slots, 0);
    for (auto& slot : plan->timing) slot.fill(nullptr);
    for (auto& slot : plan->timing)
      for (auto& e : slot) {
        hipError_t err = hipEventCreate(&e);
        if (err != hipSuccess) {
          destroy_timing(plan);
          return fail(RAFHIP_ERR_HIP, "rafhip_lans_timing_enable: hipEventCreate: %s",
                      hipGetErrorString(err));
        }
      }
    return RAFHIP_OK;
  });
}

int rafhip_lans_timing_read(rafhip_lans_plan* plan, int32_t slot, float* ms_out5) {
  clear_error();
  if (!plan || !ms_out5) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_read: null argument");
  if (slot < 0 || (size_t)slot >= plan->timing.size() || plan->steps_done <= slot)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_read: slot %d holds no step", slot);
  auto& ev = plan->timing[(size_t)slot];
  const int recorded = plan->timing_marks[(size_t)slot];
  if ((recorded & 1) == 0) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_read: slot %d holds no step", slot);
  int last = 0;
  for (int j = 1; j < 6; ++j) {
    ms_out5[j - 1] = 0.0f;
    if (recorded & (1 << j)) {  // the interval that ends at event j started at the last recorded event
      RAFHIP_HIP_TRY(hipEventSynchronize(ev[j]));
      RAFHIP_HIP_TRY(hipEventElapsedTime(&ms_out5[j - 1], ev[last], ev[j]));
      last = j;
    }
  }
  return RAFHIP_OK;
}

}  // extern "C"

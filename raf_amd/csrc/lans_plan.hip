// Host side of the multi-tensor LANS step: the plan (chunk table, tensor table, timing events) and
// the C-ABI entry points.  The plan plays the part of the reference's LansImpl constructor
// (src/op/dialect/cuda/lans.cc:27-83) and rafhip_lans_step that of LansImpl::Execute (:92-131),
// without its blocking copy of `step` to the host and without its per-element scratch buffer.
#include <hip/hip_runtime.h>

#include <array>
#include <cstring>
#include <limits>
#include <new>
#include <vector>

#include "lans_kernels.h"
#include "status.h"

using namespace rafhip;

namespace {

constexpr int64_t kAlign = 256;
inline int64_t align_up(int64_t x) { return (x + kAlign - 1) / kAlign * kAlign; }

struct WorkspaceLayout {
  int64_t scalars_off, stats_off, partials_off, total;
};

}  // namespace

struct rafhip_lans_plan {
  int device = 0;
  int32_t n_tensors = 0;
  int32_t grad_dtype = RAFHIP_F32;
  int64_t n_chunks = 0;
  int64_t total_elements = 0;
  std::vector<int64_t> numel;
  std::vector<int32_t> first_chunk;
  WorkspaceLayout ws{};

  // Device tables: [TensorRec x n_tensors][ChunkRec x n_chunks] in one allocation.
  void* d_tables = nullptr;
  TensorRec* d_tensors = nullptr;
  ChunkRec* d_chunks = nullptr;

  // Tensor-table upload: pinned staging + the records last sent, so a step whose pointers did not
  // move sends nothing.
  TensorRec* h_staging = nullptr;
  std::vector<TensorRec> last_sent;
  bool sent_once = false;
  hipEvent_t staging_free = nullptr;  // recorded after the last upload was enqueued

  // Optional per-kernel timing: slots x 6 events.
  std::vector<std::array<hipEvent_t, 6>> timing;
  int64_t steps_done = 0;
};

namespace {

void destroy_timing(rafhip_lans_plan* p) {
  for (auto& slot : p->timing)
    for (auto& e : slot)
      if (e) (void)hipEventDestroy(e);
  p->timing.clear();
}

void free_plan(rafhip_lans_plan* p) {
  if (!p) return;
  destroy_timing(p);
  if (p->staging_free) (void)hipEventDestroy(p->staging_free);
  if (p->h_staging) (void)hipHostFree(p->h_staging);
  if (p->d_tables) (void)hipFree(p->d_tables);
  delete p;
}

inline bool aligned_to(const void* p, uintptr_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

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

int rafhip_lans_query_layout(int32_t n_tensors, const int64_t* numel, int64_t* n_chunks_out,
                             int64_t* workspace_bytes_out) {
  clear_error();
  if (n_tensors < 0 || (n_tensors > 0 && !numel))
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_query_layout: bad tensor list");
  int64_t chunks = 0;
  for (int32_t t = 0; t < n_tensors; ++t) {
    if (numel[t] < 0)
      return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_query_layout: numel[%d] = %lld < 0", t,
                  (long long)numel[t]);
    chunks += (numel[t] + kChunk - 1) / kChunk;
  }
  if (n_chunks_out) *n_chunks_out = chunks;
  if (workspace_bytes_out)
    *workspace_bytes_out = align_up((int64_t)sizeof(StepScalars)) +
                           align_up((int64_t)sizeof(TensorStats) * n_tensors) +
                           align_up((int64_t)sizeof(double) * 2 * chunks);
  return RAFHIP_OK;
}

int rafhip_lans_plan_create(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                            rafhip_lans_plan** out_plan) {
  clear_error();
  if (!out_plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_create: out_plan is NULL");
  *out_plan = nullptr;
  if (n_tensors < 0)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_create: n_tensors = %d < 0", n_tensors);
  if (n_tensors > 0 && !numel)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_create: numel is NULL");
  if (grad_dtype != RAFHIP_F32 && grad_dtype != RAFHIP_F16)
    return fail(RAFHIP_ERR_UNSUPPORTED,
                "rafhip_lans_plan_create: gradient dtype %d (LANS takes fp32 weights and state; "
                "gradients may be fp32 or fp16)",
                grad_dtype);

  rafhip_lans_plan* p = new (std::nothrow) rafhip_lans_plan();
  if (!p) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_create: out of host memory");
  p->n_tensors = n_tensors;
  p->grad_dtype = grad_dtype;
  p->numel.assign(numel, numel + n_tensors);
  p->first_chunk.resize(n_tensors);
  int64_t chunks = 0, total = 0;
  for (int32_t t = 0; t < n_tensors; ++t) {
    if (numel[t] < 0) {
      free_plan(p);
      return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_plan_create: numel[%d] = %lld < 0", t,
                  (long long)numel[t]);
    }
    p->first_chunk[t] = (int32_t)chunks;
    chunks += (numel[t] + kChunk - 1) / kChunk;
    total += numel[t];
    if (chunks > std::numeric_limits<int32_t>::max()) {
      free_plan(p);
      return fail(RAFHIP_ERR_UNSUPPORTED, "rafhip_lans_plan_create: more than 2^31 chunks");
    }
  }
  p->n_chunks = chunks;
  p->total_elements = total;
  p->ws.scalars_off = 0;
  p->ws.stats_off = align_up((int64_t)sizeof(StepScalars));
  p->ws.partials_off = p->ws.stats_off + align_up((int64_t)sizeof(TensorStats) * n_tensors);
  p->ws.total = p->ws.partials_off + align_up((int64_t)sizeof(double) * 2 * chunks);

  if (hipGetDevice(&p->device) != hipSuccess) {
    (void)hipGetLastError();
    free_plan(p);
    return fail(RAFHIP_ERR_NO_DEVICE, "rafhip_lans_plan_create: no HIP device available");
  }

  if (n_tensors > 0) {
    const size_t tensors_bytes = (size_t)align_up((int64_t)sizeof(TensorRec) * n_tensors);
    const size_t chunk_bytes = sizeof(ChunkRec) * (size_t)chunks;
    hipError_t e = hipMalloc(&p->d_tables, tensors_bytes + (chunk_bytes ? chunk_bytes : 8));
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void**>(&p->h_staging),
                                           sizeof(TensorRec) * (size_t)n_tensors, hipHostMallocDefault);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&p->staging_free, hipEventDisableTiming);
    if (e != hipSuccess) {
      free_plan(p);
      return fail(RAFHIP_ERR_HIP, "rafhip_lans_plan_create: allocation failed: %s",
                  hipGetErrorString(e));
    }
    p->d_tensors = static_cast<TensorRec*>(p->d_tables);
    p->d_chunks = reinterpret_cast<ChunkRec*>(static_cast<char*>(p->d_tables) + tensors_bytes);
    if (chunks > 0) {
      std::vector<ChunkRec> table((size_t)chunks);
      size_t k = 0;
      for (int32_t t = 0; t < n_tensors; ++t) {
        const int64_t nc = (numel[t] + kChunk - 1) / kChunk;
        for (int64_t i = 0; i < nc; ++i) table[k++] = ChunkRec{t, (int32_t)i};
      }
      e = hipMemcpy(p->d_chunks, table.data(), chunk_bytes, hipMemcpyHostToDevice);
      if (e != hipSuccess) {
        free_plan(p);
        return fail(RAFHIP_ERR_HIP, "rafhip_lans_plan_create: chunk table upload failed: %s",
                    hipGetErrorString(e));
      }
    }
  }
  *out_plan = p;
  return RAFHIP_OK;
}

int rafhip_lans_plan_destroy(rafhip_lans_plan* plan) {
  clear_error();
  free_plan(plan);
  return RAFHIP_OK;
}

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

int rafhip_lans_step(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                     float* const* m, float* const* v, const float* step_dev, int32_t step_host,
                     const rafhip_lans_hparams* hp, void* workspace, int64_t workspace_bytes,
                     void* stream) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: plan is NULL");
  if (!hp) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: hparams is NULL");
  if (hp->mode != 0 && hp->mode != 1)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: mode = %d (0 = L2, 1 = decoupled)",
                hp->mode);
  const int32_t n = plan->n_tensors;
  if (n == 0 || plan->n_chunks == 0) return RAFHIP_OK;  // nothing to update
  if (!g || !w || !m || !v)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: null pointer list");
  if (!workspace || workspace_bytes < plan->ws.total)
    return fail(RAFHIP_ERR_WORKSPACE, "rafhip_lans_step: workspace %p of %lld bytes, need %lld",
                workspace, (long long)workspace_bytes, (long long)plan->ws.total);
  if (!aligned_to(workspace, kAlign))
    return fail(RAFHIP_ERR_WORKSPACE, "rafhip_lans_step: workspace %p is not 256-byte aligned",
                workspace);

  // Build this call's tensor table; 4-byte (fp16 g: 2-byte) alignment is the hard requirement,
  // wider alignment only selects the vector path.
  const uintptr_t g_elem = plan->grad_dtype == RAFHIP_F16 ? 2 : 4;
  const uintptr_t g_vec = plan->grad_dtype == RAFHIP_F16 ? 8 : 16;
  std::vector<TensorRec> recs((size_t)n);
  for (int32_t t = 0; t < n; ++t) {
    TensorRec& r = recs[t];
    r.g = g[t];
    r.w = w[t];
    r.m = m[t];
    r.v = v[t];
    r.numel = plan->numel[t];
    r.first_chunk = plan->first_chunk[t];
    r.vec_ok = 0;
    if (r.numel == 0) continue;
    if (!r.g || !r.w || !r.m || !r.v)
      return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: tensor %d has a null data pointer", t);
    if (!aligned_to(r.g, g_elem) || !aligned_to(r.w, 4) || !aligned_to(r.m, 4) ||
        !aligned_to(r.v, 4))
      return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_step: tensor %d is not element-aligned", t);
    r.vec_ok = aligned_to(r.g, g_vec) && aligned_to(r.w, 16) && aligned_to(r.m, 16) &&
               aligned_to(r.v, 16);
  }

  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t table_bytes = sizeof(TensorRec) * (size_t)n;
  if (!plan->sent_once ||
      std::memcmp(plan->last_sent.data(), recs.data(), table_bytes) != 0) {
    // The previous upload may still be reading the staging buffer.
    if (plan->sent_once) RAFHIP_HIP_TRY(hipEventSynchronize(plan->staging_free));
    std::memcpy(plan->h_staging, recs.data(), table_bytes);
    RAFHIP_HIP_TRY(hipMemcpyAsync(plan->d_tensors, plan->h_staging, table_bytes,
                                  hipMemcpyHostToDevice, s));
    RAFHIP_HIP_TRY(hipEventRecord(plan->staging_free, s));
    plan->last_sent.swap(recs);
    plan->sent_once = true;
  }

  char* ws = static_cast<char*>(workspace);
  StepScalars* scalars = reinterpret_cast<StepScalars*>(ws + plan->ws.scalars_off);
  TensorStats* stats = reinterpret_cast<TensorStats*>(ws + plan->ws.stats_off);
  double* partials = reinterpret_cast<double*>(ws + plan->ws.partials_off);

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

  const unsigned chunk_grid = (unsigned)(plan->n_chunks < (1 << 20) ? plan->n_chunks : (1 << 20));
  const unsigned finish_grid = (unsigned)((n + kLansWaves - 1) / kLansWaves);

  std::array<hipEvent_t, 6>* ev = nullptr;
  if (!plan->timing.empty()) ev = &plan->timing[plan->steps_done % (int64_t)plan->timing.size()];
#define RAFHIP_MARK(i) \
  if (ev) RAFHIP_HIP_TRY(hipEventRecord((*ev)[i], s))

  RAFHIP_MARK(0);
  launch_norm_gw(plan->grad_dtype, chunk_grid, s, plan->d_tensors, plan->d_chunks, plan->n_chunks,
                 hp->grad_unscale, partials);
  RAFHIP_MARK(1);
  launch_finish_a(finish_grid, s, plan->d_tensors, n, partials, stats, scalars, step_dev, step_host,
                  pod);
  RAFHIP_MARK(2);
  launch_norm_u(plan->grad_dtype, chunk_grid, s, plan->d_tensors, plan->d_chunks, plan->n_chunks,
                hp->grad_unscale, scalars, stats, partials);
  RAFHIP_MARK(3);
  launch_finish_b(finish_grid, s, plan->d_tensors, n, partials, stats, scalars);
  RAFHIP_MARK(4);
  launch_apply(plan->grad_dtype, chunk_grid, s, plan->d_tensors, plan->d_chunks, plan->n_chunks,
               hp->grad_unscale, scalars, stats);
  RAFHIP_MARK(5);
#undef RAFHIP_MARK
  RAFHIP_HIP_TRY(hipGetLastError());
  plan->steps_done++;
  return RAFHIP_OK;
}

int rafhip_lans_read_norms(const rafhip_lans_plan* plan, const void* workspace, double* host_out,
                           void* stream) {
  clear_error();
  if (!plan || !workspace || !host_out)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_read_norms: null argument");
  const int32_t n = plan->n_tensors;
  if (n == 0) return RAFHIP_OK;
  std::vector<TensorStats> st((size_t)n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  RAFHIP_HIP_TRY(hipMemcpyAsync(st.data(),
                                static_cast<const char*>(workspace) + plan->ws.stats_off,
                                sizeof(TensorStats) * (size_t)n, hipMemcpyDeviceToHost, s));
  RAFHIP_HIP_TRY(hipStreamSynchronize(s));
  for (int32_t t = 0; t < n; ++t) {
    host_out[4 * t + 0] = st[t].grad_norm;
    host_out[4 * t + 1] = st[t].param_norm;
    host_out[4 * t + 2] = st[t].um_norm;
    host_out[4 * t + 3] = st[t].ug_norm;
  }
  return RAFHIP_OK;
}

int rafhip_lans_timing_enable(rafhip_lans_plan* plan, int32_t slots) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_enable: plan is NULL");
  if (slots < 0 || slots > 4096)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_enable: slots = %d", slots);
  destroy_timing(plan);
  plan->steps_done = 0;
  plan->timing.resize((size_t)slots);
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
}

int rafhip_lans_timing_read(rafhip_lans_plan* plan, int32_t slot, float* ms_out5) {
  clear_error();
  if (!plan || !ms_out5) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_read: null argument");
  if (slot < 0 || (size_t)slot >= plan->timing.size() || plan->steps_done <= slot)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_lans_timing_read: slot %d holds no step", slot);
  auto& ev = plan->timing[(size_t)slot];
  RAFHIP_HIP_TRY(hipEventSynchronize(ev[5]));
  for (int i = 0; i < 5; ++i) RAFHIP_HIP_TRY(hipEventElapsedTime(&ms_out5[i], ev[i], ev[i + 1]));
  return RAFHIP_OK;
}

}  // extern "C"

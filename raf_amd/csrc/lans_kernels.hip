// gfx950 kernels of the multi-tensor LANS step; layout, schedules and numerics are described in
// lans_kernels.h.  The rule follows the reference's fp32 CUDA functors
// (src/op/dialect/cuda/kernels/multi_tensor_lans.cu:283-307 stage 1, :346-352 and :386 stage 2,
// :95-185 norms; host scalars src/op/dialect/cuda/lans.cc:94-109) evaluated in float64.
#include "lans_kernels.h"

#include "half_types.h"
#include "rafhip_optim.h"

// No implicit contraction of a*b+c: where a fused multiply-add is wanted it is written as
// __builtin_fma.  The same source line then gives the same bits in every kernel it is inlined
// into, which the bit-equality of the two schedules (and of all grid sizes) relies on.
#pragma clang fp contract(off)

namespace rafhip {
namespace {

typedef RAFHIP_GLOBAL const f32x4 gc_float4;
typedef RAFHIP_GLOBAL f32x4 g_float4;
typedef RAFHIP_GLOBAL const float gc_float;
typedef RAFHIP_GLOBAL float g_float;
typedef RAFHIP_GLOBAL u16x4 g_u16x4;
typedef RAFHIP_GLOBAL unsigned short g_u16;

// ------------------------------------------------------------------ cache policy
// Every pass streams far more data than the 256 MB Infinity Cache holds.  Loads and stores that
// carry the non-temporal hint do not allocate lines there, and on MI355X that alone is worth
// 10-15 % of HBM bandwidth (measured: the read-only pass goes from 6.2 to 6.9 TB/s).  The one
// stream worth caching is the gradient in passes B and C: it is the smallest array, pass B walks
// the list back to front and pass C front to back, so pass C finds the gradients of the front
// third of the list still cached.  Measured best of nine combinations on the BERT-large list.
struct CachePolicy {  // true = non-temporal
  bool a_g, b_g, b_wmv, c_g, c_wmv, c_stores;
};
constexpr CachePolicy kPhasedPolicy = {true, false, true, false, true, true};
// Pipelined: pass A leaves the gradient cached for pass B of the same group a round later, which
// consumes it (non-temporal); pass B loads w, m, v temporally so that they are cached when pass C
// of the group reads them another round later; pass C reads non-temporally (a hit is consumed, not
// kept) and writes non-temporally.  Measured best of nine combinations.
constexpr CachePolicy kPipelinedPolicy = {false, true, false, true, true, true};
constexpr bool kPipelinedAhead = true;  // issue the next trip's loads before evaluating this one
#ifndef RAFHIP_PIPELINED_A_UNROLL
#define RAFHIP_PIPELINED_A_UNROLL 8
#endif
constexpr int kPipelinedAUnroll = RAFHIP_PIPELINED_A_UNROLL;
// Lists whose whole working set fits in the cache (a few million elements) are better off cached.
constexpr CachePolicy kResidentPolicy = {false, false, false, false, false, false};

// ------------------------------------------------------------------ reductions
// Sum over the 64 lanes of a wavefront; the total is valid in lane 0.  Fixed butterfly order.
__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
  return x;
}

// Block-wide sums of N values, returned to every thread.  `red` is [4][kLansWaves] doubles of
// LDS.  The leading barrier makes the helper safe to call repeatedly on the same LDS.  With kFlag
// it also tells every thread whether `flag` was set in any thread, through the same two barriers.
template <int N, bool kFlag = false>
__device__ __forceinline__ bool block_sum(double (&x)[N], double (*red)[kLansWaves], bool flag = false) {
  static_assert(N <= 3, "red holds three rows of sums and one of flags");
#pragma unroll
  for (int j = 0; j < N; ++j) x[j] = wave_sum(x[j]);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  bool wave_flag = false;
  if constexpr (kFlag) wave_flag = __any(flag ? 1 : 0) != 0;
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < N; ++j) red[j][wave] = x[j];
    if constexpr (kFlag) red[3][wave] = wave_flag ? 1.0 : 0.0;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < N; ++j) {
    double s = red[j][0];
#pragma unroll
    for (int k = 1; k < kLansWaves; ++k) s += red[j][k];
    x[j] = s;
  }
  if constexpr (kFlag) {
    bool any = false;
#pragma unroll
    for (int k = 0; k < kLansWaves; ++k) any = any || red[3][k] != 0.0;
    return any;
  }
  return false;
}

// Loads/stores that are coherent across the whole device (they go past the per-XCD L2), used for
// the few words that workgroups exchange inside the persistent kernel.  Because every exchanged
// word moves this way, the kernel never needs a device-scope fence (which would write back and
// invalidate a whole L2 while other workgroups stream through it): "publish, then signal" only has
// to wait for the publishing stores to complete, which a workgroup-scope release fence does.
__device__ __forceinline__ double ld_dev(const double* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev(double* p, double v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

constexpr uint64_t kNotReady = 0xFFFFFFFFFFFFFFFFull;
// What is published in place of a value that could not be computed because a wait ran out: also a
// NaN pattern that no computation produces.  Whoever consumes it passes it on, and pass C skips
// the stores of an element whose parameters are lost, so that a step that ran out of a wait leaves
// every element either at its old or at its correct new value, never at garbage.
constexpr uint64_t kLost = 0xFFFFFFFFFFFFFFFEull;
__device__ __forceinline__ double lost_value() { return __longlong_as_double((long long)kLost); }
__device__ __forceinline__ bool is_lost(double v) { return (uint64_t)__double_as_longlong(v) == kLost; }

__device__ __forceinline__ uint64_t ld_bits(const double* p) {
  return __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}

// Words that travel between workgroups of the pipelined schedule (chunk partials, per-tensor
// statistics) double as their own "ready" flags: the set-up launch fills them with kNotReady (a
// NaN pattern no computation produces, because published values are canonicalised), each is
// written exactly once per step with a single 8-byte store, and a consumer re-reads a word until
// it differs.  No ordering between words is needed.  A wait that runs out raises the error word
// and returns the "lost" pattern, so the grid always drains.
__device__ __forceinline__ void publish(double* p, double v) {
  st_dev(p, v != v ? __builtin_nan("") : v);
}
// The bound of a wait travels in registers (a kernel argument): a poll loop must not touch the
// cache line of the ticket, which every workgroup hammers with atomics (reading the bound from
// there made the whole step 12 % slower).
struct WaitCtx {
  uint32_t* error;       // set to 1 when a wait runs out
  uint32_t limit;        // polls a wait may take
  uint32_t* host_error;  // the same flag in pinned host memory, which the host can read without a copy
  bool gave_up = false;  // this thread has seen a wait run out: its later waits do not poll at all
};
__device__ __forceinline__ double wait_published(const double* word, WaitCtx& wc) {
  uint64_t bits = ld_bits(word);
  uint32_t spins = 0;
  while (bits == kNotReady) {
    if (wc.gave_up || ++spins > wc.limit) {
      // The step is lost.  Raise the error word and make it visible before anything this thread
      // publishes afterwards, so that whoever consumes such a value also finds the word raised
      // (pass C then leaves the tensors as they were).  The fence is expensive, and only here.
      if (!wc.gave_up) {
        __hip_atomic_store(wc.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (wc.host_error) __hip_atomic_store(wc.host_error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        wc.gave_up = true;
      }
      bits = kLost;
      break;
    }
    __builtin_amdgcn_s_sleep(8);
    bits = ld_bits(word);
  }
  return __longlong_as_double((long long)bits);
}

// Several words at once: all loads are issued together, and only words that were not ready are
// read again.
template <int N>
__device__ __forceinline__ void wait_published_n(const double* const (&words)[N], double (&out)[N],
                                                 WaitCtx& wc) {
  uint64_t bits[N];
#pragma unroll
  for (int j = 0; j < N; ++j) bits[j] = ld_bits(words[j]);
#pragma unroll
  for (int j = 0; j < N; ++j)
    out[j] = bits[j] != kNotReady ? __longlong_as_double((long long)bits[j])
                                  : wait_published(words[j], wc);
}

// A tensor's totals from its chunk partials (kPartialSlots doubles per chunk, N of them starting
// at `slot`): thread t adds chunks t, t+256, ... in order, then the fixed block tree.  The order
// depends on nothing but the unit count.  A unit is chunks_per_unit chunks (pass A: kChunksPerA)
// and keeps its partial in its first chunk's slot.  With kWait the partials are awaited.
template <int N, bool kWait>
__device__ __forceinline__ bool tensor_totals(const double* partials, int slot, int64_t n_units,
                                              int chunks_per_unit, double (&tot)[N],
                                              double (*red)[kLansWaves], WaitCtx& wc) {
  bool lost = false;  // kWait only: a partial is lost, or this thread ran out of a wait
  if (n_units == 1) {
    // One unit: the total is that partial (0 + x, as the tree below would form it), which every
    // thread can read for itself -- no trip through LDS and two barriers for the many one-chunk
    // tensors of a list of small tensors.
    const double* p = partials + slot;
    if (kWait) {
      const double* words[N];
#pragma unroll
      for (int j = 0; j < N; ++j) words[j] = p + j;
      wait_published_n<N>(words, tot, wc);
#pragma unroll
      for (int j = 0; j < N; ++j) lost = lost || is_lost(tot[j]);
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) tot[j] = ld_dev(p + j);
    }
#pragma unroll
    for (int j = 0; j < N; ++j) tot[j] = 0.0 + tot[j];
    return lost;  // each thread's own view; the publishing thread acts on its own
  }
#pragma unroll
  for (int j = 0; j < N; ++j) tot[j] = 0.0;
  for (int64_t i = threadIdx.x; i < n_units; i += kLansBlock) {
    const double* p = partials + kPartialSlots * (i * chunks_per_unit) + slot;
    if (kWait) {
      const double* words[N];
      double val[N];
#pragma unroll
      for (int j = 0; j < N; ++j) words[j] = p + j;
      wait_published_n<N>(words, val, wc);
#pragma unroll
      for (int j = 0; j < N; ++j) {
        lost = lost || is_lost(val[j]);
        tot[j] += val[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) tot[j] += ld_dev(p + j);
    }
  }
  return block_sum<N, kWait>(tot, red, lost);
}

// ------------------------------------------------------------------ the rule, per element
// sqrt(x) for x >= 0: hardware rsq (2^-24) and one coupled Newton step (2^-47).  The clamp keeps
// x == 0 exact (0 * rsq(tiny) = 0) without a branch.
__device__ __forceinline__ double sqrt_nonneg(double x) {
  const double y = __builtin_amdgcn_rsq(fmax(x, 1e-300));
  const double g = x * y;
  const double h = 0.5 * y;
  const double r = __builtin_fma(-h, g, 0.5);
  return __builtin_fma(g, r, g);
}

// 1/d: hardware rcp (2^-24), one Newton step, then div_fixup restores the IEEE results for the
// special operands (1/0 = inf, 1/inf = 0, NaN).
__device__ __forceinline__ double reciprocal(double d) {
  const double r0 = __builtin_amdgcn_rcp(d);
  const double e = __builtin_fma(-d, r0, 1.0);
  const double r1 = __builtin_fma(r0, e, r0);
  return __builtin_amdgcn_div_fixup(r1, d, 1.0);
}

struct Directions {
  double m1, v1, um, ug;
};

// Stage 1 of the rule for one element (multi_tensor_lans.cu:283-307).  inv_gdiv is
// 1/(||g||+eps) when the gradient is normalised and 1 otherwise.  The two decay switches fold the
// L2 / decoupled modes into multiplications by 0 or 1.
__device__ __forceinline__ Directions lans_directions(double g, double w, double m, double v,
                                                      double inv_gdiv, const StepScalars& k) {
  const double wp = (k.wd != 0.0) ? w : 0.0;  // reference skips the weight when wd == 0 (:264-269)
  const double decay = k.wd * wp;
  const double sg = __builtin_fma(k.decay_into_grad, decay, g * inv_gdiv);
  const double sp = k.decay_into_dir * decay;
  Directions d;
  d.m1 = __builtin_fma(k.beta3, sg, m * k.beta1);
  d.v1 = __builtin_fma(k.one_minus_beta2 * sg, sg, v * k.beta2);
  const double inv_den = reciprocal(sqrt_nonneg(d.v1 * k.inv_bc2) + k.eps);
  d.um = __builtin_fma(d.m1 * k.inv_bc1, inv_den, sp);
  d.ug = __builtin_fma(sg, inv_den, sp);
  return d;
}

struct ChunkView {
  const void* g;
  float* w;
  float* m;
  float* v;
  unsigned short* p;  // 16-bit weight copy or null
  int len;            // elements in this chunk
  int vec_ok;
};

// `unit_chunks` is 1 for passes B and C and kChunksPerA for pass A.
__device__ __forceinline__ ChunkView chunk_view(const TensorRec& tr, uint32_t chunk,
                                                int g_elem_bytes, int unit_chunks = 1) {
  const int unit = unit_chunks << tr.chunk_shift;
  const int64_t base = (int64_t)chunk * unit;
  const int64_t rest = tr.numel - base;
  ChunkView cv;
  cv.g = static_cast<const char*>(tr.g) + base * g_elem_bytes;
  cv.w = tr.w + base;
  cv.m = tr.m + base;
  cv.v = tr.v + base;
  cv.p = tr.p ? static_cast<unsigned short*>(tr.p) + base : nullptr;
  cv.len = rest < unit ? (int)rest : unit;
  cv.vec_ok = tr.vec_ok;
  return cv;
}

// ------------------------------------------------------------------ pass A on one chunk
// Per-thread contribution to sum g^2 (block reduction is the caller's).  Only the gradient is read:
// ||w|| is not needed before the trust ratios, so its sum rides along with pass B.
// kU: 16-byte accesses in flight per lane per trip.  A lane adds its elements in ascending order
// whatever kU is, so the sum does not depend on it.
template <typename G, bool kNT, int kU = 4>
__device__ __forceinline__ double chunk_sum_g(const ChunkView& cv, float unscale) {
  constexpr int kW = GradIO<G>::kWide;  // elements per 16-byte lane access
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  if (cv.vec_ok) {
    const int nw = cv.len / kW;
    for (int i0 = threadIdx.x; i0 < nw; i0 += kLansBlock * kU) {
      typename GradIO<G>::RawWide raw[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int i = i0 + u * kLansBlock;
        if (i < nw) raw[u] = GradIO<G>::template load_raw_wide<kNT>(cv.g, i);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        if (i0 + u * kLansBlock < nw) {
          float x[kW];
          GradIO<G>::widen_wide(raw[u], unscale, x);
#pragma unroll
          for (int j = 0; j < kW; ++j) acc[j & 3] = __builtin_fma((double)x[j], (double)x[j], acc[j & 3]);
        }
      }
    }
    const int tail = nw * kW + threadIdx.x;  // the < kW leftover elements of a last chunk
    if (tail < cv.len) {
      const double gx = GradIO<G>::load1(cv.g, tail, unscale);
      acc[0] = __builtin_fma(gx, gx, acc[0]);
    }
  } else {
    for (int i = threadIdx.x; i < cv.len; i += kLansBlock) {
      const double gx = GradIO<G>::load1(cv.g, i, unscale);
      acc[0] = __builtin_fma(gx, gx, acc[0]);
    }
  }
  return (acc[0] + acc[1]) + (acc[2] + acc[3]);
}

// ------------------------------------------------------------------ passes B and C: shared loads
// One trip's worth of the four arrays for one lane: kUnroll groups of 4 consecutive elements.
// The gradient stays as loaded (widening it would wait for the load) until the trip is evaluated.
template <typename G>
struct Batch {
  typename GradIO<G>::Raw4 g[kUnroll];
  f32x4 w[kUnroll], m[kUnroll], v[kUnroll];
};

template <typename G, bool kGradNT, bool kNT>
__device__ __forceinline__ void load_batch(Batch<G>& b, const ChunkView& cv, int i0, int n4) {
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int i = i0 + u * kLansBlock;
    if (i < n4) {
      b.g[u] = GradIO<G>::template load_raw4<kGradNT>(cv.g, i);
      b.w[u] = ldg<kNT>((gc_float4*)cv.w + i);
      b.m[u] = ldg<kNT>((gc_float4*)cv.m + i);
      b.v[u] = ldg<kNT>((gc_float4*)cv.v + i);
    }
  }
}

// Walks the 4-element groups of a chunk trip by trip and hands each loaded trip to `body`.  With
// kAhead the loads of trip i+1 are issued before trip i is evaluated: one more trip of registers
// (32 VGPRs), which the persistent kernel has to spare at three workgroups per CU.
// `pre` runs once before the first trip is evaluated -- with kAhead after that trip's loads have
// been issued, so that whatever it waits for (the tensor's statistics, read past the L2 in the
// pipelined schedule) is in flight together with the data instead of ahead of it.
template <typename G, bool kGradNT, bool kNT, bool kAhead, typename Pre, typename Body>
__device__ __forceinline__ void for_each_trip(const ChunkView& cv, int n4, Pre&& pre, Body&& body) {
  constexpr int kStride = kLansBlock * kUnroll;
  if constexpr (kAhead) {
    Batch<G> nxt;
    load_batch<G, kGradNT, kNT>(nxt, cv, (int)threadIdx.x, n4);
    pre();
    for (int i0 = threadIdx.x; i0 < n4; i0 += kStride) {
      const Batch<G> cur = nxt;
      load_batch<G, kGradNT, kNT>(nxt, cv, i0 + kStride, n4);  // guarded per lane by i < n4
      body(cur, i0);
    }
  } else {
    pre();
    for (int i0 = threadIdx.x; i0 < n4; i0 += kStride) {
      Batch<G> cur;
      load_batch<G, kGradNT, kNT>(cur, cv, i0, n4);
      body(cur, i0);
    }
  }
}

// a^2 + b^2 + c^2 + d^2 as two chains of one product and one fused multiply-add each.
__device__ __forceinline__ double sum_sq4(double a, double b, double c, double d) {
  return __builtin_fma(b, b, a * a) + __builtin_fma(d, d, c * c);
}

// One trip's contribution to a lane's sums of u_m^2, u_g^2 and w^2 (pass B).
template <typename G>
__device__ __forceinline__ void sums_of_trip(const Batch<G>& cur, int i0, int n4, float unscale,
                                             double inv_gdiv, const StepScalars& k, double& am,
                                             double& au, double& aw) {
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    if (i0 + u * kLansBlock < n4) {
      const f32x4 g = GradIO<G>::widen4(cur.g[u], unscale);
      const Directions d0 = lans_directions(g.x, cur.w[u].x, cur.m[u].x, cur.v[u].x, inv_gdiv, k);
      const Directions d1 = lans_directions(g.y, cur.w[u].y, cur.m[u].y, cur.v[u].y, inv_gdiv, k);
      const Directions d2 = lans_directions(g.z, cur.w[u].z, cur.m[u].z, cur.v[u].z, inv_gdiv, k);
      const Directions d3 = lans_directions(g.w, cur.w[u].w, cur.m[u].w, cur.v[u].w, inv_gdiv, k);
      am += sum_sq4(d0.um, d1.um, d2.um, d3.um);
      au += sum_sq4(d0.ug, d1.ug, d2.ug, d3.ug);
      aw += sum_sq4((double)cur.w[u].x, (double)cur.w[u].y, (double)cur.w[u].z, (double)cur.w[u].w);
    }
  }
}

// ------------------------------------------------------------------ pass B on one chunk
// Per-thread contributions to sum u_m^2, sum u_g^2 and sum w^2.  `get_inv_gdiv` supplies the
// tensor's gradient divisor (the pipelined schedule may have to wait for it).
// (In the one-launch-per-pass kernels, issuing trip i+1's loads before evaluating trip i costs a
// wave of occupancy and makes them slower; the persistent kernel has the registers to spare.)
template <typename G, bool kGradNT, bool kNT, bool kAhead = false, typename GetInvGdiv>
__device__ __forceinline__ void chunk_sums_u(const ChunkView& cv, float unscale,
                                             const StepScalars& k, GetInvGdiv&& get_inv_gdiv,
                                             double (&sums)[3]) {
  double am = 0.0, au = 0.0, aw = 0.0;
  if (cv.vec_ok) {
    const int n4 = cv.len >> 2;
    double inv_gdiv = 1.0;
    for_each_trip<G, kGradNT, kNT, kAhead>(cv, n4, [&] { inv_gdiv = get_inv_gdiv(); },
                                           [&](const Batch<G>& cur, int i0) {
      sums_of_trip<G>(cur, i0, n4, unscale, inv_gdiv, k, am, au, aw);
    });
    const int tail = (n4 << 2) + threadIdx.x;
    if (tail < cv.len) {
      const double wx = ((gc_float*)cv.w)[tail];
      const Directions d = lans_directions(GradIO<G>::load1(cv.g, tail, unscale), wx,
                                           ((gc_float*)cv.m)[tail], ((gc_float*)cv.v)[tail],
                                           inv_gdiv, k);
      am = __builtin_fma(d.um, d.um, am);
      au = __builtin_fma(d.ug, d.ug, au);
      aw = __builtin_fma(wx, wx, aw);
    }
  } else {
    const double inv_gdiv = get_inv_gdiv();
    for (int i = threadIdx.x; i < cv.len; i += kLansBlock) {
      const double wx = ((gc_float*)cv.w)[i];
      const Directions d = lans_directions(GradIO<G>::load1(cv.g, i, unscale), wx,
                                           ((gc_float*)cv.m)[i], ((gc_float*)cv.v)[i], inv_gdiv, k);
      am = __builtin_fma(d.um, d.um, am);
      au = __builtin_fma(d.ug, d.ug, au);
      aw = __builtin_fma(wx, wx, aw);
    }
  }
  sums[0] = am;
  sums[1] = au;
  sums[2] = aw;
}

// ------------------------------------------------------------------ pass C on one chunk
struct Applied {
  float w, m, v;
};

struct ApplyParams {
  double inv_gdiv, rm, rg;
  bool valid = true;  // false: a wait ran out somewhere upstream; this thread stores nothing
};

__device__ __forceinline__ Applied apply_one(double g, double w, double m, double v,
                                             const ApplyParams& p, const StepScalars& k) {
  const Directions d = lans_directions(g, w, m, v, p.inv_gdiv, k);
  Applied o;
  // multi_tensor_lans.cu:386: p - ratio_m*update_m - ratio_g*update_g, left to right
  o.w = (float)__builtin_fma(-p.rg, d.ug, __builtin_fma(-p.rm, d.um, w));
  o.m = (float)d.m1;
  o.v = (float)d.v1;
  return o;
}

// One trip of pass C for a lane: the new w, m, v (and the optional 16-bit weight copy) of its
// kUnroll groups of four elements.
template <typename G, bool kStoreNT>
__device__ __forceinline__ void apply_trip(const Batch<G>& cur, int i0, int n4, const ChunkView& cv,
                                           float unscale, bool p_is_bf16, const ApplyParams& p,
                                           const StepScalars& k) {
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int i = i0 + u * kLansBlock;
    if (i < n4) {
      const f32x4 g = GradIO<G>::widen4(cur.g[u], unscale);
      const Applied a0 = apply_one(g.x, cur.w[u].x, cur.m[u].x, cur.v[u].x, p, k);
      const Applied a1 = apply_one(g.y, cur.w[u].y, cur.m[u].y, cur.v[u].y, p, k);
      const Applied a2 = apply_one(g.z, cur.w[u].z, cur.m[u].z, cur.v[u].z, p, k);
      const Applied a3 = apply_one(g.w, cur.w[u].w, cur.m[u].w, cur.v[u].w, p, k);
      stg<kStoreNT>((g_float4*)cv.w + i, f32x4{a0.w, a1.w, a2.w, a3.w});
      stg<kStoreNT>((g_float4*)cv.m + i, f32x4{a0.m, a1.m, a2.m, a3.m});
      stg<kStoreNT>((g_float4*)cv.v + i, f32x4{a0.v, a1.v, a2.v, a3.v});
      if (cv.p)  // uniform over the workgroup
        stg<kStoreNT>((g_u16x4*)cv.p + i,
                      u16x4{narrow16(a0.w, p_is_bf16), narrow16(a1.w, p_is_bf16),
                            narrow16(a2.w, p_is_bf16), narrow16(a3.w, p_is_bf16)});
    }
  }
}

// `get_params` supplies the tensor's divisor and trust ratios.
template <typename G, bool kGradNT, bool kNT, bool kStoreNT, bool kAhead = false, typename GetParams>
__device__ __forceinline__ void chunk_apply(const ChunkView& cv, float unscale, bool p_is_bf16,
                                            const StepScalars& k, GetParams&& get_params) {
  if (cv.vec_ok) {
    const int n4 = cv.len >> 2;
    ApplyParams p{1.0, 0.0, 0.0};
    for_each_trip<G, kGradNT, kNT, kAhead>(cv, n4, [&] { p = get_params(); },
                                           [&](const Batch<G>& cur, int i0) {
      if (p.valid) apply_trip<G, kStoreNT>(cur, i0, n4, cv, unscale, p_is_bf16, p, k);
    });
    const int tail = (n4 << 2) + threadIdx.x;
    if (tail < cv.len && p.valid) {
      const Applied o = apply_one(GradIO<G>::load1(cv.g, tail, unscale), ((gc_float*)cv.w)[tail],
                                  ((gc_float*)cv.m)[tail], ((gc_float*)cv.v)[tail], p, k);
      ((g_float*)cv.w)[tail] = o.w;
      ((g_float*)cv.m)[tail] = o.m;
      ((g_float*)cv.v)[tail] = o.v;
      if (cv.p) ((g_u16*)cv.p)[tail] = narrow16(o.w, p_is_bf16);
    }
  } else {
    const ApplyParams p = get_params();
    for (int i = threadIdx.x; p.valid && i < cv.len; i += kLansBlock) {
      const Applied o = apply_one(GradIO<G>::load1(cv.g, i, unscale), ((gc_float*)cv.w)[i],
                                  ((gc_float*)cv.m)[i], ((gc_float*)cv.v)[i], p, k);
      ((g_float*)cv.w)[i] = o.w;
      ((g_float*)cv.m)[i] = o.m;
      ((g_float*)cv.v)[i] = o.v;
      if (cv.p) ((g_u16*)cv.p)[i] = narrow16(o.w, p_is_bf16);
    }
  }
}

// ------------------------------------------------------------------ per-tensor finishes
// From the total of pass A: the gradient norm and divisor (multi_tensor_lans.cu:284-286: divide
// only when normalising and the norm is non-zero).  Executed by one thread.
__device__ __forceinline__ double grad_divisor(double gn, const StepScalars& k) {
  return (k.normalize_grad && gn != 0.0) ? 1.0 / (gn + k.eps) : 1.0;
}
__device__ __forceinline__ double stats_after_a(TensorStats* st, double sum_g,
                                                const StepScalars& k) {
  const double gn = sqrt(sum_g);
  const double inv_gdiv = grad_divisor(gn, k);
  publish(&st->grad_norm, gn);
  publish(&st->inv_grad_div, inv_gdiv);
  return inv_gdiv;
}

// From the totals of pass B: ||w|| and the two trust ratios (multi_tensor_lans.cu:349-352) with
// beta1 / beta3 folded in.  Executed by one thread.
struct NormsAfterB {
  double unm, ung, pn;
};
__device__ __forceinline__ NormsAfterB trust_ratios(const double (&tot)[3], const StepScalars& k,
                                                    double& ratio_m, double& ratio_g) {
  const double unm = sqrt(tot[0]), ung = sqrt(tot[1]), pn = sqrt(tot[2]);
  const double rm = (unm != 0.0 && pn != 0.0) ? k.lr * (pn / unm) : k.lr;
  const double rg = (ung != 0.0 && pn != 0.0) ? k.lr * (pn / ung) : k.lr;
  ratio_m = rm * k.beta1;
  ratio_g = rg * k.beta3;
  return NormsAfterB{unm, ung, pn};
}
__device__ __forceinline__ void stats_after_b(TensorStats* st, const double (&tot)[3],
                                              const StepScalars& k, double& ratio_m,
                                              double& ratio_g) {
  const NormsAfterB n = trust_ratios(tot, k, ratio_m, ratio_g);
  const double unm = n.unm, ung = n.ung, pn = n.pn;
  publish(&st->param_norm, pn);
  publish(&st->um_norm, unm);
  publish(&st->ug_norm, ung);
  publish(&st->ratio_m, ratio_m);
  publish(&st->ratio_g, ratio_g);
}

// In place of stats_after_a / stats_after_b when the totals could not be formed.
__device__ __forceinline__ void stats_lost_after_a(TensorStats* st) {
  st_dev(&st->grad_norm, lost_value());
  st_dev(&st->inv_grad_div, lost_value());
}
__device__ __forceinline__ void stats_lost_after_b(TensorStats* st) {
  st_dev(&st->param_norm, lost_value());
  st_dev(&st->um_norm, lost_value());
  st_dev(&st->ug_norm, lost_value());
  st_dev(&st->ratio_m, lost_value());
  st_dev(&st->ratio_g, lost_value());
}

__device__ __forceinline__ int64_t chunks_of(const TensorRec& tr) {
  return (tr.numel + ((int64_t)1 << tr.chunk_shift) - 1) >> tr.chunk_shift;
}
__device__ __forceinline__ int64_t units_a_of(const TensorRec& tr) {
  const int shift = tr.chunk_shift + kChunksPerAShift;
  return (tr.numel + ((int64_t)1 << shift) - 1) >> shift;
}

// Host scalars of the reference (lans.cc:94-109), evaluated on the device so that the step tensor
// never has to be copied to the host; also rewinds the ticket and clears the error word.  One thread.
__device__ __forceinline__ void write_step_scalars(const LansDeviceArgs& a, const float* step_dev,
                                                   int32_t step_host, const HParamsPod& hp) {
  a.sync->ticket = 0u;
  a.sync->error = 0u;
  const int step = step_dev ? (int)(*step_dev) : step_host;
  float bc1 = 1.0f, bc2 = 1.0f;
  if (hp.bias_correction == 1) {  // double pow, then one rounding to fp32 (lans.cc:103-104)
    bc1 = (float)(1.0 - pow((double)hp.beta1, (double)step));
    bc2 = (float)(1.0 - pow((double)hp.beta2, (double)step));
  }
  StepScalars k;
  k.beta1 = hp.beta1;
  k.beta2 = hp.beta2;
  k.one_minus_beta2 = 1.0f - hp.beta2;                             // fp32 subtraction (:291)
  k.beta3 = (hp.grad_averaging == 1) ? (1.0f - hp.beta1) : 1.0f;  // fp32 (lans.cc:107-109)
  k.eps = hp.eps;
  k.wd = hp.weight_decay;
  k.inv_bc1 = 1.0 / (double)bc1;
  k.inv_bc2 = 1.0 / (double)bc2;
  k.lr = hp.learning_rate;
  k.decay_into_grad = hp.mode == 0 ? 1.0 : 0.0;
  k.decay_into_dir = hp.mode == 0 ? 0.0 : 1.0;
  k.normalize_grad = hp.normalize_grad;
  k.pad = 0;
  *a.scalars = k;
}

// Dynamic loss scaling.  The factor every gradient element is multiplied by first comes from the
// plan's hyper-parameters or, when the caller gave one, from an fp32 word in device memory (the
// reciprocal of the current loss scale); a non-zero `found_inf` word makes the whole step a no-op:
// every kernel of the step returns at once and w, m, v (and the 16-bit copies) keep their bits.
// Both words are read when a kernel starts, so the host never has to know their values.
__device__ __forceinline__ float grad_unscale_of(const LansDeviceArgs& a) {
  return a.unscale_dev ? *a.unscale_dev : a.unscale;
}
__device__ __forceinline__ bool step_is_skipped(const LansDeviceArgs& a) {
  return a.found_inf_dev != nullptr && *a.found_inf_dev != 0.0f;
}

// ------------------------------------------------------------------ set-up launch
// Set-up of a pipelined step: the step scalars, and every word the schedule waits on (chunk
// partials, per-tensor statistics) marked as not ready.  The phased schedule waits on nothing and
// writes its scalars from the first pass instead.
__global__ __launch_bounds__(kLansBlock) void lans_prepare(LansDeviceArgs a, const float* step_dev,
                                                           int32_t step_host, HParamsPod hp) {
  const uint64_t tid = (uint64_t)blockIdx.x * kLansBlock + threadIdx.x;
  const uint64_t nthr = (uint64_t)gridDim.x * kLansBlock;
  uint64_t* stat_words = reinterpret_cast<uint64_t*>(a.stats);
  for (uint64_t i = tid; i < 8u * (uint64_t)a.n_tensors; i += nthr) stat_words[i] = kNotReady;
  uint64_t* part_words = reinterpret_cast<uint64_t*>(a.partials);
  for (uint64_t i = tid; i < (uint64_t)kPartialSlots * (uint64_t)a.n_chunks; i += nthr)
    part_words[i] = kNotReady;
  if (tid == 0) write_step_scalars(a, step_dev, step_host, hp);
}

// ------------------------------------------------------------------ phased schedule
// Three variants: streaming (lists far larger than the Infinity Cache), resident (lists that fit),
// and resident with inline finishes for lists of short tensors only: there every workgroup of pass
// B (C) adds the few chunk partials of its tensor itself -- the same sums in the same order as the
// finish launch would -- and the two one-workgroup-per-tensor launches disappear, which is a fifth
// of the step for a list of thousands of small tensors.
enum PhasedMode { kModeStreaming = 0, kModeResident = 1, kModeResidentInline = 2 };

template <typename G, int kMode>
__global__ __launch_bounds__(kLansBlock) void lans_norm_g(LansDeviceArgs a, const float* step_dev,
                                                          int32_t step_host, HParamsPod hp) {
  constexpr CachePolicy kP = kMode == kModeStreaming ? kPhasedPolicy : kResidentPolicy;
  __shared__ double red[4][kLansWaves];
  if (step_is_skipped(a)) return;
  const float unscale = grad_unscale_of(a);
  // This pass needs no scalars; the later launches find them written by the first workgroup.
  if (blockIdx.x == 0 && threadIdx.x == 0) write_step_scalars(a, step_dev, step_host, hp);
  for (int64_t i = blockIdx.x; i < a.n_items_a; i += gridDim.x) {
    const WorkItem it = a.items_a[i];
    const TensorRec tr = a.tensors[it.tensor];
    const uint32_t unit = it.chunk_phase & kChunkMask;
    const ChunkView cv = chunk_view(tr, unit, (int)sizeof(G), kChunksPerA);
    double s[1] = {chunk_sum_g<G, kP.a_g>(cv, unscale)};
    block_sum<1>(s, red);
    if (threadIdx.x == 0)
      publish(&a.partials[kPartialSlots * ((int64_t)tr.first_chunk + (int64_t)unit * kChunksPerA)], s[0]);
  }
}

// One workgroup per tensor.
__global__ __launch_bounds__(kLansBlock) void lans_finish(LansDeviceArgs a, int after_b) {
  __shared__ double red[4][kLansWaves];
  if (step_is_skipped(a)) return;
  WaitCtx no_wait{nullptr, 0, nullptr};
  const int t = blockIdx.x;
  const TensorRec tr = a.tensors[t];
  const double* part = a.partials + kPartialSlots * (int64_t)tr.first_chunk;
  const StepScalars k = *a.scalars;
  if (after_b) {
    double tot[3], r0, r1;
    tensor_totals<3, false>(part, 1, chunks_of(tr), 1, tot, red, no_wait);
    if (threadIdx.x == 0) stats_after_b(&a.stats[t], tot, k, r0, r1);
  } else {
    double tot[1];
    tensor_totals<1, false>(part, 0, units_a_of(tr), kChunksPerA, tot, red, no_wait);
    if (threadIdx.x == 0) stats_after_a(&a.stats[t], tot[0], k);
  }
}

template <typename G, int kMode>
__global__ __launch_bounds__(kLansBlock) void lans_norm_u(LansDeviceArgs a) {
  constexpr CachePolicy kP = kMode == kModeStreaming ? kPhasedPolicy : kResidentPolicy;
  __shared__ double red[4][kLansWaves];
  if (step_is_skipped(a)) return;
  const float unscale = grad_unscale_of(a);
  WaitCtx no_wait{nullptr, 0, nullptr};
  const StepScalars k = *a.scalars;
  // Back to front: pass A has just streamed the gradients front to back, so the end of the list is
  // what the Infinity Cache still holds; pass C then starts at the front, where this pass ends.
  for (int64_t b = blockIdx.x; b < a.n_chunks; b += gridDim.x) {
    const int64_t c = a.n_chunks - 1 - b;
    const WorkItem it = a.items[c];
    const TensorRec tr = a.tensors[it.tensor];
    const uint32_t chunk = it.chunk_phase & kChunkMask;
    const ChunkView cv = chunk_view(tr, chunk, (int)sizeof(G));
    double inv_gdiv;
    if constexpr (kMode == kModeResidentInline) {
      double tot[1];
      tensor_totals<1, false>(a.partials + kPartialSlots * (int64_t)tr.first_chunk, 0, units_a_of(tr),
                              kChunksPerA, tot, red, no_wait);
      if (chunk == 0 && threadIdx.x == 0)  // one workgroup per tensor leaves the statistics
        inv_gdiv = stats_after_a(&a.stats[it.tensor], tot[0], k);
      else
        inv_gdiv = grad_divisor(sqrt(tot[0]), k);
    } else {
      inv_gdiv = a.stats[it.tensor].inv_grad_div;
    }
    double s[3];
    chunk_sums_u<G, kP.b_g, kP.b_wmv>(cv, unscale, k, [&] { return inv_gdiv; }, s);
    block_sum<3>(s, red);
    if (threadIdx.x == 0) {
      publish(&a.partials[kPartialSlots * c + 1], s[0]);
      publish(&a.partials[kPartialSlots * c + 2], s[1]);
      publish(&a.partials[kPartialSlots * c + 3], s[2]);
    }
  }
}

// `slice_shift` > 0: a chunk is applied in slices of 2^slice_shift elements, one workgroup each
// (pass C adds nothing up, so how a chunk is cut changes no result); the grid provides
// kChunk >> slice_shift workgroups per chunk, and those beyond a shorter chunk's end do nothing.
// A workgroup that makes one short trip and ends never holds loads back behind its own stores:
// with 1024-element slices the streaming pass runs 3.5 % (BERT-large) to 6 % (BERT-base) faster.
template <typename G, int kMode>
__global__ __launch_bounds__(kLansBlock) void lans_apply(LansDeviceArgs a, int slice_shift) {
  constexpr CachePolicy kP = kMode == kModeStreaming ? kPhasedPolicy : kResidentPolicy;
  __shared__ double red[4][kLansWaves];
  if (step_is_skipped(a)) return;
  const float unscale = grad_unscale_of(a);
  WaitCtx no_wait{nullptr, 0, nullptr};
  const StepScalars k = *a.scalars;
  const int split_shift = slice_shift > 0 ? kChunkShift - slice_shift : 0;
  const int64_t n_slices = a.n_chunks << split_shift;
  for (int64_t b = blockIdx.x; b < n_slices; b += gridDim.x) {
    const int64_t c = b >> split_shift;
    const WorkItem it = a.items[c];
    const TensorRec tr = a.tensors[it.tensor];
    const uint32_t chunk = it.chunk_phase & kChunkMask;
    ChunkView cv = chunk_view(tr, chunk, (int)sizeof(G));
    if (split_shift > 0) {
      const int begin = (int)(b & ((1 << split_shift) - 1)) << slice_shift;
      if (begin >= cv.len) continue;
      cv.g = static_cast<const char*>(cv.g) + (int64_t)begin * (int)sizeof(G);
      cv.w += begin;
      cv.m += begin;
      cv.v += begin;
      if (cv.p) cv.p += begin;
      const int slice = 1 << slice_shift;
      cv.len = cv.len - begin < slice ? cv.len - begin : slice;
    }
    ApplyParams p;
    if constexpr (kMode == kModeResidentInline) {
      double tot[3];
      tensor_totals<3, false>(a.partials + kPartialSlots * (int64_t)tr.first_chunk, 1, chunks_of(tr), 1,
                              tot, red, no_wait);
      p.inv_gdiv = a.stats[it.tensor].inv_grad_div;  // left by pass B
      if (chunk == 0 && b == (c << split_shift) && threadIdx.x == 0)
        stats_after_b(&a.stats[it.tensor], tot, k, p.rm, p.rg);
      else
        (void)trust_ratios(tot, k, p.rm, p.rg);
    } else {
      const TensorStats st = a.stats[it.tensor];
      p = ApplyParams{st.inv_grad_div, st.ratio_m, st.ratio_g};
    }
    chunk_apply<G, kP.c_g, kP.c_wmv, kP.c_stores>(cv, unscale, a.p_is_bf16 != 0, k, [&] { return p; });
  }
}

// ------------------------------------------------------------------ pipelined schedule
template <typename G>
__global__ __launch_bounds__(kLansBlock) void lans_pipelined(LansDeviceArgs a) {
  __shared__ double red[4][kLansWaves];
  __shared__ double s_bcast[3];
  __shared__ uint32_t s_ticket;
  if (step_is_skipped(a)) return;
  const float unscale = grad_unscale_of(a);
  const StepScalars k = *a.scalars;
  WaitCtx wc{&a.sync->error, a.spin_limit, a.host_error};

  // Thread 0 draws tickets two items ahead, so an atomic's round trip is hidden behind a whole
  // item, and every thread reads the NEXT item's descriptor and tensor record while the current
  // item is being processed.  Every workgroup draws exactly two tickets past the end of the list.
  auto draw = [&]() -> uint32_t {
    return __hip_atomic_fetch_add(&a.sync->ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  uint32_t ahead = 0;  // thread 0 only: the ticket after next
  if (threadIdx.x == 0) {
    s_ticket = draw();
    ahead = draw();
  }
  __syncthreads();
  // readfirstlane tells the compiler the value is wave-uniform: the descriptor and tensor-record
  // reads below become scalar loads into SGPRs instead of per-lane loads into VGPRs.
  uint32_t ticket = __builtin_amdgcn_readfirstlane(s_ticket);
  WorkItem it = ticket < a.n_items ? a.pipeline_items[ticket] : WorkItem{0, 0};
  TensorRec tr = ticket < a.n_items ? a.tensors[it.tensor] : TensorRec{};

  while (ticket < a.n_items) {  // uniform
    __syncthreads();            // everyone has read s_ticket and is done with the previous item
    if (threadIdx.x == 0) {
      s_ticket = ahead;
      ahead = draw();
    }
    __syncthreads();
    const uint32_t next_ticket = __builtin_amdgcn_readfirstlane(s_ticket);
    const WorkItem next_it =
        next_ticket < a.n_items ? a.pipeline_items[next_ticket] : WorkItem{0, 0};
    const TensorRec next_tr = next_ticket < a.n_items ? a.tensors[next_it.tensor] : TensorRec{};

    uint64_t t_claim = 0;
    if (a.trace && threadIdx.x == 0) t_claim = wall_clock64();
    const int t = it.tensor;
    const uint32_t phase = it.chunk_phase >> kPhaseShift;
    const uint32_t chunk = it.chunk_phase & kChunkMask;
    const bool streaming = (it.chunk_phase & kStreamBit) != 0;  // uniform, like everything read off the item
    const bool unit_a = phase == kPhaseA;  // pass-A items count in units of kChunksPerA chunks
    const ChunkView cv = chunk_view(tr, chunk, (int)sizeof(G), unit_a ? kChunksPerA : 1);
    const int64_t n_chunks = chunks_of(tr);
    double* part = a.partials + kPartialSlots * ((int64_t)tr.first_chunk +
                                                  (int64_t)chunk * (unit_a ? kChunksPerA : 1));
    const double* tensor_part = a.partials + kPartialSlots * (int64_t)tr.first_chunk;
    TensorStats* st = &a.stats[t];

    if (phase == kPhaseA) {
      double s[1];
      // Three workgroups per CU have to keep the gradient stream busy on their own here: twice
      // the accesses in flight of the one-launch-per-pass kernel, which runs five.
      if (streaming)
        s[0] = chunk_sum_g<G, true, kPipelinedAUnroll>(cv, unscale);
      else
        s[0] = chunk_sum_g<G, kPipelinedPolicy.a_g, kPipelinedAUnroll>(cv, unscale);
      block_sum<1>(s, red);
      if (threadIdx.x == 0) publish(part, s[0]);
    } else if (phase == kPhaseFinishA) {
      double tot[1];
      const bool lost = tensor_totals<1, true>(tensor_part, 0, units_a_of(tr), kChunksPerA, tot, red, wc);
      if (threadIdx.x == 0) {
        if (lost)
          stats_lost_after_a(st);
        else
          stats_after_a(st, tot[0], k);
      }
    } else if (phase == kPhaseB) {
      double s[3];
      bool lost = false;  // this thread's divisor never arrived
      auto divisor = [&] {
        const double d = wait_published(&st->inv_grad_div, wc);
        lost = is_lost(d);
        return d;
      };
      if (streaming)
        chunk_sums_u<G, true, true, kPipelinedAhead>(cv, unscale, k, divisor, s);
      else
        chunk_sums_u<G, kPipelinedPolicy.b_g, kPipelinedPolicy.b_wmv, kPipelinedAhead>(cv, unscale, k, divisor, s);
      const bool any_lost = block_sum<3, true>(s, red, lost);
      if (threadIdx.x == 0) {
        if (any_lost) {
          st_dev(part + 1, lost_value());
          st_dev(part + 2, lost_value());
          st_dev(part + 3, lost_value());
        } else {
          publish(part + 1, s[0]);
          publish(part + 2, s[1]);
          publish(part + 3, s[2]);
        }
      }
    } else if (phase == kPhaseFinishB) {
      double tot[3], r0, r1;
      const bool lost = tensor_totals<3, true>(tensor_part, 1, n_chunks, 1, tot, red, wc);
      if (threadIdx.x == 0) {
        if (lost)
          stats_lost_after_b(st);
        else
          stats_after_b(st, tot, k, r0, r1);
      }
    } else if (phase == kPhaseC) {
      auto params = [&] {
        const double* const words[3] = {&st->inv_grad_div, &st->ratio_m, &st->ratio_g};
        double val[3];
        wait_published_n<3>(words, val, wc);
        return ApplyParams{val[0], val[1], val[2], !(is_lost(val[0]) || is_lost(val[1]) || is_lost(val[2]))};
      };
      if (streaming)
        chunk_apply<G, true, true, true, kPipelinedAhead>(cv, unscale, a.p_is_bf16 != 0, k, params);
      else
        chunk_apply<G, kPipelinedPolicy.c_g, kPipelinedPolicy.c_wmv, kPipelinedPolicy.c_stores, kPipelinedAhead>(
            cv, unscale, a.p_is_bf16 != 0, k, params);
    } else {
      // A one-chunk tensor: all three passes here, no other workgroup involved.  The totals equal
      // the single chunk partials, exactly as the general path computes them, and travel between
      // the threads through LDS.
      double s1[1] = {chunk_sum_g<G, false>(cv, unscale)};
      block_sum<1>(s1, red);
      if (threadIdx.x == 0) s_bcast[0] = stats_after_a(st, s1[0], k);
      __syncthreads();
      const double inv_gdiv = s_bcast[0];
      double s3[3];
      chunk_sums_u<G, false, false>(cv, unscale, k, [&] { return inv_gdiv; }, s3);
      block_sum<3>(s3, red);
      if (threadIdx.x == 0) stats_after_b(st, s3, k, s_bcast[1], s_bcast[2]);
      __syncthreads();
      const ApplyParams p{inv_gdiv, s_bcast[1], s_bcast[2]};
      chunk_apply<G, false, false, true>(cv, unscale, a.p_is_bf16 != 0, k, [&] { return p; });
    }
    if (a.trace && threadIdx.x == 0) {  // diagnostics: when the item was started and finished
      uint64_t* rec = a.trace + 4 * (uint64_t)ticket;
      rec[0] = t_claim;
      rec[1] = t_claim;
      rec[2] = wall_clock64();
      rec[3] = blockIdx.x;
    }
    ticket = next_ticket;
    it = next_it;
    tr = next_tr;
  }
}

}  // namespace

// ------------------------------------------------------------------ launchers
void launch_prepare(hipStream_t s, const LansDeviceArgs& a, const float* step_dev,
                    int32_t step_host, HParamsPod hp) {
  const uint64_t words = 8u * (uint64_t)a.n_tensors + (uint64_t)kPartialSlots * (uint64_t)a.n_chunks;
  uint64_t grid = (words + kLansBlock * 4 - 1) / (kLansBlock * 4);
  if (grid < 1) grid = 1;
  if (grid > 256) grid = 256;
  hipLaunchKernelGGL(lans_prepare, dim3((unsigned)grid), dim3(kLansBlock), 0, s, a, step_dev,
                     step_host, hp);
}

namespace {
template <typename G, int kMode>
void launch_phased_t(hipStream_t s, const LansDeviceArgs& a, const float* step_dev,
                     int32_t step_host, const HParamsPod& hp, hipEvent_t* marks,
                     int apply_slice_shift) {
  const unsigned grid = (unsigned)(a.n_chunks < (1 << 20) ? a.n_chunks : (1 << 20));
  const unsigned grid_a = (unsigned)(a.n_items_a < (1 << 20) ? a.n_items_a : (1 << 20));
  auto mark = [&](int i) {
    if (marks) (void)hipEventRecord(marks[i], s);
  };
  mark(0);
  constexpr bool kFinishLaunches = kMode != kModeResidentInline;
  hipLaunchKernelGGL((lans_norm_g<G, kMode>), dim3(grid_a), dim3(kLansBlock), 0, s, a, step_dev,
                     step_host, hp);
  mark(1);
  if (kFinishLaunches) {
    hipLaunchKernelGGL(lans_finish, dim3((unsigned)a.n_tensors), dim3(kLansBlock), 0, s, a, 0);
    mark(2);
  }
  hipLaunchKernelGGL((lans_norm_u<G, kMode>), dim3(grid), dim3(kLansBlock), 0, s, a);
  mark(3);
  if (kFinishLaunches) {
    hipLaunchKernelGGL(lans_finish, dim3((unsigned)a.n_tensors), dim3(kLansBlock), 0, s, a, 1);
    mark(4);
  }
  // Slices only where the pass streams from HBM: a cache-resident list is short of parallelism,
  // not of bandwidth, and finer items cost it 30 % of the pass.
  const int slice_shift = kMode == kModeStreaming ? apply_slice_shift : 0;
  const int64_t slices = (int64_t)a.n_chunks << (slice_shift > 0 ? kChunkShift - slice_shift : 0);
  const unsigned grid_c = (unsigned)(slices < (1 << 24) ? slices : (1 << 24) - 1);  // 2^32 threads are refused
  hipLaunchKernelGGL((lans_apply<G, kMode>), dim3(grid_c), dim3(kLansBlock), 0, s, a, slice_shift);
  mark(5);
}
}  // namespace

void launch_phased(int grad_dtype, bool streaming, bool inline_finish, hipStream_t s,
                   const LansDeviceArgs& a, const float* step_dev, int32_t step_host,
                   HParamsPod hp, hipEvent_t* marks, int apply_slice_shift) {
  auto go = [&](auto tag) {
    using G = decltype(tag);
    if (streaming)
      launch_phased_t<G, kModeStreaming>(s, a, step_dev, step_host, hp, marks, apply_slice_shift);
    else if (inline_finish)
      launch_phased_t<G, kModeResidentInline>(s, a, step_dev, step_host, hp, marks, apply_slice_shift);
    else
      launch_phased_t<G, kModeResident>(s, a, step_dev, step_host, hp, marks, apply_slice_shift);
  };
  if (grad_dtype == RAFHIP_F16)
    go(_Float16{});
  else if (grad_dtype == RAFHIP_BF16)
    go(Bf16{});
  else
    go(float{});
}

void launch_pipelined(int grad_dtype, unsigned grid, hipStream_t s, const LansDeviceArgs& a) {
  if (grad_dtype == RAFHIP_F16)
    hipLaunchKernelGGL(lans_pipelined<_Float16>, dim3(grid), dim3(kLansBlock), 0, s, a);
  else if (grad_dtype == RAFHIP_BF16)
    hipLaunchKernelGGL(lans_pipelined<Bf16>, dim3(grid), dim3(kLansBlock), 0, s, a);
  else
    hipLaunchKernelGGL(lans_pipelined<float>, dim3(grid), dim3(kLansBlock), 0, s, a);
}

int pipelined_blocks_per_cu(int grad_dtype) {
  int n = 0;
  hipError_t e;
  if (grad_dtype == RAFHIP_F16)
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, lans_pipelined<_Float16>, kLansBlock, 0);
  else if (grad_dtype == RAFHIP_BF16)
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, lans_pipelined<Bf16>, kLansBlock, 0);
  else
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, lans_pipelined<float>, kLansBlock, 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

}  // namespace rafhip

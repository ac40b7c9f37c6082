// gfx950 kernels of the multi-tensor LANS step; layout and phase order are described in
// lans_kernels.h.  The rule follows the reference's fp32 CUDA functors
// (src/op/dialect/cuda/kernels/multi_tensor_lans.cu:283-307 stage 1, :346-352 and :386 stage 2,
// :95-185 norms) evaluated in float64.
#include "lans_kernels.h"

#include <hip/hip_fp16.h>

#include "rafhip_optim.h"

namespace rafhip {
namespace {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------ gradient ingest
// Four consecutive gradients as fp32, already multiplied by the unscale factor (one fp32 rounding,
// exact for power-of-two loss scales).
template <typename G>
struct GradIO;

template <>
struct GradIO<float> {
  static __device__ __forceinline__ float4 load4(const float* g, int i4, float us) {
    const float4 r = reinterpret_cast<const float4*>(g)[i4];
    return make_float4(__fmul_rn(r.x, us), __fmul_rn(r.y, us), __fmul_rn(r.z, us),
                       __fmul_rn(r.w, us));
  }
  static __device__ __forceinline__ float load1(const float* g, int i, float us) {
    return __fmul_rn(g[i], us);
  }
};

template <>
struct GradIO<_Float16> {
  static __device__ __forceinline__ float4 load4(const _Float16* g, int i4, float us) {
    const half4_t r = reinterpret_cast<const half4_t*>(g)[i4];
    return make_float4(__fmul_rn((float)r.x, us), __fmul_rn((float)r.y, us),
                       __fmul_rn((float)r.z, us), __fmul_rn((float)r.w, us));
  }
  static __device__ __forceinline__ float load1(const _Float16* g, int i, float us) {
    return __fmul_rn((float)g[i], us);
  }
};

// ------------------------------------------------------------------ reductions
// Sum over the 64 lanes of a wavefront; the total is valid in lane 0.  Fixed butterfly order.
__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
  return x;
}

// Block-wide sums of two values; results valid in thread 0.  `red` is [2][kLansWaves] doubles of
// LDS.  The leading barrier makes the helper safe to call once per trip of a chunk loop.
__device__ __forceinline__ void block_sum2(double& a, double& b, double (*red)[kLansWaves]) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) {
    red[0][wave] = a;
    red[1][wave] = b;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double sa = red[0][0], sb = red[1][0];
#pragma unroll
    for (int k = 1; k < kLansWaves; ++k) {
      sa += red[0][k];
      sb += red[1][k];
    }
    a = sa;
    b = sb;
  }
}

// ------------------------------------------------------------------ the rule, per element
struct Directions {
  double m1, v1, um, ug;
};

// Stage 1 of the rule for one element (multi_tensor_lans.cu:283-307).  inv_gdiv is
// 1/(||g||+eps) when the gradient is normalised and 1 otherwise.
__device__ __forceinline__ Directions lans_directions(double g, double w, double m, double v,
                                                      double inv_gdiv, const StepScalars& k) {
  double sg = g * inv_gdiv;
  const double wp = (k.wd != 0.0) ? w : 0.0;  // reference skips the weight when wd == 0 (:264-269)
  const double decay = k.wd * wp;
  double sp = decay;
  if (k.mode == 0) {  // L2 mode: decay joins the scaled gradient, nothing is added afterwards
    sg += decay;
    sp = 0.0;
  }
  Directions d;
  d.m1 = m * k.beta1 + k.beta3 * sg;
  d.v1 = v * k.beta2 + k.one_minus_beta2 * sg * sg;
  const double den = sqrt(d.v1 * k.inv_bc2) + k.eps;
  const double inv_den = 1.0 / den;
  d.um = (d.m1 * k.inv_bc1) * inv_den + sp;
  d.ug = sg * inv_den + sp;
  return d;
}

struct ChunkView {
  const void* g;
  float* w;
  float* m;
  float* v;
  int len;     // elements in this chunk
  int vec_ok;
  int tensor;
};

__device__ __forceinline__ ChunkView chunk_view(const TensorRec* tensors, const ChunkRec* chunks,
                                                int64_t c, int g_elem_bytes) {
  const ChunkRec cr = chunks[c];
  const TensorRec tr = tensors[cr.tensor];
  const int64_t base = (int64_t)cr.index * kChunk;
  const int64_t rest = tr.numel - base;
  ChunkView cv;
  cv.g = static_cast<const char*>(tr.g) + base * g_elem_bytes;
  cv.w = tr.w + base;
  cv.m = tr.m + base;
  cv.v = tr.v + base;
  cv.len = rest < kChunk ? (int)rest : kChunk;
  cv.vec_ok = tr.vec_ok;
  cv.tensor = cr.tensor;
  return cv;
}

// ------------------------------------------------------------------ phase 1: sum g^2, sum w^2
template <typename G>
__global__ __launch_bounds__(kLansBlock) void lans_norm_gw(const TensorRec* __restrict__ tensors,
                                                           const ChunkRec* __restrict__ chunks,
                                                           int64_t n_chunks, float unscale,
                                                           double* __restrict__ partials) {
  __shared__ double red[2][kLansWaves];
  for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
    const ChunkView cv = chunk_view(tensors, chunks, c, (int)sizeof(G));
    const G* g = static_cast<const G*>(cv.g);
    double ag[4] = {0.0, 0.0, 0.0, 0.0}, aw[4] = {0.0, 0.0, 0.0, 0.0};
    if (cv.vec_ok) {
      const int n4 = cv.len >> 2;
      for (int i0 = threadIdx.x; i0 < n4; i0 += kLansBlock * kUnroll) {
        float4 gv[kUnroll], wv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int i = i0 + u * kLansBlock;
          if (i < n4) {
            gv[u] = GradIO<G>::load4(g, i, unscale);
            wv[u] = reinterpret_cast<const float4*>(cv.w)[i];
          } else {
            gv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            wv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
          }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          ag[0] += (double)gv[u].x * (double)gv[u].x;
          ag[1] += (double)gv[u].y * (double)gv[u].y;
          ag[2] += (double)gv[u].z * (double)gv[u].z;
          ag[3] += (double)gv[u].w * (double)gv[u].w;
          aw[0] += (double)wv[u].x * (double)wv[u].x;
          aw[1] += (double)wv[u].y * (double)wv[u].y;
          aw[2] += (double)wv[u].z * (double)wv[u].z;
          aw[3] += (double)wv[u].w * (double)wv[u].w;
        }
      }
      const int tail = (n4 << 2) + threadIdx.x;  // the < 4 leftover elements of a last chunk
      if (tail < cv.len) {
        const double gx = GradIO<G>::load1(g, tail, unscale), wx = cv.w[tail];
        ag[0] += gx * gx;
        aw[0] += wx * wx;
      }
    } else {
      for (int i = threadIdx.x; i < cv.len; i += kLansBlock) {
        const double gx = GradIO<G>::load1(g, i, unscale), wx = cv.w[i];
        ag[0] += gx * gx;
        aw[0] += wx * wx;
      }
    }
    double sg = (ag[0] + ag[1]) + (ag[2] + ag[3]);
    double sw = (aw[0] + aw[1]) + (aw[2] + aw[3]);
    block_sum2(sg, sw, red);
    if (threadIdx.x == 0) {
      partials[2 * c] = sg;
      partials[2 * c + 1] = sw;
    }
  }
}

// ------------------------------------------------------------------ phases 2 and 4: per-tensor finish
// One wavefront per tensor adds that tensor's chunk partials: lane l takes chunks l, l+64, ... in
// order, then the fixed butterfly.  The order depends on nothing but the chunk count.
__device__ __forceinline__ void tensor_totals(const TensorRec& tr, const double* partials,
                                              int lane, double& a, double& b) {
  const int64_t n_chunks = (tr.numel + kChunk - 1) / kChunk;
  const double* p = partials + 2 * (int64_t)tr.first_chunk;
  a = 0.0;
  b = 0.0;
  for (int64_t i = lane; i < n_chunks; i += 64) {
    a += p[2 * i];
    b += p[2 * i + 1];
  }
  a = wave_sum(a);
  b = wave_sum(b);
}

__global__ __launch_bounds__(kLansBlock) void lans_finish_a(
    const TensorRec* __restrict__ tensors, int32_t n_tensors, const double* __restrict__ partials,
    TensorStats* __restrict__ stats, StepScalars* __restrict__ scalars,
    const float* __restrict__ step_dev, int32_t step_host, HParamsPod hp) {
  const int t = (int)((blockIdx.x * (unsigned)kLansBlock + threadIdx.x) >> 6);
  const int lane = threadIdx.x & 63;
  if (t < n_tensors) {
    double sg, sw;
    tensor_totals(tensors[t], partials, lane, sg, sw);
    if (lane == 0) {
      const double gn = sqrt(sg), pn = sqrt(sw);
      TensorStats st;
      st.grad_norm = gn;
      st.param_norm = pn;
      // multi_tensor_lans.cu:284-286: divide only when normalising and the norm is non-zero
      st.inv_grad_div = (hp.normalize_grad && gn != 0.0) ? 1.0 / (gn + (double)hp.eps) : 1.0;
      st.um_norm = st.ug_norm = st.ratio_m = st.ratio_g = st.reserved = 0.0;
      stats[t] = st;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    // Host scalars of the reference (src/op/dialect/cuda/lans.cc:94-109), evaluated on the device so
    // the step tensor never has to be copied to the host.
    const int step = step_dev ? (int)(*step_dev) : step_host;
    float bc1 = 1.0f, bc2 = 1.0f;
    if (hp.bias_correction == 1) {  // double pow, then one rounding to fp32 (lans.cc:103-104)
      bc1 = (float)(1.0 - pow((double)hp.beta1, (double)step));
      bc2 = (float)(1.0 - pow((double)hp.beta2, (double)step));
    }
    const float beta3 = (hp.grad_averaging == 1) ? __fsub_rn(1.0f, hp.beta1) : 1.0f;
    StepScalars k;
    k.beta1 = hp.beta1;
    k.beta2 = hp.beta2;
    k.one_minus_beta2 = __fsub_rn(1.0f, hp.beta2);  // fp32 subtraction (multi_tensor_lans.cu:291)
    k.beta3 = beta3;
    k.eps = hp.eps;
    k.wd = hp.weight_decay;
    k.inv_bc1 = 1.0 / (double)bc1;
    k.inv_bc2 = 1.0 / (double)bc2;
    k.lr = hp.learning_rate;
    k.mode = hp.mode;
    k.pad = 0;
    *scalars = k;
  }
}

__global__ __launch_bounds__(kLansBlock) void lans_finish_b(
    const TensorRec* __restrict__ tensors, int32_t n_tensors, const double* __restrict__ partials,
    TensorStats* __restrict__ stats, const StepScalars* __restrict__ scalars) {
  const int t = (int)((blockIdx.x * (unsigned)kLansBlock + threadIdx.x) >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= n_tensors) return;
  double sm, sgg;
  tensor_totals(tensors[t], partials, lane, sm, sgg);
  if (lane == 0) {
    const StepScalars k = *scalars;
    const double unm = sqrt(sm), ung = sqrt(sgg);
    const double pn = stats[t].param_norm;
    // multi_tensor_lans.cu:349-352
    double rm = (unm != 0.0 && pn != 0.0) ? k.lr * (pn / unm) : k.lr;
    double rg = (ung != 0.0 && pn != 0.0) ? k.lr * (pn / ung) : k.lr;
    stats[t].um_norm = unm;
    stats[t].ug_norm = ung;
    stats[t].ratio_m = rm * k.beta1;
    stats[t].ratio_g = rg * k.beta3;
  }
}

// ------------------------------------------------------------------ phase 3: sum u_m^2, sum u_g^2
template <typename G>
__global__ __launch_bounds__(kLansBlock) void lans_norm_u(
    const TensorRec* __restrict__ tensors, const ChunkRec* __restrict__ chunks, int64_t n_chunks,
    float unscale, const StepScalars* __restrict__ scalars, const TensorStats* __restrict__ stats,
    double* __restrict__ partials) {
  __shared__ double red[2][kLansWaves];
  const StepScalars k = *scalars;
  for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
    const ChunkView cv = chunk_view(tensors, chunks, c, (int)sizeof(G));
    const G* g = static_cast<const G*>(cv.g);
    const double inv_gdiv = stats[cv.tensor].inv_grad_div;
    double am = 0.0, au = 0.0;
    if (cv.vec_ok) {
      const int n4 = cv.len >> 2;
      for (int i0 = threadIdx.x; i0 < n4; i0 += kLansBlock * kUnroll) {
        float4 gv[kUnroll], wv[kUnroll], mv[kUnroll], vv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int i = i0 + u * kLansBlock;
          if (i < n4) {
            gv[u] = GradIO<G>::load4(g, i, unscale);
            wv[u] = reinterpret_cast<const float4*>(cv.w)[i];
            mv[u] = reinterpret_cast<const float4*>(cv.m)[i];
            vv[u] = reinterpret_cast<const float4*>(cv.v)[i];
          }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int i = i0 + u * kLansBlock;
          if (i < n4) {
            const Directions d0 = lans_directions(gv[u].x, wv[u].x, mv[u].x, vv[u].x, inv_gdiv, k);
            const Directions d1 = lans_directions(gv[u].y, wv[u].y, mv[u].y, vv[u].y, inv_gdiv, k);
            const Directions d2 = lans_directions(gv[u].z, wv[u].z, mv[u].z, vv[u].z, inv_gdiv, k);
            const Directions d3 = lans_directions(gv[u].w, wv[u].w, mv[u].w, vv[u].w, inv_gdiv, k);
            am += (d0.um * d0.um + d1.um * d1.um) + (d2.um * d2.um + d3.um * d3.um);
            au += (d0.ug * d0.ug + d1.ug * d1.ug) + (d2.ug * d2.ug + d3.ug * d3.ug);
          }
        }
      }
      const int tail = (n4 << 2) + threadIdx.x;
      if (tail < cv.len) {
        const Directions d = lans_directions(GradIO<G>::load1(g, tail, unscale), cv.w[tail],
                                             cv.m[tail], cv.v[tail], inv_gdiv, k);
        am += d.um * d.um;
        au += d.ug * d.ug;
      }
    } else {
      for (int i = threadIdx.x; i < cv.len; i += kLansBlock) {
        const Directions d = lans_directions(GradIO<G>::load1(g, i, unscale), cv.w[i], cv.m[i],
                                             cv.v[i], inv_gdiv, k);
        am += d.um * d.um;
        au += d.ug * d.ug;
      }
    }
    block_sum2(am, au, red);
    if (threadIdx.x == 0) {
      partials[2 * c] = am;
      partials[2 * c + 1] = au;
    }
  }
}

// ------------------------------------------------------------------ phase 5: apply
__device__ __forceinline__ void apply_one(double g, double w, double m, double v, double inv_gdiv,
                                          const StepScalars& k, double rm, double rg, float& w_out,
                                          float& m_out, float& v_out) {
  const Directions d = lans_directions(g, w, m, v, inv_gdiv, k);
  // multi_tensor_lans.cu:386: p - ratio_m*update_m - ratio_g*update_g, left to right
  w_out = (float)((w - rm * d.um) - rg * d.ug);
  m_out = (float)d.m1;
  v_out = (float)d.v1;
}

template <typename G>
__global__ __launch_bounds__(kLansBlock) void lans_apply(
    const TensorRec* __restrict__ tensors, const ChunkRec* __restrict__ chunks, int64_t n_chunks,
    float unscale, const StepScalars* __restrict__ scalars,
    const TensorStats* __restrict__ stats) {
  const StepScalars k = *scalars;
  for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
    const ChunkView cv = chunk_view(tensors, chunks, c, (int)sizeof(G));
    const G* g = static_cast<const G*>(cv.g);
    const TensorStats st = stats[cv.tensor];
    const double inv_gdiv = st.inv_grad_div, rm = st.ratio_m, rg = st.ratio_g;
    if (cv.vec_ok) {
      const int n4 = cv.len >> 2;
      for (int i0 = threadIdx.x; i0 < n4; i0 += kLansBlock * kUnroll) {
        float4 gv[kUnroll], wv[kUnroll], mv[kUnroll], vv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int i = i0 + u * kLansBlock;
          if (i < n4) {
            gv[u] = GradIO<G>::load4(g, i, unscale);
            wv[u] = reinterpret_cast<const float4*>(cv.w)[i];
            mv[u] = reinterpret_cast<const float4*>(cv.m)[i];
            vv[u] = reinterpret_cast<const float4*>(cv.v)[i];
          }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int i = i0 + u * kLansBlock;
          if (i < n4) {
            float4 wo, mo, vo;
            apply_one(gv[u].x, wv[u].x, mv[u].x, vv[u].x, inv_gdiv, k, rm, rg, wo.x, mo.x, vo.x);
            apply_one(gv[u].y, wv[u].y, mv[u].y, vv[u].y, inv_gdiv, k, rm, rg, wo.y, mo.y, vo.y);
            apply_one(gv[u].z, wv[u].z, mv[u].z, vv[u].z, inv_gdiv, k, rm, rg, wo.z, mo.z, vo.z);
            apply_one(gv[u].w, wv[u].w, mv[u].w, vv[u].w, inv_gdiv, k, rm, rg, wo.w, mo.w, vo.w);
            reinterpret_cast<float4*>(cv.w)[i] = wo;
            reinterpret_cast<float4*>(cv.m)[i] = mo;
            reinterpret_cast<float4*>(cv.v)[i] = vo;
          }
        }
      }
      const int tail = (n4 << 2) + threadIdx.x;
      if (tail < cv.len) {
        float wo, mo, vo;
        apply_one(GradIO<G>::load1(g, tail, unscale), cv.w[tail], cv.m[tail], cv.v[tail], inv_gdiv,
                  k, rm, rg, wo, mo, vo);
        cv.w[tail] = wo;
        cv.m[tail] = mo;
        cv.v[tail] = vo;
      }
    } else {
      for (int i = threadIdx.x; i < cv.len; i += kLansBlock) {
        float wo, mo, vo;
        apply_one(GradIO<G>::load1(g, i, unscale), cv.w[i], cv.m[i], cv.v[i], inv_gdiv, k, rm, rg,
                  wo, mo, vo);
        cv.w[i] = wo;
        cv.m[i] = mo;
        cv.v[i] = vo;
      }
    }
  }
}

}  // namespace

// ------------------------------------------------------------------ launchers
void launch_norm_gw(int grad_dtype, unsigned grid, hipStream_t s, const TensorRec* tensors,
                    const ChunkRec* chunks, int64_t n_chunks, float unscale, double* partials) {
  if (grad_dtype == RAFHIP_F16)
    hipLaunchKernelGGL(lans_norm_gw<_Float16>, dim3(grid), dim3(kLansBlock), 0, s, tensors, chunks,
                       n_chunks, unscale, partials);
  else
    hipLaunchKernelGGL(lans_norm_gw<float>, dim3(grid), dim3(kLansBlock), 0, s, tensors, chunks,
                       n_chunks, unscale, partials);
}

void launch_finish_a(unsigned grid, hipStream_t s, const TensorRec* tensors, int32_t n_tensors,
                     const double* partials, TensorStats* stats, StepScalars* scalars,
                     const float* step_dev, int32_t step_host, HParamsPod hp) {
  hipLaunchKernelGGL(lans_finish_a, dim3(grid), dim3(kLansBlock), 0, s, tensors, n_tensors,
                     partials, stats, scalars, step_dev, step_host, hp);
}

void launch_norm_u(int grad_dtype, unsigned grid, hipStream_t s, const TensorRec* tensors,
                   const ChunkRec* chunks, int64_t n_chunks, float unscale,
                   const StepScalars* scalars, const TensorStats* stats, double* partials) {
  if (grad_dtype == RAFHIP_F16)
    hipLaunchKernelGGL(lans_norm_u<_Float16>, dim3(grid), dim3(kLansBlock), 0, s, tensors, chunks,
                       n_chunks, unscale, scalars, stats, partials);
  else
    hipLaunchKernelGGL(lans_norm_u<float>, dim3(grid), dim3(kLansBlock), 0, s, tensors, chunks,
                       n_chunks, unscale, scalars, stats, partials);
}

void launch_finish_b(unsigned grid, hipStream_t s, const TensorRec* tensors, int32_t n_tensors,
                     const double* partials, TensorStats* stats, const StepScalars* scalars) {
  hipLaunchKernelGGL(lans_finish_b, dim3(grid), dim3(kLansBlock), 0, s, tensors, n_tensors,
                     partials, stats, scalars);
}

void launch_apply(int grad_dtype, unsigned grid, hipStream_t s, const TensorRec* tensors,
                  const ChunkRec* chunks, int64_t n_chunks, float unscale,
                  const StepScalars* scalars, const TensorStats* stats) {
  if (grad_dtype == RAFHIP_F16)
    hipLaunchKernelGGL(lans_apply<_Float16>, dim3(grid), dim3(kLansBlock), 0, s, tensors, chunks,
                       n_chunks, unscale, scalars, stats);
  else
    hipLaunchKernelGGL(lans_apply<float>, dim3(grid), dim3(kLansBlock), 0, s, tensors, chunks,
                       n_chunks, unscale, scalars, stats);
}

}  // namespace rafhip

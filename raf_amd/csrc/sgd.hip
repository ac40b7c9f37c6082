// Momentum-SGD step for gfx950: the HIP stand-in for the TVM-generated `raf.op.tvm.sgd` kernel
// (python/raf/_tvm_op/sgd.py:13-30 in the reference).
//
// The rule is four fp32 operations, each rounded on its own:
//     t = mu*v0 ; v1 = t + dx ; s = lr*v1 ; x1 = x0 - s
// HIP contracts a*b+c into an FMA by default (-ffp-contract=fast), and its __fmul_rn/__fadd_rn are
// plain operators that do not stop that, so contraction is switched off for this whole file with
// the pragma below: the output is then bit-identical to the reference's CPU lowering (generic
// x86-64, no FMA).  fp32 denormals are kept (no flush-to-zero), as on the CPU.
//
// Memory-bound: 12 B read + 8 B written per element.  Each lane moves 16 bytes per access
// (four floats), a wavefront covers 1 KiB per access, and the grid is a fixed multiple of the CU count
// walking the tensor with a grid stride, so consecutive wavefronts touch consecutive 1 KiB lines.
#include <hip/hip_runtime.h>

//
// The multi-tensor step further down applies the same four operations, in place, to a whole list
// of parameters in ONE launch; it stands in for what the reference's traced optimizer emits per
// parameter -- cast(dx), multiply, add(out=v), multiply, subtract(out=w), cast, add(out=p)
// (python/raf/optim/sgd.py:187-215) -- and for the one-op-call-per-parameter loop of its imperative
// optimizer (sgd.py:51-58).
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <new>
#include <vector>

#include "device_table.h"
#include "half_types.h"
#include "status.h"

#pragma clang fp contract(off)

namespace rafhip {
namespace {

constexpr int kSgdBlock = 256;
constexpr int kSgdUnroll = 2;  // float4 groups in flight per lane per trip (cache-resident lists)

__device__ __forceinline__ void sgd_elem(float x0, float dx, float v0, float lr, float mu,
                                         float& v1, float& x1) {
  const float t = mu * v0;
  v1 = t + dx;
  const float s = lr * v1;
  x1 = x0 - s;
}

// Vector path: all five pointers 16-byte aligned.  n4 = number of whole float4 groups.
template <int kSgdUnroll>
__global__ __launch_bounds__(kSgdBlock) void sgd_vec4_kernel(
    const f32x4* x, const f32x4* dx, const f32x4* v, f32x4* v_out, f32x4* x_out, int64_t n4,
    float lr, float mu) {
  const int64_t stride = (int64_t)gridDim.x * kSgdBlock * kSgdUnroll;
  for (int64_t base = (int64_t)blockIdx.x * kSgdBlock * kSgdUnroll + threadIdx.x; base < n4;
       base += stride) {
    f32x4 rx[kSgdUnroll], rd[kSgdUnroll], rv[kSgdUnroll];
#pragma unroll
    for (int u = 0; u < kSgdUnroll; ++u) {
      const int64_t i = base + (int64_t)u * kSgdBlock;
      if (i < n4) {  // streamed once: non-temporal, so the Infinity Cache does not allocate lines
        rx[u] = __builtin_nontemporal_load(&x[i]);
        rd[u] = __builtin_nontemporal_load(&dx[i]);
        rv[u] = __builtin_nontemporal_load(&v[i]);
      }
    }
#pragma unroll
    for (int u = 0; u < kSgdUnroll; ++u) {
      const int64_t i = base + (int64_t)u * kSgdBlock;
      if (i < n4) {
        float v1[4], x1[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) sgd_elem(rx[u][j], rd[u][j], rv[u][j], lr, mu, v1[j], x1[j]);
        const f32x4 nv = {v1[0], v1[1], v1[2], v1[3]};
        const f32x4 nx = {x1[0], x1[1], x1[2], x1[3]};
        __builtin_nontemporal_store(nv, &v_out[i]);
        __builtin_nontemporal_store(nx, &x_out[i]);
      }
    }
  }
}

// Scalar path: unaligned tensors, and the < 4-element tail of the vector path.
__global__ __launch_bounds__(kSgdBlock) void sgd_scalar_kernel(
    const float* x, const float* dx, const float* v,
    float* v_out, float* x_out, int64_t begin, int64_t n, float lr,
    float mu) {
  const int64_t stride = (int64_t)gridDim.x * kSgdBlock;
  for (int64_t i = begin + (int64_t)blockIdx.x * kSgdBlock + threadIdx.x; i < n; i += stride) {
    float nv, nx;
    sgd_elem(x[i], dx[i], v[i], lr, mu, nv, nx);
    v_out[i] = nv;
    x_out[i] = nx;
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ------------------------------------------------------------------ other element types
// The reference's compute is written in the dtype of x0 (tir.const(value, dtype=x0.dtype),
// python/raf/_tvm_op/sgd.py:18-19), so the op also exists for float64 and the 16-bit types.  Each
// of the four operations is rounded to the element type on its own.  For binary16 and bfloat16
// the operation is done the way a CPU without half arithmetic does it (the reference's CPU target
// is bare `llvm`, include/raf/device.h:97-104): widen to fp32, operate there, round the result
// back.  fp32 carries 24 >= 2p + 2 significant bits for both 16-bit formats (p = 11 and 8), so
// the two roundings in a row give the correctly rounded 16-bit result: the same bits as native
// half arithmetic would.
template <typename T>
struct SgdElem;
template <>
struct SgdElem<double> {
  typedef double Store;
  static constexpr int kWide = 2;  // elements per 16-byte access
  static __device__ __forceinline__ double mul(double a, double b) { return a * b; }
  static __device__ __forceinline__ double add(double a, double b) { return a + b; }
  static __device__ __forceinline__ double sub(double a, double b) { return a - b; }
  static double from_double(double x) { return x; }
};
template <>
struct SgdElem<_Float16> {
  typedef _Float16 Store;
  static constexpr int kWide = 8;
  static __device__ __forceinline__ _Float16 mul(_Float16 a, _Float16 b) { return (_Float16)((float)a * (float)b); }
  static __device__ __forceinline__ _Float16 add(_Float16 a, _Float16 b) { return (_Float16)((float)a + (float)b); }
  static __device__ __forceinline__ _Float16 sub(_Float16 a, _Float16 b) { return (_Float16)((float)a - (float)b); }
  static _Float16 from_double(double x) { return (_Float16)x; }  // one rounding, like the constant's
};
template <>
struct SgdElem<Bf16> {
  typedef unsigned short Store;
  static constexpr int kWide = 8;
  static __device__ __forceinline__ unsigned short mul(unsigned short a, unsigned short b) {
    return bf16_narrow(bf16_widen(a) * bf16_widen(b));
  }
  static __device__ __forceinline__ unsigned short add(unsigned short a, unsigned short b) {
    return bf16_narrow(bf16_widen(a) + bf16_widen(b));
  }
  static __device__ __forceinline__ unsigned short sub(unsigned short a, unsigned short b) {
    return bf16_narrow(bf16_widen(a) - bf16_widen(b));
  }
  // double -> bfloat16 with one rounding to nearest even (the value is finite and far from the
  // range limits for any usable learning rate or momentum)
  static unsigned short from_double(double x) {
    const float f = (float)x;  // candidate; fix the double rounding by comparing neighbours
    unsigned u;
    std::memcpy(&u, &f, 4);
    unsigned lo = u & 0xFFFF0000u, hi = lo + 0x10000u;
    float flo, fhi;
    std::memcpy(&flo, &lo, 4);
    std::memcpy(&fhi, &hi, 4);
    const double dlo = std::fabs(x - (double)flo), dhi = std::fabs((double)fhi - x);
    const bool up = dhi < dlo || (dhi == dlo && ((lo >> 16) & 1u));
    return (unsigned short)((up ? hi : lo) >> 16);
  }
};

template <typename T>
__device__ __forceinline__ void sgd_elem_t(typename SgdElem<T>::Store x0, typename SgdElem<T>::Store dx,
                                           typename SgdElem<T>::Store v0, typename SgdElem<T>::Store lr,
                                           typename SgdElem<T>::Store mu, typename SgdElem<T>::Store& v1,
                                           typename SgdElem<T>::Store& x1) {
  v1 = SgdElem<T>::add(SgdElem<T>::mul(mu, v0), dx);
  x1 = SgdElem<T>::sub(x0, SgdElem<T>::mul(lr, v1));
}

// One 16-byte access per lane and array and trip; `vec` = every pointer is 16-byte aligned, else
// element by element.
template <typename T>
__global__ __launch_bounds__(kSgdBlock) void sgd_typed_kernel(
    const typename SgdElem<T>::Store* x, const typename SgdElem<T>::Store* dx,
    const typename SgdElem<T>::Store* v, typename SgdElem<T>::Store* v_out,
    typename SgdElem<T>::Store* x_out, int64_t n, typename SgdElem<T>::Store lr,
    typename SgdElem<T>::Store mu, int vec) {
  typedef typename SgdElem<T>::Store E;
  constexpr int kW = SgdElem<T>::kWide;
  typedef E Wide __attribute__((ext_vector_type(kW)));
  const int64_t stride = (int64_t)gridDim.x * kSgdBlock;
  const int64_t first = (int64_t)blockIdx.x * kSgdBlock + threadIdx.x;
  int64_t done = 0;
  if (vec) {
    const int64_t nw = n / kW;
    for (int64_t i = first; i < nw; i += stride) {
      const Wide rx = __builtin_nontemporal_load(reinterpret_cast<const Wide*>(x) + i);
      const Wide rd = __builtin_nontemporal_load(reinterpret_cast<const Wide*>(dx) + i);
      const Wide rv = __builtin_nontemporal_load(reinterpret_cast<const Wide*>(v) + i);
      Wide nv, nx;
#pragma unroll
      for (int j = 0; j < kW; ++j) {
        E a, b;
        sgd_elem_t<T>(rx[j], rd[j], rv[j], lr, mu, a, b);
        nv[j] = a;
        nx[j] = b;
      }
      __builtin_nontemporal_store(nv, reinterpret_cast<Wide*>(v_out) + i);
      __builtin_nontemporal_store(nx, reinterpret_cast<Wide*>(x_out) + i);
    }
    done = nw * kW;
  }
  for (int64_t i = done + first; i < n; i += stride) {
    E a, b;
    sgd_elem_t<T>(x[i], dx[i], v[i], lr, mu, a, b);
    v_out[i] = a;
    x_out[i] = b;
  }
}

template <typename T>
void launch_sgd_typed(const void* x, const void* dx, const void* v, void* v_out, void* x_out, int64_t n,
                      double learning_rate, double mu, hipStream_t s) {
  typedef typename SgdElem<T>::Store E;
  const bool vec = aligned16(x) && aligned16(dx) && aligned16(v) && aligned16(v_out) && aligned16(x_out);
  const int64_t items = vec ? (n + SgdElem<T>::kWide - 1) / SgdElem<T>::kWide : n;
  int64_t blocks = (items + kSgdBlock - 1) / kSgdBlock;
  if (blocks > kMaxGridBlocks) blocks = kMaxGridBlocks;
  // One rounding double -> element type, as tir.const(value, dtype) makes the constant.
  hipLaunchKernelGGL(sgd_typed_kernel<T>, dim3((unsigned)blocks), dim3(kSgdBlock), 0, s,
                     static_cast<const E*>(x), static_cast<const E*>(dx), static_cast<const E*>(v),
                     static_cast<E*>(v_out), static_cast<E*>(x_out), n,
                     SgdElem<T>::from_double(learning_rate), SgdElem<T>::from_double(mu), vec ? 1 : 0);
}

// ------------------------------------------------------------------ multi-tensor, in place
// 1024 elements per work item: a workgroup makes one trip (one 16-byte access per lane and array)
// and ends, so no wavefront ever holds loads back behind its own stores.  Measured on the
// BERT-large list: 6.29 TB/s, against 5.80-5.86 with 2048 and 5.67-5.85 with 4096 elements per item.
constexpr int kSgdChunkShift = 10;

struct SgdRec {  // 48 bytes, one per parameter
  float* x;      // fp32 (master) weight, updated in place
  const void* dx;  // gradient: fp32, binary16 or bfloat16
  float* v;      // fp32 velocity, updated in place
  void* p;       // optional 16-bit copy of the new weight (the model's parameter) or null
  int64_t numel;
  int32_t vec_ok;  // every pointer aligned for 4-element lane accesses
  int32_t reserved;
};

struct SgdItem {
  int32_t tensor;
  int32_t chunk;
};

template <typename G, bool kNT, int kSgdUnroll>
__global__ __launch_bounds__(kSgdBlock) void sgd_multi_kernel(const SgdRec* recs,
                                                              const SgdItem* items,
                                                              int64_t n_items, float lr, float mu,
                                                              int p_is_bf16, int chunk_shift) {
  const int kSgdChunk = 1 << chunk_shift;
  for (int64_t it = blockIdx.x; it < n_items; it += gridDim.x) {
    const SgdItem item = items[it];
    const SgdRec r = recs[item.tensor];
    const int64_t begin = (int64_t)item.chunk << chunk_shift;
    const int64_t rest = r.numel - begin;
    const int len = rest < kSgdChunk ? (int)rest : kSgdChunk;
    float* x = r.x + begin;
    float* v = r.v + begin;
    const char* dx = static_cast<const char*>(r.dx) + begin * (int64_t)sizeof(G);
    unsigned short* p = r.p ? static_cast<unsigned short*>(r.p) + begin : nullptr;
    int done = 0;
    if (r.vec_ok) {
      const int n4 = len >> 2;
      RAFHIP_GLOBAL f32x4* x4 = (RAFHIP_GLOBAL f32x4*)x;
      RAFHIP_GLOBAL f32x4* v4 = (RAFHIP_GLOBAL f32x4*)v;
      for (int i0 = threadIdx.x; i0 < n4; i0 += kSgdBlock * kSgdUnroll) {
        f32x4 rx[kSgdUnroll], rd[kSgdUnroll], rv[kSgdUnroll];
#pragma unroll
        for (int u = 0; u < kSgdUnroll; ++u) {
          const int i = i0 + u * kSgdBlock;
          if (i < n4) {
            rx[u] = ldg<kNT>((const RAFHIP_GLOBAL f32x4*)x4 + i);
            rd[u] = GradIO<G>::template load4<kNT>(dx, i, 1.0f);  // exact widening, no scaling
            rv[u] = ldg<kNT>((const RAFHIP_GLOBAL f32x4*)v4 + i);
          }
        }
#pragma unroll
        for (int u = 0; u < kSgdUnroll; ++u) {
          const int i = i0 + u * kSgdBlock;
          if (i < n4) {
            float v1[4], x1[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) sgd_elem(rx[u][j], rd[u][j], rv[u][j], lr, mu, v1[j], x1[j]);
            stg<kNT>(v4 + i, f32x4{v1[0], v1[1], v1[2], v1[3]});
            stg<kNT>(x4 + i, f32x4{x1[0], x1[1], x1[2], x1[3]});
            if (p)  // uniform over the workgroup
              stg<kNT>((RAFHIP_GLOBAL u16x4*)p + i,
                       u16x4{narrow16(x1[0], p_is_bf16 != 0), narrow16(x1[1], p_is_bf16 != 0),
                             narrow16(x1[2], p_is_bf16 != 0), narrow16(x1[3], p_is_bf16 != 0)});
          }
        }
      }
      done = n4 << 2;
    }
    for (int i = done + (int)threadIdx.x; i < len; i += kSgdBlock) {
      float nv, nx;
      sgd_elem(x[i], GradIO<G>::load1(dx, i, 1.0f), v[i], lr, mu, nv, nx);
      v[i] = nv;
      x[i] = nx;
      if (p) p[i] = narrow16(nx, p_is_bf16 != 0);
    }
  }
}

// A list whose x, dx, v total less than this sits in the 256 MB Infinity Cache between steps and
// is better off cached; larger ones stream with the non-temporal hint.
constexpr int64_t kSgdStreamFromBytes = 160LL << 20;

template <typename G>
void launch_sgd_multi(bool stream_nt, unsigned grid, hipStream_t s, const SgdRec* recs,
                      const SgdItem* items, int64_t n_items, float lr, float mu, int p_is_bf16) {
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kSgdBlock), 0, s, recs, items, n_items, lr, mu,
                       p_is_bf16, kSgdChunkShift);
  };
  if (stream_nt)
    go(sgd_multi_kernel<G, true, 1>);  // 1024-element items: one access per lane and array
  else
    go(sgd_multi_kernel<G, false, kSgdUnroll>);
}

}  // namespace
}  // namespace rafhip

extern "C" int rafhip_sgd_f32(const float* x, const float* dx, const float* v, float* v_out,
                              float* x_out, int64_t n, double learning_rate, double mu,
                              void* stream) {
  using namespace rafhip;
  clear_error();
  if (n < 0) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_f32: n = %lld < 0", (long long)n);
  if (n == 0) return RAFHIP_OK;
  if (!x || !dx || !v || !v_out || !x_out)
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_f32: null tensor pointer");
  // One rounding double -> fp32, as tir.const(value, "float32") does (sgd.py:18-19).
  const float lr32 = static_cast<float>(learning_rate);
  const float mu32 = static_cast<float>(mu);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int cap = streaming_grid_cap();

  const bool vec = aligned16(x) && aligned16(dx) && aligned16(v) && aligned16(v_out) &&
                   aligned16(x_out);
  int64_t done = 0;
  if (vec && n >= 4) {
    const int64_t n4 = n / 4;
    constexpr int unroll_short = 8;
    constexpr int per_cu = 8;
    // A long tensor is better served by workgroups that make one trip and end (see the
    // multi-tensor kernel): 6.2 against 6.0 TB/s at 16 Mi elements, 6.15 against 5.5 at 256 Mi,
    // equal at 8 Mi.  A short one is launch-bound and wants few, deep workgroups (4 Mi elements:
    // 5.8 against 5.3 TB/s).
    constexpr int64_t one_trip_from = (int64_t)8 << 20;
    const bool one_trip = n >= one_trip_from;
    const int unroll = one_trip ? 1 : unroll_short;
    const int64_t per_block = (int64_t)kSgdBlock * unroll;
    int64_t blocks = (n4 + per_block - 1) / per_block;
    const int64_t gcap = one_trip ? kMaxGridBlocks : (int64_t)cap / 8 * per_cu;
    if (blocks > gcap) blocks = gcap;
    auto go = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kSgdBlock), 0, s,
                         reinterpret_cast<const f32x4*>(x), reinterpret_cast<const f32x4*>(dx),
                         reinterpret_cast<const f32x4*>(v), reinterpret_cast<f32x4*>(v_out),
                         reinterpret_cast<f32x4*>(x_out), n4, lr32, mu32);
    };
    if (one_trip)
      go(sgd_vec4_kernel<1>);
    else
      go(sgd_vec4_kernel<unroll_short>);
    RAFHIP_HIP_TRY(hipGetLastError());
    done = n4 * 4;
  }
  if (done < n) {
    const int64_t rest = n - done;
    int64_t blocks = (rest + kSgdBlock - 1) / kSgdBlock;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(sgd_scalar_kernel, dim3((unsigned)blocks), dim3(kSgdBlock), 0, s, x, dx, v,
                       v_out, x_out, done, n, lr32, mu32);
    RAFHIP_HIP_TRY(hipGetLastError());
  }
  return RAFHIP_OK;
}

extern "C" int rafhip_sgd(const void* x, const void* dx, const void* v, void* v_out, void* x_out,
                          int64_t n, int32_t dtype, double learning_rate, double mu, void* stream) {
  using namespace rafhip;
  if (dtype == RAFHIP_F32)
    return rafhip_sgd_f32(static_cast<const float*>(x), static_cast<const float*>(dx),
                          static_cast<const float*>(v), static_cast<float*>(v_out),
                          static_cast<float*>(x_out), n, learning_rate, mu, stream);
  clear_error();
  if (dtype != RAFHIP_F64 && dtype != RAFHIP_F16 && dtype != RAFHIP_BF16)
    return fail(RAFHIP_ERR_UNSUPPORTED, "rafhip_sgd: dtype %d", dtype);
  if (n < 0) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd: n = %lld < 0", (long long)n);
  if (n == 0) return RAFHIP_OK;
  if (!x || !dx || !v || !v_out || !x_out) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd: null tensor pointer");
  const uintptr_t eb = dtype == RAFHIP_F64 ? 8 : 2;
  for (const void* p : {x, dx, v, (const void*)v_out, (const void*)x_out})
    if (reinterpret_cast<uintptr_t>(p) % eb != 0)
      return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd: a tensor is not element-aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == RAFHIP_F64)
    launch_sgd_typed<double>(x, dx, v, v_out, x_out, n, learning_rate, mu, s);
  else if (dtype == RAFHIP_F16)
    launch_sgd_typed<_Float16>(x, dx, v, v_out, x_out, n, learning_rate, mu, s);
  else
    launch_sgd_typed<Bf16>(x, dx, v, v_out, x_out, n, learning_rate, mu, s);
  RAFHIP_HIP_TRY(hipGetLastError());
  return RAFHIP_OK;
}

// ------------------------------------------------------------------ multi-tensor plan + entry
struct rafhip_sgd_plan {
  int32_t n = 0;
  int32_t grad_dtype = RAFHIP_F32;
  int device = 0;
  std::vector<int64_t> numel;
  int64_t total_elements = 0;
  int64_t n_items = 0;
  void* d_tables = nullptr;
  rafhip::SgdItem* d_items = nullptr;
  rafhip::RecordTables<rafhip::SgdRec> tables;  // device record tables that follow the caller's pointers
  std::vector<rafhip::SgdRec> recs;             // this call's records, built in place: a step allocates nothing
};

namespace {
void free_sgd_plan(rafhip_sgd_plan* p) {
  if (!p) return;
  p->tables.release();
  if (p->d_tables) (void)hipFree(p->d_tables);
  delete p;
}
inline bool aligned_to(const void* p, uintptr_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}
}  // namespace

extern "C" int rafhip_sgd_plan_create(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                                      rafhip_sgd_plan** out_plan) {
  using namespace rafhip;
  clear_error();
  if (!out_plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_plan_create: out_plan is NULL");
  *out_plan = nullptr;
  if (n_tensors < 0 || (n_tensors > 0 && !numel))
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_plan_create: bad tensor list");
  if (grad_dtype != RAFHIP_F32 && grad_dtype != RAFHIP_F16 && grad_dtype != RAFHIP_BF16)
    return fail(RAFHIP_ERR_UNSUPPORTED,
                "rafhip_sgd_plan_create: gradient dtype %d (fp32, fp16 or bf16)", grad_dtype);
  return guarded("rafhip_sgd_plan_create", [&]() -> int {
    std::unique_ptr<rafhip_sgd_plan, void (*)(rafhip_sgd_plan*)> p(new rafhip_sgd_plan(), free_sgd_plan);
    p->n = n_tensors;
    p->grad_dtype = grad_dtype;
    const int64_t kSgdChunk = (int64_t)1 << kSgdChunkShift;
    std::vector<SgdItem> items;
    for (int32_t t = 0; t < n_tensors; ++t) {
      if (numel[t] < 0)
        return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_plan_create: numel[%d] = %lld < 0", t,
                    (long long)numel[t]);
      const int64_t chunks = (numel[t] + kSgdChunk - 1) / kSgdChunk;
      if (chunks > INT32_MAX)
        return fail(RAFHIP_ERR_UNSUPPORTED, "rafhip_sgd_plan_create: tensor %d is too large", t);
      p->numel.push_back(numel[t]);
      p->total_elements += numel[t];
      for (int64_t c = 0; c < chunks; ++c) items.push_back(SgdItem{t, (int32_t)c});
    }
    p->n_items = (int64_t)items.size();
    if (p->n_items == 0) {  // nothing to update: valid, nothing to launch
      *out_plan = p.release();
      return RAFHIP_OK;
    }
    if (hipGetDevice(&p->device) != hipSuccess) {
      (void)hipGetLastError();
      return fail(RAFHIP_ERR_NO_DEVICE, "rafhip_sgd_plan_create: no HIP device available");
    }
    p->recs.resize((size_t)n_tensors);
    hipError_t e = hipMalloc(&p->d_tables, sizeof(SgdItem) * items.size());
    if (e == hipSuccess) {
      p->d_items = static_cast<SgdItem*>(p->d_tables);
      e = p->tables.init((size_t)n_tensors);
    }
    if (e == hipSuccess)
      e = hipMemcpy(p->d_items, items.data(), sizeof(SgdItem) * items.size(), hipMemcpyHostToDevice);
    if (e != hipSuccess) return fail(RAFHIP_ERR_HIP, "rafhip_sgd_plan_create: %s", hipGetErrorString(e));
    *out_plan = p.release();
    return RAFHIP_OK;
  });
}

extern "C" int rafhip_sgd_plan_destroy(rafhip_sgd_plan* plan) {
  rafhip::clear_error();
  free_sgd_plan(plan);
  return RAFHIP_OK;
}

extern "C" int rafhip_sgd_multi_step(rafhip_sgd_plan* plan, float* const* x, const void* const* dx,
                                     float* const* v, void* const* p, int32_t p_dtype,
                                     double learning_rate, double mu, void* stream) {
  using namespace rafhip;
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_multi_step: plan is NULL");
  if (p && p_dtype != RAFHIP_F16 && p_dtype != RAFHIP_BF16)
    return fail(RAFHIP_ERR_UNSUPPORTED,
                "rafhip_sgd_multi_step: weight-copy dtype %d (binary16 or bfloat16)", p_dtype);
  if (plan->n_items == 0) return RAFHIP_OK;
  if (int st = check_plan_device("rafhip_sgd_multi_step", plan->device)) return st;
  if (!x || !dx || !v) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_multi_step: null pointer list");
  return guarded("rafhip_sgd_multi_step", [&]() -> int {
    const uintptr_t g_elem = plan->grad_dtype == RAFHIP_F32 ? 4 : 2;
    std::vector<SgdRec>& recs = plan->recs;  // already n long
    for (int32_t t = 0; t < plan->n; ++t) {
      SgdRec& r = recs[t];
      r = SgdRec{x[t], dx[t], v[t], p ? p[t] : nullptr, plan->numel[t], 0, 0};
      if (r.numel == 0) continue;
      if (!r.x || !r.dx || !r.v)
        return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_multi_step: tensor %d has a null data pointer", t);
      if (!aligned_to(r.x, 4) || !aligned_to(r.v, 4) || !aligned_to(r.dx, g_elem) || !aligned_to(r.p, 2))
        return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_sgd_multi_step: tensor %d is not element-aligned", t);
      r.vec_ok = aligned_to(r.x, 16) && aligned_to(r.v, 16) && aligned_to(r.dx, 4 * g_elem) &&
                 aligned_to(r.p, 8);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const SgdRec* table = nullptr;
    if (int st = sync_tables("rafhip_sgd_multi_step", plan->tables, recs, s, &table)) return st;
    // One rounding double -> fp32, as for the single-tensor op.
    const float lr32 = static_cast<float>(learning_rate);
    const float mu32 = static_cast<float>(mu);
    // One workgroup per item; the kernel strides over what a launch cannot hold.
    const unsigned grid = (unsigned)(plan->n_items < kMaxGridBlocks ? plan->n_items : kMaxGridBlocks);
    const bool nt = plan->total_elements * (int64_t)(8 + g_elem) > kSgdStreamFromBytes;
    const int bf = p_dtype == RAFHIP_BF16 ? 1 : 0;
    if (plan->grad_dtype == RAFHIP_F16)
      launch_sgd_multi<_Float16>(nt, grid, s, table, plan->d_items, plan->n_items, lr32, mu32, bf);
    else if (plan->grad_dtype == RAFHIP_BF16)
      launch_sgd_multi<Bf16>(nt, grid, s, table, plan->d_items, plan->n_items, lr32, mu32, bf);
    else
      launch_sgd_multi<float>(nt, grid, s, table, plan->d_items, plan->n_items, lr32, mu32, bf);
    RAFHIP_HIP_TRY(hipGetLastError());
    return RAFHIP_OK;
  });
}

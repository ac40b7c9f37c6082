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

#include <cstdint>

#include "status.h"

#pragma clang fp contract(off)

namespace rafhip {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));  // native vector (HIP's float4 is a class)

constexpr int kSgdBlock = 256;
constexpr int kSgdUnroll = 2;  // float4 groups in flight per lane per trip

__device__ __forceinline__ void sgd_elem(float x0, float dx, float v0, float lr, float mu,
                                         float& v1, float& x1) {
  const float t = mu * v0;
  v1 = t + dx;
  const float s = lr * v1;
  x1 = x0 - s;
}

// Vector path: all five pointers 16-byte aligned.  n4 = number of whole float4 groups.
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

int grid_cap() {
  // Enough resident wavefronts to cover HBM latency on every CU; the grid-stride loop does the rest.
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
  const int cap = grid_cap();

  const bool vec = aligned16(x) && aligned16(dx) && aligned16(v) && aligned16(v_out) &&
                   aligned16(x_out);
  int64_t done = 0;
  if (vec && n >= 4) {
    const int64_t n4 = n / 4;
    const int64_t per_block = (int64_t)kSgdBlock * kSgdUnroll;
    int64_t blocks = (n4 + per_block - 1) / per_block;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(sgd_vec4_kernel, dim3((unsigned)blocks), dim3(kSgdBlock), 0, s,
                       reinterpret_cast<const f32x4*>(x), reinterpret_cast<const f32x4*>(dx),
                       reinterpret_cast<const f32x4*>(v), reinterpret_cast<f32x4*>(v_out),
                       reinterpret_cast<f32x4*>(x_out), n4, lr32, mu32);
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

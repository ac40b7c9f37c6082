// Device-side data layout and kernels of the multi-tensor LANS step for gfx950.
//
// Work decomposition.  Every tensor is cut into chunks of kChunk elements; the plan keeps, in HBM,
// a tensor table (pointers, element count, first chunk) and a chunk table (tensor, index within
// the tensor).  One workgroup handles one chunk per trip; a phase is ONE launch over all chunks of
// all tensors, however many tensors there are.
//
// A step is five launches on one stream:
//   1. lans_norm_gw   read g,w            -> per-chunk partial sums of g^2 and w^2
//   2. lans_finish_a  per tensor: add the chunk partials in a fixed order -> ||g||, ||w||,
//                     1/(||g||+eps); also turns the device-resident step into bc1, bc2
//   3. lans_norm_u    read g,w,m,v        -> per-chunk partial sums of u_m^2 and u_g^2
//   4. lans_finish_b  per tensor: ||u_m||, ||u_g|| -> the two trust ratios
//   5. lans_apply     read g,w,m,v, recompute the directions, write w,m,v
// No per-element scratch exists: the two update directions are recomputed in 5 instead of being
// stored (the reference stores them: 16 B/element of extra traffic plus a 4 B/element buffer).
//
// Determinism.  A chunk's partial sum depends only on the chunk (fixed lane order, fixed wave
// tree), and the per-tensor finish adds the partials in a fixed order, so results are bit-identical
// from run to run and independent of the grid size.  No atomics anywhere.
//
// Arithmetic.  Loads and stores are fp32 (fp16 for the optional half gradients); every
// per-element operation and every accumulation is float64, rounded once on store.  The weight
// update subtracts a ~1e-5-sized step from the weight, so an fp32 evaluation of the step (or of the
// norms behind the trust ratio) would leave errors far above 1e-5 *relative* on the weights that
// land near zero; float64 keeps every element within an fp32 ulp of the exactly rounded rule.
// gfx950 issues FP64 FMAs at the full vector rate, and the kernels stay HBM-bound.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace rafhip {

constexpr int kLansBlock = 256;                 // 4 wavefronts
constexpr int kLansWaves = kLansBlock / 64;
constexpr int kChunk = 16384;                   // elements per chunk (multiple of 4 * kLansBlock)
constexpr int kUnroll = 2;                      // 4-element groups in flight per lane per trip

struct TensorRec {  // 48 bytes, one per tensor
  const void* g;
  float* w;
  float* m;
  float* v;
  int64_t numel;
  int32_t first_chunk;
  int32_t vec_ok;  // 1: every base pointer allows 128-bit (fp16 g: 64-bit) lane accesses
};

struct ChunkRec {  // 8 bytes, one per chunk
  int32_t tensor;
  int32_t index;  // chunk number inside its tensor
};

// Global scalars of a step, produced on the device by lans_finish_a (256 bytes reserved).
struct StepScalars {
  double beta1, beta2, one_minus_beta2, beta3;
  double eps, wd, inv_bc1, inv_bc2;
  double lr;
  int32_t mode;
  int32_t pad;
};

struct TensorStats {  // 64 bytes, one per tensor
  double grad_norm, param_norm, inv_grad_div;  // inv_grad_div = 1/(||g||+eps) or 1
  double um_norm, ug_norm;
  double ratio_m, ratio_g;  // beta1 * trust ratio of u_m, beta3 * trust ratio of u_g
  double reserved;
};

// Host-side copy of the hyper-parameters handed to lans_finish_a by value.
struct HParamsPod {
  float learning_rate, beta1, beta2, eps, weight_decay;
  int32_t bias_correction, grad_averaging, mode, normalize_grad;
};

void launch_norm_gw(int grad_dtype, unsigned grid, hipStream_t s, const TensorRec* tensors,
                    const ChunkRec* chunks, int64_t n_chunks, float unscale, double* partials);
void launch_finish_a(unsigned grid, hipStream_t s, const TensorRec* tensors, int32_t n_tensors,
                     const double* partials, TensorStats* stats, StepScalars* scalars,
                     const float* step_dev, int32_t step_host, HParamsPod hp);
void launch_norm_u(int grad_dtype, unsigned grid, hipStream_t s, const TensorRec* tensors,
                   const ChunkRec* chunks, int64_t n_chunks, float unscale,
                   const StepScalars* scalars, const TensorStats* stats, double* partials);
void launch_finish_b(unsigned grid, hipStream_t s, const TensorRec* tensors, int32_t n_tensors,
                     const double* partials, TensorStats* stats, const StepScalars* scalars);
void launch_apply(int grad_dtype, unsigned grid, hipStream_t s, const TensorRec* tensors,
                  const ChunkRec* chunks, int64_t n_chunks, float unscale,
                  const StepScalars* scalars, const TensorStats* stats);

}  // namespace rafhip

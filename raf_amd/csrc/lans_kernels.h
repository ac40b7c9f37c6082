// Device-side data layout and launchers of the multi-tensor LANS step for gfx950.
//
// Work decomposition.  Every tensor is cut into chunks of kChunk elements (kSmallChunk for small
// tensors); the plan keeps, in HBM,
// a tensor table (pointers, element count, first chunk) and a work list of (phase, tensor, chunk)
// items.  One workgroup handles one item at a time.
//
// The rule needs three passes over a tensor, separated by tensor-wide reductions:
//   A  read g             -> per-chunk partial sums of g^2                  -> ||g||
//   B  read g,w,m,v       -> per-chunk partial sums of u_m^2, u_g^2, w^2  -> ||w||, trust ratios
//   C  read g,w,m,v, recompute the update directions, write w,m,v
// No per-element scratch exists: the directions are recomputed in C instead of being stored (the
// reference stores them: 16 B/element of extra traffic plus a 4 B/element buffer).
//
// Two schedules run the same per-chunk code and give bit-identical results:
//   phased     five launches (A, finish, B, finish, C), each over all chunks of all tensors; the
//              first also writes the step scalars.  Lists of short tensors need no finish launches.
//   pipelined  one small set-up launch plus ONE persistent launch.  Tensors are packed into groups
//              whose working set is a fraction of the 256 MB Infinity Cache, and the work list
//              interleaves pass A of group s with pass B of group s-1 and pass C of group s-2, so
//              that pass B finds the group's gradient, and pass C its w, m, v, in the cache
//              instead of HBM.  Workgroups
//              draw items from an atomic ticket.  Chunk items of pass A and B just store their
//              partial sums; a "finish" item per tensor and pass, placed after them in the list,
//              waits for those partials, adds them and publishes the tensor's statistics; items of
//              pass B (C) wait for the statistics they need.  All waiting is on single 8-byte words
//              that go from a "not ready" pattern to their final value exactly once per step, so
//              no counters, flags or fences are involved.  Every item a waiter depends on has an
//              earlier ticket and is therefore already held by a running workgroup, so the waits
//              always end; they are bounded anyway, and a time-out raises an error flag instead
//              of hanging.
//
// Determinism.  A chunk's partial sum depends only on the chunk (fixed lane order, fixed wave
// tree); a tensor's total adds its chunk partials in a fixed order whichever workgroup does it.
// Results are bit-identical from run to run, across grid sizes and across the two schedules.
// The only atomic read-modify-write is the work-list ticket; values are never accumulated
// atomically.
//
// Mixed precision.  Gradients may arrive as binary16 or bfloat16 (widened exactly on load, which
// replaces the reference's group_cast, python/raf/optim/lans.py:261-265), and pass C can write,
// next to the fp32 weight, its round-to-nearest-even 16-bit copy (replacing the cast + copy into
// the model's parameter, lans.py:289-291, :303-305).
//
// Arithmetic.  Loads and stores are fp32 (16-bit for the optional half gradients); every
// per-element operation and every accumulation is float64, rounded once on store.  The weight
// update subtracts a ~1e-5-sized step from the weight, so an fp32 evaluation of the step (or of the
// norms behind the trust ratio) would leave errors far above 1e-5 *relative* on the weights that
// land near zero.  gfx950 issues FP64 FMAs at the full vector rate; square root and reciprocal are
// the hardware approximations (2^-24) plus one Newton step (2^-47), ample for an fp32 result.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace rafhip {

constexpr int kLansBlock = 256;  // 4 wavefronts
constexpr int kLansWaves = kLansBlock / 64;
constexpr int kChunk = 8192;     // elements per chunk (multiple of 4 * kLansBlock) ...
constexpr int kSmallChunk = 4096;              // ... and of tensors below kSmallTensorBelow elements:
constexpr int64_t kSmallTensorBelow = 1 << 19;  // finer work for lists of small tensors, which are
                                                // short of parallelism, not of bandwidth
constexpr int kChunksPerAShift = 3;
constexpr int kChunksPerA = 1 << kChunksPerAShift;   // pass A reads 2-4 bytes per element, so its unit of work (and of
                                 // partial sums) is 8 chunks; its partial lives in the first one's slot
#ifndef RAFHIP_LANS_UNROLL
#define RAFHIP_LANS_UNROLL 2
#endif
constexpr int kUnroll = RAFHIP_LANS_UNROLL;  // 4-element groups in flight per lane per trip
constexpr int kPartialSlots = 4; // doubles per chunk: [0] sum g^2 | [1] sum u_m^2 [2] sum u_g^2 [3] sum w^2

// A tensor's chunk size depends on its own element count alone, so its result does not depend on
// which list it is part of.
__host__ __device__ inline int chunk_shift_for(int64_t numel) {  // chunks are powers of two
  return numel < kSmallTensorBelow ? 12 : 13;
}
__host__ __device__ inline int chunk_elems_for(int64_t numel) { return 1 << chunk_shift_for(numel); }
constexpr int kChunkShift = 13;  // log2 of the largest chunk
static_assert(kSmallChunk == 1 << 12 && kChunk == 1 << kChunkShift, "chunk_shift_for must match the chunk sizes");

struct TensorRec {  // 64 bytes, one per tensor
  const void* g;
  float* w;
  float* m;
  float* v;
  void* p;  // optional 16-bit copy of the new weight (the model's half-precision parameter) or null
  int64_t numel;
  int32_t first_chunk;
  int32_t vec_ok;  // 1: every base pointer is aligned for 4-element lane accesses
  int32_t chunk_shift;  // chunk_shift_for(numel): the tensor's chunks hold 1 << chunk_shift elements
  int32_t reserved;
};

// One unit of work: kind in the top three bits of `chunk_phase`, chunk number within the tensor
// below.  A/B/C: one chunk of that pass.  FinishA/FinishB: add the tensor's chunk partials of the
// pass and publish its statistics.  Whole: a one-chunk tensor taken through all three passes by
// one workgroup.
enum : uint32_t {
  kPhaseA = 0,
  kPhaseB = 1,
  kPhaseC = 2,
  kPhaseWhole = 3,
  kPhaseFinishA = 4,
  kPhaseFinishB = 5
};
struct WorkItem {
  int32_t tensor;
  uint32_t chunk_phase;
};
// chunk_phase: [31..29] kind | [28] streaming | [27..0] chunk.
//   streaming  the item belongs to a tensor too large for the Infinity Cache: all of its accesses
//              carry the non-temporal hint, so that it flows past the cache without evicting the
//              groups that live there between their passes.
constexpr uint32_t kPhaseShift = 29;
constexpr uint32_t kStreamBit = 1u << 28;
constexpr uint32_t kChunkMask = kStreamBit - 1;

// Global scalars of a step, produced on the device from the step tensor (256 bytes reserved).
struct StepScalars {
  double beta1, beta2, one_minus_beta2, beta3;
  double eps, wd, inv_bc1, inv_bc2;
  double lr;
  double decay_into_grad;  // 1 in L2 mode (decay joins the scaled gradient), else 0
  double decay_into_dir;   // 1 in decoupled mode (decay is added to both directions), else 0
  int32_t normalize_grad;
  int32_t pad;
};

struct TensorStats {  // 64 bytes = 8 words, one per tensor; "not ready" pattern until published
  double grad_norm, param_norm, inv_grad_div;  // inv_grad_div = 1/(||g||+eps) or 1
  double um_norm, ug_norm;
  double ratio_m, ratio_g;  // beta1 * trust ratio of u_m, beta3 * trust ratio of u_g
  double reserved;
};

// Synchronisation words of the pipelined schedule; reset by the set-up launch of every step.
struct SyncHeader {
  uint32_t ticket;  // next work item
  uint32_t error;   // 1 if a bounded wait ran out
  uint32_t pad[2];
};

struct HParamsPod {
  float learning_rate, beta1, beta2, eps, weight_decay;
  int32_t bias_correction, grad_averaging, mode, normalize_grad;
};

struct LansDeviceArgs {
  const TensorRec* tensors;
  int32_t n_tensors;
  const WorkItem* items;  // phased, passes B and C: every chunk of every tensor, n_chunks long
  int64_t n_chunks;
  const WorkItem* items_a;  // phased, pass A: every pass-A unit (kChunksPerA chunks), n_items_a long
  int64_t n_items_a;
  uint32_t n_items;       // pipelined work-list length
  const WorkItem* pipeline_items;
  uint32_t spin_limit;    // pipelined: bound of every wait, in polls
  uint32_t* host_error;   // pipelined: pinned host word raised together with sync->error, or nullptr
  float unscale;          // every gradient element is multiplied by this first (loss-scale undo) ...
  const float* unscale_dev;    // ... or, when not null, by the fp32 value this device pointer holds
  const float* found_inf_dev;  // optional: a non-zero fp32 value here turns the whole step into a no-op
  int32_t p_is_bf16;      // dtype of the optional 16-bit weight copies: 0 binary16, 1 bfloat16
  StepScalars* scalars;
  TensorStats* stats;
  double* partials;       // kPartialSlots doubles per chunk
  SyncHeader* sync;
  uint64_t* trace;        // optional diagnostics: 4 words per pipelined item, or nullptr
};

void launch_prepare(hipStream_t s, const LansDeviceArgs& a, const float* step_dev,
                    int32_t step_host, HParamsPod hp);
// `streaming`: the list is much larger than the Infinity Cache (non-temporal accesses) or fits in it.
// `inline_finish` (non-streaming lists only): every tensor has at most kInlineFinishChunks chunks,
// so the passes add the partials themselves and the two finish launches are skipped.
constexpr int kInlineFinishChunks = 32;
// The first pass also writes the step scalars: no set-up launch in this schedule.
// `apply_slice_shift`: a streaming list's last pass works in slices of 2^that many elements
// (10 to the chunk shift), 0 for whole chunks.
void launch_phased(int grad_dtype, bool streaming, bool inline_finish, hipStream_t s,
                   const LansDeviceArgs& a, const float* step_dev, int32_t step_host,
                   HParamsPod hp, hipEvent_t* marks, int apply_slice_shift);
void launch_pipelined(int grad_dtype, unsigned grid, hipStream_t s, const LansDeviceArgs& a);
// Resident workgroups per CU of the pipelined kernel (occupancy query), 0 on failure.
int pipelined_blocks_per_cu(int grad_dtype);

}  // namespace rafhip

/*
 * rafhip_optim.h -- C ABI of the gfx950 (MI355X) fused optimizer-step kernels that stand in for
 * awslabs/raf's `raf.op.sgd` and `raf.op.lans` backends.
 *
 * Plain C: raw device pointers, element counts, a HIP stream passed as void*.  No C++ or torch
 * types cross this boundary.  Every function returns a rafhip_status (0 = success) unless noted;
 * the text of the last failure on the calling thread is available from rafhip_last_error().
 * No function throws, and none of the *step* functions allocates or frees device memory.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   rafhip_sgd_f32          the TVM-built packed function behind `raf.op.tvm.sgd`:
 *                           python/raf/_tvm_op/sgd.py:13-30, registered at
 *                           src/op/dialect/tvm/optimizer.cc:44-45 and invoked with
 *                           [x, dx, v, v1, x1] at src/op/dialect/tvm/tvm_utils.cc:92-133.
 *   rafhip_l2norm           cublasSnrm2 / cublasDnrm2 in device-pointer mode behind
 *                           `raf.op.cublas.l2norm`, src/op/dialect/cublas/l2_norm.cc:52-75.
 *   rafhip_fuse_* / defuse  the per-tensor cudaMemcpyAsync loops of `raf.op.cuda.fuse_tensor` and
 *                           `raf.op.cuda.defuse_tensor`, src/op/dialect/cuda/memory.cc:55-68, :120-134.
 *   rafhip_lans_*           multi_tensor_lans_cuda<float>(...) declared at
 *                           src/op/dialect/cuda/kernels/kernel_util.cuh:25-34 and called from
 *                           LansImpl::Execute, src/op/dialect/cuda/lans.cc:124-130; the plan object
 *                           takes the role of LansImpl's constructor state (lans.cc:27-83) and
 *                           rafhip_lans_workspace_bytes that of its RequestWorkspace calls
 *                           (lans.cc:66-77).
 */
#ifndef RAFHIP_OPTIM_H_
#define RAFHIP_OPTIM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RAFHIP_ABI_VERSION 1

typedef enum rafhip_status {
  RAFHIP_OK = 0,
  RAFHIP_ERR_INVALID_ARG = 1, /* null pointer, negative size, bad enum, n % 4 != 0 ...        */
  RAFHIP_ERR_UNSUPPORTED = 2, /* dtype or size the kernels do not handle                       */
  RAFHIP_ERR_WORKSPACE = 3,   /* workspace missing, too small or misaligned                    */
  RAFHIP_ERR_HIP = 4,         /* a HIP runtime call failed; message carries hipGetErrorString  */
  RAFHIP_ERR_NO_DEVICE = 5,   /* no usable gfx950 device in this process                       */
  RAFHIP_ERR_HOST = 6         /* host side: out of memory or an unexpected C++ exception       */
} rafhip_status;

typedef enum rafhip_dtype {
  RAFHIP_F32 = 0,
  RAFHIP_F16 = 1, /* IEEE binary16; LANS gradients and 16-bit weight copies only */
  RAFHIP_BF16 = 2, /* bfloat16; LANS gradients and 16-bit weight copies only      */
  RAFHIP_F64 = 3   /* IEEE binary64; rafhip_l2norm only                            */
} rafhip_dtype;

/* ABI version of the loaded library (== RAFHIP_ABI_VERSION it was built with). */
int rafhip_abi_version(void);

/* Message of the last failing call on this thread ("" if none).  Never NULL. */
const char* rafhip_last_error(void);

/* Number of HIP devices visible (0 on a host without a GPU; never fails). */
int rafhip_device_count(void);

/* ------------------------------------------------------------------------------------------ SGD
 * Momentum SGD step of `raf.op.sgd` (python/raf/_tvm_op/sgd.py:16-30):
 *     v_out = fl32(fl32(mu32 * v) + dx)        x_out = fl32(x - fl32(lr32 * v_out))
 * with mu32 = (float)mu, lr32 = (float)learning_rate: four separately rounded fp32 operations,
 * never fused, so the result is bit-identical to the reference's CPU (LLVM) lowering.
 * Out of place like the reference op (src/op/declare/optimizer.cc:22-44); v_out may alias v and
 * x_out may alias x (element i is read before it is written by the same lane).
 * n == 0 is a successful no-op.  All pointers are device pointers of n floats.
 */
int rafhip_sgd_f32(const float* x, const float* dx, const float* v, float* v_out, float* x_out,
                   int64_t n, double learning_rate, double mu, void* stream);

/*
 * The same step in the element type of x, which is how the reference writes the compute
 * (tir.const(value, dtype=x0.dtype), python/raf/_tvm_op/sgd.py:18-19): dtype RAFHIP_F32 (the call
 * above), RAFHIP_F64, RAFHIP_F16 or RAFHIP_BF16; x, dx, v and both outputs share it.  mu and
 * learning_rate are rounded once to the element type; each of the four operations is rounded to
 * the element type on its own -- for the 16-bit types by widening to fp32, operating there and
 * rounding the result back, which is what a CPU without half arithmetic does (the reference's CPU
 * target is bare `llvm`) and gives the correctly rounded 16-bit result.  No test of the reference
 * pins the 16-bit or fp64 bits.
 */
int rafhip_sgd(const void* x, const void* dx, const void* v, void* v_out, void* x_out, int64_t n,
               int32_t dtype, double learning_rate, double mu, void* stream);

/*
 * Multi-tensor momentum SGD, IN PLACE on x and v, one launch for a whole parameter list.  Per
 * element exactly the four roundings above.  It replaces, per step, the op sequence the reference's
 * traced optimizer emits for EVERY parameter -- cast(dx, fp32), multiply, add(out=v), multiply,
 * subtract(out=w), cast(w, dtype), add(out=p) (python/raf/optim/sgd.py:187-215) -- and the
 * one-call-per-parameter loop of its imperative optimizer (sgd.py:51-58).
 *   plan       fixes the element counts and the gradient dtype (RAFHIP_F32, _F16, _BF16; half
 *              gradients are widened exactly, as cast does); owns a small device table.
 *   x, dx, v   host arrays of n_tensors device pointers: fp32 (master) weights, gradients,
 *              fp32 velocities.
 *   p          NULL, or host array of device pointers (entries may be NULL) that receive the new
 *              weight narrowed to p_dtype (RAFHIP_F16 / RAFHIP_BF16), round to nearest even: the
 *              half-precision model parameters.
 * Allocates nothing; one call at a time per plan.
 */
typedef struct rafhip_sgd_plan rafhip_sgd_plan;
int rafhip_sgd_plan_create(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                           rafhip_sgd_plan** out_plan);
int rafhip_sgd_plan_destroy(rafhip_sgd_plan* plan);
int rafhip_sgd_multi_step(rafhip_sgd_plan* plan, float* const* x, const void* const* dx,
                          float* const* v, void* const* p, int32_t p_dtype, double learning_rate,
                          double mu, void* stream);

/* ----------------------------------------------------------------------------------------- LANS
 * Hyper-parameters: the non-tensor schema fields of `raf.op.lans`
 * (scripts/src_codegen/def_schema.py:685-693) in schema order, fp32 like the schema's `float`.
 */
typedef struct rafhip_lans_hparams {
  float learning_rate;
  float beta1;
  float beta2;
  float eps;
  int32_t bias_correction; /* 1: bc_k = 1 - beta_k^step (lans.cc:102-105); else bc_k = 1      */
  float weight_decay;
  int32_t grad_averaging;  /* 1: beta3 = 1 - beta1 (lans.cc:107-109); else beta3 = 1          */
  int32_t mode;            /* 1: decoupled weight decay; 0: L2 on the scaled gradient          */
  int32_t normalize_grad;  /* bool: divide g by (||g|| + eps) when ||g|| != 0                  */
  float grad_unscale;      /* extension: g is multiplied by this first (loss-scale undo); 1.0  */
} rafhip_lans_hparams;

/* Defaults of raf.optim.LANS (python/raf/optim/lans.py:44-55) with grad_unscale = 1. */
void rafhip_lans_default_hparams(rafhip_lans_hparams* hp);

/*
 * A plan fixes what LansImpl's constructor fixes: the number of tensors and their element counts
 * (lans.cc:51-72), plus the gradient dtype.  Creation builds the device-side chunk table (one
 * hipMalloc + upload); the step calls then launch a fixed kernel sequence (see the schedules
 * below) without touching the allocator.  A plan belongs to the device that was current at creation and is not
 * thread-safe: one step at a time per plan.
 */
typedef struct rafhip_lans_plan rafhip_lans_plan;

/* Pure host arithmetic, usable without a GPU: how many chunks a tensor list is cut into and how
 * many workspace bytes a step over it needs (what LansImpl computes at lans.cc:66-77).  Either
 * output pointer may be NULL. */
int rafhip_lans_query_layout(int32_t n_tensors, const int64_t* numel, int64_t* n_chunks_out,
                             int64_t* workspace_bytes_out);

/* Elements per chunk -- the unit of work and of the partial sums of the second and third pass --
 * for a tensor of numel elements (it depends on the tensor's own size only: small tensors are cut
 * finer), and elements per unit of the first pass (a multiple of the chunk: that pass reads the
 * gradient only). */
int32_t rafhip_lans_chunk_elements(int64_t numel);
int32_t rafhip_lans_pass_a_unit_elements(int64_t numel);

/*
 * Schedules of a step; both run the same per-chunk code and give bit-identical results.
 *   PHASED     one launch per pass over all chunks of all tensors plus two small per-tensor
 *              launches between them (5 launches; 3 for a list of short tensors only).
 *   PIPELINED  set-up + ONE persistent launch whose work list interleaves the three passes of
 *              neighbouring cache-sized tensor groups, so that a group's second and third reads
 *              come from the 256 MB Infinity Cache instead of HBM.
 * A plan picks PIPELINED for lists of 64 Mi elements or more and PHASED below (short lists are
 * launch- and latency-bound); RAFHIP_LANS_SCHEDULE=phased|pipelined overrides that per process,
 * rafhip_lans_plan_options.schedule and rafhip_lans_plan_set_schedule per plan.
 */
typedef enum rafhip_lans_schedule {
  RAFHIP_LANS_PHASED = 0,
  RAFHIP_LANS_PIPELINED = 1
} rafhip_lans_schedule;

/*
 * Pure host arithmetic: the work list of the pipelined schedule (as made for a device of 256 CUs)
 * as int32 triples (kind, tensor, index), kind being 0 = pass A unit, 1 = pass B chunk, 2 = pass C
 * chunk, 3 = a one-chunk tensor taken through all three passes by one workgroup, 4 = finish pass A
 * (add the tensor's partials, publish ||g||), 5 = finish pass B (publish ||w|| and the trust
 * ratios); + 8 for an item of a tensor too large for the Infinity Cache, whose accesses bypass it
 * and whose items are spread over the whole list.
 * group_elements <= 0 selects the default group size.  triples_out may be NULL to query the count.
 * The kernel's bounded waits rely on this order, per tensor: every pass-A unit, then finish A,
 * then every pass-B chunk, then finish B, then every pass-C chunk.
 */
int rafhip_lans_pipeline_order(int32_t n_tensors, const int64_t* numel, int64_t group_elements,
                               int32_t* triples_out, int64_t capacity, int64_t* n_items_out);

/* numel[i] >= 0 (zero-sized tensors are allowed and untouched); n_tensors >= 0. */
int rafhip_lans_plan_create(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                            rafhip_lans_plan** out_plan);

/*
 * How a plan cuts and orders its work, for callers that want something else than the measured
 * defaults (the tests force every code path onto small lists this way).  None of it changes a
 * result.  Fill the struct with rafhip_lans_default_plan_options first; a field left at its
 * default value keeps the library's choice.  What the environment sets (RAFHIP_LANS_SCHEDULE,
 * RAFHIP_LANS_GROUP_ELEMS, RAFHIP_LANS_SPIN_LIMIT) stands between the two: it overrides the
 * built-in defaults and is overridden by a field set here.
 */
typedef struct rafhip_lans_plan_options {
  int32_t schedule;             /* -1: by list length; RAFHIP_LANS_PHASED / RAFHIP_LANS_PIPELINED        */
  int32_t round_slices;         /* pipelined: slices per round in which passes B and C alternate; 0: 8  */
  int64_t group_elements;       /* pipelined: elements per cache group; 0: 13,000,000                   */
  int64_t stream_from_elements; /* pipelined: tensors from this size bypass the cache; 0: 22,369,621    */
  int32_t stream_hold_items;    /* pipelined: cached items drawn after a streamed finish; -1: 4 x grid  */
  int32_t blocks_per_cu;        /* pipelined: resident workgroups per CU; 0: 3, or 2 for long tensors   */
  int32_t resident_mib;         /* phased: lists up to this size use temporal accesses; -1: 192         */
  int32_t apply_slice_shift;    /* phased, streaming lists: log2 of the last pass's slice, 0 = whole
                                   chunks; -1: 10                                                       */
  int64_t spin_limit;           /* pipelined: polls a wait may take before the step is flagged invalid;
                                   -1: 2^22 (0 makes every wait give up at once: the tests' way of
                                   forcing the time-out path while every kernel still exits normally) */
} rafhip_lans_plan_options;
void rafhip_lans_default_plan_options(rafhip_lans_plan_options* options);
/* options may be NULL (= rafhip_lans_plan_create). */
int rafhip_lans_plan_create_with(int32_t n_tensors, const int64_t* numel, int32_t grad_dtype,
                                 const rafhip_lans_plan_options* options,
                                 rafhip_lans_plan** out_plan);
/* rafhip_lans_pipeline_order with the cutting taken from `options` (group_elements,
 * round_slices, stream_from_elements, stream_hold_items; NULL = defaults). */
int rafhip_lans_pipeline_order_with(int32_t n_tensors, const int64_t* numel,
                                    const rafhip_lans_plan_options* options, int32_t* triples_out,
                                    int64_t capacity, int64_t* n_items_out);
int rafhip_lans_plan_destroy(rafhip_lans_plan* plan);
int rafhip_lans_plan_set_schedule(rafhip_lans_plan* plan, int32_t schedule);
int32_t rafhip_lans_plan_schedule(const rafhip_lans_plan* plan); /* the schedule in force; -1 on NULL */

/* Bytes of caller-provided scratch a step needs (partial sums, per-tensor norms, flags); 16-byte
 * alignment required (RAF's pools hand out 64-byte aligned blocks, include/raf/memory_pool.h).
 * Returns a negative value on a NULL plan. */
int64_t rafhip_lans_workspace_bytes(const rafhip_lans_plan* plan);
int32_t rafhip_lans_plan_num_tensors(const rafhip_lans_plan* plan);
int64_t rafhip_lans_plan_num_chunks(const rafhip_lans_plan* plan);
int64_t rafhip_lans_plan_total_elements(const rafhip_lans_plan* plan);
/* A plan keeps RAFHIP_TABLE_SLOTS device tables of tensor pointers, each with the pointer lists it
 * was last sent; a step whose lists equal one of them sends nothing, any other replaces the least
 * recently used through pinned staging memory of its own, without waiting for the device.  An
 * executor whose gradients alternate between two allocations (the reference's VM allocates them
 * per iteration, src/impl/vm/vm.cc:1099-1105) therefore stops uploading after two steps.  This
 * counts the uploads made so far (-1 on NULL).
 * A step made while its stream is being captured into a HIP graph leaves nodes that read one of
 * the tables at every replay; that table is held from then on and never given to other pointers,
 * so replays keep updating the tensors they were captured with.  A plan can thus serve up to
 * RAFHIP_TABLE_SLOTS captured pointer sets; once all tables are held, a step with pointers that
 * match none of them returns RAFHIP_ERR_UNSUPPORTED (use another plan).  The same holds for the
 * tables of the multi-tensor SGD and fuse / defuse plans. */
#define RAFHIP_TABLE_SLOTS 4
int64_t rafhip_lans_plan_table_uploads(const rafhip_lans_plan* plan);

/*
 * One LANS step, in place on w/m/v; g is read-only (the reference overwrites it with an
 * intermediate, multi_tensor_lans.cu:314, which no caller reads).
 *
 *   g, w, m, v   host arrays of n_tensors device pointers (the four quarters of the reference's
 *                tensor_list, python/raf/optim/lans.py:89).  g[i] has the plan's gradient dtype.
 *   step_dev     device pointer to the 0-d fp32 step tensor (lans.cc:92-99), read on the device
 *                so the call never blocks the host; or NULL to use step_host.
 *   workspace    device scratch of at least rafhip_lans_workspace_bytes(plan); contents need not
 *                be preserved between calls and need no initialisation.
 *   stream       hipStream_t (NULL = the default stream).  All work is enqueued on it.
 *
 * Arithmetic: scalars are the fp32 schema values; everything per element and every norm is
 * evaluated in float64 and rounded once to fp32 on store.
 */
/* A pipelined step whose bounded waits ran out (which no correct run does) leaves the list partly
 * updated: every element holds either its old or its correct new value (tensors whose waits ran out
 * keep the old ones), never garbage.  The failure is reported by rafhip_lans_read_norms of that step, or else by the NEXT step call on
 * the plan, which then returns RAFHIP_ERR_HIP without launching anything; either report clears it. */
int rafhip_lans_step(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                     float* const* m, float* const* v, const float* step_dev, int32_t step_host,
                     const rafhip_lans_hparams* hp, void* workspace, int64_t workspace_bytes,
                     void* stream);

/*
 * The same step for a half-precision model with fp32 master weights, i.e. what the reference's
 * traced optimizer builds around raf.op.lans out of three more ops (python/raf/optim/lans.py):
 *   - gradients of the plan's dtype (binary16 / bfloat16) are widened on load, replacing
 *     `_op.group_cast(g_list, "float32")` (:261-265) and the fp32 gradient copies it materialises;
 *   - p[i], when p is not NULL, receives the NEW fp32 weight narrowed to p_dtype (RAFHIP_F16 or
 *     RAFHIP_BF16) with round to nearest even, replacing `_op.cast(new_w, dtype)` and the copy into
 *     the model's parameter `_op.add(new_w, zero, out=p)` (:289-291, :303-305).
 * p is a host array of n_tensors device pointers (2-byte elements, numel[i] each; an entry may be
 * NULL to skip that tensor).  With p == NULL this is rafhip_lans_step.
 */
int rafhip_lans_step_mixed(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                           float* const* m, float* const* v, void* const* p, int32_t p_dtype,
                           const float* step_dev, int32_t step_host,
                           const rafhip_lans_hparams* hp, void* workspace,
                           int64_t workspace_bytes, void* stream);

/*
 * Bound form, for tensors that stay where they are (a training loop updates the same buffers every
 * step; the reference's VM likewise hands its cached OpEnv the same storage every iteration):
 * rafhip_lans_plan_bind checks the pointers and builds the tensor table once, and every
 * rafhip_lans_step_bound afterwards neither walks nor compares nor uploads the pointer lists.
 * Same arguments and same results as rafhip_lans_step_mixed (p may be NULL).  Binding again
 * replaces the bound tensors; other step calls on the plan may be mixed in freely.
 */
int rafhip_lans_plan_bind(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                          float* const* m, float* const* v, void* const* p, int32_t p_dtype);
int rafhip_lans_step_bound(rafhip_lans_plan* plan, const float* step_dev, int32_t step_host,
                           const rafhip_lans_hparams* hp, void* workspace, int64_t workspace_bytes,
                           void* stream);

/*
 * Dynamic loss scaling without host round trips (extension; the reference unscales with graph ops
 * in front of the optimizer and has no skip).  From this call on, every step on the plan
 *   - multiplies the gradients by the fp32 value at grad_unscale_dev (the reciprocal of the current
 *     loss scale) instead of hp->grad_unscale, when grad_unscale_dev is not NULL;
 *   - does nothing at all -- w, m, v and the 16-bit copies keep their bits, the norms of that step
 *     are undefined -- when the fp32 value at found_inf_dev is non-zero (the flag an overflow check
 *     of the gradients leaves), when found_inf_dev is not NULL.
 * Both are device pointers read by the kernels when they start, so the scale may change and a step
 * may be skipped without a new plan, a host synchronisation or a copy.  NULL switches either off.
 */
int rafhip_lans_plan_set_dynamic_scale(rafhip_lans_plan* plan, const float* grad_unscale_dev,
                                       const float* found_inf_dev);

/*
 * rafhip_lans_step_mixed without the workspace arguments, for callers that cannot allocate device
 * memory and have no workspace to hand over: code running under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose executors
 * allocate the requested workspaces around every call).  The step scalars, per-tensor statistics
 * and chunk partial sums live in an array of RAFHIP_LANS_STATIC_SCRATCH_BYTES that is part of the
 * library's device code: every GPU the library is used on holds its own copy until the process
 * ends.  The call itself allocates nothing, on the device or on the host, and gives the same bits
 * as rafhip_lans_step_mixed.  A plan whose rafhip_lans_workspace_bytes exceeds
 * RAFHIP_LANS_STATIC_SCRATCH_BYTES (lists beyond roughly two billion elements or 80 000 tensors)
 * is refused with RAFHIP_ERR_WORKSPACE.  All calls on one GPU share that GPU's array: two such
 * steps that overlap in time on one GPU (different streams or threads) race; calls on one stream
 * are ordered and safe.  p may be NULL.
 */
#define RAFHIP_LANS_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)
int rafhip_lans_step_noalloc(rafhip_lans_plan* plan, const void* const* g, float* const* w,
                             float* const* m, float* const* v, void* const* p, int32_t p_dtype,
                             const float* step_dev, int32_t step_host,
                             const rafhip_lans_hparams* hp, void* stream);

/* Copies the per-tensor norms left in the workspace by the last step on `stream`
 * (4 doubles per tensor: ||g||, ||w||, ||u_m||, ||u_g||) to host memory; synchronises `stream`. */
int rafhip_lans_read_norms(const rafhip_lans_plan* plan, const void* workspace, double* host_out,
                           void* stream);

/*
 * Optional per-kernel timing.  slots > 0 makes each following step record HIP events around its
 * kernels on the step's stream into slot (step_index % slots); slots == 0 turns it off.
 * rafhip_lans_timing_read waits for that slot's last event and returns five durations in
 * milliseconds.  Phased schedule: [0] norm of g  [1] finish  [2] norms of u_m, u_g, w  [3] finish
 * [4] apply ([1] and [3] zero for a list of short tensors, which has no finish launches).
 * Pipelined schedule: [0] set-up  [1] the persistent kernel  [2..4] zero.  Only the events that
 * delimit a launch are recorded: each costs a few microseconds of the step.
 */
int rafhip_lans_timing_enable(rafhip_lans_plan* plan, int32_t slots);
int rafhip_lans_timing_read(rafhip_lans_plan* plan, int32_t slot, float* ms_out5);

/*
 * Diagnostics of the pipelined schedule.  When the process runs with RAFHIP_LANS_TRACE=1, every
 * pipelined step leaves four 64-bit words per work item, in work-list order: the 100 MHz device
 * clock when the item was drawn, when its wait (if any) ended and when it finished, and the index
 * of the workgroup that ran it.  n_items_out receives 0 when tracing is off.  Synchronises the
 * device.
 */
int rafhip_lans_debug_trace(rafhip_lans_plan* plan, uint64_t* words_out, int64_t capacity_items,
                            int64_t* n_items_out);

/* --------------------------------------------------------------------------------------- l2norm
 * `raf.op.l2norm(x)`: out = sqrt(sum x_i^2) as ONE element of x's dtype on the device
 * (src/op/declare/reduce.cc:118-124).  dtype: RAFHIP_F32, RAFHIP_F64 (the two the reference's
 * cuBLAS backend takes, l2_norm.cc:57-71), RAFHIP_F16, RAFHIP_BF16.  Squares are accumulated in
 * float64 in a fixed order (the result is bit-identical from run to run and device to device) and
 * rounded once to the output dtype.  n == 0 gives 0.  workspace: device scratch of at least
 * rafhip_l2norm_workspace_bytes(n) bytes, 8-byte aligned, no initialisation needed (0 bytes, and
 * workspace may be NULL, for tensors of at most 16384 elements).
 */
int64_t rafhip_l2norm_workspace_bytes(int64_t n);
int rafhip_l2norm(const void* x, int32_t dtype, int64_t n, void* out, void* workspace,
                  int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- fuse / defuse tensor
 * `raf.op.fuse_tensor(data)` packs a list of tensors back to back into one flat buffer and
 * `raf.op.defuse_tensor(data, sizes, ...)` unpacks it (src/op/declare/memory.cc:43-93); offsets are
 * the running sums of the tensors' byte sizes (memory.cc:61-66).  A plan fixes the byte sizes, as
 * the reference's OpEnv constructors do (memory.cc:33-43, :95-103), and owns a small device
 * table; each call is ONE kernel launch whatever the number of tensors, and allocates nothing.
 * nbytes[i] >= 0; empty tensors and empty lists are valid.  Pointers need no alignment (16-byte
 * lane accesses are used when source and destination agree modulo 4).  One call at a time per plan.
 */
typedef struct rafhip_fuse_plan rafhip_fuse_plan;
int rafhip_fuse_plan_create(int32_t n_tensors, const int64_t* nbytes, rafhip_fuse_plan** out_plan);
int rafhip_fuse_plan_destroy(rafhip_fuse_plan* plan);
int64_t rafhip_fuse_plan_total_bytes(const rafhip_fuse_plan* plan); /* -1 on NULL */
/* parts: host array of n_tensors device pointers; fused: device buffer of total_bytes. */
int rafhip_fuse_tensors(rafhip_fuse_plan* plan, const void* const* parts, void* fused,
                        void* stream);
int rafhip_defuse_tensor(rafhip_fuse_plan* plan, const void* fused, void* const* parts,
                         void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RAFHIP_OPTIM_H_ */

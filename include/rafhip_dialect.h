/*
 * rafhip_dialect.h -- C entry points into the C++ host layer (OpEnv / dialect registry mirror and
 * the `hip` dialect ops).  They exist so that a non-C++ caller (the Python mirror of RAF's
 * frontend, ctypes) can drive an operator the way RAF's executors do:
 *
 *     make   = declare + dispatch + OpEnv construction   (src/impl/interpreter.cc:247-270,
 *                                                          src/impl/op.cc:127-180)
 *     execute = bind workspaces, set the stream, OpEnv::Execute(inputs, output), unbind
 *                                                         (src/impl/vm/vm.cc:818-855, :1099-1111)
 *
 * Tensors cross as rafhip_tensor_desc (the DLTensor fields the ops read).  Every function returns
 * 0 on success; on failure the message (a raf::Error text or a kernel-library error) is available
 * from rafhip_raf_last_error() on the same thread.
 */
#ifndef RAFHIP_DIALECT_H_
#define RAFHIP_DIALECT_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rafhip_tensor_desc {
  void* data;
  int32_t device_type; /* 1 cpu, 2 cuda, 10 rocm (include/raf/device.h:37-50) */
  int32_t device_id;
  int32_t dtype_code;  /* DLPack: 0 int, 1 uint, 2 float, 4 bfloat */
  int32_t dtype_bits;
  int32_t ndim;
  const int64_t* shape;
} rafhip_tensor_desc;

typedef struct rafhip_raf_env rafhip_raf_env; /* an OpEnv made by dispatch */

const char* rafhip_raf_last_error(void);

/* "dialect:dialect_op:plevel" entries joined by ';' in dispatch order for a base op on a device
 * type, honouring the current preference; truncated to buflen. */
int rafhip_raf_dispatch_list(const char* base_op, int32_t device_type, char* buf, int32_t buflen);

/* Scoped dialect preference for this thread (the reference tests' with_dialect): names joined by
 * ','; pass NULL or "" to clear. */
int rafhip_raf_set_dialect_preference(const char* dialects_csv);

/* raf.op.sgd(x, dx, v, learning_rate, mu) -> (v1, x1); python/raf/optim/sgd.py:56 */
int rafhip_raf_sgd_make(const rafhip_tensor_desc* x, const rafhip_tensor_desc* dx,
                        const rafhip_tensor_desc* v, double learning_rate, double mu,
                        rafhip_raf_env** env_out);
int rafhip_raf_sgd_execute(rafhip_raf_env* env, const rafhip_tensor_desc* x,
                           const rafhip_tensor_desc* dx, const rafhip_tensor_desc* v,
                           const rafhip_tensor_desc* v1, const rafhip_tensor_desc* x1,
                           void* stream);

/* raf.op.lans(tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction, weight_decay,
 * grad_averaging, mode, normalize_grad); python/raf/optim/lans.py:90-102.  tensor_list holds 4n
 * descriptors ordered g..., w..., m..., v... */
int rafhip_raf_lans_make(int32_t list_len, const rafhip_tensor_desc* tensor_list,
                         const rafhip_tensor_desc* step, float learning_rate, float beta1,
                         float beta2, float eps, int32_t bias_correction, float weight_decay,
                         int32_t grad_averaging, int32_t mode, int32_t normalize_grad,
                         rafhip_raf_env** env_out);
/* Extension op raf.op.lans_mixed (no counterpart in the reference's op set): the same arguments
 * with a tensor_list of 5n descriptors g..., w..., m..., v..., p..., where p are the model's
 * float16 / bfloat16 parameters; they receive the new fp32 weights narrowed to 16 bits, which the
 * reference's traced optimizer does with a cast and a copy after raf.op.lans
 * (python/raf/optim/lans.py:289-291, :303-305).  Execute with rafhip_raf_lans_execute. */
int rafhip_raf_lans_mixed_make(int32_t list_len, const rafhip_tensor_desc* tensor_list,
                               const rafhip_tensor_desc* step, float learning_rate, float beta1,
                               float beta2, float eps, int32_t bias_correction, float weight_decay,
                               int32_t grad_averaging, int32_t mode, int32_t normalize_grad,
                               rafhip_raf_env** env_out);
int rafhip_raf_lans_execute(rafhip_raf_env* env, int32_t list_len,
                            const rafhip_tensor_desc* tensor_list, const rafhip_tensor_desc* step,
                            void* workspace, int64_t workspace_bytes, void* stream);

/* A tensor list held as a value: RAF's TupleValue of TensorValues (include/raf/value.h), which is
 * what its executors keep between calls -- the interpreter in the argument object, the VM in its
 * registers (src/impl/vm/vm.cc:764-769) -- so that no call converts the list again.  Immutable.
 * _replace makes a new tuple that shares every field of `base` except [first, first + count),
 * which are made from `fields`: one step's list against the previous one when only the gradients
 * were allocated anew. */
typedef struct rafhip_raf_tuple rafhip_raf_tuple;
int rafhip_raf_tuple_make(int32_t n, const rafhip_tensor_desc* fields, rafhip_raf_tuple** tuple_out);
int rafhip_raf_tuple_replace(const rafhip_raf_tuple* base, int32_t first, int32_t count,
                             const rafhip_tensor_desc* fields, rafhip_raf_tuple** tuple_out);
/* Rebinds fields [first, first + count) of a tuple to the storage `fields` name, in place, the way
 * the reference's ndarray.update rebinds an array to another value (python/raf/_core/ndarray.py:
 * 191-195): for a holder that owns its tuple alone and whose caller has let go of the tensors the
 * range held.  Done (*done_out = 1) only if nothing else shares the tuple or a tensor value of the
 * range and every field keeps its dtype, device and shape; otherwise nothing is changed
 * (*done_out = 0) and the caller makes a new tuple with _replace. */
int rafhip_raf_tuple_rebind(rafhip_raf_tuple* tuple, int32_t first, int32_t count,
                            const rafhip_tensor_desc* fields, int32_t* done_out);
int32_t rafhip_raf_tuple_size(const rafhip_raf_tuple* tuple); /* -1 on NULL */
int rafhip_raf_tuple_destroy(rafhip_raf_tuple* tuple);
/* rafhip_raf_lans_execute / rafhip_raf_sgd_multi_execute on a tuple made beforehand.  as_vm != 0
 * hands Execute a NEW TupleValue over the same tensor values, which is what the VM does at every
 * iteration (vm.cc:764-769 allocates the tuple afresh from its registers); 0 hands over the
 * tuple itself, as the interpreter does with the call's argument. */
int rafhip_raf_lans_execute_tuple(rafhip_raf_env* env, const rafhip_raf_tuple* tensor_list,
                                  const rafhip_tensor_desc* step, void* workspace,
                                  int64_t workspace_bytes, void* stream, int32_t as_vm);
int rafhip_raf_sgd_multi_execute_tuple(rafhip_raf_env* env, const rafhip_raf_tuple* tensor_list,
                                       void* stream, int32_t as_vm);

/* Extension ops raf.op.sgd_multi(tensor_list, learning_rate, mu) with tensor_list = x..., dx...,
 * v... (3n descriptors) and raf.op.sgd_multi_mixed with a fourth block p... (the model's float16 /
 * bfloat16 parameters): momentum SGD over the whole list, in place on x and v, per element the
 * four roundings of raf.op.sgd.  No counterpart in the reference's op set; they replace the
 * per-parameter op sequence of its traced optimizer (python/raf/optim/sgd.py:187-215). */
int rafhip_raf_sgd_multi_make(int32_t mixed, int32_t list_len, const rafhip_tensor_desc* tensor_list,
                              double learning_rate, double mu, rafhip_raf_env** env_out);
int rafhip_raf_sgd_multi_execute(rafhip_raf_env* env, int32_t list_len,
                                 const rafhip_tensor_desc* tensor_list, void* stream);

/* raf.op.l2norm(x) -> 0-d tensor of x's dtype; scripts/src_codegen/def_schema.py:425-427,
 * src/op/declare/reduce.cc:118-126. */
int rafhip_raf_l2norm_make(const rafhip_tensor_desc* x, rafhip_raf_env** env_out);
int rafhip_raf_l2norm_execute(rafhip_raf_env* env, const rafhip_tensor_desc* x,
                              const rafhip_tensor_desc* out, void* workspace,
                              int64_t workspace_bytes, void* stream);

/* raf.op.fuse_tensor(data) -> 1-d tensor holding every tensor's elements back to back
 * (def_schema.py:829-835, src/op/declare/memory.cc:43-63).  An empty list declares no output:
 * make succeeds, the env has no outputs and execute does nothing. */
int rafhip_raf_fuse_tensor_make(int32_t n, const rafhip_tensor_desc* data,
                                rafhip_raf_env** env_out);
int rafhip_raf_fuse_tensor_execute(rafhip_raf_env* env, int32_t n, const rafhip_tensor_desc* data,
                                   const rafhip_tensor_desc* out, void* stream);

/* raf.op.defuse_tensor(data, sizes, shapes, shape_indices) -> tuple of tensors
 * (def_schema.py:836-841, src/op/declare/memory.cc:65-93). */
int rafhip_raf_defuse_tensor_make(const rafhip_tensor_desc* data, int32_t n_sizes,
                                  const int64_t* sizes, int32_t n_shapes, const int64_t* shapes,
                                  int32_t n_indices, const int64_t* shape_indices,
                                  rafhip_raf_env** env_out);
int rafhip_raf_defuse_tensor_execute(rafhip_raf_env* env, const rafhip_tensor_desc* data,
                                     int32_t n_out, const rafhip_tensor_desc* outs, void* stream);

/* OpEnv::RequestStream (include/raf/op.h:87).  The fuse_tensor and defuse_tensor OpEnvs request a
 * copy stream the way the reference's do (src/op/dialect/cuda/memory.cc:34, :89).  By default this
 * window leaves such requests unserved and the OpEnv launches on the `stream` argument.  With
 * enable != 0 (per calling thread) the execute calls serve them from a pool of streams per
 * (device, tag) and order that stream behind `stream` before Execute and `stream` behind it
 * afterwards, so the results are still in `stream`'s order. */
int rafhip_raf_serve_stream_requests(int32_t enable);

/* What the op's declare function produced (call->out): number of output tensors (a tuple counts
 * its fields; -1 on NULL) and each one's dtype and shape, so that the caller can allocate them the
 * way an executor does (src/impl/interpreter.cc:397-426).  shape_out may be NULL to query ndim. */
int32_t rafhip_raf_env_num_outputs(const rafhip_raf_env* env);
int rafhip_raf_env_output(const rafhip_raf_env* env, int32_t index, int32_t* dtype_code,
                          int32_t* dtype_bits, int32_t* ndim, int64_t* shape_out,
                          int32_t shape_capacity);

/* ------------------------------------------------------------- device API and memory pools
 * The `rocm` DeviceAPI (the ROCm counterpart of src/device_api/cuda/cuda.cc:25-248; interface
 * include/raf/device_api.h:19-177) and the memory-pool front end (include/raf/memory_pool.h:28-56,
 * src/impl/memory_pool.cc:89-180) seen from C.  device_type: 1 cpu, 10 rocm.  The default pool of
 * a rocm device is "no_pool" (stream-ordered allocation from the HIP memory pool), of the cpu
 * "page_unit_pool".
 */
int rafhip_raf_device_count(int32_t device_type, int32_t* count_out);
/* DeviceAPI::CopyDataFromTo on two contiguous tensors of equal byte size; stream may be NULL. */
int rafhip_raf_device_copy(const rafhip_tensor_desc* from, const rafhip_tensor_desc* to, void* stream);
int rafhip_raf_stream_create(int32_t device_type, int32_t device_id, void** stream_out);
int rafhip_raf_stream_free(int32_t device_type, int32_t device_id, void* stream);
int rafhip_raf_event_create(int32_t device_type, int32_t device_id, uint32_t flags, void** event_out);
int rafhip_raf_event_free(int32_t device_type, int32_t device_id, void* event);
int rafhip_raf_event_record(int32_t device_type, void* event, void* stream);
int rafhip_raf_event_elapsed_ms(int32_t device_type, void* start_event, void* end_event, float* ms_out);
int rafhip_raf_stream_wait_event(int32_t device_type, void* stream, void* event);
/* WaitDevice (what = 0, handle ignored), WaitStream (1) or WaitEvent (2). */
int rafhip_raf_wait(int32_t device_type, int32_t device_id, int32_t what, void* handle);

/* Memory::Alloc (stream_ordered = 0) or Memory::AllocAsync on the device's pool; alignment <= 0
 * selects the default (64).  The handle keeps the chunk alive; freeing it hands the chunk back to
 * its pool (or, stream-ordered, to the stream it came from). */
typedef struct rafhip_raf_memory rafhip_raf_memory;
int rafhip_raf_memory_alloc(int32_t device_type, int32_t device_id, int64_t nbytes, int64_t alignment,
                            int32_t stream_ordered, void* stream, rafhip_raf_memory** mem_out);
void* rafhip_raf_memory_data(const rafhip_raf_memory* mem);
int rafhip_raf_memory_free(rafhip_raf_memory* mem);
/* raf.memory_pool.InitPool / RemovePool / ResetPool (src/impl/memory_pool.cc:144-180). */
int rafhip_raf_pool_init(int32_t device_type, int32_t device_id, const char* pool_name);
int rafhip_raf_pool_remove(int32_t device_type, int32_t device_id);
int rafhip_raf_pool_reset(int32_t device_type, int32_t device_id);
/* Name of the device's pool and <used, pool> sizes in MB; any output may be NULL. */
int rafhip_raf_pool_info(int32_t device_type, int32_t device_id, char* name_buf, int32_t buflen,
                         float* used_mb_out, float* pool_mb_out);
/* Memory::GetAllocBytes: what a request of nbytes really takes from the pool; -1 on error. */
int64_t rafhip_raf_pool_alloc_bytes(int32_t device_type, int32_t device_id, int64_t nbytes);

/* Dialect fusion.  The reference's traced SGD optimizer emits, per parameter,
 *     new_v = add(multiply(momentum, v), dx, out=v)
 *     new_w = subtract(w, multiply(learning_rate, new_v), out=w)
 * with a cast(dx, "float32") in front for 16-bit gradients (python/raf/optim/sgd.py:192-200).
 * rafhip_raf_traced_sgd_make builds that graph for one parameter from the descriptors' types, runs
 * the FuseDialect pass (src/pass/fuse_dialect.cc:179-198) for their device type with the `hip`
 * dialect's "sgd_update" pattern, and dispatches the fused function the way
 * DispatchFusedOp does (src/impl/op.cc:182-203: maker raf.op.hip._fused_op).  If nothing fuses
 * (other device, other dtypes) it fails like a dispatch with no backend, and *env_out still
 * holds the graphs for rafhip_raf_env_ir_text.  _execute runs the fused function IN PLACE on w
 * and v (that is what out= means) as one kernel launch.
 * rafhip_raf_env_ir_text copies the text of the graph before (fused = 0) or after the pass. */
int rafhip_raf_traced_sgd_make(const rafhip_tensor_desc* w, const rafhip_tensor_desc* dx,
                               const rafhip_tensor_desc* v, double learning_rate, double momentum,
                               rafhip_raf_env** env_out);
int rafhip_raf_traced_sgd_execute(rafhip_raf_env* env, const rafhip_tensor_desc* w,
                                  const rafhip_tensor_desc* dx, const rafhip_tensor_desc* v,
                                  void* stream);
int rafhip_raf_env_ir_text(const rafhip_raf_env* env, int32_t fused, char* buf, int32_t buflen);

/* Whole traced optimizers.  Builds the optimizer part of the function that the reference's traced
 * optimizer makes for a model with n parameters -- kind 0: SGD (python/raf/optim/sgd.py:187-215;
 * g = the gradients, m unused), kind 1: LANS for a half-precision model
 * (python/raf/optim/lans.py:244-312: group_cast, raf.op.lans, cast, add(out=p)) -- runs FuseDialect
 * with the hip dialect's graph rewrites and patterns, and makes one OpEnv per call of the result.
 * Every list holds n descriptors; p (the model's 16-bit parameters) may be NULL for SGD on a
 * float32 model.  zero_is_constant tells whether the optimizer's zero tensor is already bound into
 * the graph as a constant (then cast and copy are folded into the multi-tensor op) or is a free
 * variable as traced (then they stay, and have no backend in this library: the make call fails
 * unless allow_partial, which skips the result fields that need them).  hyper: SGD
 * {learning_rate, momentum}; LANS the nine schema values in order (ints and bools as numbers).
 * _execute runs the OpEnvs in order, in place on the caller's tensors; workspace as reported by
 * rafhip_raf_env_workspace_bytes.  rafhip_raf_env_graph_ops lists what the fused graph calls, in
 * order, joined by ';': dialect ops, "<dialect>._fused_op(<pattern>)", and with a leading '!' ops
 * that were left without a backend.  On failure *env_out still holds the graphs for
 * rafhip_raf_env_ir_text. */
int rafhip_raf_traced_optimizer_make(int32_t kind, int32_t n, const rafhip_tensor_desc* g,
                                     const rafhip_tensor_desc* w, const rafhip_tensor_desc* m,
                                     const rafhip_tensor_desc* v, const rafhip_tensor_desc* p,
                                     const rafhip_tensor_desc* step, int32_t zero_is_constant,
                                     const double* hyper, int32_t n_hyper, int32_t allow_partial,
                                     rafhip_raf_env** env_out);
int rafhip_raf_traced_optimizer_execute(rafhip_raf_env* env, int32_t n, const rafhip_tensor_desc* g,
                                        const rafhip_tensor_desc* w, const rafhip_tensor_desc* m,
                                        const rafhip_tensor_desc* v, const rafhip_tensor_desc* p,
                                        const rafhip_tensor_desc* step, int32_t allow_partial,
                                        void* workspace, int64_t workspace_bytes, void* stream);
int rafhip_raf_env_graph_ops(const rafhip_raf_env* env, char* buf, int32_t buflen);

/* hip-dialect extension for learning-rate schedules: moves the learning rate of an OpEnv made by
 * the sgd, sgd_multi, lans or lans_mixed makers, so that a new value every step does not mean a
 * new OpEnv (in the reference the learning rate is a schema constant and part of the OpEnv cache
 * key, src/impl/vm/vm.cc:1012-1015).  Fails for any other OpEnv. */
int rafhip_raf_env_set_learning_rate(rafhip_raf_env* env, double learning_rate);

/* hip-dialect extensions for loss scaling, on an OpEnv made by the lans or lans_mixed makers (the
 * reference's LansArgs has no such field; its optimizers unscale with graph ops in front of the
 * op).  _set_grad_unscale: every gradient element is multiplied by `factor` first (1 by default).
 * _set_dynamic_scale: device-resident one-element float32 tensors holding that factor (the
 * reciprocal of the current loss scale) and an overflow flag; the kernels read them when they
 * start, and a non-zero flag turns the step into a no-op.  Either descriptor may be NULL.  None
 * of this identifies the OpEnv: a scale change keeps the OpEnv, its plan and its tables.  On the
 * env of a traced optimizer (rafhip_raf_traced_optimizer_make) they reach every call of the graph
 * that takes a gradient scale. */
int rafhip_raf_env_set_grad_unscale(rafhip_raf_env* env, float factor);
int rafhip_raf_env_set_dynamic_scale(rafhip_raf_env* env, const rafhip_tensor_desc* grad_unscale,
                                     const rafhip_tensor_desc* found_inf);

/* Total bytes of the OpEnv's workspace requests (each rounded up to 256). */
int64_t rafhip_raf_env_workspace_bytes(const rafhip_raf_env* env);
/* OpEnv::name() and the dialect op the dispatcher picked; pointers stay valid until destroy. */
const char* rafhip_raf_env_name(const rafhip_raf_env* env);
const char* rafhip_raf_env_op(const rafhip_raf_env* env);
int rafhip_raf_env_destroy(rafhip_raf_env* env);

#ifdef __cplusplus
}
#endif
#endif /* RAFHIP_DIALECT_H_ */

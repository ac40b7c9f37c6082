// Knobs of the `hip` dialect that have no field in the reference's schemas.
#pragma once

#include <string>

#include "raf_ir.h"

namespace raf {
namespace op {
namespace hip {

// Loss scaling.  The reference's LansArgs has no field for it: there, gradients are cast and
// unscaled by separate ops before LANS runs.  The hip LANS OpEnvs fold the unscaling into the
// kernels and implement this interface, through which the executor that owns the OpEnv sets,
// between two Execute calls,
//   - the factor every gradient element is multiplied by first (e.g. 1/1024; 1 by default), or
//   - for dynamic loss scaling, device pointers to that factor and to an overflow flag (fp32 words
//     read by the kernels: a non-zero flag makes the step a no-op), either of which may be null.
// Neither is part of what identifies the OpEnv, so a scale change keeps the OpEnv and its plan.
class HasGradScaling {
 public:
  virtual ~HasGradScaling() = default;
  virtual void SetGradUnscale(float factor) = 0;
  virtual void SetDynamicScale(const float* grad_unscale_dev, const float* found_inf_dev) = 0;
};

// A learning-rate schedule changes one hyper-parameter every step.  The reference's schemas carry
// the learning rate as a constant, so there every new value means a new OpEnv (the VM's cache key
// holds the constants, src/impl/vm/vm.cc:1012-1015).  The hip OpEnvs of the optimizer ops
// implement this interface instead: the executor that owns the OpEnv may move its learning rate
// between two Execute calls and keep the OpEnv, its plan and its device tables.
class HasLearningRate {
 public:
  virtual ~HasLearningRate() = default;
  virtual void SetLearningRate(double learning_rate) = 0;
  virtual double GetLearningRate() const = 0;
};

// The per-parameter update of the reference's traced SGD optimizer
// (python/raf/optim/sgd.py:192-200) as a dataflow pattern, with handles on its leaves:
//     subtract(w, multiply(lr, add(multiply(mu, v), dx | cast(dx_half, "float32"), v, null)), w, null)
// `op_prefix` is "raf.op." for the pattern registered with the FuseDialect pass and
// "raf.op.hip." for the body of the fused function.  Inside the function every outside value
// (constants included) is a parameter of its own, so there the leaves are all wildcards and the
// `out` arguments are separate leaves.
struct SgdUpdatePattern {
  ir::DFPattern root;
  ir::DFPattern w, w_out, v, v_out, dx, dx_half, lr, mu, null_v, null_w, cast_dtype;
};
SgdUpdatePattern MakeSgdUpdatePattern(const std::string& op_prefix, bool inside_function);
constexpr const char* kSgdUpdatePatternName = "sgd_update";
constexpr int kSgdUpdatePatternPlevel = 60;  // above every pattern of the reference (8..55)

// The expression the traced optimizer emits for one parameter (w, v float32; dx float32, or a
// 16-bit float that is cast first); the result is new_w.
ir::Expr TracedSgdUpdate(const ir::Expr& w, const ir::Expr& dx, const ir::Expr& v,
                         double learning_rate, double momentum);

// The optimizer part of the function that the reference's traced SGD optimizer builds for a model
// with n parameters (python/raf/optim/sgd.py:187-215): TracedSgdUpdate for every parameter and,
// when `p` is not empty (a half-precision model with fp32 master weights), the cast to the model's
// dtype and the copy `add(new_w, zero, out=p)` behind it.  The result is the tuple of the n new
// model weights.  `zero` is the optimizer's zero tensor: a variable as traced, or a zeros constant
// once the model's constant attributes are bound into the graph.
ir::Expr TracedSgdOptimizer(const std::vector<ir::Expr>& w, const std::vector<ir::Expr>& dx,
                            const std::vector<ir::Expr>& v, const std::vector<ir::Expr>& p,
                            const ir::Expr& zero, double learning_rate, double momentum);

// Hyper-parameters of raf.op.lans in schema order (scripts/src_codegen/def_schema.py:685-693).
struct LansHyper {
  double learning_rate = 1e-3, beta1 = 0.9, beta2 = 0.999, eps = 1e-6;
  int bias_correction = 1;
  double weight_decay = 0.01;
  int grad_averaging = 1, mode = 1, normalize_grad = 1;
};

// The optimizer part of what the reference's traced LANS optimizer builds for a half-precision
// model (python/raf/optim/lans.py:244-312): group_cast of the n gradients to float32, raf.op.lans
// over [g32..., w..., m..., v...], and per parameter cast(new_w, dtype) and add(_, zero, out=p).
// The result is the tuple (new model weights..., new m..., new v...).  The increment of the step
// counter in front of it (lans.py:240, a scalar add) is left out: `step` is passed as it is.
ir::Expr TracedLansOptimizer(const std::vector<ir::Expr>& g, const std::vector<ir::Expr>& w,
                             const std::vector<ir::Expr>& m, const std::vector<ir::Expr>& v,
                             const std::vector<ir::Expr>& p, const ir::Expr& zero, const ir::Expr& step,
                             const LansHyper& hyper);

}  // namespace hip
}  // namespace op
}  // namespace raf

// Dialect fusion for the `hip` dialect: the operator sequence that the reference's traced SGD
// optimizer emits for every parameter,
//     new_v = add(multiply(momentum, v), dx, out=v)
//     new_w = subtract(w, multiply(learning_rate, new_v), out=w)
// with dx = cast(dx, "float32") in front when the model is not float32
// (python/raf/optim/sgd.py:192-200), is registered as a fuse pattern, and the primitive function
// that the FuseDialect pass makes of it is executed as ONE launch of the gfx950 SGD kernel: five
// streams over the parameter instead of four element-wise kernels and two temporaries.
//
// The reference registers its patterns from Python (python/raf/_op/dialect_pattern.py:120-143,
// through raf.op.AddDialectPattern, src/impl/dialect.cc:284) and builds fused functions in a
// maker named raf.op.<dialect>._fused_op (src/op/dialect/cutlass/cutlass_fusion.cc:117-141);
// the maker below has that name and shape.  The element-wise base ops get `hip` dialect ops with
// plevel -1: like the reference's raf.op.cutlass.add (plevel 0,
// src/op/dialect/cutlass/cutlass_utils.cc:114) they exist so that a fused function has ops to
// call, are never picked for a single op (src/impl/dialect.cc:183-186 skips plevel <= 0) and
// have no OpEnv of their own.
#include <sstream>

#include "hip_dialect.h"
#include "raf_iface.h"
#include "raf_ir.h"
#include "rafhip_optim.h"

namespace raf {
namespace op {
namespace hip {

using device_api::DeviceAPI;
using value::Value;

namespace {

bool IsF32(const DType& t) { return t.code == kDLFloat && t.bits == 32; }
bool IsF16(const DType& t) { return t.code == kDLFloat && t.bits == 16; }
bool IsBF16(const DType& t) { return t.code == kDLBfloat && t.bits == 16; }

}  // namespace

SgdUpdatePattern MakeSgdUpdatePattern(const std::string& op_prefix, bool inside_function) {
  using namespace ir;
  SgdUpdatePattern p;
  if (inside_function) {
    p.w = wildcard();
    p.v = wildcard();
    p.dx = wildcard();
    p.dx_half = wildcard();
    // Every outside value was lifted into a parameter of its own: constants are variables now,
    // and the two uses of v (and of w) are two parameters bound to the same argument.
    p.lr = wildcard();
    p.mu = wildcard();
    p.v_out = wildcard();
    p.w_out = wildcard();
    p.null_v = wildcard();
    p.null_w = wildcard();
    p.cast_dtype = wildcard();
  } else {
    // Only what the kernel can run may be fused: a fused function has no other dialect to fall
    // back to.  Types must be known, as for the reference's pass (it runs after InferType).
    const DType f32{kDLFloat, 32};
    p.w = has_dtype(f32);
    p.v = has_dtype(f32);
    p.dx = has_dtype(f32);
    p.dx_half = alt(has_dtype(DType{kDLFloat, 16}), has_dtype(DType{kDLBfloat, 16}));
    p.lr = is_constant();
    p.mu = is_constant();
    p.v_out = p.v;  // out=v: the very same expression
    p.w_out = p.w;
    p.null_v = is_constant(MakeNull());
    p.null_w = is_constant(MakeNull());
    p.cast_dtype = is_constant(MakeString("float32"));
  }
  DFPattern widened = call(is_op(op_prefix + "cast"), {p.dx_half, p.cast_dtype});
  DFPattern grad = alt(widened, p.dx);
  DFPattern new_v = call(is_op(op_prefix + "add"),
                         {call(is_op(op_prefix + "multiply"), {p.mu, p.v}), grad, p.v_out, p.null_v});
  p.root = call(is_op(op_prefix + "subtract"),
                {p.w, call(is_op(op_prefix + "multiply"), {p.lr, new_v}), p.w_out, p.null_w});
  return p;
}

ir::Expr TracedSgdUpdate(const ir::Expr& w, const ir::Expr& dx, const ir::Expr& v,
                         double learning_rate, double momentum) {
  using namespace ir;
  const TensorType wt = TypeOf(w);
  Expr grad = dx;
  const TensorType gt = TypeOf(dx);
  if (gt.defined && !IsF32(gt.dtype)) {  // sgd.py:192-194
    TensorType widened = gt;
    widened.dtype = DType{kDLFloat, 32};
    grad = MakeCall(GetOp("raf.op.cast"), {dx, MakeString("float32")}, widened);
  }
  Expr scaled_v = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(momentum), v}, TypeOf(v));
  Expr new_v = MakeCall(GetOp("raf.op.add"), {scaled_v, grad, v, MakeNull()}, TypeOf(v));  // :197
  Expr step = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(learning_rate), new_v}, TypeOf(v));
  return MakeCall(GetOp("raf.op.subtract"), {w, step, w, MakeNull()}, wt);  // :198-200
}

namespace {

// The OpEnv of a fused function made from the "sgd_update" pattern.  Arguments arrive as
// ListArgs in parameter order; which parameter plays which role is read off the function body.
class SgdUpdateFusedEnv : public OpEnv {
 public:
  explicit SgdUpdateFusedEnv(const CallValues& cv) {
    const auto* func = ir::AsFunction(cv->closure);
    const auto* args = cv->args_as<schema::ListArgs>();
    if (!func || !args) {
      error_msgs.push_back(kName + std::string(": call does not carry a function and ListArgs"));
      return;
    }
    SgdUpdatePattern pat = MakeSgdUpdatePattern("raf.op.hip.", true);
    ir::NodeMap nm;
    if (!ir::MatchPattern(pat.root, func->body, &nm)) {
      error_msgs.push_back(kName + std::string(": the function body is not an SGD update:\n") +
                           ir::AsText(cv->closure));
      return;
    }
    half_grad_ = nm.count(pat.dx_half.get()) != 0;
    auto index_of = [&](const ir::DFPattern& leaf, const char* what) -> int {
      auto it = nm.find(leaf.get());
      if (it != nm.end())
        for (size_t i = 0; i < func->params.size(); ++i)
          if (func->params[i].get() == it->second.get()) return (int)i;
      error_msgs.push_back(kName + std::string(": ") + what + " is not a parameter of the function");
      return -1;
    };
    i_w_ = index_of(pat.w, "w");
    i_w_out_ = index_of(pat.w_out, "out of subtract");
    i_v_ = index_of(pat.v, "v");
    i_v_out_ = index_of(pat.v_out, "out of add");
    i_dx_ = index_of(half_grad_ ? pat.dx_half : pat.dx, "dx");
    i_lr_ = index_of(pat.lr, "learning rate");
    i_mu_ = index_of(pat.mu, "momentum");
    const int i_null_v = index_of(pat.null_v, "where of add");
    const int i_null_w = index_of(pat.null_w, "where of subtract");
    const int i_dtype = half_grad_ ? index_of(pat.cast_dtype, "dtype of cast") : -1;
    if (!error_msgs.empty()) return;
    if (args->args.size() != func->params.size()) {
      error_msgs.push_back(kName + std::string(": argument count differs from parameter count"));
      return;
    }
    for (size_t i = 0; i < func->params.size(); ++i) arg_indices.push_back((int)i);
    if (cv->device.device_type() != DevType::kROCM())
      error_msgs.push_back(kName + std::string(": device is not rocm"));
    if (!Scalar(args->args[(size_t)i_lr_], &learning_rate_) || !Scalar(args->args[(size_t)i_mu_], &mu_))
      error_msgs.push_back(kName + std::string(": learning rate and momentum must be scalar constants"));
    if (args->args[(size_t)i_null_v] || args->args[(size_t)i_null_w])
      error_msgs.push_back(kName + std::string(": `where` is not supported"));
    if (half_grad_) {
      auto s = std::dynamic_pointer_cast<StringValueObj>(args->args[(size_t)i_dtype]);
      if (!s || s->value != "float32")
        error_msgs.push_back(kName + std::string(": the gradient must be cast to float32"));
    }
    if (!error_msgs.empty()) return;
    auto tensor = [&](int i) -> const TensorView* {
      auto t = std::dynamic_pointer_cast<value::TensorValueObj>(args->args[(size_t)i]);
      return t ? &t->tensor : nullptr;
    };
    const TensorView *w = tensor(i_w_), *v = tensor(i_v_), *dx = tensor(i_dx_);
    if (!w || !v || !dx || !tensor(i_w_out_) || !tensor(i_v_out_)) {
      error_msgs.push_back(kName + std::string(": w, v, dx and the two `out` arguments must be tensors"));
      return;
    }
    if (!IsF32(w->dtype) || !IsF32(v->dtype))
      error_msgs.push_back(kName + std::string(": w and v must be float32"));
    if (half_grad_ ? !(IsF16(dx->dtype) || IsBF16(dx->dtype)) : !IsF32(dx->dtype))
      error_msgs.push_back(kName + std::string(": dx must be float32, or float16 / bfloat16 under a cast"));
    if (w->shape != v->shape || w->shape != dx->shape)
      error_msgs.push_back(kName + std::string(": w, v and dx differ in shape (broadcasting is not fused)"));
    if (error_msgs.empty() && rafhip_device_count() <= 0)
      error_msgs.push_back(kName + std::string(": no HIP device is visible"));
    if (!error_msgs.empty()) return;
    numel_ = w->numel();
    if (half_grad_) {
      int st = rafhip_sgd_plan_create(1, &numel_, IsF16(dx->dtype) ? RAFHIP_F16 : RAFHIP_BF16, &plan_);
      if (st != RAFHIP_OK)
        error_msgs.push_back(std::string("rafhip_sgd_plan_create: ") + rafhip_last_error());
    }
  }

  ~SgdUpdateFusedEnv() override {
    if (plan_) (void)rafhip_sgd_plan_destroy(plan_);
  }

  std::string name() const override { return name_; }

  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::ListArgs>();
    RAF_CHECK(args != nullptr, "the fused SGD update expects ListArgs");
    Execute(args->args, cv->out);
  }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    RAF_CHECK(inputs.size() == arg_indices.size(), "the fused SGD update: wrong number of inputs");
    const TensorView& w = value::AsTensor(inputs[(size_t)i_w_])->tensor;
    const TensorView& v = value::AsTensor(inputs[(size_t)i_v_])->tensor;
    const TensorView& dx = value::AsTensor(inputs[(size_t)i_dx_])->tensor;
    // out=v and out=w: the kernel updates in place, so the `out` tensors must be v and w.
    RAF_CHECK(value::AsTensor(inputs[(size_t)i_v_out_])->tensor.data == v.data,
              "the fused SGD update: `out` of add is not v");
    RAF_CHECK(value::AsTensor(inputs[(size_t)i_w_out_])->tensor.data == w.data,
              "the fused SGD update: `out` of subtract is not w");
    if (output) {
      RAF_CHECK(value::AsTensor(output)->tensor.data == w.data,
                "the fused SGD update: the output must share w's memory (out=w)");
    }
    RAF_CHECK(w.numel() == numel_ && v.numel() == numel_ && dx.numel() == numel_,
              "the fused SGD update: tensor sizes differ from those it was built for");
    void* stream = DeviceAPI::Get(DevType::kROCM())->GetStream();
    int st;
    if (half_grad_) {
      float* xs[1] = {static_cast<float*>(w.data)};
      const void* gs[1] = {dx.data};
      float* vs[1] = {static_cast<float*>(v.data)};
      st = rafhip_sgd_multi_step(plan_, xs, gs, vs, nullptr, RAFHIP_F16, learning_rate_, mu_, stream);
    } else {
      st = rafhip_sgd_f32(static_cast<const float*>(w.data), static_cast<const float*>(dx.data),
                          static_cast<const float*>(v.data), static_cast<float*>(v.data),
                          static_cast<float*>(w.data), numel_, learning_rate_, mu_, stream);
    }
    if (st != RAFHIP_OK) {
      std::ostringstream ss;
      ss << "the fused SGD update failed with status " << st << ": " << rafhip_last_error();
      throw Error(ss.str());
    }
  }

  static OpEnv* make(const CallValues& cv) { return new SgdUpdateFusedEnv(cv); }

 private:
  // A Python float reaches the traced graph as a float64 scalar constant
  // (src/op/regs/ffi2expr.h:41-43); the kernel entry points round it to fp32 once, as raf.op.sgd
  // does with tir.const(value, dtype) (python/raf/_tvm_op/sgd.py:18-19).
  static bool Scalar(const Value& v, double* out) {
    if (auto f = std::dynamic_pointer_cast<FloatValueObj>(v)) {
      *out = f->value;
      return true;
    }
    if (auto i = std::dynamic_pointer_cast<IntValueObj>(v)) {
      *out = (double)i->value;
      return true;
    }
    return false;
  }

  static constexpr const char* kName = "raf.op.hip._fused_op(sgd_update)";
  int i_w_ = -1, i_w_out_ = -1, i_v_ = -1, i_v_out_ = -1, i_dx_ = -1, i_lr_ = -1, i_mu_ = -1;
  bool half_grad_ = false;
  double learning_rate_ = 0.0, mu_ = 0.0;
  int64_t numel_ = 0;
  rafhip_sgd_plan* plan_ = nullptr;
  std::string name_ = TruncateName(GetUniqueName("raf.op.hip._fused_op.sgd_update"));
};

// Like the reference's cutlass FusedFuncBuild: the pattern name picks the implementation.
OpEnv* FusedFuncBuild(const CallValues& call) {
  const auto* func = ir::AsFunction(call->closure);
  RAF_CHECK(func != nullptr, "raf.op.hip._fused_op: the callee is not a function");
  auto it = func->attrs.find(ir::kPatternName);
  RAF_CHECK(it != func->attrs.end(), "No pattern name marked for the function");
  if (it->second == kSgdUpdatePatternName) return SgdUpdateFusedEnv::make(call);
  throw Error("Unknown hip fusion pattern: " + it->second);
}

__attribute__((unused)) const bool g_pattern_registered = [] {
  DialectFusePattern::AddPattern(MakeSgdUpdatePattern("raf.op.", false).root, "hip",
                                 kSgdUpdatePatternPlevel, kSgdUpdatePatternName);
  return true;
}();

}  // namespace

RAF_REGISTER_DIALECT_OP(hip, add, -1);
RAF_REGISTER_DIALECT_OP(hip, subtract, -1);
RAF_REGISTER_DIALECT_OP(hip, multiply, -1);
RAF_REGISTER_DIALECT_OP(hip, cast, -1);
RAF_OP_ENV_MAKER("raf.op.hip._fused_op", FusedFuncBuild);

}  // namespace hip
}  // namespace op
}  // namespace raf

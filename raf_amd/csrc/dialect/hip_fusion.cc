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
//
// Two more rewrites work on the whole graph, because what they gather has one root per parameter
// and as many parameters as the model has (see DialectGraphRewrite in raf_ir.h):
//   sgd_multi   every per-parameter SGD update of a traced function (same learning rate, momentum
//               and dtypes) becomes ONE call of raf.op.hip.sgd_multi over the tuple of all
//               weights, gradients and velocities -- one launch instead of one per parameter --
//               and, for a half-precision model, the cast and the copy into the model's parameter
//               behind every update (python/raf/optim/sgd.py:203-215) join it as
//               raf.op.hip.sgd_multi_mixed;
//   lans_mixed  the group_cast in front of raf.op.lans (python/raf/optim/lans.py:261-265) is
//               dropped -- the kernels widen half gradients themselves -- and the per-parameter
//               cast and copy behind it (lans.py:289-291, :303-305) join it as
//               raf.op.hip.lans_mixed.
// The copy is `add(new_w, zero, out=p)` with `zero` a tensor attribute of the optimizer; it can
// only be folded away when the graph shows that tensor to be all zeros, i.e. after the model's
// constant attributes have been bound into the graph (a zeros constant here).  While `zero` is a
// free variable the cast and the copy stay as they are and only the part in front of them fuses.
#include <set>
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
const char* DTypeName(const DType& t) { return IsBF16(t) ? "bfloat16" : IsF16(t) ? "float16" : "float32"; }
}  // namespace

ir::Expr TracedSgdOptimizer(const std::vector<ir::Expr>& w, const std::vector<ir::Expr>& dx,
                            const std::vector<ir::Expr>& v, const std::vector<ir::Expr>& p,
                            const ir::Expr& zero, double learning_rate, double momentum) {
  using namespace ir;
  RAF_CHECK(w.size() == dx.size() && w.size() == v.size() && (p.empty() || p.size() == w.size()),
            "TracedSgdOptimizer: the lists differ in length");
  std::vector<Expr> outs;
  for (size_t i = 0; i < w.size(); ++i) {
    Expr new_w = TracedSgdUpdate(w[i], dx[i], v[i], learning_rate, momentum);
    if (!p.empty()) {  // sgd.py:203-215
      const TensorType pt = TypeOf(p[i]);
      Expr narrowed = MakeCall(GetOp("raf.op.cast"), {new_w, MakeString(DTypeName(pt.dtype))}, pt);
      new_w = MakeCall(GetOp("raf.op.add"), {narrowed, zero, p[i], MakeNull()}, pt);
    }
    outs.push_back(new_w);
  }
  return MakeTuple(outs);
}

ir::Expr TracedLansOptimizer(const std::vector<ir::Expr>& g, const std::vector<ir::Expr>& w,
                             const std::vector<ir::Expr>& m, const std::vector<ir::Expr>& v,
                             const std::vector<ir::Expr>& p, const ir::Expr& zero, const ir::Expr& step,
                             const LansHyper& hyper) {
  using namespace ir;
  const size_t n = w.size();
  RAF_CHECK(g.size() == n && m.size() == n && v.size() == n && p.size() == n,
            "TracedLansOptimizer: the lists differ in length");
  std::vector<TensorType> g32_types;
  for (size_t i = 0; i < n; ++i) {
    TensorType t = TypeOf(g[i]);
    t.dtype = DType{kDLFloat, 32};
    g32_types.push_back(t);
  }
  Expr fp32_g = MakeTupleCall(GetOp("raf.op.group_cast"), {MakeTuple(g), MakeString("float32")}, g32_types);
  std::vector<Expr> list;
  for (size_t i = 0; i < n; ++i) list.push_back(MakeTupleGetItem(fp32_g, (int)i));  // lans.py:261-265
  list.insert(list.end(), w.begin(), w.end());
  list.insert(list.end(), m.begin(), m.end());
  list.insert(list.end(), v.begin(), v.end());
  std::vector<TensorType> out_types;
  for (const Expr& e : list) out_types.push_back(TypeOf(e));
  Expr out = MakeTupleCall(
      GetOp("raf.op.lans"),
      {MakeTuple(list), step, MakeFloat(hyper.learning_rate), MakeFloat(hyper.beta1), MakeFloat(hyper.beta2),
       MakeFloat(hyper.eps), MakeInt(hyper.bias_correction), MakeFloat(hyper.weight_decay),
       MakeInt(hyper.grad_averaging), MakeInt(hyper.mode), MakeInt(hyper.normalize_grad)},
      out_types);  // lans.py:268-280
  std::vector<Expr> next_w, next_m, next_v;
  for (size_t i = 0; i < n; ++i) {
    const TensorType pt = TypeOf(p[i]);
    Expr new_w = MakeTupleGetItem(out, (int)(n + i));
    Expr narrowed = MakeCall(GetOp("raf.op.cast"), {new_w, MakeString(DTypeName(pt.dtype))}, pt);  // :289-291
    next_w.push_back(MakeCall(GetOp("raf.op.add"), {narrowed, zero, p[i], MakeNull()}, pt));      // :303-305
    next_m.push_back(MakeTupleGetItem(out, (int)(2 * n + i)));
    next_v.push_back(MakeTupleGetItem(out, (int)(3 * n + i)));
  }
  std::vector<Expr> result = next_w;
  result.insert(result.end(), next_m.begin(), next_m.end());
  result.insert(result.end(), next_v.begin(), next_v.end());
  return MakeTuple(result);
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

// ------------------------------------------------------------------ whole-graph rewrites
using ir::Expr;
using ir::ExprNode;

// Who uses what: every argument slot, tuple field, tuple projection and function body counts.
struct UseMap {
  std::map<const ExprNode*, std::vector<const ExprNode*>> users;
  explicit UseMap(const std::vector<Expr>& nodes) {
    for (const Expr& e : nodes) {
      if (const auto* c = ir::AsCall(e)) {
        for (const auto& a : c->args) users[a.get()].push_back(e.get());
      } else if (const auto* t = ir::AsTupleNode(e)) {
        for (const auto& f : t->fields) users[f.get()].push_back(e.get());
      } else if (const auto* g = ir::AsTupleGetItem(e)) {
        users[g->tuple.get()].push_back(e.get());
      } else if (const auto* f = ir::AsFunction(e)) {
        users[f->body.get()].push_back(e.get());
      }
    }
  }
  const std::vector<const ExprNode*>& of(const ExprNode* n) const {
    static const std::vector<const ExprNode*> none;
    auto it = users.find(n);
    return it == users.end() ? none : it->second;
  }
};

bool IsCallOf(const Expr& e, const char* op_name) {
  const auto* c = ir::AsCall(e);
  const auto* o = c ? ir::AsOp(c->op) : nullptr;
  return o && o->name == op_name;
}

bool SameShape(const ir::TensorType& a, const ir::TensorType& b) {
  return a.defined && b.defined && a.shape == b.shape;
}

// The half-precision tail behind a new fp32 weight `new_w`:
//     p_new = add(cast(new_w, "float16" | "bfloat16"), zeros, out=p, where=null)
// with nothing else using new_w or the cast, `zeros` an all-zero constant and p a 16-bit tensor of
// new_w's shape and the cast's dtype.  Returns the add call and p, or nulls.
struct HalfTail {
  Expr add, p;
  bool bf16 = false;
};
HalfTail FindHalfTail(const Expr& new_w, const UseMap& uses, const std::map<const ExprNode*, Expr>& by_ptr) {
  HalfTail none;
  const auto& u1 = uses.of(new_w.get());
  if (u1.size() != 1) return none;
  const Expr cast = by_ptr.at(u1[0]);
  if (!IsCallOf(cast, "raf.op.cast")) return none;
  const auto* cc = ir::AsCall(cast);
  const auto* dt = cc->args.size() == 2 ? ir::AsConstant(cc->args[1]) : nullptr;
  if (!dt || dt->value_kind != ir::ConstantNode::kString || cc->args[0].get() != new_w.get()) return none;
  const bool bf16 = dt->s == "bfloat16";
  if (!bf16 && dt->s != "float16") return none;
  const auto& u2 = uses.of(cast.get());
  if (u2.size() != 1) return none;
  const Expr add = by_ptr.at(u2[0]);
  if (!IsCallOf(add, "raf.op.add")) return none;
  const auto* ac = ir::AsCall(add);
  if (ac->args.size() != 4 || ac->args[0].get() != cast.get()) return none;
  const auto* zero = ir::AsConstant(ac->args[1]);
  const auto* where = ir::AsConstant(ac->args[3]);
  if (!zero || zero->value_kind != ir::ConstantNode::kZeros) return none;
  if (!where || where->value_kind != ir::ConstantNode::kNull) return none;
  const ir::TensorType pt = ir::TypeOf(ac->args[2]);
  if (!SameShape(pt, ir::TypeOf(new_w))) return none;
  if (!(bf16 ? IsBF16(pt.dtype) : IsF16(pt.dtype))) return none;
  HalfTail t;
  t.add = add;
  t.p = ac->args[2];
  t.bf16 = bf16;
  return t;
}

// True if any expression of `roots` can reach a node of `stops` through its operands.
bool Reaches(const std::vector<Expr>& roots, const std::set<const ExprNode*>& stops) {
  for (const Expr& r : roots)
    for (const Expr& e : ir::PostOrder(r))
      if (stops.count(e.get())) return true;
  return false;
}

std::vector<ir::TensorType> TypesOf(const std::vector<Expr>& fields) {
  std::vector<ir::TensorType> out;
  for (const Expr& f : fields) out.push_back(ir::TypeOf(f));
  return out;
}

bool ScalarConstant(const Expr& e, double* out) {
  const auto* k = ir::AsConstant(e);
  if (!k) return false;
  if (k->value_kind == ir::ConstantNode::kFloat) {
    *out = k->f;
    return true;
  }
  if (k->value_kind == ir::ConstantNode::kInt) {
    *out = (double)k->i;
    return true;
  }
  return false;
}

// ---- every per-parameter SGD update of the graph in one raf.op.hip.sgd_multi[_mixed] call
Expr FuseMultiTensorSgd(const Expr& root) {
  const std::vector<Expr> nodes = ir::PostOrder(root);
  std::map<const ExprNode*, Expr> by_ptr;
  for (const Expr& e : nodes) by_ptr[e.get()] = e;
  const UseMap uses(nodes);
  const SgdUpdatePattern pat = MakeSgdUpdatePattern("raf.op.", false);
  const std::vector<const ir::DFPatternNode*> call_patterns = ir::CallPatternsOf(pat.root);

  struct Match {
    Expr root, w, dx, v, out;  // out: what stands for this parameter's result (root or the tail's add)
    HalfTail tail;
    std::set<const ExprNode*> calls;
  };
  // key: learning rate, momentum, gradient dtype (32, 16, -16 for bfloat16), tail (0, 16, -16)
  std::map<std::tuple<double, double, int, int>, std::vector<Match>> groups;
  for (const Expr& e : nodes) {
    if (!IsCallOf(e, "raf.op.subtract")) continue;
    ir::NodeMap nm;
    if (!ir::MatchPattern(pat.root, e, &nm)) continue;
    Match m;
    m.root = e;
    m.w = nm.at(pat.w.get());
    m.v = nm.at(pat.v.get());
    const bool half = nm.count(pat.dx_half.get()) != 0;
    m.dx = half ? nm.at(pat.dx_half.get()) : nm.at(pat.dx.get());
    double lr = 0, mu = 0;
    if (!ScalarConstant(nm.at(pat.lr.get()), &lr) || !ScalarConstant(nm.at(pat.mu.get()), &mu)) continue;
    const ir::TensorType wt = ir::TypeOf(m.w), gt = ir::TypeOf(m.dx);
    if (!SameShape(wt, ir::TypeOf(m.v)) || !SameShape(wt, gt)) continue;  // no broadcasting
    for (const auto* cp : call_patterns) {
      auto it = nm.find(cp);
      if (it != nm.end()) m.calls.insert(it->second.get());
    }
    // the calls inside the match must have no user outside it (the old out= call would stay alive)
    bool is_private = true;
    for (const ExprNode* inner : m.calls) {
      if (inner == e.get()) continue;
      for (const ExprNode* user : uses.of(inner)) is_private = is_private && m.calls.count(user) != 0;
    }
    if (!is_private) continue;
    m.tail = FindHalfTail(e, uses, by_ptr);
    m.out = m.tail.add ? m.tail.add : e;
    const int g_kind = !half ? 32 : (IsBF16(gt.dtype) ? -16 : 16);
    const int t_kind = !m.tail.add ? 0 : (m.tail.bf16 ? -16 : 16);
    groups[std::make_tuple(lr, mu, g_kind, t_kind)].push_back(std::move(m));
  }

  std::map<const ExprNode*, Expr> replace;
  for (auto& kv : groups) {
    std::vector<Match>& ms = kv.second;
    if (ms.size() < 2) continue;  // a single update is what the sgd_update pattern is for
    std::vector<Expr> ws, dxs, vs, ps, leaves;
    std::set<const ExprNode*> produced, seen_w;
    bool distinct = true;
    for (const Match& m : ms) {
      ws.push_back(m.w);
      dxs.push_back(m.dx);
      vs.push_back(m.v);
      if (m.tail.add) ps.push_back(m.tail.p);
      produced.insert(m.calls.begin(), m.calls.end());
      if (m.tail.add) produced.insert(m.tail.add.get());
      distinct = distinct && seen_w.insert(m.w.get()).second && seen_w.insert(m.v.get()).second;
    }
    leaves = ws;
    leaves.insert(leaves.end(), dxs.begin(), dxs.end());
    leaves.insert(leaves.end(), vs.begin(), vs.end());
    leaves.insert(leaves.end(), ps.begin(), ps.end());
    // gathering is only a reordering of independent updates: no input may come out of another one
    if (!distinct || Reaches(leaves, produced)) continue;
    const bool mixed = !ps.empty();
    const Expr op = LowerOp(mixed ? "raf.op.sgd_multi_mixed" : "raf.op.sgd_multi", "hip");
    if (!op) continue;
    const size_t n = ms.size();
    Expr call = ir::MakeTupleCall(op, {ir::MakeTuple(leaves), ir::MakeFloat(std::get<0>(kv.first)),
                                       ir::MakeFloat(std::get<1>(kv.first))},
                                  TypesOf(leaves));
    // the op returns its list: the new weights are fields 0..n-1, the model's parameters 3n..4n-1
    for (size_t i = 0; i < n; ++i)
      replace[ms[i].out.get()] = ir::MakeTupleGetItem(call, (int)(mixed ? 3 * n + i : i));
  }
  return replace.empty() ? root : ir::Substitute(root, replace);
}

// ---- group_cast -> lans -> cast -> add(out=p) as one raf.op.hip.lans[_mixed] call
Expr FuseLansMixed(const Expr& root) {
  const std::vector<Expr> nodes = ir::PostOrder(root);
  std::map<const ExprNode*, Expr> by_ptr;
  for (const Expr& e : nodes) by_ptr[e.get()] = e;
  const UseMap uses(nodes);
  std::map<const ExprNode*, Expr> replace;
  for (const Expr& e : nodes) {
    if (!IsCallOf(e, "raf.op.lans")) continue;
    const auto* lans = ir::AsCall(e);
    if (lans->args.size() != 11) continue;
    const auto* list = ir::AsTupleNode(lans->args[0]);
    if (!list || list->fields.empty() || list->fields.size() % 4 != 0) continue;
    const size_t n = list->fields.size() / 4;
    // the gradients: field i of ONE group_cast(tuple of n half tensors, "float32")
    const auto* first = ir::AsTupleGetItem(list->fields[0]);
    if (!first || !IsCallOf(first->tuple, "raf.op.group_cast")) continue;
    const Expr gc = first->tuple;
    const auto* gcc = ir::AsCall(gc);
    const auto* halves = gcc->args.size() == 2 ? ir::AsTupleNode(gcc->args[0]) : nullptr;
    const auto* to = gcc->args.size() == 2 ? ir::AsConstant(gcc->args[1]) : nullptr;
    if (!halves || halves->fields.size() != n || !to || to->value_kind != ir::ConstantNode::kString ||
        to->s != "float32")
      continue;
    bool ok = true;
    int g_kind = 0;
    for (size_t i = 0; ok && i < n; ++i) {
      const auto* gi = ir::AsTupleGetItem(list->fields[i]);
      ok = gi && gi->tuple.get() == gc.get() && gi->index == (int)i;
      const ir::TensorType ht = ir::TypeOf(halves->fields[i]);
      const int kind = !ht.defined ? 0 : IsF16(ht.dtype) ? 16 : IsBF16(ht.dtype) ? -16 : 0;
      ok = ok && kind != 0 && (i == 0 || kind == g_kind);
      g_kind = kind;
      for (size_t q = 1; ok && q < 4; ++q) {  // w, m, v: fp32 tensors of the gradient's shape
        const ir::TensorType t = ir::TypeOf(list->fields[q * n + i]);
        ok = t.defined && IsF32(t.dtype) && SameShape(t, ht);
      }
    }
    if (!ok) continue;
    // what is taken from the op's result: only w, m, v may be (the fp32 gradients would be gone)
    // A field may be projected by more than one TupleGetItem node; every one of them is replaced,
    // or the old call would stay alive beside the new one and update the tensors twice.
    std::map<int, std::vector<Expr>> taken;  // field index -> its TupleGetItem nodes
    bool only_projections = true;
    for (const ExprNode* user : uses.of(e.get())) {
      const auto* g = ir::AsTupleGetItem(by_ptr.at(user));
      only_projections = only_projections && g != nullptr && g->index >= (int)n && g->index < (int)(4 * n);
      if (g) taken[g->index].push_back(by_ptr.at(user));
    }
    if (!only_projections) continue;
    // the half-precision tails, all or none; a new weight that is projected twice has other users
    // than its cast, so it has no tail
    std::vector<HalfTail> tails;
    for (size_t i = 0; i < n; ++i) {
      auto it = taken.find((int)(n + i));
      HalfTail t = it == taken.end() || it->second.size() != 1 ? HalfTail()
                                                              : FindHalfTail(it->second[0], uses, by_ptr);
      if (!t.add || (!tails.empty() && t.bf16 != tails[0].bf16)) break;
      tails.push_back(t);
    }
    const bool mixed = tails.size() == n;
    std::vector<Expr> fields(halves->fields.begin(), halves->fields.end());
    fields.insert(fields.end(), list->fields.begin() + (std::ptrdiff_t)n, list->fields.end());
    if (mixed) {
      std::set<const ExprNode*> produced = {e.get()};
      std::vector<Expr> ps;
      for (const HalfTail& t : tails) ps.push_back(t.p);
      if (Reaches(ps, produced)) continue;
      fields.insert(fields.end(), ps.begin(), ps.end());
    }
    const Expr op = LowerOp(mixed ? "raf.op.lans_mixed" : "raf.op.lans", "hip");
    if (!op) continue;
    std::vector<Expr> args(lans->args.begin(), lans->args.end());
    args[0] = ir::MakeTuple(fields);
    const Expr call = ir::MakeTupleCall(op, args, TypesOf(fields));
    for (const auto& kv : taken)
      for (const Expr& projection : kv.second) replace[projection.get()] = ir::MakeTupleGetItem(call, kv.first);
    if (mixed)
      for (size_t i = 0; i < n; ++i) replace[tails[i].add.get()] = ir::MakeTupleGetItem(call, (int)(4 * n + i));
  }
  return replace.empty() ? root : ir::Substitute(root, replace);
}

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
  DialectGraphRewrite::Add("hip", 20, "sgd_multi", FuseMultiTensorSgd);
  DialectGraphRewrite::Add("hip", 10, "lans_mixed", FuseLansMixed);
  return true;
}();

}  // namespace

RAF_REGISTER_DIALECT_OP(hip, add, -1);
RAF_REGISTER_DIALECT_OP(hip, subtract, -1);
RAF_REGISTER_DIALECT_OP(hip, multiply, -1);
RAF_REGISTER_DIALECT_OP(hip, cast, -1);
// raf.op.group_cast has no hip backend: the lans_mixed rewrite removes it from in front of LANS.
RAF_OP_ENV_MAKER("raf.op.hip._fused_op", FusedFuncBuild);

}  // namespace hip
}  // namespace op
}  // namespace raf

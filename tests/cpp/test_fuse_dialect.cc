// Host-side checks of the graph IR mirror, the dataflow patterns and the FuseDialect pass, in the
// manner of the reference's tests/python/pass/test_pass_fuse_dialect.py: build the graph the
// traced SGD optimizer emits (python/raf/optim/sgd.py:192-200), run the pass, and compare with
// the expected graph structurally (:41-105 fusion, :108-138 single call, :142-163 no fusion,
// :166-215 identical functions are shared).  Runs without a GPU.
#include <cstdio>
#include <cstdlib>
#include <string>

#include "hip_dialect.h"
#include "raf_iface.h"
#include "raf_ir.h"

using namespace raf;
using namespace raf::ir;
using namespace raf::op;

#define EXPECT(cond)                                                         \
  do {                                                                       \
    if (!(cond)) {                                                           \
      std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                          \
    }                                                                        \
  } while (0)

template <typename F>
static std::string Raises(F&& f) {
  try {
    f();
  } catch (const raf::Error& e) {
    return e.what();
  }
  return "";
}

static bool Contains(const std::string& s, const char* what) { return s.find(what) != std::string::npos; }

static TensorType Ty(std::vector<int64_t> shape, int bits = 32, int code = kDLFloat) {
  TensorType t;
  t.defined = true;
  t.shape = std::move(shape);
  t.dtype = DType{code, bits};
  return t;
}

// A fake CPU dialect with a one-call pattern and a two-call pattern, like the reference's cublas
// and cutlass entries for dense (python/raf/_op/dialect_pattern.py:139-143).
RAF_REGISTER_DIALECT("fakeblas").set_enable(DevType::kCPU());
RAF_REGISTER_DIALECT_OP(fakeblas, dense, 7);
RAF_REGISTER_DIALECT_OP(fakeblas, relu, 7);

// What FuseDialect must make of one traced update (parameter order: depth-first over the root's
// arguments, one parameter per use of an outside value).
static Expr ExpectedFusedUpdate(const Expr& w, const Expr& dx, const Expr& v, double lr, double mu,
                                Expr* func_out = nullptr, const Expr& reuse = nullptr) {
  const TensorType wt = TypeOf(w), none;
  const bool half = TypeOf(dx).dtype.bits == 16;
  Expr p_w = MakeVar("p", wt), p_lr = MakeVar("p", none), p_mu = MakeVar("p", none);
  Expr p_v = MakeVar("p", wt), p_dx = MakeVar("p", TypeOf(dx)), p_ty = MakeVar("p", none);
  Expr p_vout = MakeVar("p", wt), p_n1 = MakeVar("p", none), p_wout = MakeVar("p", wt), p_n2 = MakeVar("p", none);
  Expr grad = p_dx;
  if (half) grad = MakeCall(GetOp("raf.op.hip.cast"), {p_dx, p_ty}, wt);
  Expr mv = MakeCall(GetOp("raf.op.hip.multiply"), {p_mu, p_v}, wt);
  Expr nv = MakeCall(GetOp("raf.op.hip.add"), {mv, grad, p_vout, p_n1}, wt);
  Expr st = MakeCall(GetOp("raf.op.hip.multiply"), {p_lr, nv}, wt);
  Expr body = MakeCall(GetOp("raf.op.hip.subtract"), {p_w, st, p_wout, p_n2}, wt);
  std::vector<Expr> params = {p_w, p_lr, p_mu, p_v, p_dx};
  if (half) params.push_back(p_ty);
  params.insert(params.end(), {p_vout, p_n1, p_wout, p_n2});
  Expr func = reuse ? reuse
                    : MakeFunction(params, body,
                                   {{"Primitive", "1"}, {"Dialect", "hip"}, {"PatternName", "sgd_update"}});
  if (func_out) *func_out = func;
  std::vector<Expr> args = {w, MakeFloat(lr), MakeFloat(mu), v, dx};
  if (half) args.push_back(MakeString("float32"));
  args.insert(args.end(), {v, MakeNull(), w, MakeNull()});
  return MakeCall(func, args, wt);
}

int main() {
  std::puts("pattern registry: plevel-descending, duplicate plevel refused");
  {
    auto* list = DialectFusePattern::Get();
    EXPECT(list->size() == 1 && list->front().dialect == "hip" && list->front().name == "sgd_update" &&
           list->front().plevel == 60);
    DialectFusePattern::AddPattern(call(is_op("raf.op.dense"), {wildcard(), wildcard()}), "fakeblas", 9, "dense");
    DialectFusePattern::AddPattern(
        call(is_op("raf.op.relu"), {call(is_op("raf.op.dense"), {wildcard(), wildcard()})}), "fakeblas", 70,
        "dense_relu");
    std::vector<int> plevels;
    for (const auto& p : *list) plevels.push_back(p.plevel);
    EXPECT((plevels == std::vector<int>{70, 60, 9}));
    EXPECT(Contains(Raises([] { DialectFusePattern::AddPattern(wildcard(), "hip", 60, "again"); }),
                    "dialect pattern with plevel 60 is already registered"));
    EXPECT(OpDialect::Lower("raf.op.add", "hip") == "raf.op.hip.add");
    EXPECT(OpDialect::Lower("raf.op.add", "fakeblas").empty());
    // fusion-only dialect ops are never picked for a single op
    EXPECT(OpDialect::Dispatch("raf.op.add", DevType::kROCM()).empty());
    EXPECT(OpEnvMaker::Get("raf.op.hip.add") == nullptr && OpEnvMaker::Get("raf.op.hip._fused_op") != nullptr);
  }

  std::puts("patterns: shared nodes, alternatives, constants, dtypes");
  {
    Expr a = MakeVar("a", Ty({4})), b = MakeVar("b", Ty({4}, 16));
    DFPattern x = wildcard();
    DFPattern twice = call(is_op("raf.op.add"), {x, x, is_constant(MakeNull()), is_constant(MakeNull())});
    EXPECT(MatchPattern(twice, MakeCall(GetOp("raf.op.add"), {a, a, MakeNull(), MakeNull()})));
    EXPECT(!MatchPattern(twice, MakeCall(GetOp("raf.op.add"), {a, b, MakeNull(), MakeNull()})));
    EXPECT(!MatchPattern(twice, MakeCall(GetOp("raf.op.add"), {a, a, MakeNull(), MakeInt(0)})));
    EXPECT(!MatchPattern(twice, MakeCall(GetOp("raf.op.add"), {a, a})));
    EXPECT(!MatchPattern(twice, MakeCall(GetOp("raf.op.subtract"), {a, a, MakeNull(), MakeNull()})));
    // a failed left alternative must not leave bindings behind: (x, x) fails on (a, b), then (x, y) fits
    DFPattern y = wildcard();
    DFPattern either = alt(call(is_op("raf.op.multiply"), {x, x}), call(is_op("raf.op.multiply"), {x, y}));
    NodeMap nm;
    EXPECT(MatchPattern(either, MakeCall(GetOp("raf.op.multiply"), {b, a}), &nm));
    EXPECT(nm.at(x.get()).get() == b.get() && nm.at(y.get()).get() == a.get());
    EXPECT(MatchPattern(has_dtype(DType{kDLFloat, 16}), b) && !MatchPattern(has_dtype(DType{kDLFloat, 16}), a));
    EXPECT(!MatchPattern(has_dtype(DType{kDLFloat, 32}), MakeVar("untyped")));
    EXPECT(MatchPattern(is_constant(MakeFloat(0.5)), MakeFloat(0.5)) &&
           !MatchPattern(is_constant(MakeFloat(0.5)), MakeFloat(0.25)) &&
           !MatchPattern(is_constant(MakeFloat(1)), MakeInt(1)) && MatchPattern(is_constant(), MakeString("s")) &&
           !MatchPattern(is_constant(), a));
    EXPECT(MatchPattern(is_ops({"raf.op.relu", "raf.op.gelu"}), GetOp("raf.op.gelu")));
    EXPECT(GetOp("raf.op.relu").get() == GetOp("raf.op.relu").get());
  }

  std::puts("structural equality");
  {
    Expr a = MakeVar("a", Ty({4})), b = MakeVar("b", Ty({4})), c = MakeVar("c", Ty({5}));
    Expr ab = MakeCall(GetOp("raf.op.multiply"), {a, b}), ba = MakeCall(GetOp("raf.op.multiply"), {b, a});
    EXPECT(StructuralEqual(ab, ba));  // free variables correspond in order of use
    EXPECT(!StructuralEqual(ab, MakeCall(GetOp("raf.op.multiply"), {a, a})));
    EXPECT(!StructuralEqual(MakeCall(GetOp("raf.op.multiply"), {a, a}), ab));
    EXPECT(!StructuralEqual(ab, MakeCall(GetOp("raf.op.multiply"), {a, c})));
    EXPECT(!StructuralEqual(ab, MakeCall(GetOp("raf.op.add"), {a, b})));
    EXPECT(StructuralEqual(MakeFunction({a, b}, ab), MakeFunction({b, a}, ba)));
    EXPECT(!StructuralEqual(MakeFunction({a, b}, ab), MakeFunction({a, b}, ba)));
    EXPECT(!StructuralEqual(MakeFunction({a, b}, ab), MakeFunction({a, b}, ab, {{"Primitive", "1"}})));
    Expr p = MakeVar("p", Ty({4})), q = MakeVar("p", Ty({4}));  // equal hints: equal text
    EXPECT(AsText(MakeFunction({a, b}, ab)) != AsText(MakeFunction({b, a}, ba)));
    EXPECT(AsText(MakeFunction({p, q}, MakeCall(GetOp("raf.op.multiply"), {p, q}))) ==
           AsText(MakeFunction({q, p}, MakeCall(GetOp("raf.op.multiply"), {q, p}))));
  }

  std::puts("the traced float32 update becomes one call of a primitive hip function");
  Expr w = MakeVar("w", Ty({1024, 1024})), dx = MakeVar("dx", Ty({1024, 1024})), v = MakeVar("v", Ty({1024, 1024}));
  Expr fused_fn;
  {
    Expr traced = hip::TracedSgdUpdate(w, dx, v, 0.01, 0.9);
    EXPECT(Contains(AsText(traced), "raf.op.subtract(%w") && !Contains(AsText(traced), "hip"));
    Expr fused = pass::FuseDialect(traced, DevType::kROCM());
    Expr expected = ExpectedFusedUpdate(w, dx, v, 0.01, 0.9, &fused_fn);
    if (!StructuralEqual(fused, expected))
      std::fprintf(stderr, "got:\n%s\nexpected:\n%s\n", AsText(fused).c_str(), AsText(expected).c_str());
    EXPECT(StructuralEqual(fused, expected));
    // the arguments are the original expressions, `out` included
    const auto* c = AsCall(fused);
    EXPECT(c->args[0].get() == w.get() && c->args[3].get() == v.get() && c->args[4].get() == dx.get() &&
           c->args[5].get() == v.get() && c->args[7].get() == w.get());
    EXPECT(AsFunction(c->op)->params.size() == 9);
    // a second run finds nothing left to fuse
    EXPECT(pass::FuseDialect(fused, DevType::kROCM()).get() == fused.get());
  }

  std::puts("a 16-bit gradient is fused together with its cast");
  for (int code : {kDLFloat, kDLBfloat}) {
    Expr dx16 = MakeVar("dx", Ty({1024, 1024}, 16, code));
    Expr fused = pass::FuseDialect(hip::TracedSgdUpdate(w, dx16, v, 0.01, 0.9), DevType::kROCM());
    EXPECT(StructuralEqual(fused, ExpectedFusedUpdate(w, dx16, v, 0.01, 0.9)));
    EXPECT(AsFunction(AsCall(fused)->op)->params.size() == 10);
  }

  std::puts("no fusion: other device, unknown or unsupported types, out= elsewhere, where=");
  {
    Expr traced = hip::TracedSgdUpdate(w, dx, v, 0.01, 0.9);
    EXPECT(pass::FuseDialect(traced, DevType::kCPU()).get() == traced.get());
    EXPECT(pass::FuseDialect(traced, DevType::kCUDA()).get() == traced.get());
    EXPECT(pass::FuseDialect(traced, DevType::kUnknown()).get() == traced.get());
    Expr uw = MakeVar("w"), udx = MakeVar("dx"), uv = MakeVar("v");
    Expr untyped = hip::TracedSgdUpdate(uw, udx, uv, 0.01, 0.9);
    EXPECT(pass::FuseDialect(untyped, DevType::kROCM()).get() == untyped.get());
    Expr w64 = MakeVar("w", Ty({8}, 64)), dx64 = MakeVar("dx", Ty({8}, 64)), v64 = MakeVar("v", Ty({8}, 64));
    Expr f64 = hip::TracedSgdUpdate(w64, dx64, v64, 0.01, 0.9);
    EXPECT(!Contains(AsText(pass::FuseDialect(f64, DevType::kROCM())), "hip"));
    // the velocity written somewhere else than v is another computation
    Expr other = MakeVar("other", Ty({1024, 1024}));
    Expr mv = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.9), v}, TypeOf(v));
    Expr nv = MakeCall(GetOp("raf.op.add"), {mv, dx, other, MakeNull()}, TypeOf(v));
    Expr st = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.01), nv}, TypeOf(v));
    Expr elsewhere = MakeCall(GetOp("raf.op.subtract"), {w, st, w, MakeNull()}, TypeOf(w));
    EXPECT(pass::FuseDialect(elsewhere, DevType::kROCM()).get() == elsewhere.get());
    Expr nv2 = MakeCall(GetOp("raf.op.add"), {mv, dx, v, other}, TypeOf(v));  // where=other
    Expr st2 = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.01), nv2}, TypeOf(v));
    Expr masked = MakeCall(GetOp("raf.op.subtract"), {w, st2, w, MakeNull()}, TypeOf(w));
    EXPECT(pass::FuseDialect(masked, DevType::kROCM()).get() == masked.get());
    // a learning rate that is a tensor, not a constant
    Expr lr_t = MakeVar("lr", Ty({}));
    Expr nv3 = MakeCall(GetOp("raf.op.add"), {mv, dx, v, MakeNull()}, TypeOf(v));
    Expr st3 = MakeCall(GetOp("raf.op.multiply"), {lr_t, nv3}, TypeOf(v));
    Expr sched = MakeCall(GetOp("raf.op.subtract"), {w, st3, w, MakeNull()}, TypeOf(w));
    EXPECT(pass::FuseDialect(sched, DevType::kROCM()).get() == sched.get());
  }

  std::puts("no fusion when a value inside the match is also used outside it");
  {
    // new_v feeds the weight update and is returned as well: fusing would leave the old add(out=v)
    // alive beside the fused function, and v would be updated twice
    Expr mv = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.9), v}, TypeOf(v));
    Expr nv = MakeCall(GetOp("raf.op.add"), {mv, dx, v, MakeNull()}, TypeOf(v));
    Expr st = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.01), nv}, TypeOf(v));
    Expr nw = MakeCall(GetOp("raf.op.subtract"), {w, st, w, MakeNull()}, TypeOf(w));
    Expr both = MakeCall(GetOp("raf.op.tuple3"), {nw, nv, dx});
    EXPECT(pass::FuseDialect(both, DevType::kROCM()).get() == both.get());
    // the same update without the second consumer is fused, also below another call
    Expr alone = MakeCall(GetOp("raf.op.tuple3"), {nw, dx, dx});
    Expr fused = pass::FuseDialect(alone, DevType::kROCM());
    EXPECT(fused.get() != alone.get() && AsFunction(AsCall(AsCall(fused)->args[0])->op) != nullptr);
    // a shared dense: dense+relu may not swallow it, the one-call pattern still lowers it once
    Expr x = MakeVar("x", Ty({10, 20})), k = MakeVar("k", Ty({30, 20}));
    Expr dense = MakeCall(GetOp("raf.op.dense"), {x, k}, Ty({10, 30}));
    Expr act = MakeCall(GetOp("raf.op.relu"), {dense}, Ty({10, 30}));
    Expr shared = MakeCall(GetOp("raf.op.tuple3"), {act, dense, x});
    Expr got = pass::FuseDialect(shared, DevType::kCPU());
    Expr low = MakeCall(GetOp("raf.op.fakeblas.dense"), {x, k}, Ty({10, 30}));
    Expr want = MakeCall(GetOp("raf.op.tuple3"), {MakeCall(GetOp("raf.op.relu"), {low}, Ty({10, 30})), low, x});
    EXPECT(StructuralEqual(got, want));
  }

  std::puts("updates of equal type share one fused function; another shape gets its own");
  {
    Expr w2 = MakeVar("w2", Ty({1024, 1024})), dx2 = MakeVar("dx2", Ty({1024, 1024})), v2 = MakeVar("v2", Ty({1024, 1024}));
    Expr w3 = MakeVar("w3", Ty({1024})), dx3 = MakeVar("dx3", Ty({1024})), v3 = MakeVar("v3", Ty({1024}));
    // the three updates hang under one root, as outputs of the traced function would; their
    // learning rates differ, so they are not gathered into one multi-tensor call (the constants
    // are lifted into parameters, so the functions are still identical)
    Expr root = MakeCall(GetOp("raf.op.tuple3"),
                         {hip::TracedSgdUpdate(w, dx, v, 0.01, 0.9), hip::TracedSgdUpdate(w2, dx2, v2, 0.02, 0.9),
                          hip::TracedSgdUpdate(w3, dx3, v3, 0.03, 0.9)});
    Expr fused = pass::FuseDialect(root, DevType::kROCM());
    const auto* c = AsCall(fused);
    EXPECT(c && c->args.size() == 3);
    const auto *c0 = AsCall(c->args[0]), *c1 = AsCall(c->args[1]), *c2 = AsCall(c->args[2]);
    EXPECT(AsFunction(c0->op) && c0->op.get() == c1->op.get() && c2->op.get() != c0->op.get());
    Expr fn;
    Expr e0 = ExpectedFusedUpdate(w, dx, v, 0.01, 0.9, &fn);
    Expr expected = MakeCall(GetOp("raf.op.tuple3"),
                             {e0, ExpectedFusedUpdate(w2, dx2, v2, 0.02, 0.9, nullptr, fn),
                              ExpectedFusedUpdate(w3, dx3, v3, 0.03, 0.9)});
    EXPECT(StructuralEqual(fused, expected));
    // sharing is part of the structure: three separate functions are a different graph
    Expr separate = MakeCall(GetOp("raf.op.tuple3"),
                             {ExpectedFusedUpdate(w, dx, v, 0.01, 0.9), ExpectedFusedUpdate(w2, dx2, v2, 0.02, 0.9),
                              ExpectedFusedUpdate(w3, dx3, v3, 0.03, 0.9)});
    EXPECT(!StructuralEqual(fused, separate));
  }

  std::puts("plevel order; a one-call match is lowered without a function");
  {
    Expr x = MakeVar("x", Ty({10, 20})), k = MakeVar("k", Ty({30, 20}));
    Expr dense = MakeCall(GetOp("raf.op.dense"), {x, k}, Ty({10, 30}));
    Expr alone = MakeCall(GetOp("raf.op.multiply"), {dense, MakeFloat(2.0)}, Ty({10, 30}));
    Expr got = pass::FuseDialect(alone, DevType::kCPU());
    Expr want = MakeCall(GetOp("raf.op.multiply"),
                         {MakeCall(GetOp("raf.op.fakeblas.dense"), {x, k}, Ty({10, 30})), MakeFloat(2.0)}, Ty({10, 30}));
    EXPECT(StructuralEqual(got, want));
    // dense+relu (plevel 70) wins over dense alone (plevel 9)
    Expr act = MakeCall(GetOp("raf.op.relu"), {dense}, Ty({10, 30}));
    got = pass::FuseDialect(act, DevType::kCPU());
    const auto* c = AsCall(got);
    const auto* f = c ? AsFunction(c->op) : nullptr;
    EXPECT(f && f->attrs.at("Dialect") == "fakeblas" && f->attrs.at("PatternName") == "dense_relu" &&
           f->attrs.at("Primitive") == "1" && f->params.size() == 2 && c->args[0].get() == x.get());
    EXPECT(Contains(AsText(got), "raf.op.fakeblas.relu") && Contains(AsText(got), "raf.op.fakeblas.dense"));
    // a dialect without an op for a matched call is an error, as in the reference
    DialectFusePattern::AddPattern(call(is_op("raf.op.gelu"), {wildcard()}), "fakeblas", 3, "gelu");
    EXPECT(Contains(Raises([&] { pass::FuseDialect(MakeCall(GetOp("raf.op.gelu"), {x}), DevType::kCPU()); }),
                    "Cannot find dialect \"fakeblas\" registered to operator raf.op.gelu"));
  }

  std::puts("fused dispatch: the maker is found by dialect, the implementation by pattern name");
  {
    Expr fused = pass::FuseDialect(hip::TracedSgdUpdate(w, dx, v, 0.01, 0.9), DevType::kROCM());
    auto tensor = [](const Expr& var, DevType dev, void* data) {
      TensorView t;
      t.shape = AsVar(var)->type.shape;
      t.dtype = AsVar(var)->type.dtype;
      t.device = Device(dev, 0);
      t.data = data;
      return value::MakeTensor(t);
    };
    std::map<const ExprNode*, value::Value> on_cpu = {{w.get(), tensor(w, DevType::kCPU(), nullptr)},
                                                      {dx.get(), tensor(dx, DevType::kCPU(), nullptr)},
                                                      {v.get(), tensor(v, DevType::kCPU(), nullptr)}};
    CallValues cv = BindCall(fused, on_cpu, Device(DevType::kCPU(), 0));
    EXPECT(cv->closure && cv->args_as<schema::ListArgs>()->args.size() == 9);
    EXPECT(cv->args_as<schema::ListArgs>()->args[6] == nullptr);  // null constant
    std::string err = Raises([&] { Dispatch(cv); });
    EXPECT(Contains(err, "Failed to dispatch fused op:") && Contains(err, "device is not rocm") &&
           Contains(err, "Name: raf.op.hip._fused_op") && Contains(err, "PatternName=sgd_update"));
    EXPECT(Contains(Raises([&] { BindCall(fused, {}, Device(DevType::kROCM(), 0)); }), "bound variable"));

    const auto* c = AsCall(fused);
    const auto* f = AsFunction(c->op);
    auto attrs = f->attrs;
    attrs["PatternName"] = "conv";
    CallValues unknown = BindCall(MakeCall(MakeFunction(f->params, f->body, attrs), c->args), on_cpu,
                                  Device(DevType::kROCM(), 0));
    EXPECT(Contains(Raises([&] { Dispatch(unknown); }), "Unknown hip fusion pattern: conv"));
    attrs.erase("PatternName");
    CallValues unnamed = BindCall(MakeCall(MakeFunction(f->params, f->body, attrs), c->args), on_cpu,
                                  Device(DevType::kROCM(), 0));
    EXPECT(Contains(Raises([&] { Dispatch(unnamed); }), "No pattern name marked"));
    attrs = f->attrs;
    attrs.erase("Primitive");
    CallValues plain = BindCall(MakeCall(MakeFunction(f->params, f->body, attrs), c->args), on_cpu,
                                Device(DevType::kROCM(), 0));
    EXPECT(Contains(Raises([&] { Dispatch(plain); }), "non-primitive function"));
    attrs = f->attrs;
    attrs["Dialect"] = "fakeblas";
    CallValues nomaker = BindCall(MakeCall(MakeFunction(f->params, f->body, attrs), c->args), on_cpu,
                                  Device(DevType::kCPU(), 0));
    EXPECT(Contains(Raises([&] { Dispatch(nomaker); }), "Name: raf.op.fakeblas._fused_op"));
    // a body that is not the update is refused by the implementation, not run
    Expr p0 = MakeVar("p", Ty({4})), p1 = MakeVar("p", Ty({4}));
    Expr wrong = MakeFunction({p0, p1}, MakeCall(GetOp("raf.op.hip.multiply"), {p0, p1}, Ty({4})), f->attrs);
    Expr a4 = MakeVar("a", Ty({4}));
    CallValues bad = BindCall(MakeCall(wrong, {a4, a4}), {{a4.get(), tensor(a4, DevType::kROCM(), nullptr)}},
                              Device(DevType::kROCM(), 0));
    EXPECT(Contains(Raises([&] { Dispatch(bad); }), "the function body is not an SGD update"));

    // on a rocm device: an OpEnv if a GPU is there, a clear refusal if not; never a CPU fallback
    std::map<const ExprNode*, value::Value> on_rocm = {{w.get(), tensor(w, DevType::kROCM(), nullptr)},
                                                       {dx.get(), tensor(dx, DevType::kROCM(), nullptr)},
                                                       {v.get(), tensor(v, DevType::kROCM(), nullptr)}};
    CallValues rocm = BindCall(fused, on_rocm, Device(DevType::kROCM(), 0));
    if (device_api::DeviceAPI::Get(DevType::kROCM())->GetDeviceCount() == 0) {
      EXPECT(Contains(Raises([&] { Dispatch(rocm); }), "no HIP device is visible"));
    } else {
      OpEnvPtr env = Dispatch(rocm);
      EXPECT(env && Contains(env->name(), "raf_op_hip__fused_op_sgd_update") && env->arg_indices.size() == 9);
    }
  }

  std::puts("ALL OK");
  return 0;
}

// Host-side checks of the `hip` dialect's whole-graph rewrites: the per-parameter updates of the
// reference's traced SGD optimizer (python/raf/optim/sgd.py:187-215) gathered into one
// multi-tensor call, and the group_cast / cast / add(out=p) ops around raf.op.lans in its traced
// LANS optimizer (python/raf/optim/lans.py:244-312) folded into the LANS call.  As in the
// reference's tests/python/pass/test_pass_fuse_dialect.py the graph after the pass is compared
// structurally with an expected graph built by hand, and variants that must not fuse come back
// untouched.  Runs without a GPU.
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

static bool Contains(const std::string& s, const char* what) { return s.find(what) != std::string::npos; }

static TensorType Ty(std::vector<int64_t> shape, int bits = 32, int code = kDLFloat) {
  TensorType t;
  t.defined = true;
  t.shape = std::move(shape);
  t.dtype = DType{code, bits};
  return t;
}

static std::vector<TensorType> Types(const std::vector<Expr>& es) {
  std::vector<TensorType> out;
  for (const auto& e : es) out.push_back(TypeOf(e));
  return out;
}

static void ExpectEqual(const Expr& got, const Expr& want, int line) {
  if (!StructuralEqual(got, want)) {
    std::fprintf(stderr, "line %d, got:\n%s\nexpected:\n%s\n", line, AsText(got).c_str(), AsText(want).c_str());
    std::exit(1);
  }
}

struct Params {
  std::vector<Expr> g, w, m, v, p;
};

static Params MakeParams(const std::vector<std::vector<int64_t>>& shapes, int grad_bits, int grad_code, int p_code) {
  Params q;
  for (size_t i = 0; i < shapes.size(); ++i) {
    const std::string k = std::to_string(i);
    q.g.push_back(MakeVar("g" + k, Ty(shapes[i], grad_bits, grad_code)));
    q.w.push_back(MakeVar("w" + k, Ty(shapes[i])));
    q.m.push_back(MakeVar("m" + k, Ty(shapes[i])));
    q.v.push_back(MakeVar("v" + k, Ty(shapes[i])));
    q.p.push_back(MakeVar("p" + k, Ty(shapes[i], 16, p_code)));
  }
  return q;
}

static std::vector<Expr> Concat(std::initializer_list<std::vector<Expr>> parts) {
  std::vector<Expr> out;
  for (const auto& p : parts) out.insert(out.end(), p.begin(), p.end());
  return out;
}

int main() {
  const std::vector<std::vector<int64_t>> shapes = {{1024, 1024}, {1024}, {30522, 1024}};
  const size_t n = shapes.size();

  std::puts("registry: two graph rewrites of the hip dialect, by descending plevel");
  {
    auto* list = DialectGraphRewrite::Get();
    EXPECT(list->size() == 2 && list->front().name == "sgd_multi" && list->back().name == "lans_mixed");
    EXPECT(list->front().dialect == "hip" && list->front().plevel > list->back().plevel);
  }

  std::puts("tuples: types, text, equality, substitution");
  {
    Expr a = MakeVar("a", Ty({4})), b = MakeVar("b", Ty({4}, 16));
    Expr t = MakeTuple({a, b});
    EXPECT(TypeOf(MakeTupleGetItem(t, 1)).dtype.bits == 16 && TypeOf(MakeTupleGetItem(t, 0)).dtype.bits == 32);
    Expr c = MakeTupleCall(GetOp("raf.op.some"), {t}, {Ty({4}), Ty({7})});
    EXPECT(TypeOf(MakeTupleGetItem(c, 1)).shape == std::vector<int64_t>{7} && !TypeOf(c).defined);
    EXPECT(Contains(AsText(MakeTupleGetItem(c, 1)), ".1") && Contains(AsText(t), "(%a0, %b1)"));
    Expr a2 = MakeVar("a2", Ty({4}));
    EXPECT(StructuralEqual(MakeTuple({a, a2}), MakeTuple({a2, a})) && !StructuralEqual(MakeTuple({a, a}), MakeTuple({a, a2})));
    EXPECT(!StructuralEqual(MakeTupleGetItem(t, 0), MakeTupleGetItem(t, 1)));
    EXPECT(StructuralEqual(MakeZeros(Ty({4}, 16)), MakeZeros(Ty({4}, 16))) &&
           !StructuralEqual(MakeZeros(Ty({4}, 16)), MakeZeros(Ty({4}))));
    Expr repl = MakeVar("r", Ty({4}));
    Expr s = Substitute(MakeTupleGetItem(c, 0), {{a.get(), repl}});
    EXPECT(AsTupleNode(AsCall(AsTupleGetItem(s)->tuple)->args[0])->fields[0].get() == repl.get());
    EXPECT(PostOrder(c).back().get() == c.get() && PostOrder(c).size() == 5);  // a, b, t, op, c
  }

  std::puts("SGD: the updates of all float32 parameters become one raf.op.hip.sgd_multi call");
  {
    Params q = MakeParams(shapes, 32, kDLFloat, kDLFloat);
    Expr traced = hip::TracedSgdOptimizer(q.w, q.g, q.v, {}, nullptr, 0.01, 0.9);
    EXPECT(!Contains(AsText(traced), "hip"));
    Expr fused = pass::FuseDialect(traced, DevType::kROCM());
    std::vector<Expr> list = Concat({q.w, q.g, q.v});
    Expr call = MakeTupleCall(GetOp("raf.op.hip.sgd_multi"), {MakeTuple(list), MakeFloat(0.01), MakeFloat(0.9)},
                              Types(list));
    ExpectEqual(fused, MakeTuple({MakeTupleGetItem(call, 0), MakeTupleGetItem(call, 1), MakeTupleGetItem(call, 2)}),
                __LINE__);
    // the list holds the original expressions, in the op's order x..., dx..., v...
    const auto* c = AsCall(AsTupleGetItem(AsTupleNode(fused)->fields[0])->tuple);
    const auto* t = AsTupleNode(c->args[0]);
    EXPECT(t->fields.size() == 3 * n && t->fields[0].get() == q.w[0].get() && t->fields[n].get() == q.g[0].get() &&
           t->fields[2 * n + 2].get() == q.v[2].get());
    EXPECT(TypeOf(AsTupleNode(fused)->fields[1]).shape == shapes[1]);
    EXPECT(pass::FuseDialect(fused, DevType::kROCM()).get() == fused.get());  // nothing left to do
    // other devices: untouched
    EXPECT(pass::FuseDialect(traced, DevType::kCPU()).get() == traced.get());
    EXPECT(pass::FuseDialect(traced, DevType::kCUDA()).get() == traced.get());
  }

  std::puts("SGD, half-precision model: gradient cast, weight cast and copy join as sgd_multi_mixed");
  for (int code : {kDLFloat, kDLBfloat}) {
    Params q = MakeParams(shapes, 16, code, code);
    Expr zero = MakeZeros(Ty({}, 16, code));
    Expr fused = pass::FuseDialect(hip::TracedSgdOptimizer(q.w, q.g, q.v, q.p, zero, 0.01, 0.9), DevType::kROCM());
    std::vector<Expr> list = Concat({q.w, q.g, q.v, q.p});
    Expr call = MakeTupleCall(GetOp("raf.op.hip.sgd_multi_mixed"),
                              {MakeTuple(list), MakeFloat(0.01), MakeFloat(0.9)}, Types(list));
    ExpectEqual(fused,
                MakeTuple({MakeTupleGetItem(call, (int)(3 * n)), MakeTupleGetItem(call, (int)(3 * n + 1)),
                           MakeTupleGetItem(call, (int)(3 * n + 2))}),
                __LINE__);
    EXPECT(!Contains(AsText(fused), "raf.op.cast") && !Contains(AsText(fused), "raf.op.add"));
  }

  std::puts("SGD: while `zero` is a free variable the cast and the copy stay, the updates still gather");
  {
    Params q = MakeParams(shapes, 16, kDLFloat, kDLFloat);
    Expr zero = MakeVar("zero", Ty({}, 16));
    Expr fused = pass::FuseDialect(hip::TracedSgdOptimizer(q.w, q.g, q.v, q.p, zero, 0.01, 0.9), DevType::kROCM());
    std::vector<Expr> list = Concat({q.w, q.g, q.v});
    Expr call = MakeTupleCall(GetOp("raf.op.hip.sgd_multi"), {MakeTuple(list), MakeFloat(0.01), MakeFloat(0.9)},
                              Types(list));
    std::vector<Expr> outs;
    for (size_t i = 0; i < n; ++i) {
      Expr narrowed = MakeCall(GetOp("raf.op.cast"), {MakeTupleGetItem(call, (int)i), MakeString("float16")},
                               TypeOf(q.p[i]));
      outs.push_back(MakeCall(GetOp("raf.op.add"), {narrowed, zero, q.p[i], MakeNull()}, TypeOf(q.p[i])));
    }
    ExpectEqual(fused, MakeTuple(outs), __LINE__);
  }

  std::puts("SGD: only what is alike and independent is gathered");
  {
    Params q = MakeParams(shapes, 32, kDLFloat, kDLFloat);
    // another learning rate for the third parameter: two gather, one goes to the per-parameter pattern
    Expr mixed_lr = MakeTuple({hip::TracedSgdUpdate(q.w[0], q.g[0], q.v[0], 0.01, 0.9),
                               hip::TracedSgdUpdate(q.w[1], q.g[1], q.v[1], 0.01, 0.9),
                               hip::TracedSgdUpdate(q.w[2], q.g[2], q.v[2], 0.05, 0.9)});
    Expr fused = pass::FuseDialect(mixed_lr, DevType::kROCM());
    const auto* t = AsTupleNode(fused);
    EXPECT(t && AsTupleGetItem(t->fields[0]) && AsTupleGetItem(t->fields[1]) &&
           AsTupleGetItem(t->fields[0])->tuple.get() == AsTupleGetItem(t->fields[1])->tuple.get());
    EXPECT(AsTupleNode(AsCall(AsTupleGetItem(t->fields[0])->tuple)->args[0])->fields.size() == 6);
    const auto* single = AsCall(t->fields[2]);
    EXPECT(single && AsFunction(single->op) && AsFunction(single->op)->attrs.at("PatternName") == "sgd_update");
    // float32 and float16 gradients do not share a call (the kernel widens one dtype per list)
    Expr g16 = MakeVar("g16", Ty(shapes[1], 16));
    Expr two_dtypes = MakeTuple({hip::TracedSgdUpdate(q.w[0], q.g[0], q.v[0], 0.01, 0.9),
                                 hip::TracedSgdUpdate(q.w[1], g16, q.v[1], 0.01, 0.9)});
    EXPECT(!Contains(AsText(pass::FuseDialect(two_dtypes, DevType::kROCM())), "sgd_multi"));
    // a parameter whose new velocity is also an output keeps its separate ops (the out= call would
    // run twice otherwise); the other two still gather
    Expr mv = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.9), q.v[2]}, TypeOf(q.v[2]));
    Expr nv = MakeCall(GetOp("raf.op.add"), {mv, q.g[2], q.v[2], MakeNull()}, TypeOf(q.v[2]));
    Expr st = MakeCall(GetOp("raf.op.multiply"), {MakeFloat(0.01), nv}, TypeOf(q.v[2]));
    Expr nw = MakeCall(GetOp("raf.op.subtract"), {q.w[2], st, q.w[2], MakeNull()}, TypeOf(q.w[2]));
    Expr leaky = MakeTuple({hip::TracedSgdUpdate(q.w[0], q.g[0], q.v[0], 0.01, 0.9),
                            hip::TracedSgdUpdate(q.w[1], q.g[1], q.v[1], 0.01, 0.9), nw, nv});
    Expr got = pass::FuseDialect(leaky, DevType::kROCM());
    EXPECT(AsTupleNode(got)->fields[2].get() == nw.get() && AsTupleNode(got)->fields[3].get() == nv.get());
    EXPECT(AsTupleGetItem(AsTupleNode(got)->fields[0]) != nullptr);
    // a gradient computed from another parameter's new weight: the two updates are ordered, not gathered
    Expr first = hip::TracedSgdUpdate(q.w[0], q.g[0], q.v[0], 0.01, 0.9);
    Expr dependent = MakeCall(GetOp("raf.op.relu"), {first}, TypeOf(first));
    Expr chained = MakeTuple({first, hip::TracedSgdUpdate(q.w[1], q.g[1], q.v[1], 0.01, 0.9),
                              hip::TracedSgdUpdate(MakeVar("w9", Ty(shapes[0])), dependent, MakeVar("v9", Ty(shapes[0])),
                                                   0.01, 0.9)});
    EXPECT(!Contains(AsText(pass::FuseDialect(chained, DevType::kROCM())), "sgd_multi"));
    // the same weight twice is not a list of independent updates
    Expr twice = MakeTuple({hip::TracedSgdUpdate(q.w[0], q.g[0], q.v[0], 0.01, 0.9),
                            hip::TracedSgdUpdate(q.w[0], q.g[1], q.v[0], 0.01, 0.9)});
    EXPECT(!Contains(AsText(pass::FuseDialect(twice, DevType::kROCM())), "sgd_multi"));
  }

  hip::LansHyper hyper;
  auto lans_args = [&](const Expr& list, const Expr& step) {
    return std::vector<Expr>{list, step, MakeFloat(hyper.learning_rate), MakeFloat(hyper.beta1),
                             MakeFloat(hyper.beta2), MakeFloat(hyper.eps), MakeInt(hyper.bias_correction),
                             MakeFloat(hyper.weight_decay), MakeInt(hyper.grad_averaging), MakeInt(hyper.mode),
                             MakeInt(hyper.normalize_grad)};
  };

  std::puts("LANS, half-precision model: group_cast, cast and copy fold into raf.op.hip.lans_mixed");
  for (int code : {kDLFloat, kDLBfloat}) {
    Params q = MakeParams(shapes, 16, code, code);
    Expr step = MakeVar("step", Ty({}));
    Expr traced = hip::TracedLansOptimizer(q.g, q.w, q.m, q.v, q.p, MakeZeros(Ty({}, 16, code)), step, hyper);
    EXPECT(Contains(AsText(traced), "raf.op.group_cast") && Contains(AsText(traced), "raf.op.lans("));
    Expr fused = pass::FuseDialect(traced, DevType::kROCM());
    std::vector<Expr> list = Concat({q.g, q.w, q.m, q.v, q.p});
    Expr call = MakeTupleCall(GetOp("raf.op.hip.lans_mixed"), lans_args(MakeTuple(list), step), Types(list));
    std::vector<Expr> outs;
    for (size_t i = 0; i < n; ++i) outs.push_back(MakeTupleGetItem(call, (int)(4 * n + i)));  // the model's weights
    for (size_t i = 0; i < n; ++i) outs.push_back(MakeTupleGetItem(call, (int)(2 * n + i)));  // m
    for (size_t i = 0; i < n; ++i) outs.push_back(MakeTupleGetItem(call, (int)(3 * n + i)));  // v
    ExpectEqual(fused, MakeTuple(outs), __LINE__);
    const std::string text = AsText(fused);
    EXPECT(!Contains(text, "group_cast") && !Contains(text, "raf.op.cast") && !Contains(text, "raf.op.add"));
    // the gradients handed to the op are the model's half-precision ones, untouched
    EXPECT(AsTupleNode(AsCall(AsTupleGetItem(AsTupleNode(fused)->fields[0])->tuple)->args[0])->fields[0].get() ==
           q.g[0].get());
    EXPECT(pass::FuseDialect(traced, DevType::kCUDA()).get() == traced.get());
  }

  std::puts("LANS: while `zero` is a free variable only the group_cast folds, into raf.op.hip.lans");
  {
    Params q = MakeParams(shapes, 16, kDLFloat, kDLFloat);
    Expr step = MakeVar("step", Ty({})), zero = MakeVar("zero", Ty({}, 16));
    Expr fused = pass::FuseDialect(hip::TracedLansOptimizer(q.g, q.w, q.m, q.v, q.p, zero, step, hyper),
                                   DevType::kROCM());
    std::vector<Expr> list = Concat({q.g, q.w, q.m, q.v});
    Expr call = MakeTupleCall(GetOp("raf.op.hip.lans"), lans_args(MakeTuple(list), step), Types(list));
    std::vector<Expr> outs;
    for (size_t i = 0; i < n; ++i) {
      Expr narrowed = MakeCall(GetOp("raf.op.cast"), {MakeTupleGetItem(call, (int)(n + i)), MakeString("float16")},
                               TypeOf(q.p[i]));
      outs.push_back(MakeCall(GetOp("raf.op.add"), {narrowed, zero, q.p[i], MakeNull()}, TypeOf(q.p[i])));
    }
    for (size_t i = 0; i < n; ++i) outs.push_back(MakeTupleGetItem(call, (int)(2 * n + i)));
    for (size_t i = 0; i < n; ++i) outs.push_back(MakeTupleGetItem(call, (int)(3 * n + i)));
    ExpectEqual(fused, MakeTuple(outs), __LINE__);
  }

  std::puts("LANS: what does not fit stays as it is");
  {
    Params q = MakeParams(shapes, 16, kDLFloat, kDLFloat);
    Expr step = MakeVar("step", Ty({})), zero = MakeZeros(Ty({}, 16));
    // float32 gradients, no group_cast: nothing for this rewrite to do
    Params f = MakeParams(shapes, 32, kDLFloat, kDLFloat);
    std::vector<Expr> list = Concat({f.g, f.w, f.m, f.v});
    Expr plain = MakeTupleCall(GetOp("raf.op.lans"), lans_args(MakeTuple(list), step), Types(list));
    Expr plain_out = MakeTuple({MakeTupleGetItem(plain, (int)n)});
    EXPECT(pass::FuseDialect(plain_out, DevType::kROCM()).get() == plain_out.get());
    // someone reads the float32 gradient the op returns: it must keep existing
    Expr traced = hip::TracedLansOptimizer(q.g, q.w, q.m, q.v, q.p, zero, step, hyper);
    Expr lans_call;
    for (const Expr& e : PostOrder(traced))
      if (AsCall(e) && AsOp(AsCall(e)->op) && AsOp(AsCall(e)->op)->name == "raf.op.lans") lans_call = e;
    std::vector<Expr> fields = AsTupleNode(traced)->fields;
    fields.push_back(MakeTupleGetItem(lans_call, 0));
    Expr reads_g = MakeTuple(fields);
    EXPECT(pass::FuseDialect(reads_g, DevType::kROCM()).get() == reads_g.get());
    // the gradients are cast in another order than they are listed
    std::vector<Expr> g32;
    Expr gc = MakeTupleCall(GetOp("raf.op.group_cast"), {MakeTuple(q.g), MakeString("float32")},
                            Types(Concat({f.g})));
    g32 = {MakeTupleGetItem(gc, 1), MakeTupleGetItem(gc, 0), MakeTupleGetItem(gc, 2)};
    std::vector<Expr> shuffled = Concat({g32, q.w, q.m, q.v});
    Expr odd = MakeTupleCall(GetOp("raf.op.lans"), lans_args(MakeTuple(shuffled), step), Types(shuffled));
    Expr odd_out = MakeTuple({MakeTupleGetItem(odd, (int)n)});
    EXPECT(pass::FuseDialect(odd_out, DevType::kROCM()).get() == odd_out.get());
    // a float16 model with one bfloat16 parameter: the tails differ, so none is folded in
    Params mixed = MakeParams(shapes, 16, kDLFloat, kDLFloat);
    mixed.p[1] = MakeVar("pb", Ty(shapes[1], 16, kDLBfloat));
    Expr got = pass::FuseDialect(hip::TracedLansOptimizer(mixed.g, mixed.w, mixed.m, mixed.v, mixed.p, zero, step, hyper),
                                 DevType::kROCM());
    EXPECT(Contains(AsText(got), "raf.op.hip.lans(") && !Contains(AsText(got), "lans_mixed") &&
           Contains(AsText(got), "raf.op.cast"));
  }

  std::puts("LANS: a result field projected by two TupleGetItem nodes: both move to the new call");
  {
    Params q = MakeParams(shapes, 16, kDLFloat, kDLFloat);
    Expr step = MakeVar("step", Ty({})), zero = MakeZeros(Ty({}, 16));
    Expr traced = hip::TracedLansOptimizer(q.g, q.w, q.m, q.v, q.p, zero, step, hyper);
    Expr lans_call;
    for (const Expr& e : PostOrder(traced))
      if (AsCall(e) && AsOp(AsCall(e)->op) && AsOp(AsCall(e)->op)->name == "raf.op.lans") lans_call = e;
    // a second, separate projection of the first moment of parameter 0 and of the new weight of
    // parameter 1 (which thereby has a user besides its cast: no 16-bit tails are folded in)
    std::vector<Expr> fields = AsTupleNode(traced)->fields;
    fields.push_back(MakeTupleGetItem(lans_call, (int)(2 * n)));
    Expr twice_m = MakeTuple(fields);
    Expr got = pass::FuseDialect(twice_m, DevType::kROCM());
    std::string text = AsText(got);
    EXPECT(Contains(text, "raf.op.hip.lans_mixed") && !Contains(text, "raf.op.lans(") && !Contains(text, "group_cast"));
    fields.push_back(MakeTupleGetItem(lans_call, (int)(n + 1)));
    Expr twice_w = MakeTuple(fields);
    got = pass::FuseDialect(twice_w, DevType::kROCM());
    text = AsText(got);
    EXPECT(Contains(text, "raf.op.hip.lans(") && !Contains(text, "lans_mixed") && !Contains(text, "raf.op.lans(") &&
           !Contains(text, "group_cast") && Contains(text, "raf.op.cast"));
    // every call of the rewritten graph is reached through the ONE new call
    size_t calls = 0;
    for (const Expr& e : PostOrder(got))
      if (AsCall(e) && AsOp(AsCall(e)->op) && AsOp(AsCall(e)->op)->name == "raf.op.hip.lans") ++calls;
    EXPECT(calls == 1);
  }

  std::puts("ALL OK");
  return 0;
}

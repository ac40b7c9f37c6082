// Graph IR, dataflow patterns, the dialect fuse-pattern registry, the FuseDialect pass and the
// dispatch of fused functions; see raf_ir.h for what each part mirrors in the reference.
#include "raf_ir.h"

#include <cstdio>
#include <mutex>
#include <set>
#include <sstream>
#include <unordered_map>

namespace raf {
namespace ir {

// ----------------------------------------------------------------------------------- builders
Expr MakeVar(const std::string& name_hint, const TensorType& type) {
  auto n = std::make_shared<VarNode>();
  n->name_hint = name_hint;
  n->type = type;
  return n;
}

Expr MakeNull() { return std::make_shared<ConstantNode>(); }

Expr MakeFloat(double v) {
  auto n = std::make_shared<ConstantNode>();
  n->value_kind = ConstantNode::kFloat;
  n->f = v;
  return n;
}

Expr MakeInt(int64_t v) {
  auto n = std::make_shared<ConstantNode>();
  n->value_kind = ConstantNode::kInt;
  n->i = v;
  return n;
}

Expr MakeString(const std::string& v) {
  auto n = std::make_shared<ConstantNode>();
  n->value_kind = ConstantNode::kString;
  n->s = v;
  return n;
}

Expr MakeZeros(const TensorType& type) {
  RAF_CHECK(type.defined, "a zeros constant needs a type");
  auto n = std::make_shared<ConstantNode>();
  n->value_kind = ConstantNode::kZeros;
  n->type = type;
  return n;
}

Expr MakeTuple(std::vector<Expr> fields) {
  for (const auto& f : fields) RAF_CHECK(f != nullptr, "undefined tuple field");
  auto n = std::make_shared<TupleNode>();
  n->fields = std::move(fields);
  return n;
}

Expr MakeTupleGetItem(const Expr& tuple, int index) {
  RAF_CHECK(tuple != nullptr && index >= 0, "TupleGetItem needs a tuple and a non-negative index");
  if (const auto* t = AsTupleNode(tuple))
    RAF_CHECK((size_t)index < t->fields.size(), "TupleGetItem: index out of range");
  auto n = std::make_shared<TupleGetItemNode>();
  n->tuple = tuple;
  n->index = index;
  return n;
}

Expr MakeTupleCall(const Expr& op, std::vector<Expr> args, std::vector<TensorType> field_types) {
  RAF_CHECK(AsOp(op) || AsFunction(op), "the callee must be an operator or a function");
  auto n = std::make_shared<CallNode>();
  n->op = op;
  n->args = std::move(args);
  n->field_types = std::move(field_types);
  return n;
}

Expr GetOp(const std::string& name) {
  static std::mutex mu;
  static std::map<std::string, Expr> ops;
  std::lock_guard<std::mutex> lock(mu);
  auto it = ops.find(name);
  if (it != ops.end()) return it->second;
  auto n = std::make_shared<OpNode>();
  n->name = name;
  ops[name] = n;
  return n;
}

Expr MakeCall(const Expr& op, std::vector<Expr> args, const TensorType& type) {
  RAF_CHECK(AsOp(op) || AsFunction(op), "the callee must be an operator or a function");
  auto n = std::make_shared<CallNode>();
  n->op = op;
  n->args = std::move(args);
  n->type = type;
  return n;
}

Expr MakeFunction(std::vector<Expr> params, const Expr& body,
                  std::map<std::string, std::string> attrs) {
  for (const auto& p : params) RAF_CHECK(AsVar(p) != nullptr, "function parameters must be variables");
  auto n = std::make_shared<FunctionNode>();
  n->params = std::move(params);
  n->body = body;
  n->attrs = std::move(attrs);
  return n;
}

TensorType TypeOf(const Expr& e) {
  if (const auto* v = AsVar(e)) return v->type;
  if (const auto* c = AsCall(e)) return c->type;
  if (const auto* k = AsConstant(e)) return k->value_kind == ConstantNode::kZeros ? k->type : TensorType();
  if (const auto* g = AsTupleGetItem(e)) {
    if (const auto* t = AsTupleNode(g->tuple))
      return (size_t)g->index < t->fields.size() ? TypeOf(t->fields[(size_t)g->index]) : TensorType();
    if (const auto* c = AsCall(g->tuple))
      return (size_t)g->index < c->field_types.size() ? c->field_types[(size_t)g->index] : TensorType();
  }
  return TensorType();
}

namespace {
void PostOrderVisit(const Expr& e, std::set<const ExprNode*>* seen, std::vector<Expr>* out) {
  if (!e || !seen->insert(e.get()).second) return;
  if (const auto* c = AsCall(e)) {
    PostOrderVisit(c->op, seen, out);
    for (const auto& a : c->args) PostOrderVisit(a, seen, out);
  } else if (const auto* f = AsFunction(e)) {
    for (const auto& p : f->params) PostOrderVisit(p, seen, out);
    PostOrderVisit(f->body, seen, out);
  } else if (const auto* t = AsTupleNode(e)) {
    for (const auto& x : t->fields) PostOrderVisit(x, seen, out);
  } else if (const auto* g = AsTupleGetItem(e)) {
    PostOrderVisit(g->tuple, seen, out);
  }
  out->push_back(e);
}

class Substituter {
 public:
  explicit Substituter(const std::map<const ExprNode*, Expr>& replace) : replace_(replace) {}
  Expr Mutate(const Expr& e) {
    if (!e) return e;
    auto r = replace_.find(e.get());
    if (r != replace_.end()) return r->second;
    auto it = memo_.find(e.get());
    if (it != memo_.end()) return it->second;
    Expr post = e;
    if (const auto* c = AsCall(e)) {
      Expr op = Mutate(c->op);
      bool changed = op.get() != c->op.get();
      std::vector<Expr> args;
      for (const auto& a : c->args) {
        args.push_back(Mutate(a));
        changed = changed || args.back().get() != a.get();
      }
      if (changed) {
        auto n = std::make_shared<CallNode>();
        n->op = op;
        n->args = std::move(args);
        n->type = c->type;
        n->field_types = c->field_types;
        post = n;
      }
    } else if (const auto* t = AsTupleNode(e)) {
      bool changed = false;
      std::vector<Expr> fields;
      for (const auto& x : t->fields) {
        fields.push_back(Mutate(x));
        changed = changed || fields.back().get() != x.get();
      }
      if (changed) post = MakeTuple(std::move(fields));
    } else if (const auto* g = AsTupleGetItem(e)) {
      Expr tuple = Mutate(g->tuple);
      if (tuple.get() != g->tuple.get()) post = MakeTupleGetItem(tuple, g->index);
    } else if (const auto* f = AsFunction(e)) {
      Expr body = Mutate(f->body);
      if (body.get() != f->body.get()) post = MakeFunction(f->params, body, f->attrs);
    }
    memo_[e.get()] = post;
    return post;
  }

 private:
  const std::map<const ExprNode*, Expr>& replace_;
  std::map<const ExprNode*, Expr> memo_;
};
}  // namespace

std::vector<Expr> PostOrder(const Expr& root) {
  std::set<const ExprNode*> seen;
  std::vector<Expr> out;
  PostOrderVisit(root, &seen, &out);
  return out;
}

Expr Substitute(const Expr& root, const std::map<const ExprNode*, Expr>& replace) {
  return Substituter(replace).Mutate(root);
}

// --------------------------------------------------------------------------------------- text
namespace {

std::string DTypeText(const DType& t) {
  const char* base = t.code == kDLFloat ? "float" : t.code == kDLBfloat ? "bfloat" : t.code == 0 ? "int" : "uint";
  return std::string(base) + std::to_string(t.bits);
}

std::string TypeText(const TensorType& t) {
  if (!t.defined) return "?";
  std::ostringstream ss;
  ss << "Tensor[(";
  for (size_t i = 0; i < t.shape.size(); ++i) ss << (i ? ", " : "") << t.shape[i];
  ss << "), " << DTypeText(t.dtype) << "]";
  return ss.str();
}

std::string ConstantText(const ConstantNode* c) {
  switch (c->value_kind) {
    case ConstantNode::kNull:
      return "null";
    case ConstantNode::kFloat: {
      char buf[40];
      std::snprintf(buf, sizeof(buf), "%.17gf64", c->f);
      return buf;
    }
    case ConstantNode::kInt:
      return std::to_string(c->i) + "i64";
    case ConstantNode::kZeros:
      return "zeros(" + TypeText(c->type) + ")";
    default:
      return "\"" + c->s + "\"";
  }
}

class Printer {
 public:
  std::string Print(const Expr& e) {
    std::string last = Ref(e, 0);
    os_ << last << "\n";
    return os_.str();
  }

 private:
  std::string Indent(int depth) { return std::string((size_t)depth * 2, ' '); }

  // Returns the name under which `e` can be referred to, emitting its definition first if needed.
  std::string Ref(const Expr& e, int depth) {
    RAF_CHECK(e != nullptr, "undefined expression");
    auto it = names_.find(e.get());
    if (it != names_.end()) return it->second;
    std::string name;
    if (const auto* v = AsVar(e)) {
      name = "%" + v->name_hint + std::to_string(n_vars_++);
    } else if (const auto* c = AsConstant(e)) {
      return ConstantText(c);  // constants are printed in place
    } else if (const auto* o = AsOp(e)) {
      return o->name;
    } else if (const auto* call = AsCall(e)) {
      std::string callee = Ref(call->op, depth);
      std::vector<std::string> args;
      for (const auto& a : call->args) args.push_back(Ref(a, depth));
      name = "%" + std::to_string(n_values_++);
      os_ << Indent(depth) << name << " = " << callee << "(";
      for (size_t i = 0; i < args.size(); ++i) os_ << (i ? ", " : "") << args[i];
      os_ << ")";
      if (call->type.defined) os_ << " /* ty=" << TypeText(call->type) << " */";
      os_ << ";\n";
    } else if (const auto* t = AsTupleNode(e)) {
      std::vector<std::string> fields;
      for (const auto& x : t->fields) fields.push_back(Ref(x, depth));
      name = "%" + std::to_string(n_values_++);
      os_ << Indent(depth) << name << " = (";
      for (size_t i = 0; i < fields.size(); ++i) os_ << (i ? ", " : "") << fields[i];
      os_ << (fields.size() == 1 ? ",)" : ")") << ";\n";
    } else if (const auto* g = AsTupleGetItem(e)) {
      return Ref(g->tuple, depth) + "." + std::to_string(g->index);  // printed in place
    } else {
      const auto* f = AsFunction(e);
      name = "%fn" + std::to_string(n_funcs_++);
      std::vector<std::string> params;
      for (const auto& p : f->params) params.push_back(Ref(p, depth) + ": " + TypeText(AsVar(p)->type));
      os_ << Indent(depth) << name << " = fn (";
      for (size_t i = 0; i < params.size(); ++i) os_ << (i ? ", " : "") << params[i];
      os_ << ")";
      for (const auto& kv : f->attrs) os_ << " " << kv.first << "=" << kv.second;
      os_ << " {\n";
      std::string body = Ref(f->body, depth + 1);
      os_ << Indent(depth + 1) << body << "\n" << Indent(depth) << "};\n";
    }
    names_[e.get()] = name;
    return name;
  }

  std::ostringstream os_;
  std::map<const ExprNode*, std::string> names_;
  int n_vars_ = 0, n_values_ = 0, n_funcs_ = 0;
};

bool SameDType(const DType& a, const DType& b) { return a.code == b.code && a.bits == b.bits; }

bool SameType(const TensorType& a, const TensorType& b) {
  if (a.defined != b.defined) return false;
  return !a.defined || (a.shape == b.shape && SameDType(a.dtype, b.dtype));
}

bool SameConstant(const ConstantNode* a, const ConstantNode* b) {
  if (a->value_kind != b->value_kind) return false;
  switch (a->value_kind) {
    case ConstantNode::kNull:
      return true;
    case ConstantNode::kFloat:
      return a->f == b->f;
    case ConstantNode::kInt:
      return a->i == b->i;
    case ConstantNode::kZeros:
      return SameType(a->type, b->type);
    default:
      return a->s == b->s;
  }
}

class Equal {
 public:
  bool Check(const Expr& a, const Expr& b) {
    if (!a || !b) return !a && !b;
    if (a->kind != b->kind) return false;
    auto it = lhs_to_rhs_.find(a.get());
    if (it != lhs_to_rhs_.end()) return it->second == b.get();
    auto rit = rhs_to_lhs_.find(b.get());
    if (rit != rhs_to_lhs_.end()) return false;  // b already stands for another expression of a
    bool ok = false;
    switch (a->kind) {
      case ExprNode::kVar:
        ok = SameType(AsVar(a)->type, AsVar(b)->type);
        break;
      case ExprNode::kConstant:
        return SameConstant(AsConstant(a), AsConstant(b));  // constants are not identity-mapped
      case ExprNode::kOp:
        return a.get() == b.get();
      case ExprNode::kCall: {
        const auto *ca = AsCall(a), *cb = AsCall(b);
        ok = ca->args.size() == cb->args.size() && Check(ca->op, cb->op);
        for (size_t i = 0; ok && i < ca->args.size(); ++i) ok = Check(ca->args[i], cb->args[i]);
        break;
      }
      case ExprNode::kFunction: {
        const auto *fa = AsFunction(a), *fb = AsFunction(b);
        ok = fa->params.size() == fb->params.size() && fa->attrs == fb->attrs;
        for (size_t i = 0; ok && i < fa->params.size(); ++i) ok = Check(fa->params[i], fb->params[i]);
        ok = ok && Check(fa->body, fb->body);
        break;
      }
      case ExprNode::kTuple: {
        const auto *ta = AsTupleNode(a), *tb = AsTupleNode(b);
        ok = ta->fields.size() == tb->fields.size();
        for (size_t i = 0; ok && i < ta->fields.size(); ++i) ok = Check(ta->fields[i], tb->fields[i]);
        break;
      }
      case ExprNode::kTupleGetItem: {
        const auto *ga = AsTupleGetItem(a), *gb = AsTupleGetItem(b);
        ok = ga->index == gb->index && Check(ga->tuple, gb->tuple);
        break;
      }
    }
    if (ok) {
      lhs_to_rhs_[a.get()] = b.get();
      rhs_to_lhs_[b.get()] = a.get();
    }
    return ok;
  }

 private:
  std::map<const ExprNode*, const ExprNode*> lhs_to_rhs_, rhs_to_lhs_;
};

}  // namespace

std::string AsText(const Expr& e) { return Printer().Print(e); }

bool StructuralEqual(const Expr& a, const Expr& b) { return Equal().Check(a, b); }

// ------------------------------------------------------------------------------------ patterns
namespace {
std::shared_ptr<DFPatternNode> NewPattern(DFPatternNode::Kind kind) {
  auto p = std::make_shared<DFPatternNode>();
  p->kind = kind;
  return p;
}
}  // namespace

DFPattern wildcard() { return NewPattern(DFPatternNode::kWildcard); }

DFPattern is_constant() { return NewPattern(DFPatternNode::kConstant); }

DFPattern is_constant(const Expr& value) {
  RAF_CHECK(AsConstant(value) != nullptr, "is_constant takes a constant");
  auto p = NewPattern(DFPatternNode::kConstant);
  p->constant = value;
  return p;
}

DFPattern is_op(const std::string& name) {
  auto p = NewPattern(DFPatternNode::kOp);
  p->op_name = name;
  return p;
}

DFPattern is_ops(const std::vector<std::string>& names) {
  RAF_CHECK(!names.empty(), "is_ops needs at least one operator");
  DFPattern p = is_op(names[0]);
  for (size_t i = 1; i < names.size(); ++i) p = alt(p, is_op(names[i]));
  return p;
}

DFPattern call(const DFPattern& op, std::vector<DFPattern> args) {
  auto p = NewPattern(DFPatternNode::kCall);
  p->op = op;
  p->args = std::move(args);
  return p;
}

DFPattern alt(const DFPattern& left, const DFPattern& right) {
  auto p = NewPattern(DFPatternNode::kAlt);
  p->left = left;
  p->right = right;
  return p;
}

DFPattern has_dtype(const DType& dtype, DFPattern inner) {
  auto p = NewPattern(DFPatternNode::kDType);
  p->inner = inner ? inner : wildcard();
  p->dtype = dtype;
  return p;
}

namespace {

class Matcher {
 public:
  bool Match(const DFPattern& p, const Expr& e) {
    auto it = memo_.find(p.get());
    if (it != memo_.end()) return it->second.get() == e.get();
    const size_t mark = trail_.size();
    if (MatchNode(p.get(), e)) {
      memo_[p.get()] = e;
      trail_.push_back(p.get());
      return true;
    }
    while (trail_.size() > mark) {  // forget what the failed attempt bound
      memo_.erase(trail_.back());
      trail_.pop_back();
    }
    return false;
  }
  const NodeMap& node_map() const { return memo_; }

 private:
  bool MatchNode(const DFPatternNode* p, const Expr& e) {
    switch (p->kind) {
      case DFPatternNode::kWildcard:
        return e != nullptr;
      case DFPatternNode::kConstant: {
        const auto* c = AsConstant(e);
        return c && (!p->constant || SameConstant(c, AsConstant(p->constant)));
      }
      case DFPatternNode::kOp: {
        const auto* o = AsOp(e);
        return o && o->name == p->op_name;
      }
      case DFPatternNode::kCall: {
        const auto* c = AsCall(e);
        if (!c || c->args.size() != p->args.size() || !Match(p->op, c->op)) return false;
        for (size_t i = 0; i < p->args.size(); ++i)
          if (!Match(p->args[i], c->args[i])) return false;
        return true;
      }
      case DFPatternNode::kAlt:
        return Match(p->left, e) || Match(p->right, e);
      case DFPatternNode::kDType: {
        if (!Match(p->inner, e)) return false;
        const TensorType t = TypeOf(e);
        return t.defined && SameDType(t.dtype, p->dtype);
      }
    }
    return false;
  }

  NodeMap memo_;
  std::vector<const DFPatternNode*> trail_;
};

bool IsPrimitive(const FunctionNode* f) {
  auto it = f->attrs.find(kPrimitive);
  return it != f->attrs.end() && it->second != "0";
}

// Every kCall node of a pattern.
void CollectCallPatternNodes(const DFPattern& p, std::set<const DFPatternNode*>* seen,
                             std::vector<const DFPatternNode*>* calls) {
  if (!p || !seen->insert(p.get()).second) return;
  if (p->kind == DFPatternNode::kCall) calls->push_back(p.get());
  CollectCallPatternNodes(p->op, seen, calls);
  for (const auto& a : p->args) CollectCallPatternNodes(a, seen, calls);
  CollectCallPatternNodes(p->left, seen, calls);
  CollectCallPatternNodes(p->right, seen, calls);
  CollectCallPatternNodes(p->inner, seen, calls);
}

class Rewriter {
 public:
  Rewriter(const DFPattern& pattern, const RewriteCallback& cb, const Expr& root)
      : pattern_(pattern), cb_(cb), call_patterns_(CallPatternsOf(pattern)) {
    CountUses(root);
  }

  Expr Mutate(const Expr& e) {
    auto it = memo_.find(e.get());
    if (it != memo_.end()) return it->second;
    Expr post = e;
    if (const auto* c = AsCall(e)) {
      Expr op = Mutate(c->op);
      std::vector<Expr> args;
      bool changed = op.get() != c->op.get();
      for (const auto& a : c->args) {
        args.push_back(Mutate(a));
        changed = changed || args.back().get() != a.get();
      }
      if (changed) {
        auto n = std::make_shared<CallNode>();
        n->op = op;
        n->args = args;
        n->type = c->type;
        n->field_types = c->field_types;
        post = n;
      }
      origin_[post.get()] = e.get();
      NodeMap node_map;
      if (MatchPattern(pattern_, post, &node_map) && InteriorIsPrivate(post, node_map))
        post = cb_(e, post, node_map);
    } else if (const auto* f = AsFunction(e)) {
      if (!IsPrimitive(f)) {
        Expr body = Mutate(f->body);
        if (body.get() != f->body.get()) post = MakeFunction(f->params, body, f->attrs);
      }
    } else if (const auto* t = AsTupleNode(e)) {
      bool changed = false;
      std::vector<Expr> fields;
      for (const auto& x : t->fields) {
        fields.push_back(Mutate(x));
        changed = changed || fields.back().get() != x.get();
      }
      if (changed) post = MakeTuple(std::move(fields));
    } else if (const auto* g = AsTupleGetItem(e)) {
      Expr tuple = Mutate(g->tuple);
      if (tuple.get() != g->tuple.get()) post = MakeTupleGetItem(tuple, g->index);
    }
    memo_[e.get()] = post;
    keep_alive_.push_back(e);
    return post;
  }

 private:
  // How many argument slots of the graph refer to each expression.
  void CountUses(const Expr& e) {
    if (!e || !counted_.insert(e.get()).second) return;
    if (const auto* c = AsCall(e)) {
      CountUses(c->op);
      for (const auto& a : c->args) {
        ++uses_[a.get()];
        CountUses(a);
      }
    } else if (const auto* f = AsFunction(e)) {
      ++uses_[f->body.get()];
      CountUses(f->body);
    } else if (const auto* t = AsTupleNode(e)) {
      for (const auto& x : t->fields) {
        ++uses_[x.get()];
        CountUses(x);
      }
    } else if (const auto* g = AsTupleGetItem(e)) {
      ++uses_[g->tuple.get()];
      CountUses(g->tuple);
    }
  }

  // A match of several calls is replaced by its root alone, so the calls inside it must have no
  // consumer outside it: such a consumer would keep the old call alive next to the fused one, and
  // an operator with out= would then run twice.  (The reference leaves this to the pattern writer.)
  bool InteriorIsPrivate(const Expr& root, const NodeMap& node_map) const {
    std::vector<const CallNode*> matched;
    for (const auto* cp : call_patterns_) {
      auto it = node_map.find(cp);
      if (it != node_map.end()) matched.push_back(AsCall(it->second));
    }
    for (const CallNode* inner : matched) {
      if (inner == root.get()) continue;
      size_t inside = 0;
      for (const CallNode* user : matched)
        for (const auto& a : user->args) inside += a.get() == inner;
      auto org = origin_.find(inner);
      auto total = uses_.find(org == origin_.end() ? inner : org->second);
      if (total == uses_.end() || total->second != inside) return false;
    }
    return true;
  }

  const DFPattern& pattern_;
  const RewriteCallback& cb_;
  std::vector<const DFPatternNode*> call_patterns_;
  std::set<const ExprNode*> counted_;
  std::map<const ExprNode*, size_t> uses_;
  std::map<const ExprNode*, const ExprNode*> origin_;  // rebuilt call -> the call it was made from
  std::map<const ExprNode*, Expr> memo_;
  std::vector<Expr> keep_alive_;
};

}  // namespace

std::vector<const DFPatternNode*> CallPatternsOf(const DFPattern& pattern) {
  std::set<const DFPatternNode*> seen;
  std::vector<const DFPatternNode*> calls;
  CollectCallPatternNodes(pattern, &seen, &calls);
  return calls;
}

bool MatchPattern(const DFPattern& pattern, const Expr& expr, NodeMap* node_map) {
  Matcher m;
  if (!m.Match(pattern, expr)) return false;
  if (node_map) *node_map = m.node_map();
  return true;
}

Expr RewritePatterns(const DFPattern& pattern, const RewriteCallback& callback, const Expr& expr) {
  return Rewriter(pattern, callback, expr).Mutate(expr);
}

}  // namespace ir

namespace op {

// ----------------------------------------------------------------------- fuse-pattern registry
DialectFusePattern::PatternList* DialectFusePattern::Get() {
  static PatternList patterns;
  return &patterns;
}

void DialectFusePattern::AddPattern(const ir::DFPattern& pattern, const std::string& dialect,
                                    int plevel, const std::string& name) {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  PatternList* list = Get();
  DialectFusePattern entry;
  entry.pattern = pattern;
  entry.dialect = dialect;
  entry.plevel = plevel;
  entry.name = name;
  auto it = list->begin();
  for (; it != list->end(); ++it) {
    RAF_CHECK(plevel != it->plevel, "InternalError: dialect pattern with plevel " +
                                        std::to_string(plevel) + " is already registered");
    if (plevel > it->plevel) break;
  }
  list->insert(it, entry);
}

std::list<DialectGraphRewrite>* DialectGraphRewrite::Get() {
  static std::list<DialectGraphRewrite> rewrites;
  return &rewrites;
}

void DialectGraphRewrite::Add(const std::string& dialect, int plevel, const std::string& name, Fn fn) {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  auto* list = Get();
  DialectGraphRewrite entry;
  entry.dialect = dialect;
  entry.plevel = plevel;
  entry.name = name;
  entry.fn = std::move(fn);
  auto it = list->begin();
  for (; it != list->end(); ++it) {
    RAF_CHECK(!(plevel == it->plevel && dialect == it->dialect),
              "InternalError: dialect " + dialect + " already has a graph rewrite with plevel " +
                  std::to_string(plevel));
    if (plevel > it->plevel) break;
  }
  list->insert(it, entry);
}

ir::Expr LowerOp(const std::string& base_op, const std::string& dialect) {
  std::string name = OpDialect::Lower(base_op, dialect);
  return name.empty() ? ir::Expr() : ir::GetOp(name);
}

// ------------------------------------------------------------------------------ fused dispatch
CallValues BindCall(const ir::Expr& call, const std::map<const ir::ExprNode*, value::Value>& bindings,
                    const Device& device) {
  const auto* c = ir::AsCall(call);
  RAF_CHECK(c != nullptr, "BindCall takes a call");
  RAF_CHECK(ir::AsFunction(c->op) != nullptr, "BindCall takes a call of a fused function");
  auto args = std::make_shared<schema::ListArgs>();
  for (const auto& a : c->args) {
    if (const auto* k = ir::AsConstant(a)) {
      switch (k->value_kind) {
        case ir::ConstantNode::kNull:
          args->args.push_back(nullptr);
          break;
        case ir::ConstantNode::kFloat: {
          auto v = std::make_shared<FloatValueObj>();
          v->value = k->f;
          args->args.push_back(v);
          break;
        }
        case ir::ConstantNode::kInt: {
          auto v = std::make_shared<IntValueObj>();
          v->value = k->i;
          args->args.push_back(v);
          break;
        }
        default: {
          auto v = std::make_shared<StringValueObj>();
          v->value = k->s;
          args->args.push_back(v);
        }
      }
    } else {
      auto it = bindings.find(a.get());
      RAF_CHECK(it != bindings.end(), "BindCall: an argument is neither a constant nor a bound variable");
      args->args.push_back(it->second);
    }
  }
  auto cv = std::make_shared<CallValuesNode>();
  cv->callee = "";
  cv->closure = c->op;
  cv->args = args;
  cv->device = device;
  return cv;
}

OpEnvPtr DispatchFusedOp(const CallValues& call) {
  const auto* func = ir::AsFunction(call->closure);
  RAF_CHECK(func != nullptr, "DispatchFusedOp: the callee is not a function");
  RAF_CHECK(func->attrs.count(ir::kPrimitive) && func->attrs.at(ir::kPrimitive) != "0",
            "Encountered a non-primitive function when dispatching a call");
  auto dialect = func->attrs.find(ir::kDialect);
  RAF_CHECK(dialect != func->attrs.end(),
            "Fused function doesn't have dialect attribute: " + ir::AsText(call->closure));
  const std::string name = "raf.op." + dialect->second + "._fused_op";
  const OpEnvMaker* maker = OpEnvMaker::Get(name);
  OpEnvPtr env(maker ? (*maker)(call) : nullptr);
  if (!env || env->HasError()) {
    std::ostringstream ss;
    ss << "Failed to dispatch fused op:";
    if (env)
      for (const auto& m : env->error_msgs) ss << "\n\t" << m;
    ss << "\nName: " << name << "\n" << ir::AsText(call->closure);
    throw Error(ss.str());
  }
  return env;
}

OpEnvPtr Dispatch(const CallValues& call) {
  if (call->closure) return DispatchFusedOp(call);
  return DispatchSingleOp(call);
}

}  // namespace op

// ------------------------------------------------------------------------------------ the pass
namespace pass {
namespace {

using ir::Expr;

class FuseMutator {
 public:
  FuseMutator(const std::string& dialect, const std::set<const ir::ExprNode*>& call_set,
              const std::string& pattern_name, std::unordered_map<std::string, Expr>* cache)
      : dialect_(dialect), call_set_(call_set), pattern_name_(pattern_name), cache_(cache) {}

  Expr Rewrite(const Expr& expr) {
    const bool single = call_set_.size() == 1;
    Expr body = Mutate(expr, single);
    if (single) return body;  // one call needs no function around it
    std::map<std::string, std::string> attrs;
    attrs[ir::kPrimitive] = "1";
    attrs[ir::kDialect] = dialect_;
    if (!pattern_name_.empty()) attrs[ir::kPatternName] = pattern_name_;
    Expr func = ir::MakeFunction(params_, body, attrs);
    const std::string key = ir::AsText(func);
    auto it = cache_->find(key);
    if (it != cache_->end())
      func = it->second;
    else
      (*cache_)[key] = func;
    return ir::MakeCall(func, args_, ir::TypeOf(expr));
  }

 private:
  Expr Mutate(const Expr& e, bool single) {
    auto it = memo_.find(e.get());
    if (it != memo_.end()) return it->second;
    const auto* c = ir::AsCall(e);
    RAF_CHECK(c != nullptr && ir::AsOp(c->op) != nullptr, "a fuse pattern matched a call of a non-operator");
    const std::string& base = ir::AsOp(c->op)->name;
    Expr dialect_op = op::LowerOp(base, dialect_);
    RAF_CHECK(dialect_op != nullptr,
              "Cannot find dialect \"" + dialect_ + "\" registered to operator " + base);
    std::vector<Expr> new_args;
    for (const auto& a : c->args) {
      if (single) {
        new_args.push_back(a);
      } else if (call_set_.count(a.get())) {
        new_args.push_back(Mutate(a, single));
      } else {  // an outside value: lift it into a parameter, one per use like the reference
        Expr var = ir::MakeVar("p", ir::TypeOf(a));
        new_args.push_back(var);
        params_.push_back(var);
        args_.push_back(a);
      }
    }
    Expr out = ir::MakeCall(dialect_op, new_args, c->type);
    memo_[e.get()] = out;
    return out;
  }

  std::string dialect_;
  const std::set<const ir::ExprNode*>& call_set_;
  std::string pattern_name_;
  std::unordered_map<std::string, Expr>* cache_;
  std::vector<Expr> params_, args_;
  std::map<const ir::ExprNode*, Expr> memo_;
};

}  // namespace

ir::Expr FuseDialect(const ir::Expr& expr, DevType device_type) {
  if (device_type == DevType::kUnknown()) return expr;  // the reference warns and skips the pass
  Expr ret = expr;
  const std::list<op::DialectGraphRewrite> rewrites = *op::DialectGraphRewrite::Get();
  for (const auto& rw : rewrites)
    if (op::Dialect::IsEnabled(rw.dialect, device_type)) ret = rw.fn(ret);
  // A snapshot: makers may not register patterns while the pass runs.
  const op::DialectFusePattern::PatternList patterns = *op::DialectFusePattern::Get();
  for (const auto& pat : patterns) {
    if (!op::Dialect::IsEnabled(pat.dialect, device_type)) continue;
    const std::vector<const ir::DFPatternNode*> call_patterns = ir::CallPatternsOf(pat.pattern);
    std::unordered_map<std::string, Expr> func_cache;
    auto callback = [&](const Expr& pre, const Expr& post, const ir::NodeMap& node_map) -> Expr {
      (void)pre;
      std::set<const ir::ExprNode*> call_set;
      for (const auto* cp : call_patterns) {
        auto it = node_map.find(cp);
        if (it != node_map.end()) call_set.insert(it->second.get());
      }
      return FuseMutator(pat.dialect, call_set, pat.name, &func_cache).Rewrite(post);
    };
    ret = ir::RewritePatterns(pat.pattern, callback, ret);
  }
  return ret;
}

}  // namespace pass
}  // namespace raf

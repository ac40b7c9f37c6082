// The slice of RAF's graph IR that dialect fusion needs, restated without TVM: expressions in
// graph normal form (variables, constants, operators, calls, primitive functions), dataflow
// patterns over them, the dialect fuse-pattern registry, the FuseDialect pass and the dispatch of
// the fused functions it creates.  The `hip` dialect uses it to turn the operator sequence that
// the reference's traced SGD optimizer emits per parameter into one call of the gfx950 SGD kernel.
//
// What each piece mirrors in the reference tree:
//   Expr nodes ................ relay Var / Constant / Op / Call / Function as RAF uses them
//                               (include/raf/ir.h; function attributes "Primitive", "Dialect",
//                               "PatternName": include/raf/ir.h:185-192)
//   DFPattern, is_op, wildcard, is_constant, has_dtype, `|`
//                               python/raf/ir/dataflow_pattern.py as used by
//                               python/raf/_op/dialect_pattern.py:8-118
//   DialectFusePattern ........ include/raf/dialect.h:171-197, src/impl/dialect.cc:218-239
//   OpDialect::Lower .......... src/impl/dialect.cc:204-214
//   FuseDialect ............... src/pass/fuse_dialect.cc:27-213
//   DispatchFusedOp, Dispatch . src/impl/op.cc:182-215
//   ListArgs .................. src/impl/op.cc:255-264
#pragma once

#include <functional>
#include <list>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "raf_iface.h"

namespace raf {
namespace ir {

struct ExprNode;
using Expr = std::shared_ptr<const ExprNode>;

// A tensor type; `defined` is false for an expression whose type is not known.
struct TensorType {
  bool defined = false;
  std::vector<int64_t> shape;
  DType dtype;
};

struct ExprNode {
  enum Kind { kVar, kConstant, kOp, kCall, kFunction, kTuple, kTupleGetItem };
  explicit ExprNode(Kind k) : kind(k) {}
  virtual ~ExprNode() = default;
  const Kind kind;
};

struct VarNode : ExprNode {
  VarNode() : ExprNode(kVar) {}
  std::string name_hint;
  TensorType type;
};

// A constant holds a value: null (the reference's `const(None)`), a float, an integer, a string,
// or a tensor all of whose elements are zero (what binding a model's constant attribute such as
// `self.zero` and folding constants leaves in the graph; only its type matters to a pass).
struct ConstantNode : ExprNode {
  enum ValueKind { kNull, kFloat, kInt, kString, kZeros };
  ConstantNode() : ExprNode(kConstant) {}
  ValueKind value_kind = kNull;
  double f = 0.0;
  int64_t i = 0;
  std::string s;
  TensorType type;  // kZeros
};

struct OpNode : ExprNode {
  OpNode() : ExprNode(kOp) {}
  std::string name;
};

struct CallNode : ExprNode {
  CallNode() : ExprNode(kCall) {}
  Expr op;  // an OpNode or a FunctionNode
  std::vector<Expr> args;
  TensorType type;  // result type, when known
  std::vector<TensorType> field_types;  // for a call that returns a tuple: its fields' types, when known
};

// Tuples: the tensor lists of the multi-tensor ops and the results of ops that return several
// tensors (relay Tuple / TupleGetItem).
struct TupleNode : ExprNode {
  TupleNode() : ExprNode(kTuple) {}
  std::vector<Expr> fields;
};

struct TupleGetItemNode : ExprNode {
  TupleGetItemNode() : ExprNode(kTupleGetItem) {}
  Expr tuple;
  int index = 0;
};

struct FunctionNode : ExprNode {
  FunctionNode() : ExprNode(kFunction) {}
  std::vector<Expr> params;  // VarNodes
  Expr body;
  std::map<std::string, std::string> attrs;
};

constexpr const char* kPrimitive = "Primitive";
constexpr const char* kDialect = "Dialect";
constexpr const char* kPatternName = "PatternName";

Expr MakeVar(const std::string& name_hint, const TensorType& type = TensorType());
Expr MakeNull();
Expr MakeFloat(double v);
Expr MakeInt(int64_t v);
Expr MakeString(const std::string& v);
Expr MakeZeros(const TensorType& type);
Expr MakeTuple(std::vector<Expr> fields);
Expr MakeTupleGetItem(const Expr& tuple, int index);
// A call whose result is a tuple of tensors of the given types.
Expr MakeTupleCall(const Expr& op, std::vector<Expr> args, std::vector<TensorType> field_types);
Expr GetOp(const std::string& name);  // one node per operator name
Expr MakeCall(const Expr& op, std::vector<Expr> args, const TensorType& type = TensorType());
Expr MakeFunction(std::vector<Expr> params, const Expr& body,
                  std::map<std::string, std::string> attrs = {});

template <typename T>
const T* As(const Expr& e, ExprNode::Kind kind) {
  return e && e->kind == kind ? static_cast<const T*>(e.get()) : nullptr;
}
inline const VarNode* AsVar(const Expr& e) { return As<VarNode>(e, ExprNode::kVar); }
inline const ConstantNode* AsConstant(const Expr& e) { return As<ConstantNode>(e, ExprNode::kConstant); }
inline const OpNode* AsOp(const Expr& e) { return As<OpNode>(e, ExprNode::kOp); }
inline const CallNode* AsCall(const Expr& e) { return As<CallNode>(e, ExprNode::kCall); }
inline const FunctionNode* AsFunction(const Expr& e) { return As<FunctionNode>(e, ExprNode::kFunction); }
inline const TupleNode* AsTupleNode(const Expr& e) { return As<TupleNode>(e, ExprNode::kTuple); }
inline const TupleGetItemNode* AsTupleGetItem(const Expr& e) {
  return As<TupleGetItemNode>(e, ExprNode::kTupleGetItem);
}

// The type of a variable, a call that returns a tensor, a zeros constant, or a field taken from a
// tuple or from a call that returns a tuple; undefined for everything else.
TensorType TypeOf(const Expr& e);

// Every expression reachable from `root` (function bodies included), each once, arguments before
// the expressions that use them.
std::vector<Expr> PostOrder(const Expr& root);

// `root` rebuilt with every expression that is a key of `replace` swapped for its value (the
// values are taken as they are, not rewritten again); untouched sub-graphs are shared.
Expr Substitute(const Expr& root, const std::map<const ExprNode*, Expr>& replace);

// Text form for messages and for the cache of fused functions; shared sub-expressions are bound
// to %n names, so the text is linear in the size of the graph.
std::string AsText(const Expr& e);

// Equality up to the names of variables: bound variables (function parameters) correspond by
// position, free variables one to one in order of first use; types of variables must agree.
bool StructuralEqual(const Expr& a, const Expr& b);

// ------------------------------------------------------------------------------------ patterns
struct DFPatternNode;
using DFPattern = std::shared_ptr<const DFPatternNode>;

struct DFPatternNode {
  enum Kind { kWildcard, kConstant, kOp, kCall, kAlt, kDType };
  Kind kind = kWildcard;
  Expr constant;                // kConstant: the value to equal, or empty for any constant
  std::string op_name;          // kOp
  DFPattern op;                 // kCall
  std::vector<DFPattern> args;  // kCall
  DFPattern left, right;        // kAlt
  DFPattern inner;              // kDType: the pattern whose match must have this dtype
  DType dtype;                  // kDType
};

DFPattern wildcard();
DFPattern is_constant();                    // any constant
DFPattern is_constant(const Expr& value);   // a constant equal to `value` (null, float, int, string)
DFPattern is_op(const std::string& name);
DFPattern is_ops(const std::vector<std::string>& names);
DFPattern call(const DFPattern& op, std::vector<DFPattern> args);
DFPattern alt(const DFPattern& left, const DFPattern& right);
DFPattern has_dtype(const DType& dtype, DFPattern inner = nullptr);  // inner defaults to wildcard()

// pattern node -> the expression it matched.  A pattern node that occurs several times in a
// pattern must match one and the same expression everywhere.
using NodeMap = std::map<const DFPatternNode*, Expr>;
// Every call node of a pattern (the reference's CallPatternExtractor, src/pass/fuse_dialect.cc:27-43).
std::vector<const DFPatternNode*> CallPatternsOf(const DFPattern& pattern);
bool MatchPattern(const DFPattern& pattern, const Expr& expr, NodeMap* node_map = nullptr);

// Rewrites bottom-up: every sub-expression (after its arguments were rewritten) that matches
// `pattern` is replaced by callback(pre, post, node_map); the bodies of primitive functions are
// left alone.  A match whose inner calls have consumers outside the match is skipped: the
// replacement keeps the root only, so those consumers would hold on to the old calls.
using RewriteCallback = std::function<Expr(const Expr& pre, const Expr& post, const NodeMap&)>;
Expr RewritePatterns(const DFPattern& pattern, const RewriteCallback& callback, const Expr& expr);

}  // namespace ir

namespace op {

class DialectFusePattern {
 public:
  using PatternList = std::list<DialectFusePattern>;
  ir::DFPattern pattern;
  std::string dialect;
  int plevel = 0;
  std::string name;
  static PatternList* Get();
  // Keeps the list sorted by descending plevel; a plevel that is already taken is an error.
  static void AddPattern(const ir::DFPattern& pattern, const std::string& dialect, int plevel,
                         const std::string& name = "");
};

// A rewrite of a whole graph on behalf of a dialect.  DialectFusePattern covers what a dataflow
// pattern can say: a fixed number of calls under ONE root.  A multi-tensor optimizer step gathers a
// variable number of per-parameter roots (every parameter's update, or every parameter's cast and
// copy behind raf.op.lans) into one call that returns a tuple, which no such pattern expresses;
// dialects register those as functions over the graph.  FuseDialect runs them, for the dialects
// enabled on the device, in descending plevel order ahead of the patterns.  (Inside RAF proper
// each is one more pass in front of FuseDialect in the pass sequence.)
class DialectGraphRewrite {
 public:
  using Fn = std::function<ir::Expr(const ir::Expr&)>;
  std::string dialect;
  int plevel = 0;
  std::string name;
  Fn fn;
  static std::list<DialectGraphRewrite>* Get();
  static void Add(const std::string& dialect, int plevel, const std::string& name, Fn fn);
};

// The dialect op registered for `base_op` by `dialect` (an OpNode), or an empty Expr.
ir::Expr LowerOp(const std::string& base_op, const std::string& dialect);

namespace schema {
struct ListArgs : ArgsBase {  // the arguments of a fused function, in parameter order
  std::vector<value::Value> args;
  int FieldIndex(const std::string&) const override { return -1; }
};
}  // namespace schema

// Scalar values for constants handed to a fused function.
struct FloatValueObj : value::ValueObj {
  double value = 0.0;
};
struct IntValueObj : value::ValueObj {
  int64_t value = 0;
};
struct StringValueObj : value::ValueObj {
  std::string value;
};

// CallValues for `call`, whose callee is a primitive function: variables take their values from
// `bindings`, constants become scalar values (null: an empty Value).  The arguments go into
// ListArgs and the function into call->closure.
CallValues BindCall(const ir::Expr& call, const std::map<const ir::ExprNode*, value::Value>& bindings,
                    const Device& device);

// raf.op.<dialect>._fused_op's maker builds the OpEnv of a primitive function; no OpEnv, or one
// with error_msgs, is fatal here (there is no other dialect to fall back to).
OpEnvPtr DispatchFusedOp(const CallValues& call);
OpEnvPtr Dispatch(const CallValues& call);

}  // namespace op

namespace pass {

// Applies every registered fuse pattern whose dialect is enabled on `device_type`, in plevel
// order.  A match of several calls becomes a call of a primitive function (attributes Primitive,
// Dialect, PatternName) whose body calls the dialect's ops and whose parameters are the matched
// calls' outside arguments; a match of one call becomes a call of the dialect op.  Identical fused
// functions are shared.
ir::Expr FuseDialect(const ir::Expr& expr, DevType device_type);

}  // namespace pass
}  // namespace raf

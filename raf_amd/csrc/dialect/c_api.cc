// C entry points declared in rafhip_dialect.h: a minimal executor around the OpEnv mirror.
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <sstream>
#include <string>

#include "hip_dialect.h"
#include "memory_pool.h"
#include "raf_iface.h"
#include "raf_ir.h"
#include "rafhip_dialect.h"

using namespace raf;
using namespace raf::op;

struct rafhip_raf_memory {
  std::shared_ptr<memory_pool::Memory> mem;
};

struct rafhip_raf_tuple {
  value::TupleValue value;
};

struct rafhip_raf_env {
  OpEnvPtr env;
  CallValues call;
  std::string name;
  std::string op;
  // Only for an env made from a graph (rafhip_raf_traced_sgd_make): the graph before and after
  // the FuseDialect pass and the variables to bind at Execute time.
  ir::Expr traced, fused;
  std::vector<ir::Expr> vars;
  // The tensor list of the last execute call, as descriptors and as the tuple value made from
  // them: a training loop passes the same tensors every step, and an executor proper would hold
  // them as values already, so the tuple is made once and handed over again while the descriptors
  // stay the same.
  std::vector<rafhip_tensor_desc> list_descs;
  std::vector<int64_t> list_shapes;
  value::Value list_tuple;
  // Only for an env made from a whole optimizer graph (rafhip_raf_traced_optimizer_make): one
  // OpEnv per call of the fused graph, in execution order.
  struct GraphCall {
    const ir::ExprNode* node = nullptr;
    std::string what;       // the dialect op, or "<dialect>._fused_op(<pattern>)"; "!" + op if it has no backend
    OpEnvPtr env;           // empty if unsupported
    int out_arg = -1;       // fused function: the argument whose memory the result shares
  };
  std::vector<GraphCall> graph_calls;
  std::vector<size_t> var_counts;  // how many variables each descriptor list of the make call bound
  int kind = -1;                   // 0 SGD, 1 LANS
};

namespace {

thread_local std::string g_error;
thread_local std::unique_ptr<DialectPreference> g_pref;

template <typename F>
int Guard(F&& f) {
  try {
    g_error.clear();
    f();
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 1;
  } catch (...) {
    g_error = "unknown C++ exception";
    return 1;
  }
}

value::TensorValue FromDesc(const rafhip_tensor_desc* d, const char* what) {
  if (!d) throw Error(std::string(what) + ": null tensor descriptor");
  if (d->ndim < 0 || (d->ndim > 0 && !d->shape)) throw Error(std::string(what) + ": bad shape");
  TensorView t;
  t.data = d->data;
  t.device = Device(DevType(d->device_type), d->device_id);
  t.dtype.code = d->dtype_code;
  t.dtype.bits = d->dtype_bits;
  t.shape.assign(d->shape, d->shape + d->ndim);
  return value::MakeTensor(t);
}

// The tuple value of a tensor list, remade only when a descriptor differs from the last call's.
value::Value ListTuple(rafhip_raf_env* env, int32_t n, const rafhip_tensor_desc* list, const char* what) {
  bool same = env->list_tuple != nullptr && (size_t)n == env->list_descs.size();
  size_t dim = 0;
  for (int32_t i = 0; same && i < n; ++i) {
    const rafhip_tensor_desc& a = list[i];
    const rafhip_tensor_desc& b = env->list_descs[(size_t)i];
    same = a.data == b.data && a.ndim == b.ndim && a.dtype_code == b.dtype_code &&
           a.dtype_bits == b.dtype_bits && a.device_type == b.device_type && a.device_id == b.device_id &&
           (a.ndim <= 0 || a.shape != nullptr);
    for (int32_t d = 0; same && d < a.ndim; ++d) same = a.shape[d] == env->list_shapes[dim + (size_t)d];
    dim += (size_t)(b.ndim > 0 ? b.ndim : 0);
  }
  if (same) return env->list_tuple;
  std::vector<value::Value> fields;
  fields.reserve((size_t)n);
  env->list_tuple = nullptr;
  env->list_descs.assign(list, list + n);
  env->list_shapes.clear();
  for (int32_t i = 0; i < n; ++i) {
    fields.push_back(FromDesc(&list[i], what));
    env->list_shapes.insert(env->list_shapes.end(), list[i].shape, list[i].shape + list[i].ndim);
    env->list_descs[(size_t)i].shape = nullptr;  // the caller's array may go away; the copy above is compared
  }
  env->list_tuple = value::MakeTuple(std::move(fields));
  return env->list_tuple;
}

constexpr int64_t kWsAlign = 256;
int64_t RoundUp(int64_t x) { return (x + kWsAlign - 1) / kWsAlign * kWsAlign; }

// What the executors do around Execute: point every requested workspace into the block the caller
// provides, run, then take the pointers back (src/impl/vm/vm.cc:1099-1105, :846-853).
struct WorkspaceBinding {
  const std::vector<WorkspaceRequest>& reqs;
  WorkspaceBinding(OpEnv* env, void* block, int64_t bytes) : reqs(env->workspace_requests()) {
    int64_t need = 0;
    for (const auto& r : reqs) need += RoundUp(r.nbytes);
    if (need > 0 && (!block || bytes < need))
      throw Error("workspace of " + std::to_string(bytes) + " bytes given, OpEnv requested " +
                  std::to_string(need));
    char* p = static_cast<char*>(block);
    for (const auto& r : reqs) {
      *r.dest = p;
      p += RoundUp(r.nbytes);
    }
  }
  ~WorkspaceBinding() {
    for (const auto& r : reqs) *r.dest = nullptr;
  }
};

// Stream requests (OpEnv::RequestStream).  Off by default: the requests stay unserved (*dest is
// null) and an OpEnv launches on the compute stream.  Switched on, the executor serves them from a
// pool of streams per (device, tag), like Stream::Get in the reference (src/impl/interpreter.cc:384-389),
// and -- since a caller of this window expects an operator's results in stream order -- makes the
// requested stream wait for the compute stream before Execute and the compute stream wait for
// the requested stream after it.
thread_local bool g_serve_stream_requests = false;

struct StreamPool {
  std::mutex mu;
  std::map<std::tuple<int, int, int, int>, void*> streams;  // (device type, device id, tag, index)
  void* Get(const Device& dev, int tag, int index) {
    std::lock_guard<std::mutex> lock(mu);
    void*& s = streams[std::make_tuple((int)dev.device_type(), dev.device_id(), tag, index)];
    if (!s) s = device_api::DeviceAPI::Get(dev.device_type())->CreateStream(dev);
    return s;
  }
};
// The two events that order a served stream against the compute stream, made once per thread and
// device (an event may be recorded again as soon as the wait on its previous record has been
// enqueued; two threads must not share one).  They live as long as the process.
std::pair<void*, void*> OrderingEvents(const Device& dev, device_api::DeviceAPI* api) {
  thread_local std::map<std::pair<int, int>, std::pair<void*, void*>> events;
  auto& ev = events[{(int)dev.device_type(), dev.device_id()}];
  constexpr uint32_t kNoTiming = 0x2;  // hipEventDisableTiming: ordering only
  if (!ev.first) ev.first = api->CreateEvent(dev, kNoTiming);
  if (!ev.second) ev.second = api->CreateEvent(dev, kNoTiming);
  return ev;
}
StreamPool& Streams() {
  static StreamPool* pool = new StreamPool();  // streams live as long as the process
  return *pool;
}

struct StreamBinding {
  const std::vector<StreamRequest>& reqs;
  std::shared_ptr<device_api::DeviceAPI> api;
  Device device;
  void* compute = nullptr;
  void* after = nullptr;
  std::vector<void*> served;
  StreamBinding(OpEnv* env, const Device& dev, void* compute_stream)
      : reqs(env->stream_requests()), device(dev), compute(compute_stream) {
    if (!g_serve_stream_requests || reqs.empty()) {
      for (const auto& r : reqs) *r.dest = nullptr;
      return;
    }
    api = device_api::DeviceAPI::Get(dev.device_type());
    const auto events = OrderingEvents(dev, api.get());
    after = events.second;
    api->EventRecordOnStream(events.first, compute);
    for (const auto& r : reqs) {
      void* s = Streams().Get(r.device, r.tag_idx, r.stream_idx);
      api->StreamWaitEvent(s, events.first);
      *r.dest = s;
      served.push_back(s);
    }
  }
  // Ordering the compute stream behind the served streams can fail; call it on the normal path.
  void Finish() {
    for (void* s : served) {
      api->EventRecordOnStream(after, s);
      api->StreamWaitEvent(compute, after);
    }
    served.clear();
  }
  ~StreamBinding() {
    for (const auto& r : reqs) *r.dest = nullptr;
  }
};

rafhip_raf_env* Finish(const CallValues& call) {
  RunDeclare(call);
  auto* h = new rafhip_raf_env();
  h->call = call;
  if (call->callee.empty()) return h;  // declared as a no-op (an empty tensor list): nothing to dispatch
  std::string picked;
  std::unique_ptr<rafhip_raf_env> guard(h);
  OpEnvPtr env = DispatchSingleOp(call, &picked);
  h->env = env;
  h->name = env->name();
  h->op = picked;
  return guard.release();
}

std::vector<int64_t> ToVector(const int64_t* p, int32_t n, const char* what) {
  if (n < 0 || (n > 0 && !p)) throw Error(std::string(what) + ": bad integer list");
  return std::vector<int64_t>(p, p + n);
}

// The declared outputs, flattened: a tensor is one output, a tuple its fields.
std::vector<value::TensorValue> Outputs(const rafhip_raf_env* env) {
  std::vector<value::TensorValue> outs;
  if (!env->call->out) return outs;
  if (auto t = std::dynamic_pointer_cast<value::TensorValueObj>(env->call->out)) {
    outs.push_back(t);
  } else {
    for (const auto& f : value::AsTuple(env->call->out)->fields) outs.push_back(value::AsTensor(f));
  }
  return outs;
}

// ------------------------------------------------------------------ running a fused graph
// A small evaluator for graphs that FuseDialect has worked on: variables take the caller's
// tensors, tuples and projections are formed, and every call is either a `hip` dialect op of the
// optimizer family or a fused function, each with an OpEnv of its own that is made once and then
// executed in order.  Anything else (an element-wise base op that nothing fused) has no backend in
// this library; a result field that needs one is skipped when the caller allows that, and the
// make call reports the op with a leading '!'.
struct Unsupported : Error {
  using Error::Error;
};

class GraphRunner {
 public:
  GraphRunner(rafhip_raf_env* env, const std::map<const ir::ExprNode*, value::Value>& bindings, bool make,
              char* workspace, int64_t workspace_bytes)
      : env_(env), bindings_(bindings), make_(make), ws_(workspace), ws_left_(workspace_bytes) {}

  value::Value Eval(const ir::Expr& e) {
    auto it = memo_.find(e.get());
    if (it != memo_.end()) return it->second;
    value::Value v = Compute(e);
    memo_[e.get()] = v;
    return v;
  }

 private:
  static double Number(const value::Value& v, const char* what) {
    if (auto f = std::dynamic_pointer_cast<FloatValueObj>(v)) return f->value;
    if (auto i = std::dynamic_pointer_cast<IntValueObj>(v)) return (double)i->value;
    throw Error(std::string(what) + " must be a scalar constant");
  }

  rafhip_raf_env::GraphCall& Slot(const ir::ExprNode* node) {
    for (auto& gc : env_->graph_calls)
      if (gc.node == node) return gc;
    RAF_CHECK(make_, "the graph was not prepared for this call");
    env_->graph_calls.emplace_back();
    env_->graph_calls.back().node = node;
    return env_->graph_calls.back();
  }

  void Run(OpEnv* op_env, const std::vector<value::Value>& inputs, const value::Value& out) {
    if (!op_env) throw Error("a call of the graph has no OpEnv: making the graph did not succeed");
    int64_t need = 0;
    for (const auto& r : op_env->workspace_requests()) need += RoundUp(r.nbytes);
    if (need > ws_left_) throw Error("the workspace is too small for the graph's operators");
    WorkspaceBinding bind(op_env, ws_, need);
    ws_ += need;
    ws_left_ -= need;
    op_env->Execute(inputs, out);
  }

  value::Value Compute(const ir::Expr& e) {
    if (ir::AsVar(e)) {
      auto it = bindings_.find(e.get());
      RAF_CHECK(it != bindings_.end(), "a variable of the graph has no value");
      return it->second;
    }
    if (const auto* k = ir::AsConstant(e)) {
      switch (k->value_kind) {
        case ir::ConstantNode::kNull:
          return nullptr;
        case ir::ConstantNode::kFloat: {
          auto v = std::make_shared<FloatValueObj>();
          v->value = k->f;
          return v;
        }
        case ir::ConstantNode::kInt: {
          auto v = std::make_shared<IntValueObj>();
          v->value = k->i;
          return v;
        }
        case ir::ConstantNode::kString: {
          auto v = std::make_shared<StringValueObj>();
          v->value = k->s;
          return v;
        }
        default:
          throw Unsupported("a tensor constant that nothing folded away has no storage here");
      }
    }
    if (const auto* t = ir::AsTupleNode(e)) {
      std::vector<value::Value> fields;
      for (const auto& f : t->fields) fields.push_back(Eval(f));
      return value::MakeTuple(std::move(fields));
    }
    if (const auto* g = ir::AsTupleGetItem(e)) {
      auto tuple = value::AsTuple(Eval(g->tuple));
      RAF_CHECK((size_t)g->index < tuple->fields.size(), "tuple index out of range");
      return tuple->fields[(size_t)g->index];
    }
    const auto* c = ir::AsCall(e);
    RAF_CHECK(c != nullptr, "unexpected expression in a graph to run");
    std::vector<value::Value> args;
    for (const auto& a : c->args) args.push_back(Eval(a));
    const Device device = env_->call->device;
    if (const auto* func = ir::AsFunction(c->op)) {
      auto& slot = Slot(e.get());
      if (make_) {
        auto list = std::make_shared<schema::ListArgs>();
        list->args = args;
        auto cv = std::make_shared<CallValuesNode>();
        cv->closure = c->op;
        cv->args = list;
        cv->device = device;
        slot.env = DispatchFusedOp(cv);
        auto name = func->attrs.find(ir::kPatternName);
        slot.what = func->attrs.at(ir::kDialect) + "._fused_op(" + (name == func->attrs.end() ? "" : name->second) + ")";
        // an element-wise root with out=: the result shares that argument's memory
        const auto* root = ir::AsCall(func->body);
        if (root && root->args.size() == 4)
          for (size_t i = 0; i < func->params.size(); ++i)
            if (func->params[i].get() == root->args[2].get()) slot.out_arg = (int)i;
        RAF_CHECK(slot.out_arg >= 0, "cannot tell where the fused function's result lives");
      } else {
        Run(slot.env.get(), args, args[(size_t)slot.out_arg]);
      }
      return args[(size_t)slot.out_arg];
    }
    const std::string& name = ir::AsOp(c->op)->name;
    const bool lans = name == "raf.op.hip.lans" || name == "raf.op.hip.lans_mixed";
    const bool sgd = name == "raf.op.hip.sgd_multi" || name == "raf.op.hip.sgd_multi_mixed";
    if (!lans && !sgd) {
      if (make_) {
        auto& slot = Slot(e.get());
        slot.what = "!" + name;
      }
      throw Unsupported("Cannot find a valid dispatch for op " + name +
                        ": outside a fused function the hip dialect has no backend for it");
    }
    auto& slot = Slot(e.get());
    auto tuple = value::AsTuple(args.at(0));
    if (make_) {
      std::shared_ptr<schema::ArgsBase> sargs;
      std::vector<value::TensorValue> tensors;
      for (const auto& f : tuple->fields) tensors.push_back(value::AsTensor(f));
      if (lans) {
        RAF_CHECK(args.size() == 11, name + " takes 11 arguments");
        auto a = std::make_shared<schema::LansArgs>();
        a->tensor_list = tensors;
        a->step = value::AsTensor(args[1]);
        a->learning_rate = (float)Number(args[2], "learning_rate");
        a->beta1 = (float)Number(args[3], "beta1");
        a->beta2 = (float)Number(args[4], "beta2");
        a->eps = (float)Number(args[5], "eps");
        a->bias_correction = (int)Number(args[6], "bias_correction");
        a->weight_decay = (float)Number(args[7], "weight_decay");
        a->grad_averaging = (int)Number(args[8], "grad_averaging");
        a->mode = (int)Number(args[9], "mode");
        a->normalize_grad = Number(args[10], "normalize_grad") != 0;
        sargs = a;
      } else {
        RAF_CHECK(args.size() == 3, name + " takes 3 arguments");
        auto a = std::make_shared<schema::SgdMultiArgs>();
        a->tensor_list = tensors;
        a->learning_rate = Number(args[1], "learning_rate");
        a->mu = Number(args[2], "mu");
        sargs = a;
      }
      CallValues cv = MakeCall(name, sargs);
      cv->device = device;
      cv->out = tuple;
      slot.env = DispatchSingleOp(cv);
      slot.what = name;
    } else {
      std::vector<value::Value> inputs = {tuple};
      if (lans) inputs.push_back(args[1]);
      Run(slot.env.get(), inputs, tuple);
    }
    return tuple;  // these ops return their list: the update is in place
  }

  rafhip_raf_env* env_;
  const std::map<const ir::ExprNode*, value::Value>& bindings_;
  bool make_;
  char* ws_;
  int64_t ws_left_;
  std::map<const ir::ExprNode*, value::Value> memo_;
};

// Evaluates the fields of the graph's result tuple one by one; a field that needs an operator
// without a backend is skipped if `allow_partial`, else the error goes up.
void RunGraph(rafhip_raf_env* env, const std::map<const ir::ExprNode*, value::Value>& bindings, bool make,
              bool allow_partial, void* workspace, int64_t workspace_bytes) {
  GraphRunner runner(env, bindings, make, static_cast<char*>(workspace), workspace_bytes);
  const auto* result = ir::AsTupleNode(env->fused);
  RAF_CHECK(result != nullptr, "the optimizer graph must end in a tuple");
  for (const auto& field : result->fields) {
    try {
      runner.Eval(field);
    } catch (const Unsupported&) {
      if (!allow_partial) throw;
    }
  }
}

}  // namespace

extern "C" {

const char* rafhip_raf_last_error(void) { return g_error.c_str(); }

int rafhip_raf_dispatch_list(const char* base_op, int32_t device_type, char* buf, int32_t buflen) {
  return Guard([&] {
    if (!base_op || !buf || buflen <= 0) throw Error("rafhip_raf_dispatch_list: bad arguments");
    std::ostringstream ss;
    bool first = true;
    for (const auto& e : OpDialect::GetDispatchList(base_op, DevType(device_type))) {
      if (!first) ss << ';';
      first = false;
      ss << e.dialect << ':' << e.dialect_op << ':' << e.plevel;
    }
    std::string s = ss.str();
    std::strncpy(buf, s.c_str(), (size_t)buflen - 1);
    buf[buflen - 1] = '\0';
  });
}

int rafhip_raf_set_dialect_preference(const char* dialects_csv) {
  return Guard([&] {
    g_pref.reset();
    if (!dialects_csv || !*dialects_csv) return;
    std::vector<std::string> names;
    std::stringstream ss(dialects_csv);
    std::string item;
    while (std::getline(ss, item, ','))
      if (!item.empty()) names.push_back(item);
    g_pref.reset(new DialectPreference(std::move(names)));
  });
}

int rafhip_raf_sgd_make(const rafhip_tensor_desc* x, const rafhip_tensor_desc* dx,
                        const rafhip_tensor_desc* v, double learning_rate, double mu,
                        rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_sgd_make: env_out is NULL");
    *env_out = nullptr;
    auto args = std::make_shared<schema::SgdArgs>();
    args->x = FromDesc(x, "x");
    args->dx = FromDesc(dx, "dx");
    args->v = FromDesc(v, "v");
    args->learning_rate = learning_rate;
    args->mu = mu;
    *env_out = Finish(MakeCall("raf.op.sgd", args));
  });
}

int rafhip_raf_sgd_execute(rafhip_raf_env* env, const rafhip_tensor_desc* x,
                           const rafhip_tensor_desc* dx, const rafhip_tensor_desc* v,
                           const rafhip_tensor_desc* v1, const rafhip_tensor_desc* x1,
                           void* stream) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_sgd_execute: env is NULL");
    std::vector<value::Value> inputs = {FromDesc(x, "x"), FromDesc(dx, "dx"), FromDesc(v, "v")};
    value::Value out = value::MakeTuple({FromDesc(v1, "v1"), FromDesc(x1, "x1")});
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), nullptr, 0);
    env->env->Execute(inputs, out);
  });
}

namespace {
int LansMake(const char* op_name, int32_t list_len, const rafhip_tensor_desc* tensor_list,
             const rafhip_tensor_desc* step, float learning_rate, float beta1, float beta2,
             float eps, int32_t bias_correction, float weight_decay, int32_t grad_averaging,
             int32_t mode, int32_t normalize_grad, rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_lans_make: env_out is NULL");
    *env_out = nullptr;
    if (list_len < 0 || (list_len > 0 && !tensor_list))
      throw Error("rafhip_raf_lans_make: bad tensor list");
    auto args = std::make_shared<schema::LansArgs>();
    for (int32_t i = 0; i < list_len; ++i)
      args->tensor_list.push_back(FromDesc(&tensor_list[i], "tensor_list"));
    args->step = FromDesc(step, "step");
    args->learning_rate = learning_rate;
    args->beta1 = beta1;
    args->beta2 = beta2;
    args->eps = eps;
    args->bias_correction = bias_correction;
    args->weight_decay = weight_decay;
    args->grad_averaging = grad_averaging;
    args->mode = mode;
    args->normalize_grad = normalize_grad != 0;
    *env_out = Finish(MakeCall(op_name, args));
  });
}
}  // namespace

int rafhip_raf_lans_make(int32_t list_len, const rafhip_tensor_desc* tensor_list,
                         const rafhip_tensor_desc* step, float learning_rate, float beta1,
                         float beta2, float eps, int32_t bias_correction, float weight_decay,
                         int32_t grad_averaging, int32_t mode, int32_t normalize_grad,
                         rafhip_raf_env** env_out) {
  return LansMake("raf.op.lans", list_len, tensor_list, step, learning_rate, beta1, beta2, eps,
                  bias_correction, weight_decay, grad_averaging, mode, normalize_grad, env_out);
}

int rafhip_raf_lans_mixed_make(int32_t list_len, const rafhip_tensor_desc* tensor_list,
                               const rafhip_tensor_desc* step, float learning_rate, float beta1,
                               float beta2, float eps, int32_t bias_correction, float weight_decay,
                               int32_t grad_averaging, int32_t mode, int32_t normalize_grad,
                               rafhip_raf_env** env_out) {
  return LansMake("raf.op.lans_mixed", list_len, tensor_list, step, learning_rate, beta1, beta2,
                  eps, bias_correction, weight_decay, grad_averaging, mode, normalize_grad, env_out);
}

int rafhip_raf_lans_execute(rafhip_raf_env* env, int32_t list_len,
                            const rafhip_tensor_desc* tensor_list, const rafhip_tensor_desc* step,
                            void* workspace, int64_t workspace_bytes, void* stream) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_lans_execute: env is NULL");
    if (list_len < 0 || (list_len > 0 && !tensor_list))
      throw Error("rafhip_raf_lans_execute: bad tensor list");
    value::Value tuple = ListTuple(env, list_len, tensor_list, "tensor_list");
    std::vector<value::Value> inputs = {tuple, FromDesc(step, "step")};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), workspace, workspace_bytes);
    env->env->Execute(inputs, tuple);  // output aliases the inputs
  });
}

int rafhip_raf_tuple_make(int32_t n, const rafhip_tensor_desc* fields, rafhip_raf_tuple** tuple_out) {
  return Guard([&] {
    if (!tuple_out) throw Error("rafhip_raf_tuple_make: tuple_out is NULL");
    *tuple_out = nullptr;
    if (n < 0 || (n > 0 && !fields)) throw Error("rafhip_raf_tuple_make: bad field list");
    std::vector<value::Value> values;
    values.reserve((size_t)n);
    for (int32_t i = 0; i < n; ++i) values.push_back(FromDesc(&fields[i], "tuple field"));
    *tuple_out = new rafhip_raf_tuple{value::MakeTuple(std::move(values))};
  });
}

int rafhip_raf_tuple_replace(const rafhip_raf_tuple* base, int32_t first, int32_t count,
                             const rafhip_tensor_desc* fields, rafhip_raf_tuple** tuple_out) {
  return Guard([&] {
    if (!tuple_out) throw Error("rafhip_raf_tuple_replace: tuple_out is NULL");
    *tuple_out = nullptr;
    if (!base) throw Error("rafhip_raf_tuple_replace: base is NULL");
    const int64_t n = (int64_t)base->value->fields.size();
    if (first < 0 || count < 0 || (int64_t)first + count > n || (count > 0 && !fields))
      throw Error("rafhip_raf_tuple_replace: range [" + std::to_string(first) + ", " +
                  std::to_string((int64_t)first + count) + ") does not fit a tuple of " + std::to_string(n));
    std::vector<value::Value> values = base->value->fields;  // shares the tensor values
    for (int32_t i = 0; i < count; ++i) values[(size_t)first + (size_t)i] = FromDesc(&fields[i], "tuple field");
    *tuple_out = new rafhip_raf_tuple{value::MakeTuple(std::move(values))};
  });
}

int rafhip_raf_tuple_rebind(rafhip_raf_tuple* tuple, int32_t first, int32_t count,
                            const rafhip_tensor_desc* fields, int32_t* done_out) {
  return Guard([&] {
    if (!done_out) throw Error("rafhip_raf_tuple_rebind: done_out is NULL");
    *done_out = 0;
    if (!tuple) throw Error("rafhip_raf_tuple_rebind: tuple is NULL");
    const int64_t n = (int64_t)tuple->value->fields.size();
    if (first < 0 || count < 0 || (int64_t)first + count > n || (count > 0 && !fields))
      throw Error("rafhip_raf_tuple_rebind: range [" + std::to_string(first) + ", " +
                  std::to_string((int64_t)first + count) + ") does not fit a tuple of " + std::to_string(n));
    if (tuple->value.use_count() != 1) return;
    std::vector<value::Value>& held = tuple->value->fields;
    for (int32_t i = 0; i < count; ++i) {
      const value::Value& v = held[(size_t)first + (size_t)i];
      const auto* t = dynamic_cast<const value::TensorValueObj*>(v.get());
      const rafhip_tensor_desc& d = fields[i];
      if (!t || v.use_count() != 1 || d.ndim < 0 || (size_t)d.ndim != t->tensor.shape.size() ||
          (d.ndim > 0 && !d.shape) || d.dtype_code != t->tensor.dtype.code ||
          d.dtype_bits != t->tensor.dtype.bits || d.device_type != (int)t->tensor.device.device_type() ||
          d.device_id != t->tensor.device.device_id())
        return;
      for (int32_t k = 0; k < d.ndim; ++k)
        if (d.shape[k] != t->tensor.shape[(size_t)k]) return;
    }
    for (int32_t i = 0; i < count; ++i)
      static_cast<value::TensorValueObj*>(held[(size_t)first + (size_t)i].get())->tensor.data = fields[i].data;
    *done_out = 1;
  });
}

int32_t rafhip_raf_tuple_size(const rafhip_raf_tuple* tuple) {
  return tuple ? (int32_t)tuple->value->fields.size() : -1;
}

int rafhip_raf_tuple_destroy(rafhip_raf_tuple* tuple) {
  return Guard([&] { delete tuple; });
}

namespace {
// The value Execute receives for a tuple handle: the tuple itself, or (as_vm) a new TupleValue
// over the same tensor values, as the VM's AllocTuple makes one per iteration (vm.cc:764-769).
value::Value TupleArgument(const rafhip_raf_tuple* tuple, int32_t as_vm, const char* who) {
  if (!tuple) throw Error(std::string(who) + ": tensor_list is NULL");
  if (!as_vm) return tuple->value;
  return value::MakeTuple(tuple->value->fields);
}
}  // namespace

int rafhip_raf_lans_execute_tuple(rafhip_raf_env* env, const rafhip_raf_tuple* tensor_list,
                                  const rafhip_tensor_desc* step, void* workspace,
                                  int64_t workspace_bytes, void* stream, int32_t as_vm) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_lans_execute_tuple: env is NULL");
    if (!env->env) return;  // declared as a no-op
    value::Value tuple = TupleArgument(tensor_list, as_vm, "rafhip_raf_lans_execute_tuple");
    std::vector<value::Value> inputs = {tuple, FromDesc(step, "step")};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), workspace, workspace_bytes);
    env->env->Execute(inputs, tuple);  // output aliases the inputs
  });
}

int rafhip_raf_sgd_multi_execute_tuple(rafhip_raf_env* env, const rafhip_raf_tuple* tensor_list,
                                       void* stream, int32_t as_vm) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_sgd_multi_execute_tuple: env is NULL");
    if (!env->env) return;  // declared as a no-op
    value::Value tuple = TupleArgument(tensor_list, as_vm, "rafhip_raf_sgd_multi_execute_tuple");
    std::vector<value::Value> inputs = {tuple};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), nullptr, 0);
    env->env->Execute(inputs, tuple);  // output aliases the inputs
  });
}

int rafhip_raf_sgd_multi_make(int32_t mixed, int32_t list_len, const rafhip_tensor_desc* tensor_list,
                              double learning_rate, double mu, rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_sgd_multi_make: env_out is NULL");
    *env_out = nullptr;
    if (list_len < 0 || (list_len > 0 && !tensor_list))
      throw Error("rafhip_raf_sgd_multi_make: bad tensor list");
    auto args = std::make_shared<schema::SgdMultiArgs>();
    for (int32_t i = 0; i < list_len; ++i)
      args->tensor_list.push_back(FromDesc(&tensor_list[i], "tensor_list"));
    args->learning_rate = learning_rate;
    args->mu = mu;
    *env_out = Finish(MakeCall(mixed ? "raf.op.sgd_multi_mixed" : "raf.op.sgd_multi", args));
  });
}

int rafhip_raf_sgd_multi_execute(rafhip_raf_env* env, int32_t list_len,
                                 const rafhip_tensor_desc* tensor_list, void* stream) {
  return Guard([&] {
    if (!env || !env->env) throw Error("rafhip_raf_sgd_multi_execute: env is NULL");
    if (list_len < 0 || (list_len > 0 && !tensor_list))
      throw Error("rafhip_raf_sgd_multi_execute: bad tensor list");
    value::Value tuple = ListTuple(env, list_len, tensor_list, "tensor_list");
    std::vector<value::Value> inputs = {tuple};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), nullptr, 0);
    env->env->Execute(inputs, tuple);  // output aliases the inputs
  });
}

int rafhip_raf_l2norm_make(const rafhip_tensor_desc* x, rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_l2norm_make: env_out is NULL");
    *env_out = nullptr;
    auto args = std::make_shared<schema::L2NormArgs>();
    args->x = FromDesc(x, "x");
    *env_out = Finish(MakeCall("raf.op.l2norm", args));
  });
}

int rafhip_raf_l2norm_execute(rafhip_raf_env* env, const rafhip_tensor_desc* x,
                              const rafhip_tensor_desc* out, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  return Guard([&] {
    if (!env || !env->env) throw Error("rafhip_raf_l2norm_execute: env is NULL");
    std::vector<value::Value> inputs = {FromDesc(x, "x")};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), workspace, workspace_bytes);
    env->env->Execute(inputs, FromDesc(out, "out"));
  });
}

int rafhip_raf_fuse_tensor_make(int32_t n, const rafhip_tensor_desc* data,
                                rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_fuse_tensor_make: env_out is NULL");
    *env_out = nullptr;
    if (n < 0 || (n > 0 && !data)) throw Error("rafhip_raf_fuse_tensor_make: bad tensor list");
    auto args = std::make_shared<schema::FuseTensorArgs>();
    for (int32_t i = 0; i < n; ++i) args->data.push_back(FromDesc(&data[i], "data"));
    *env_out = Finish(MakeCall("raf.op.fuse_tensor", args));
  });
}

int rafhip_raf_fuse_tensor_execute(rafhip_raf_env* env, int32_t n, const rafhip_tensor_desc* data,
                                   const rafhip_tensor_desc* out, void* stream) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_fuse_tensor_execute: env is NULL");
    if (!env->env) return;  // declared as a no-op
    if (n < 0 || (n > 0 && !data)) throw Error("rafhip_raf_fuse_tensor_execute: bad tensor list");
    std::vector<value::Value> fields;
    for (int32_t i = 0; i < n; ++i) fields.push_back(FromDesc(&data[i], "data"));
    std::vector<value::Value> inputs = {value::MakeTuple(std::move(fields))};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), nullptr, 0);
    StreamBinding streams(env->env.get(), env->call->device, stream);
    env->env->Execute(inputs, FromDesc(out, "out"));
    streams.Finish();
  });
}

int rafhip_raf_defuse_tensor_make(const rafhip_tensor_desc* data, int32_t n_sizes,
                                  const int64_t* sizes, int32_t n_shapes, const int64_t* shapes,
                                  int32_t n_indices, const int64_t* shape_indices,
                                  rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_defuse_tensor_make: env_out is NULL");
    *env_out = nullptr;
    auto args = std::make_shared<schema::DefuseTensorArgs>();
    args->data = FromDesc(data, "data");
    args->sizes = ToVector(sizes, n_sizes, "sizes");
    args->shapes = ToVector(shapes, n_shapes, "shapes");
    args->shape_indices = ToVector(shape_indices, n_indices, "shape_indices");
    *env_out = Finish(MakeCall("raf.op.defuse_tensor", args));
  });
}

int rafhip_raf_defuse_tensor_execute(rafhip_raf_env* env, const rafhip_tensor_desc* data,
                                     int32_t n_out, const rafhip_tensor_desc* outs, void* stream) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_defuse_tensor_execute: env is NULL");
    if (!env->env) return;  // declared as a no-op
    if (n_out < 0 || (n_out > 0 && !outs)) throw Error("rafhip_raf_defuse_tensor_execute: bad output list");
    std::vector<value::Value> fields;
    for (int32_t i = 0; i < n_out; ++i) fields.push_back(FromDesc(&outs[i], "out"));
    std::vector<value::Value> inputs = {FromDesc(data, "data")};
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    WorkspaceBinding bind(env->env.get(), nullptr, 0);
    StreamBinding streams(env->env.get(), env->call->device, stream);
    env->env->Execute(inputs, value::MakeTuple(std::move(fields)));
    streams.Finish();
  });
}

int rafhip_raf_serve_stream_requests(int32_t enable) {
  return Guard([&] { g_serve_stream_requests = enable != 0; });
}

int32_t rafhip_raf_env_num_outputs(const rafhip_raf_env* env) {
  if (!env) return -1;
  int32_t n = -1;
  Guard([&] { n = (int32_t)Outputs(env).size(); });
  return n;
}

int rafhip_raf_env_output(const rafhip_raf_env* env, int32_t index, int32_t* dtype_code,
                          int32_t* dtype_bits, int32_t* ndim, int64_t* shape_out,
                          int32_t shape_capacity) {
  return Guard([&] {
    if (!env || !dtype_code || !dtype_bits || !ndim) throw Error("rafhip_raf_env_output: null argument");
    auto outs = Outputs(env);
    if (index < 0 || (size_t)index >= outs.size()) throw Error("rafhip_raf_env_output: no such output");
    const TensorView& t = outs[(size_t)index]->tensor;
    *dtype_code = t.dtype.code;
    *dtype_bits = t.dtype.bits;
    *ndim = t.ndim();
    if (shape_out) {
      if (shape_capacity < t.ndim()) throw Error("rafhip_raf_env_output: shape buffer too small");
      for (int i = 0; i < t.ndim(); ++i) shape_out[i] = t.shape[(size_t)i];
    }
  });
}

// ------------------------------------------------------------------ device API and memory pools
int rafhip_raf_device_count(int32_t device_type, int32_t* count_out) {
  return Guard([&] {
    if (!count_out) throw Error("rafhip_raf_device_count: count_out is NULL");
    *count_out = device_api::DeviceAPI::Get(DevType(device_type))->GetDeviceCount();
  });
}

int rafhip_raf_device_copy(const rafhip_tensor_desc* from, const rafhip_tensor_desc* to, void* stream) {
  return Guard([&] {
    auto f = FromDesc(from, "from"), t = FromDesc(to, "to");
    const bool gpu = f->tensor.device.device_type() == DevType::kROCM() ||
                     t->tensor.device.device_type() == DevType::kROCM();
    device_api::DeviceAPI::Get(gpu ? DevType::kROCM() : DevType::kCPU())
        ->CopyDataFromTo(f->tensor, t->tensor, stream);
  });
}

int rafhip_raf_stream_create(int32_t device_type, int32_t device_id, void** stream_out) {
  return Guard([&] {
    if (!stream_out) throw Error("rafhip_raf_stream_create: stream_out is NULL");
    *stream_out = device_api::DeviceAPI::Get(DevType(device_type))
                      ->CreateStream(Device(DevType(device_type), device_id));
  });
}

int rafhip_raf_stream_free(int32_t device_type, int32_t device_id, void* stream) {
  return Guard([&] {
    device_api::DeviceAPI::Get(DevType(device_type))->FreeStream(Device(DevType(device_type), device_id), stream);
  });
}

int rafhip_raf_event_create(int32_t device_type, int32_t device_id, uint32_t flags, void** event_out) {
  return Guard([&] {
    if (!event_out) throw Error("rafhip_raf_event_create: event_out is NULL");
    *event_out = device_api::DeviceAPI::Get(DevType(device_type))
                     ->CreateEvent(Device(DevType(device_type), device_id), flags);
  });
}

int rafhip_raf_event_free(int32_t device_type, int32_t device_id, void* event) {
  return Guard([&] {
    device_api::DeviceAPI::Get(DevType(device_type))->FreeEvent(Device(DevType(device_type), device_id), event);
  });
}

int rafhip_raf_event_record(int32_t device_type, void* event, void* stream) {
  return Guard([&] { device_api::DeviceAPI::Get(DevType(device_type))->EventRecordOnStream(event, stream); });
}

int rafhip_raf_event_elapsed_ms(int32_t device_type, void* start_event, void* end_event, float* ms_out) {
  return Guard([&] {
    if (!ms_out) throw Error("rafhip_raf_event_elapsed_ms: ms_out is NULL");
    *ms_out = device_api::DeviceAPI::Get(DevType(device_type))
                  ->EventElapsedTimeInMilliSeconds(start_event, end_event);
  });
}

int rafhip_raf_stream_wait_event(int32_t device_type, void* stream, void* event) {
  return Guard([&] { device_api::DeviceAPI::Get(DevType(device_type))->StreamWaitEvent(stream, event); });
}

int rafhip_raf_wait(int32_t device_type, int32_t device_id, int32_t what, void* handle) {
  return Guard([&] {
    auto api = device_api::DeviceAPI::Get(DevType(device_type));
    switch (what) {
      case 0:
        api->WaitDevice(Device(DevType(device_type), device_id));
        break;
      case 1:
        api->WaitStream(handle);
        break;
      case 2:
        api->WaitEvent(handle);
        break;
      default:
        throw Error("rafhip_raf_wait: what must be 0 (device), 1 (stream) or 2 (event)");
    }
  });
}

int rafhip_raf_memory_alloc(int32_t device_type, int32_t device_id, int64_t nbytes, int64_t alignment,
                            int32_t stream_ordered, void* stream, rafhip_raf_memory** mem_out) {
  return Guard([&] {
    if (!mem_out) throw Error("rafhip_raf_memory_alloc: mem_out is NULL");
    *mem_out = nullptr;
    const Device dev(DevType(device_type), device_id);
    if (alignment <= 0) alignment = kDefaultMemoryAlignment;
    auto m = stream_ordered ? memory_pool::Memory::AllocAsync(dev, nbytes, stream, alignment)
                            : memory_pool::Memory::Alloc(dev, nbytes, alignment);
    *mem_out = new rafhip_raf_memory{std::move(m)};
  });
}

void* rafhip_raf_memory_data(const rafhip_raf_memory* mem) { return mem ? mem->mem->data : nullptr; }

int rafhip_raf_memory_free(rafhip_raf_memory* mem) {
  return Guard([&] { delete mem; });
}

int rafhip_raf_pool_init(int32_t device_type, int32_t device_id, const char* pool_name) {
  return Guard([&] {
    if (!pool_name) throw Error("rafhip_raf_pool_init: pool_name is NULL");
    memory_pool::InitPool(Device(DevType(device_type), device_id), pool_name);
  });
}

int rafhip_raf_pool_remove(int32_t device_type, int32_t device_id) {
  return Guard([&] { memory_pool::RemovePool(Device(DevType(device_type), device_id)); });
}

int rafhip_raf_pool_reset(int32_t device_type, int32_t device_id) {
  return Guard([&] { memory_pool::ResetPool(Device(DevType(device_type), device_id)); });
}

int rafhip_raf_pool_info(int32_t device_type, int32_t device_id, char* name_buf, int32_t buflen,
                         float* used_mb_out, float* pool_mb_out) {
  return Guard([&] {
    const Device dev(DevType(device_type), device_id);
    memory_pool::MemoryPool* pool = memory_pool::Memory::GetPool(dev);
    if (name_buf && buflen > 0) {
      std::strncpy(name_buf, pool->GetName().c_str(), (size_t)buflen - 1);
      name_buf[buflen - 1] = '\0';
    }
    if (used_mb_out || pool_mb_out) {
      auto sz = pool->GetPoolSize();
      if (used_mb_out) *used_mb_out = sz.first;
      if (pool_mb_out) *pool_mb_out = sz.second;
    }
  });
}

int64_t rafhip_raf_pool_alloc_bytes(int32_t device_type, int32_t device_id, int64_t nbytes) {
  int64_t r = -1;
  Guard([&] { r = memory_pool::Memory::GetAllocBytes(Device(DevType(device_type), device_id), nbytes); });
  return r;
}

int64_t rafhip_raf_env_workspace_bytes(const rafhip_raf_env* env) {
  if (!env) return -1;
  if (!env->graph_calls.empty()) {
    int64_t total = 0;
    for (const auto& gc : env->graph_calls)
      if (gc.env)
        for (const auto& r : gc.env->workspace_requests()) total += RoundUp(r.nbytes);
    return total;
  }
  if (!env->env) return 0;
  int64_t need = 0;
  for (const auto& r : env->env->workspace_requests()) need += RoundUp(r.nbytes);
  return need;
}

int rafhip_raf_traced_sgd_make(const rafhip_tensor_desc* w, const rafhip_tensor_desc* dx,
                               const rafhip_tensor_desc* v, double learning_rate, double momentum,
                               rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_traced_sgd_make: env_out is NULL");
    *env_out = nullptr;
    const rafhip_tensor_desc* descs[3] = {w, dx, v};
    const char* names[3] = {"w", "dx", "v"};
    std::unique_ptr<rafhip_raf_env> h(new rafhip_raf_env());
    std::map<const ir::ExprNode*, value::Value> bindings;
    for (int i = 0; i < 3; ++i) {
      value::TensorValue t = FromDesc(descs[i], names[i]);
      ir::TensorType ty;
      ty.defined = true;
      ty.shape = t->tensor.shape;
      ty.dtype = t->tensor.dtype;
      h->vars.push_back(ir::MakeVar(names[i], ty));
      bindings[h->vars.back().get()] = t;
    }
    const Device device = value::AsTensor(bindings[h->vars[0].get()])->tensor.device;
    h->traced = hip::TracedSgdUpdate(h->vars[0], h->vars[1], h->vars[2], learning_rate, momentum);
    h->fused = pass::FuseDialect(h->traced, device.device_type());
    const auto* call = ir::AsCall(h->fused);
    if (!call || !ir::AsFunction(call->op)) {
      // Nothing was fused; the element-wise base ops have no backend in this library.
      *env_out = h.release();
      throw Error("Cannot find a valid dispatch for op " + ir::AsOp(ir::AsCall((*env_out)->traced)->op)->name +
                  ": no fuse pattern matched on device type " + device.device_type().c_str());
    }
    h->call = BindCall(h->fused, bindings, device);
    h->env = Dispatch(h->call);
    h->name = h->env->name();
    h->op = "raf.op." + ir::AsFunction(call->op)->attrs.at(ir::kDialect) + "._fused_op";
    *env_out = h.release();
  });
}

int rafhip_raf_traced_sgd_execute(rafhip_raf_env* env, const rafhip_tensor_desc* w,
                                  const rafhip_tensor_desc* dx, const rafhip_tensor_desc* v,
                                  void* stream) {
  return Guard([&] {
    if (!env || !env->env || env->vars.size() != 3)
      throw Error("rafhip_raf_traced_sgd_execute: env was not made by rafhip_raf_traced_sgd_make");
    std::map<const ir::ExprNode*, value::Value> bindings;
    value::TensorValue wt = FromDesc(w, "w");
    bindings[env->vars[0].get()] = wt;
    bindings[env->vars[1].get()] = FromDesc(dx, "dx");
    bindings[env->vars[2].get()] = FromDesc(v, "v");
    CallValues call = BindCall(env->fused, bindings, env->call->device);
    call->out = wt;  // out=w: the result shares w's memory (src/op/declare/binary.cc:52-55)
    OpEnv::SetStreamForAllBackends(call->device, stream);
    WorkspaceBinding bind(env->env.get(), nullptr, 0);
    // the executors hand a fused function all of its arguments (arg_indices covers them all)
    env->env->Execute(call->args_as<schema::ListArgs>()->args, call->out);
  });
}

namespace {
// Binds the descriptor lists of a traced-optimizer call to the graph's variables (same order as at
// make time) and returns the bindings.
std::map<const ir::ExprNode*, value::Value> BindLists(const rafhip_raf_env* env, int32_t n,
                                                      const rafhip_tensor_desc* const* lists, int n_lists,
                                                      const rafhip_tensor_desc* step) {
  std::map<const ir::ExprNode*, value::Value> bindings;
  size_t next = 0;
  for (int l = 0; l < n_lists; ++l) {
    const size_t count = env->var_counts.at((size_t)l);
    if (count == 0) continue;
    RAF_CHECK(lists[l] != nullptr && (size_t)n == count, "a tensor list is missing or has another length than at make time");
    for (size_t i = 0; i < count; ++i) bindings[env->vars.at(next++).get()] = FromDesc(&lists[l][i], "tensor list");
  }
  if (env->var_counts.size() > (size_t)n_lists && env->var_counts[(size_t)n_lists] == 1) {
    RAF_CHECK(step != nullptr, "the step tensor is missing");
    bindings[env->vars.at(next++).get()] = FromDesc(step, "step");
  }
  return bindings;
}
}  // namespace

int rafhip_raf_traced_optimizer_make(int32_t kind, int32_t n, const rafhip_tensor_desc* g,
                                     const rafhip_tensor_desc* w, const rafhip_tensor_desc* m,
                                     const rafhip_tensor_desc* v, const rafhip_tensor_desc* p,
                                     const rafhip_tensor_desc* step, int32_t zero_is_constant,
                                     const double* hyper, int32_t n_hyper, int32_t allow_partial,
                                     rafhip_raf_env** env_out) {
  return Guard([&] {
    if (!env_out) throw Error("rafhip_raf_traced_optimizer_make: env_out is NULL");
    *env_out = nullptr;
    if (kind != 0 && kind != 1) throw Error("rafhip_raf_traced_optimizer_make: kind must be 0 (SGD) or 1 (LANS)");
    if (n <= 0 || !g || !w || !v) throw Error("rafhip_raf_traced_optimizer_make: bad tensor lists");
    if (kind == 1 && (!m || !p || !step)) throw Error("rafhip_raf_traced_optimizer_make: LANS needs m, p and step");
    if (!hyper || n_hyper != (kind == 0 ? 2 : 9))
      throw Error("rafhip_raf_traced_optimizer_make: SGD takes 2 hyper-parameters, LANS 9");
    std::unique_ptr<rafhip_raf_env> h(new rafhip_raf_env());
    h->kind = kind;
    const rafhip_tensor_desc* lists[5] = {g, w, kind == 1 ? m : nullptr, v, p};
    const char* names[5] = {"g", "w", "m", "v", "p"};
    std::vector<ir::Expr> vars[5];
    for (int l = 0; l < 5; ++l) {
      h->var_counts.push_back(lists[l] ? (size_t)n : 0);
      for (int32_t i = 0; lists[l] && i < n; ++i) {
        value::TensorValue t = FromDesc(&lists[l][i], names[l]);
        ir::TensorType ty;
        ty.defined = true;
        ty.shape = t->tensor.shape;
        ty.dtype = t->tensor.dtype;
        vars[l].push_back(ir::MakeVar(std::string(names[l]) + std::to_string(i), ty));
        h->vars.push_back(vars[l].back());
      }
    }
    const Device device = FromDesc(&w[0], "w")->tensor.device;
    ir::Expr zero;
    if (p) {
      ir::TensorType zt;
      zt.defined = true;
      zt.dtype = ir::TypeOf(vars[4][0]).dtype;
      // as traced the optimizer's zero tensor is one more input of the function; bound as a
      // constant it is a zeros constant (it then needs no storage: nothing is left to read it)
      zero = zero_is_constant ? ir::MakeZeros(zt) : ir::MakeVar("zero", zt);
    }
    if (kind == 0) {
      h->var_counts.push_back(0);
      h->traced = hip::TracedSgdOptimizer(vars[1], vars[0], vars[3], vars[4], zero, hyper[0], hyper[1]);
    } else {
      value::TensorValue st = FromDesc(step, "step");
      ir::TensorType sty;
      sty.defined = true;
      sty.shape = st->tensor.shape;
      sty.dtype = st->tensor.dtype;
      ir::Expr step_var = ir::MakeVar("step", sty);
      h->vars.push_back(step_var);
      h->var_counts.push_back(1);
      hip::LansHyper hy;
      hy.learning_rate = hyper[0];
      hy.beta1 = hyper[1];
      hy.beta2 = hyper[2];
      hy.eps = hyper[3];
      hy.bias_correction = (int)hyper[4];
      hy.weight_decay = hyper[5];
      hy.grad_averaging = (int)hyper[6];
      hy.mode = (int)hyper[7];
      hy.normalize_grad = (int)hyper[8];
      h->traced = hip::TracedLansOptimizer(vars[0], vars[1], vars[2], vars[3], vars[4], zero, step_var, hy);
    }
    h->fused = pass::FuseDialect(h->traced, device.device_type());
    h->call = std::make_shared<CallValuesNode>();
    h->call->device = device;
    h->op = kind == 0 ? "traced SGD optimizer" : "traced LANS optimizer";
    h->name = h->op;
    const rafhip_tensor_desc* all[5] = {g, w, kind == 1 ? m : nullptr, v, p};
    *env_out = h.get();  // kept on failure too: it still holds the graphs for rafhip_raf_env_ir_text
    rafhip_raf_env* raw = h.release();
    RunGraph(raw, BindLists(raw, n, all, 5, step), /*make=*/true, allow_partial != 0, nullptr, 0);
  });
}

int rafhip_raf_traced_optimizer_execute(rafhip_raf_env* env, int32_t n, const rafhip_tensor_desc* g,
                                        const rafhip_tensor_desc* w, const rafhip_tensor_desc* m,
                                        const rafhip_tensor_desc* v, const rafhip_tensor_desc* p,
                                        const rafhip_tensor_desc* step, int32_t allow_partial,
                                        void* workspace, int64_t workspace_bytes, void* stream) {
  return Guard([&] {
    if (!env || env->kind < 0) throw Error("rafhip_raf_traced_optimizer_execute: env was not made by rafhip_raf_traced_optimizer_make");
    const rafhip_tensor_desc* all[5] = {g, w, env->kind == 1 ? m : nullptr, v, p};
    auto bindings = BindLists(env, n, all, 5, step);
    OpEnv::SetStreamForAllBackends(env->call->device, stream);
    RunGraph(env, bindings, /*make=*/false, allow_partial != 0, workspace, workspace_bytes);
  });
}

int rafhip_raf_env_graph_ops(const rafhip_raf_env* env, char* buf, int32_t buflen) {
  return Guard([&] {
    if (!env || !buf || buflen <= 0) throw Error("rafhip_raf_env_graph_ops: bad arguments");
    std::string s;
    for (const auto& gc : env->graph_calls) s += (s.empty() ? "" : ";") + gc.what;
    if ((int64_t)s.size() >= (int64_t)buflen) throw Error("rafhip_raf_env_graph_ops: buffer too small");
    std::memcpy(buf, s.c_str(), s.size() + 1);
  });
}

int rafhip_raf_env_ir_text(const rafhip_raf_env* env, int32_t fused, char* buf, int32_t buflen) {
  return Guard([&] {
    if (!env || !buf || buflen <= 0) throw Error("rafhip_raf_env_ir_text: bad arguments");
    const ir::Expr& e = fused ? env->fused : env->traced;
    if (!e) throw Error("rafhip_raf_env_ir_text: env was not made from a graph");
    std::string s = ir::AsText(e);
    if ((int64_t)s.size() >= (int64_t)buflen) throw Error("rafhip_raf_env_ir_text: buffer too small");
    std::memcpy(buf, s.c_str(), s.size() + 1);
  });
}

int rafhip_raf_env_set_learning_rate(rafhip_raf_env* env, double learning_rate) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_env_set_learning_rate: env is NULL");
    if (!env->env) return;  // declared as a no-op: nothing to tell
    auto* target = dynamic_cast<hip::HasLearningRate*>(env->env.get());
    if (!target) throw Error("rafhip_raf_env_set_learning_rate: " + env->name + " has no learning rate");
    target->SetLearningRate(learning_rate);
  });
}

int rafhip_raf_env_set_grad_unscale(rafhip_raf_env* env, float factor) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_env_set_grad_unscale: env is NULL");
    if (!env->graph_calls.empty()) {  // a traced optimizer: every call of the graph that takes one
      for (auto& gc : env->graph_calls)
        if (auto* t = dynamic_cast<hip::HasGradScaling*>(gc.env.get())) t->SetGradUnscale(factor);
      return;
    }
    if (!env->env) return;  // declared as a no-op
    auto* target = dynamic_cast<hip::HasGradScaling*>(env->env.get());
    if (!target) throw Error("rafhip_raf_env_set_grad_unscale: " + env->name + " takes no gradient scale");
    target->SetGradUnscale(factor);
  });
}

int rafhip_raf_env_set_dynamic_scale(rafhip_raf_env* env, const rafhip_tensor_desc* grad_unscale,
                                     const rafhip_tensor_desc* found_inf) {
  return Guard([&] {
    if (!env) throw Error("rafhip_raf_env_set_dynamic_scale: env is NULL");
    const bool graph = !env->graph_calls.empty();
    if (!graph && !env->env) return;  // declared as a no-op
    auto* target = graph ? nullptr : dynamic_cast<hip::HasGradScaling*>(env->env.get());
    if (!graph && !target) throw Error("rafhip_raf_env_set_dynamic_scale: " + env->name + " takes no gradient scale");
    auto word = [&](const rafhip_tensor_desc* d, const char* what) -> const float* {
      if (!d) return nullptr;
      const TensorView t = FromDesc(d, what)->tensor;
      if (t.dtype.code != kDLFloat || t.dtype.bits != 32 || t.numel() != 1)
        throw Error(std::string(what) + " must be a one-element float32 tensor");
      if (t.device.device_type() != DevType::kROCM() || t.device.device_id() != env->call->device.device_id())
        throw Error(std::string(what) + " must live on the OpEnv's device");
      return static_cast<const float*>(t.data);
    };
    const float* unscale_word = word(grad_unscale, "grad_unscale");
    const float* found_inf_word = word(found_inf, "found_inf");
    if (graph) {
      for (auto& gc : env->graph_calls)
        if (auto* t = dynamic_cast<hip::HasGradScaling*>(gc.env.get())) t->SetDynamicScale(unscale_word, found_inf_word);
      return;
    }
    target->SetDynamicScale(unscale_word, found_inf_word);
  });
}

const char* rafhip_raf_env_name(const rafhip_raf_env* env) { return env ? env->name.c_str() : ""; }
const char* rafhip_raf_env_op(const rafhip_raf_env* env) { return env ? env->op.c_str() : ""; }

int rafhip_raf_env_destroy(rafhip_raf_env* env) {
  return Guard([&] { delete env; });
}

}  // extern "C"

// Registries, dispatch and the two optimizer declare functions behind raf_iface.h.
#include <algorithm>
#include <sstream>
#include <unordered_map>

#include "raf_iface.h"

namespace raf {

const char* DevType::c_str() const {
  switch (v_) {
    case 1:
      return "cpu";
    case 2:
      return "cuda";
    case 10:
      return "rocm";
    default:
      return "???";
  }
}

namespace value {

TensorValue MakeTensor(const TensorView& view) {
  auto t = std::make_shared<TensorValueObj>();
  t->tensor = view;
  return t;
}

TupleValue MakeTuple(std::vector<Value> fields) {
  auto t = std::make_shared<TupleValueObj>();
  t->fields = std::move(fields);
  return t;
}

TensorValue AsTensor(const Value& v) {
  auto t = std::dynamic_pointer_cast<TensorValueObj>(v);
  if (!t) throw Error("Downcast failed: value is not a TensorValue");
  return t;
}

TupleValue AsTuple(const Value& v) {
  auto t = std::dynamic_pointer_cast<TupleValueObj>(v);
  if (!t) throw Error("Downcast failed: value is not a TupleValue");
  return t;
}

}  // namespace value

namespace op {

// ------------------------------------------------------------------------------------- schemas
namespace schema {

static int IndexIn(const char* const* names, int n, const std::string& name) {
  for (int i = 0; i < n; ++i)
    if (name == names[i]) return i;
  throw Error("schema has no field named " + name);
}

int SgdArgs::FieldIndex(const std::string& name) const {
  static const char* const kNames[] = {"x", "dx", "v", "learning_rate", "mu"};
  return IndexIn(kNames, 5, name);
}

int LansArgs::FieldIndex(const std::string& name) const {
  static const char* const kNames[] = {"tensor_list", "step",   "learning_rate",   "beta1",
                                       "beta2",       "eps",    "bias_correction", "weight_decay",
                                       "grad_averaging", "mode", "normalize_grad"};
  return IndexIn(kNames, 11, name);
}

int SgdMultiArgs::FieldIndex(const std::string& name) const {
  static const char* const kNames[] = {"tensor_list", "learning_rate", "mu"};
  return IndexIn(kNames, 3, name);
}

int L2NormArgs::FieldIndex(const std::string& name) const {
  static const char* const kNames[] = {"x"};
  return IndexIn(kNames, 1, name);
}

int FuseTensorArgs::FieldIndex(const std::string& name) const {
  static const char* const kNames[] = {"data"};
  return IndexIn(kNames, 1, name);
}

int DefuseTensorArgs::FieldIndex(const std::string& name) const {
  static const char* const kNames[] = {"data", "sizes", "shapes", "shape_indices"};
  return IndexIn(kNames, 4, name);
}

}  // namespace schema

CallValues MakeCall(const std::string& op_name, std::shared_ptr<schema::ArgsBase> args) {
  auto call = std::make_shared<CallValuesNode>();
  call->callee = op_name;
  call->args = std::move(args);
  return call;
}

// ------------------------------------------------------------------------------------- declare
namespace {

// src/op/declare/optimizer.cc:22-44: x, dx, v agree in rank and shape; two fresh outputs (v1, x1)
// with dx's shape, dtype and device.
void SgdDecl(const CallValues& call) {
  const auto* args = call->args_as<schema::SgdArgs>();
  RAF_CHECK(args != nullptr, "raf.op.sgd expects SgdArgs");
  RAF_CHECK(args->x && args->dx && args->v, "raf.op.sgd: x, dx and v must be tensors");
  const TensorView& x0 = args->x->tensor;
  const TensorView& dx = args->dx->tensor;
  const TensorView& v0 = args->v->tensor;
  RAF_CHECK(x0.ndim() == dx.ndim(), "x and dx differ in rank");
  RAF_CHECK(v0.ndim() == dx.ndim(), "v and dx differ in rank");
  for (int i = 0; i < x0.ndim(); ++i) {
    RAF_CHECK(x0.shape[i] == dx.shape[i], "x and dx differ in shape");
    RAF_CHECK(v0.shape[i] == dx.shape[i], "v and dx differ in shape");
  }
  TensorView out;
  out.device = dx.device;
  out.dtype = dx.dtype;
  out.shape = dx.shape;  // data stays null until the executor allocates it
  call->out = value::MakeTuple({value::MakeTensor(out), value::MakeTensor(out)});
  call->device = dx.device;
}

// src/op/declare/optimizer.cc:46-58: 4n tensors; the output tuple is the input values themselves
// (the op updates them in place); device of the first tensor.
void LansDecl(const CallValues& call) {
  const auto* args = call->args_as<schema::LansArgs>();
  RAF_CHECK(args != nullptr, "raf.op.lans expects LansArgs");
  RAF_CHECK(args->tensor_list.size() % 4 == 0, "tensor_list must hold 4n tensors (g, w, m, v)");
  std::vector<value::Value> out;
  for (const auto& t : args->tensor_list) {
    RAF_CHECK(t != nullptr, "tensor_list holds a null tensor");
    out.push_back(t);
  }
  if (!args->tensor_list.empty()) call->device = args->tensor_list[0]->tensor.device;
  call->out = value::MakeTuple(std::move(out));
}

// Extension op raf.op.lans_mixed: LansArgs with a fifth block of tensors, the model's 16-bit
// parameters, that receive the narrowed new weights; declared like raf.op.lans (output = inputs).
void LansMixedDecl(const CallValues& call) {
  const auto* args = call->args_as<schema::LansArgs>();
  RAF_CHECK(args != nullptr, "raf.op.lans_mixed expects LansArgs");
  RAF_CHECK(args->tensor_list.size() % 5 == 0,
            "tensor_list must hold 5n tensors (g, w, m, v, p)");
  std::vector<value::Value> out;
  for (const auto& t : args->tensor_list) {
    RAF_CHECK(t != nullptr, "tensor_list holds a null tensor");
    out.push_back(t);
  }
  if (!args->tensor_list.empty()) call->device = args->tensor_list[0]->tensor.device;
  call->out = value::MakeTuple(std::move(out));
}

// Extension ops raf.op.sgd_multi (3n tensors: x, dx, v) and raf.op.sgd_multi_mixed (4n: and the
// 16-bit model parameters): in place like raf.op.lans, so the output tuple is the input values.
void SgdMultiDecl(const CallValues& call, size_t blocks) {
  const auto* args = call->args_as<schema::SgdMultiArgs>();
  RAF_CHECK(args != nullptr, "raf.op.sgd_multi expects SgdMultiArgs");
  RAF_CHECK(args->tensor_list.size() % blocks == 0,
            "tensor_list must hold " + std::to_string(blocks) + "n tensors");
  const size_t n = args->tensor_list.size() / blocks;
  std::vector<value::Value> out;
  for (const auto& t : args->tensor_list) {
    RAF_CHECK(t != nullptr, "tensor_list holds a null tensor");
    out.push_back(t);
  }
  for (size_t i = 0; i < n; ++i)  // x, dx, v (and p) of one parameter agree in shape
    for (size_t b = 1; b < blocks; ++b)
      RAF_CHECK(args->tensor_list[b * n + i]->tensor.shape == args->tensor_list[i]->tensor.shape,
                "tensors of one parameter differ in shape");
  if (!args->tensor_list.empty()) call->device = args->tensor_list[0]->tensor.device;
  call->out = value::MakeTuple(std::move(out));
}

// src/op/declare/reduce.cc:118-124: a 0-d output of x's dtype on x's device.
void L2NormDecl(const CallValues& call) {
  const auto* args = call->args_as<schema::L2NormArgs>();
  RAF_CHECK(args != nullptr && args->x, "raf.op.l2norm expects a tensor");
  TensorView out;
  out.device = args->x->tensor.device;
  out.dtype = args->x->tensor.dtype;
  call->out = value::MakeTensor(out);
  call->device = out.device;
}

// src/op/declare/memory.cc:43-63: a 1-d output with the total element count, dtype and device of
// the first tensor; an empty list has no output and no callee.
void FuseTensorDecl(const CallValues& call) {
  const auto* args = call->args_as<schema::FuseTensorArgs>();
  RAF_CHECK(args != nullptr, "raf.op.fuse_tensor expects FuseTensorArgs");
  if (args->data.empty()) {
    call->callee.clear();
    return;
  }
  int64_t total = 0;
  for (const auto& t : args->data) {
    RAF_CHECK(t != nullptr, "data holds a null tensor");
    total += t->tensor.numel();
  }
  const TensorView& x = args->data[0]->tensor;
  TensorView out;
  out.device = x.device;
  out.dtype = x.dtype;
  out.shape = {total};
  call->out = value::MakeTensor(out);
  call->device = x.device;
}

// src/op/declare/memory.cc:65-93: the sizes must add up to the input's element count; one output
// per entry of shape_indices, shaped by its slice of `shapes`.
void DefuseTensorDecl(const CallValues& call) {
  const auto* args = call->args_as<schema::DefuseTensorArgs>();
  RAF_CHECK(args != nullptr && args->data, "raf.op.defuse_tensor expects DefuseTensorArgs");
  const TensorView& x = args->data->tensor;
  call->device = x.device;
  int64_t total = 0;
  for (int64_t s : args->sizes) total += s;
  RAF_CHECK(total == x.numel(), "Input tensor size should be " + std::to_string(total) + ", got " +
                                    std::to_string(x.numel()) + ".");
  std::vector<value::Value> outs;
  int64_t start = 0;
  for (int64_t end : args->shape_indices) {
    RAF_CHECK(start <= end && end <= (int64_t)args->shapes.size(), "shape_indices out of range");
    TensorView t;
    t.device = x.device;
    t.dtype = x.dtype;
    t.shape.assign(args->shapes.begin() + start, args->shapes.begin() + end);
    outs.push_back(value::MakeTensor(t));
    start = end;
  }
  if (outs.empty()) {
    call->callee.clear();
    return;
  }
  call->out = value::MakeTuple(std::move(outs));
}

}  // namespace

void RunDeclare(const CallValues& call) {
  std::string op = call->callee;
  if (IsDialectOp(op)) op = GetBaseOp(op);
  if (op == "raf.op.sgd") return SgdDecl(call);
  if (op == "raf.op.lans") return LansDecl(call);
  if (op == "raf.op.lans_mixed") return LansMixedDecl(call);
  if (op == "raf.op.sgd_multi") return SgdMultiDecl(call, 3);
  if (op == "raf.op.sgd_multi_mixed") return SgdMultiDecl(call, 4);
  if (op == "raf.op.l2norm") return L2NormDecl(call);
  if (op == "raf.op.fuse_tensor") return FuseTensorDecl(call);
  if (op == "raf.op.defuse_tensor") return DefuseTensorDecl(call);
  throw Error("no declare function registered for op " + op);
}

// --------------------------------------------------------------------------------------- OpEnv
void OpEnv::RequestWorkspace(void** dest, const Device& device, int64_t nbytes) {
  workspace_.push_back(WorkspaceRequest{dest, device, nbytes});
}

void OpEnv::RequestStream(void** dest, const Device& device, int tag_idx) {  // src/impl/op.cc:66-72
  const int index = (int)stream_.size();
  stream_.push_back(StreamRequest{dest, device, tag_idx, index});
}

void OpEnv::SetStreamForAllBackends(Device device, void* stream) {
  device_api::DeviceAPI::Get(device.device_type())->SetStream(device, stream);  // src/impl/op.cc:92-96
}

// ------------------------------------------------------------------------------------ registries
namespace {

template <typename T>
struct NamedRegistry {
  std::mutex mu;
  std::map<std::string, std::unique_ptr<T>> items;
  T& get_or_add(const std::string& name) {
    std::lock_guard<std::mutex> lock(mu);
    auto& slot = items[name];
    if (!slot) slot.reset(new T());
    return *slot;
  }
  T* find(const std::string& name) {
    std::lock_guard<std::mutex> lock(mu);
    auto it = items.find(name);
    return it == items.end() ? nullptr : it->second.get();
  }
};

NamedRegistry<OpEnvMaker>& Makers() {
  static NamedRegistry<OpEnvMaker> r;
  return r;
}
NamedRegistry<Dialect>& Dialects() {
  static NamedRegistry<Dialect> r;
  return r;
}
NamedRegistry<OpDialect>& OpDialects() {
  static NamedRegistry<OpDialect> r;
  return r;
}

struct DialectOpAttrs {
  std::string dialect, base_op;
};
std::mutex& AttrMu() {
  static std::mutex m;
  return m;
}
std::map<std::string, DialectOpAttrs>& Attrs() {
  static std::map<std::string, DialectOpAttrs> m;
  return m;
}

thread_local const std::vector<std::string>* g_preference = nullptr;

}  // namespace

OpEnv* OpEnvMaker::operator()(const CallValues& call) const {
  RAF_CHECK(func_ != nullptr, "OpEnvMaker " + name + " has no function");
  return func_(call);
}
OpEnvMaker& OpEnvMaker::RegisterOrGet(const std::string& op_name) {
  return Makers().get_or_add(op_name);
}
const OpEnvMaker* OpEnvMaker::Get(const std::string& op_name) { return Makers().find(op_name); }

Dialect& Dialect::set_enable(DevType device_type) {
  enable_devices_.push_back((int)device_type);
  return *this;
}
bool Dialect::is_enabled(DevType device_type) const {
  return std::find(enable_devices_.begin(), enable_devices_.end(), (int)device_type) !=
         enable_devices_.end();
}
Dialect& Dialect::RegisterOrGet(const std::string& dialect_name) {
  return Dialects().get_or_add(dialect_name);
}
const Dialect* Dialect::Get(const std::string& dialect_name) {
  return Dialects().find(dialect_name);
}
bool Dialect::IsEnabled(const std::string& dialect, DevType device_type) {
  const Dialect* d = Get(dialect);
  RAF_CHECK(d != nullptr, "Dialect " + dialect + " is not registered.");
  return d->is_enabled(device_type);
}
std::vector<std::string> Dialect::GetEnabledDialects(DevType device_type) {
  std::vector<std::string> ret;
  auto& reg = Dialects();
  std::lock_guard<std::mutex> lock(reg.mu);
  for (auto& kv : reg.items)
    if (kv.second->is_enabled(device_type)) ret.push_back(kv.second->name);
  return ret;
}

OpDialect& OpDialect::add_dialect(const std::string& dialect_name, const std::string& dialect_op,
                                  int plevel) {
  std::lock_guard<std::mutex> lock(mu_);
  for (const auto& e : dialect_ops_) {
    if (e.dialect == dialect_name)
      throw Error("InternalError: base operator " + name +
                  " already has a registration on dialect " + dialect_name);
    if (e.plevel == plevel)
      throw Error("InternalError: base operator " + name +
                  " already has a registration on dialect " + e.dialect +
                  " with same plevel=" + std::to_string(plevel) + " as this dialect " +
                  dialect_name);
  }
  auto pos = std::find_if(dialect_ops_.begin(), dialect_ops_.end(),
                          [plevel](const DialectOpEntry& e) { return plevel > e.plevel; });
  dialect_ops_.insert(pos, DialectOpEntry{dialect_name, dialect_op, plevel});
  return *this;
}
OpDialect& OpDialect::RegisterOrGet(const std::string& base_op) {
  return OpDialects().get_or_add(base_op);
}

OpDialect::TDialectList OpDialect::GetDispatchList(const std::string& base_op,
                                                   DevType device_type) {
  OpDialect& od = OpDialects().get_or_add(base_op);
  TDialectList enabled;
  {
    std::lock_guard<std::mutex> lock(od.mu_);
    for (const auto& e : od.dialect_ops_) {
      const Dialect* d = Dialect::Get(e.dialect);
      RAF_CHECK(d != nullptr, "Dialect " + e.dialect + " is not registered.");
      if (d->is_enabled(device_type)) enabled.push_back(e);
    }
  }
  const std::vector<std::string>* pref = DialectPreference::Current();
  if (!pref) return enabled;
  TDialectList preferred;
  for (const auto& want : *pref)
    for (const auto& e : enabled)
      if (e.dialect == want) {
        preferred.push_back(e);
        break;
      }
  return preferred;
}

std::string OpDialect::Dispatch(const std::string& base_op, DevType device_type,
                                const std::vector<std::string>& skip_dialects) {
  for (const auto& e : GetDispatchList(base_op, device_type)) {
    if (e.plevel <= 0) continue;
    if (std::find(skip_dialects.begin(), skip_dialects.end(), e.dialect) != skip_dialects.end())
      continue;
    return e.dialect_op;
  }
  return "";
}

std::string OpDialect::Lower(const std::string& base_op, const std::string& dialect) {
  OpDialect& od = OpDialects().get_or_add(base_op);
  std::lock_guard<std::mutex> lock(od.mu_);
  for (const auto& e : od.dialect_ops_)
    if (e.dialect == dialect) return e.dialect_op;
  return "";
}

DialectPreference::DialectPreference(std::vector<std::string> dialects)
    : dialects_(std::move(dialects)), prev_(g_preference) {
  g_preference = &dialects_;
}
DialectPreference::~DialectPreference() { g_preference = prev_; }
const std::vector<std::string>* DialectPreference::Current() { return g_preference; }

void RegisterDialectOpAttrs(const std::string& dialect_op, const std::string& dialect,
                            const std::string& base_op) {
  std::lock_guard<std::mutex> lock(AttrMu());
  Attrs()[dialect_op] = DialectOpAttrs{dialect, base_op};
}
bool IsDialectOp(const std::string& op) {
  std::lock_guard<std::mutex> lock(AttrMu());
  return Attrs().count(op) != 0;
}
std::string GetDialect(const std::string& op) {
  std::lock_guard<std::mutex> lock(AttrMu());
  auto it = Attrs().find(op);
  RAF_CHECK(it != Attrs().end(), op + " is not a dialect op");
  return it->second.dialect;
}
std::string GetBaseOp(const std::string& op) {
  std::lock_guard<std::mutex> lock(AttrMu());
  auto it = Attrs().find(op);
  RAF_CHECK(it != Attrs().end(), op + " is not a dialect op");
  return it->second.base_op;
}

// ------------------------------------------------------------------------------------- dispatch
OpEnvPtr DispatchSingleOp(const CallValues& call, std::string* picked_op) {
  std::vector<std::string> errors;
  auto try_maker = [&](const std::string& op_name) -> OpEnvPtr {
    const OpEnvMaker* maker = OpEnvMaker::Get(op_name);
    if (!maker) return nullptr;
    OpEnvPtr env((*maker)(call));
    if (env && !env->HasError()) {
      if (picked_op) *picked_op = op_name;
      return env;
    }
    if (env) errors.insert(errors.end(), env->error_msgs.begin(), env->error_msgs.end());
    return nullptr;
  };

  std::string op = call->callee;
  if (OpEnvPtr env = try_maker(op)) return env;
  std::string skip_dialect;
  if (IsDialectOp(op)) {  // a dialect op that refused: fall back to its base op's other dialects
    skip_dialect = GetDialect(op);
    op = GetBaseOp(op);
  }
  for (const auto& entry : OpDialect::GetDispatchList(op, call->device.device_type())) {
    if (entry.dialect == skip_dialect) continue;
    if (OpEnvPtr env = try_maker(entry.dialect_op)) return env;
  }
  std::ostringstream ss;
  ss << "Cannot find a valid dispatch for op " << op << ":";
  for (const auto& m : errors) ss << "\n" << m;
  throw Error(ss.str());
}

std::string GetUniqueName(std::string name) {
  static std::mutex mu;
  static std::unordered_map<std::string, int> seen;
  std::replace(name.begin(), name.end(), '.', '_');
  std::lock_guard<std::mutex> lock(mu);
  for (;;) {
    auto it = seen.find(name);
    if (it == seen.end()) {
      seen[name] = 1;
      return name;
    }
    name += "_" + std::to_string(it->second++);
  }
}

std::string TruncateName(std::string name) {
  constexpr size_t kMax = 80;
  if (name.size() > kMax)
    name = name.substr(0, kMax) + "_" + std::to_string(std::hash<std::string>{}(name)) + "_";
  return name;
}

}  // namespace op
}  // namespace raf

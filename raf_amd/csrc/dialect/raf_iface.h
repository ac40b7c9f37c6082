// A self-contained restatement of the slice of RAF's C++ interface that a dialect backend sees:
// values, the two optimizer schemas, CallValues, OpEnv / OpEnvMaker, the Dialect and OpDialect
// registries, single-op dispatch, and the device API's "current stream".  RAF itself cannot be
// built here (it sits on TVM, an empty submodule), so the `hip` dialect in hip_dialect.cc is
// compiled and tested against this header; names, argument meaning and error behaviour follow
// the reference so that the same dialect source registers into the real RAF by swapping includes.
//
// What each piece mirrors in the reference tree:
//   DevType / Device ........ include/raf/device.h:37-75 (kCPU = 1, kCUDA = 2, kROCM = 10)
//   CallValues .............. include/raf/op.h:35-57
//   OpEnv ................... include/raf/op.h:59-101 (+ RequestWorkspace, src/impl/op.cc:58-64)
//   OpEnvMaker .............. include/raf/op.h:105-145
//   Dialect, OpDialect ...... include/raf/dialect.h:60-169, src/impl/dialect.cc:56-202
//   DispatchSingleOp ........ src/impl/op.cc:127-180
//   GetUniqueName/Truncate .. src/impl/op.cc:263-290
//   schemas ................. scripts/src_codegen/def_schema.py:671-694
//   declare ................. src/op/declare/optimizer.cc:22-62
//   registration macros ..... include/raf/dialect.h:231-243, include/raf/op.h:331-334
//   DeviceAPI ............... include/raf/device_api.h:19-177, src/impl/device_api.cc:18-50
// Failures that the reference raises through CHECK / LOG(FATAL) (a dmlc::Error) are raf::Error here.
#pragma once

#include <cstdint>
#include <functional>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace raf {

namespace ir {
struct ExprNode;  // raf_ir.h
}

class Error : public std::runtime_error {
 public:
  explicit Error(const std::string& what) : std::runtime_error(what) {}
};

#define RAF_CHECK(cond, msg)                                                         \
  do {                                                                               \
    if (!(cond)) throw ::raf::Error(std::string("Check failed: " #cond ": ") + (msg)); \
  } while (0)

// ------------------------------------------------------------------------------------- devices
class DevType {
 public:
  constexpr DevType() : v_(0) {}
  constexpr explicit DevType(int v) : v_(v) {}
  static constexpr DevType kUnknown() { return DevType(0); }
  static constexpr DevType kCPU() { return DevType(1); }
  static constexpr DevType kCUDA() { return DevType(2); }
  static constexpr DevType kROCM() { return DevType(10); }
  constexpr operator int() const { return v_; }
  const char* c_str() const;

 private:
  int v_;
};

struct Device {
  DevType device_type_{};
  int device_id_ = -1;
  Device() = default;
  Device(DevType t, int id) : device_type_(t), device_id_(id) {}
  DevType device_type() const { return device_type_; }
  int device_id() const { return device_id_; }
};

// DLPack-style dtype codes (kDLInt = 0, kDLUInt = 1, kDLFloat = 2, kDLBfloat = 4).
constexpr int kDLFloat = 2;
constexpr int kDLBfloat = 4;
struct DType {
  int code = kDLFloat;
  int bits = 32;
};

// The fields of a DLTensor that the optimizer ops look at; `data` is not owned.
struct TensorView {
  void* data = nullptr;
  Device device;
  DType dtype;
  std::vector<int64_t> shape;
  int ndim() const { return (int)shape.size(); }
  int64_t numel() const {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
  }
};

// -------------------------------------------------------------------------------------- values
namespace value {

struct ValueObj {
  virtual ~ValueObj() = default;
};
using Value = std::shared_ptr<ValueObj>;

struct TensorValueObj : ValueObj {
  TensorView tensor;
};
using TensorValue = std::shared_ptr<TensorValueObj>;

struct TupleValueObj : ValueObj {
  std::vector<Value> fields;
};
using TupleValue = std::shared_ptr<TupleValueObj>;

TensorValue MakeTensor(const TensorView& view);
TupleValue MakeTuple(std::vector<Value> fields);
// Downcasts that raise raf::Error on a kind mismatch, like ir::Downcast.
TensorValue AsTensor(const Value& v);
TupleValue AsTuple(const Value& v);

}  // namespace value

// -------------------------------------------------------------------------------------- device api
// include/raf/device.h:24 takes this from TVM's runtime (kAllocAlignment); 64 in the TVM
// generation the reference was written against.
constexpr int64_t kDefaultMemoryAlignment = 64;

namespace device_api {

// The reference's unified low-level device interface, include/raf/device_api.h:19-177, method for
// method.  Implementations register a maker under the device type's name (the reference's
// "raf.device_api._make.<devtype>" global, src/impl/device_api.cc:26-31) and Get creates one
// instance per device type on first use (:37-47).
class DeviceAPI {
 public:
  virtual ~DeviceAPI() = default;
  virtual int GetDeviceCount() = 0;
  virtual void* AllocMemory(int64_t nbytes, int64_t alignment) = 0;
  virtual void* AllocMemoryAsync(int64_t nbytes, void* stream, int64_t alignment) = 0;
  virtual void FreeMemory(void* ptr) = 0;
  virtual void FreeMemoryAsync(void* ptr, void* stream) = 0;
  // Contiguous tensors of equal byte size; `stream` may be null (synchronous copy).
  virtual void CopyDataFromTo(const TensorView& from, const TensorView& to, void* stream = nullptr) = 0;
  // <bytes handed to users, bytes taken from the system> of the device's own pool, if it has one.
  virtual std::pair<int64_t, int64_t> GetPoolSize() { return std::make_pair(0, 0); }
  virtual void SetDevice(const int device_id) = 0;
  virtual void* CreateStream(const Device& dev) = 0;
  virtual void FreeStream(const Device& dev, void* stream) = 0;
  virtual void SetStream(const Device& dev, void* stream) = 0;
  virtual void* GetStream() = 0;
  virtual void* CreateEvent(const Device& dev, uint32_t flags = 0) = 0;
  virtual void FreeEvent(const Device& dev, void* event) = 0;
  virtual float EventElapsedTimeInMilliSeconds(void* start_event, void* end_event) = 0;
  virtual void EventRecordOnStream(void* event, void* stream) = 0;
  virtual void StreamWaitEvent(void* stream, void* event) = 0;
  virtual void WaitDevice(const Device& dev) = 0;
  virtual void WaitStream(void* stream) = 0;
  virtual void WaitEvent(void* event) = 0;

  // Raises raf::Error if no maker is registered for the device type.
  static std::shared_ptr<DeviceAPI> Get(DevType device_type);
  using Maker = DeviceAPI* (*)();
  static bool RegisterMaker(const std::string& devtype_name, Maker maker);
};

}  // namespace device_api

namespace op {

// ------------------------------------------------------------------------------------- schemas
namespace schema {

struct ArgsBase {
  virtual ~ArgsBase() = default;
  // Field name -> position, the FRAFSchemaFieldIndex attribute of the reference.
  virtual int FieldIndex(const std::string& name) const = 0;
};

struct SgdArgs : ArgsBase {  // def_schema.py:671-677
  value::TensorValue x, dx, v;
  double learning_rate = 0.0;
  double mu = 0.0;
  int FieldIndex(const std::string& name) const override;
};

struct LansArgs : ArgsBase {  // def_schema.py:678-694
  std::vector<value::TensorValue> tensor_list;
  value::TensorValue step;
  float learning_rate = 0.f, beta1 = 0.f, beta2 = 0.f, eps = 0.f;
  int bias_correction = 0;
  float weight_decay = 0.f;
  int grad_averaging = 0;
  int mode = 0;
  bool normalize_grad = false;
  int FieldIndex(const std::string& name) const override;
};

// Extension ops raf.op.sgd_multi / raf.op.sgd_multi_mixed: momentum SGD over a parameter list in
// place.  tensor_list = [x..., dx..., v...] (+ [p...], the model's 16-bit parameters, for _mixed).
struct SgdMultiArgs : ArgsBase {
  std::vector<value::TensorValue> tensor_list;
  double learning_rate = 0.0;
  double mu = 0.0;
  int FieldIndex(const std::string& name) const override;
};

struct L2NormArgs : ArgsBase {  // def_schema.py:425-427
  value::TensorValue x;
  int FieldIndex(const std::string& name) const override;
};

struct FuseTensorArgs : ArgsBase {  // def_schema.py:829-835
  std::vector<value::TensorValue> data;
  int FieldIndex(const std::string& name) const override;
};

struct DefuseTensorArgs : ArgsBase {  // def_schema.py:836-841
  value::TensorValue data;
  std::vector<int64_t> sizes;          // element count of every output
  std::vector<int64_t> shapes;         // all outputs' dimensions, concatenated
  std::vector<int64_t> shape_indices;  // end of every output's dimensions in `shapes`
  int FieldIndex(const std::string& name) const override;
};

}  // namespace schema

// ---------------------------------------------------------------------------------- CallValues
struct CallValuesNode {
  std::string callee;  // operator name, e.g. "raf.op.lans" or "raf.op.hip.lans"
  // Set instead of `callee` when a fused (primitive) function is called: the reference's
  // ClosureValue callee (src/impl/op.cc:182-185).  `args` is then a schema::ListArgs.
  std::shared_ptr<const ir::ExprNode> closure;
  std::shared_ptr<schema::ArgsBase> args;
  value::Value out;
  Device device;
  template <typename T>
  const T* args_as() const {
    return dynamic_cast<const T*>(args.get());
  }
};
using CallValues = std::shared_ptr<CallValuesNode>;
CallValues MakeCall(const std::string& op_name, std::shared_ptr<schema::ArgsBase> args);

// Runs the operator's declare function: checks the arguments, fills call->out and call->device.
void RunDeclare(const CallValues& call);

// --------------------------------------------------------------------------------------- OpEnv
struct WorkspaceRequest {
  void** dest;
  Device device;
  int64_t nbytes;
};

// include/raf/stream_pool.h:52-76: what a requested stream is for.  The copy tags are the ones
// the fuse / defuse OpEnvs ask for (src/op/dialect/cuda/memory.cc:34, :89).
namespace stream_pool {
enum StreamTag : int {
  kUnknown = 0,
  kCudaCompute = 1,
  kMemCpyCpuToCuda = 2,
  kMemCpyCudaToCpu = 3,
  kCudaCommunicate = 4,
  kMemCpyCudaToCuda1 = 5,
  kMemCpyCudaToCuda2 = 6,
};
}  // namespace stream_pool

struct StreamRequest {  // requests::Requests::StreamRequest (src/requests.h)
  void** dest;
  Device device;
  int tag_idx;
  int stream_idx;
};

class OpEnv {
 public:
  OpEnv() = default;
  virtual ~OpEnv() = default;
  virtual std::string name() const = 0;
  virtual void Execute(const CallValues& call) = 0;
  virtual void Execute(const std::vector<value::Value>& inputs, value::Value output) = 0;

  std::vector<std::string> error_msgs;
  bool HasError() { return !error_msgs.empty(); }

  // Recorded at construction; the executor points *dest at nbytes of device memory before every
  // Execute and may take it back afterwards.
  void RequestWorkspace(void** dest, const Device& device, int64_t nbytes);
  const std::vector<WorkspaceRequest>& workspace_requests() const { return workspace_; }
  // Also recorded at construction; the executor points *dest at a stream of its pool for
  // (device, tag_idx) before Execute (src/impl/interpreter.cc:384-389, src/impl/vm/vm.cc:1082-1091).
  void RequestStream(void** dest, const Device& device, int tag_idx);
  const std::vector<StreamRequest>& stream_requests() const { return stream_; }

  std::vector<int> arg_indices;  // schema fields handed to Execute(inputs, output) by the VM

  static void SetStreamForAllBackends(Device device, void* stream);

 private:
  std::vector<WorkspaceRequest> workspace_;
  std::vector<StreamRequest> stream_;
};
using OpEnvPtr = std::shared_ptr<OpEnv>;

class OpEnvMaker {
 public:
  using FMakeOpEnv = std::function<OpEnv*(const CallValues& call)>;
  OpEnvMaker& set_name(const std::string& n) {
    name = n;
    return *this;
  }
  OpEnvMaker& set_func(FMakeOpEnv f) {
    func_ = std::move(f);
    return *this;
  }
  OpEnv* operator()(const CallValues& call) const;
  static OpEnvMaker& RegisterOrGet(const std::string& op_name);
  static const OpEnvMaker* Get(const std::string& op_name);  // nullptr if none
  std::string name;

 private:
  FMakeOpEnv func_;
};

// ------------------------------------------------------------------------------------ dialects
class Dialect {
 public:
  Dialect& set_name(const std::string& n) {
    name = n;
    return *this;
  }
  Dialect& set_enable(DevType device_type);
  bool is_enabled(DevType device_type) const;
  static Dialect& RegisterOrGet(const std::string& dialect_name);
  static const Dialect* Get(const std::string& dialect_name);  // nullptr if unknown
  static bool IsEnabled(const std::string& dialect, DevType device_type);
  static std::vector<std::string> GetEnabledDialects(DevType device_type);
  std::string name;

 private:
  std::vector<int> enable_devices_;
};

struct DialectOpEntry {
  std::string dialect;
  std::string dialect_op;
  int plevel;
};

class OpDialect {
 public:
  using TDialectList = std::list<DialectOpEntry>;
  OpDialect& set_name(const std::string& n) {
    name = n;
    return *this;
  }
  // Keeps the list sorted by descending plevel; a second registration of the same dialect, or of
  // the same plevel, on one base op is an error.
  OpDialect& add_dialect(const std::string& dialect_name, const std::string& dialect_op,
                         int plevel = 10);
  static OpDialect& RegisterOrGet(const std::string& base_op);
  static TDialectList GetDispatchList(const std::string& base_op, DevType device_type);
  // Highest-plevel enabled dialect op, skipping `skip_dialects`; "" if none.
  static std::string Dispatch(const std::string& base_op, DevType device_type,
                              const std::vector<std::string>& skip_dialects = {});
  // The op that `dialect` registered for `base_op`, whatever the device; "" if none
  // (src/impl/dialect.cc:204-214).
  static std::string Lower(const std::string& base_op, const std::string& dialect);
  std::string name;

 private:
  TDialectList dialect_ops_;
  std::mutex mu_;
};

// A scoped, thread-local preference list (the `with_dialect` of the reference's tests,
// include/raf/dialect.h:29-58): while alive, GetDispatchList only returns these dialects, in
// this order.
class DialectPreference {
 public:
  explicit DialectPreference(std::vector<std::string> dialects);
  ~DialectPreference();
  static const std::vector<std::string>* Current();

 private:
  std::vector<std::string> dialects_;
  const std::vector<std::string>* prev_;
};

// Records which base op / dialect a dialect op belongs to (TRAFBaseOp / TRAFDialect attributes).
void RegisterDialectOpAttrs(const std::string& dialect_op, const std::string& dialect,
                            const std::string& base_op);
bool IsDialectOp(const std::string& op);
std::string GetDialect(const std::string& op);
std::string GetBaseOp(const std::string& op);

// Tries the op's own maker, then every enabled dialect op in plevel order; an OpEnv that comes
// back with error_msgs is skipped.  Raises raf::Error listing the collected messages when nothing
// fits ("Cannot find a valid dispatch for op ...").  *picked_op, if given, receives the name of
// the op whose maker produced the OpEnv.
OpEnvPtr DispatchSingleOp(const CallValues& call, std::string* picked_op = nullptr);

std::string GetUniqueName(std::string name);
std::string TruncateName(std::string name);

}  // namespace op
}  // namespace raf

// ------------------------------------------------------------------------- registration macros
#define RAF_IFACE_CAT_(a, b) a##b
#define RAF_IFACE_CAT(a, b) RAF_IFACE_CAT_(a, b)
#define RAF_IFACE_STR_(s) #s

#define RAF_BASE_OP_NAME(NAME) RAF_IFACE_STR_(raf.op.NAME)
#define RAF_DIALECT_OP_NAME(DIALECT, NAME) RAF_IFACE_STR_(raf.op.DIALECT.NAME)

#define RAF_REGISTER_DIALECT(DIALECT_NAME)                                          \
  static __attribute__((unused))::raf::op::Dialect& RAF_IFACE_CAT(_raf_dialect_def_, __COUNTER__) = \
      ::raf::op::Dialect::RegisterOrGet(DIALECT_NAME).set_name(DIALECT_NAME)

namespace raf {
namespace op {
inline OpDialect& RegisterDialectOp_(const char* dialect, const char* base_op,
                                     const char* dialect_op, int plevel) {
  RegisterDialectOpAttrs(dialect_op, dialect, base_op);
  return OpDialect::RegisterOrGet(base_op).set_name(base_op).add_dialect(dialect, dialect_op,
                                                                         plevel);
}
}  // namespace op
}  // namespace raf

#define RAF_REGISTER_DIALECT_OP(DIALECT, OP, PLEVEL)                                               \
  static __attribute__((unused))::raf::op::OpDialect& RAF_IFACE_CAT(_raf_op_dialect_def_, __COUNTER__) = \
      ::raf::op::RegisterDialectOp_(#DIALECT, RAF_BASE_OP_NAME(OP),                                \
                                    RAF_DIALECT_OP_NAME(DIALECT, OP), PLEVEL)

#define RAF_OP_ENV_MAKER(OP_NAME, FOP_ENV_MAKER)                                                  \
  static __attribute__((unused))::raf::op::OpEnvMaker& RAF_IFACE_CAT(_raf_op_env_maker_def_, __COUNTER__) = \
      ::raf::op::OpEnvMaker::RegisterOrGet(OP_NAME).set_name(OP_NAME).set_func(FOP_ENV_MAKER)

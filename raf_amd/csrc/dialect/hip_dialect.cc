// The `hip` dialect: OpEnv backends of raf.op.sgd and raf.op.lans for ROCm devices, written
// against the OpEnv / dialect-op registration interface (raf_iface.h mirrors it) and calling the
// gfx950 kernels through the C ABI of rafhip_optim.h only.
//
// Counterparts in the reference tree:
//   LansHipEnv   LansImpl, src/op/dialect/cuda/lans.cc:25-165 (registration :164-165)
//   L2NormHipEnv       L2NormImpl, src/op/dialect/cublas/l2_norm.cc:26-86
//   FuseTensorHipEnv   CudaFuseTensor, src/op/dialect/cuda/memory.cc:27-77
//   DefuseTensorHipEnv CudaDefuseTensor, src/op/dialect/cuda/memory.cc:82-143
//   SgdHipEnv    the RAF_TVM(sgd, ...) backend, src/op/dialect/tvm/optimizer.cc:22-45, whose
//                Execute packs [x, dx, v, v1, x1] (src/op/dialect/tvm/tvm_utils.cc:92-133)
// Differences on purpose: the stream is looked up at Execute time (the reference caches it in the
// constructor, lans.cc:79-80); `step` stays on the device (the reference copies it to the host
// and blocks, lans.cc:94-99); a single workspace holds partial sums and norms and there is no
// per-element scratch (lans.cc:66); element counts are 64-bit (lans.cc:57 uses int); unsupported
// arguments are reported through error_msgs so dispatch can fall through to another dialect.
#include "hip_dialect.h"

#include <cstring>
#include <sstream>
#include <typeinfo>

#include "raf_iface.h"
#include "rafhip_optim.h"

namespace raf {
namespace op {
namespace hip {

using device_api::DeviceAPI;
using value::AsTensor;
using value::AsTuple;
using value::Value;

namespace {

std::string KernelError(const char* what, int status) {
  std::ostringstream ss;
  ss << what << " failed with status " << status << ": " << rafhip_last_error();
  return ss.str();
}

bool IsF32(const DType& t) { return t.code == kDLFloat && t.bits == 32; }
bool IsF16(const DType& t) { return t.code == kDLFloat && t.bits == 16; }
bool IsBF16(const DType& t) { return t.code == kDLBfloat && t.bits == 16; }
int32_t KernelDType(const DType& t) {
  return IsF32(t) ? RAFHIP_F32 : IsF16(t) ? RAFHIP_F16 : IsBF16(t) ? RAFHIP_BF16 : -1;
}

// The data pointers of a tuple's tensor fields into out[fields.size()].  This runs for every field
// at every Execute, so it costs one type comparison and one pointer read per field: no reference
// counting, and the exact-type test first (inside RAF the downcast is a type-index comparison,
// `field.as<TensorValueObj>()`); only a subclass would take the dynamic_cast.
void CollectDataPointers(const std::vector<Value>& fields, void** out, const std::string& op) {
  for (size_t i = 0; i < fields.size(); ++i) {
    const value::ValueObj* f = fields[i].get();
    const value::TensorValueObj* t = nullptr;
    if (f != nullptr)
      t = typeid(*f) == typeid(value::TensorValueObj) ? static_cast<const value::TensorValueObj*>(f)
                                                      : dynamic_cast<const value::TensorValueObj*>(f);
    if (!t) throw Error(op + ": field " + std::to_string(i) + " of tensor_list is not a tensor");
    out[i] = t->tensor.data;
  }
}

}  // namespace

// ----------------------------------------------------------------------------------------- SGD
class SgdHipEnv : public OpEnv, public HasLearningRate {
 public:
  explicit SgdHipEnv(const CallValues& cv) {
    const auto* args = cv->args_as<schema::SgdArgs>();
    if (!args) {
      error_msgs.push_back("raf.op.hip.sgd: call does not carry SgdArgs");
      return;
    }
    // The VM passes the tensor fields as `inputs` (optimizer.cc:26-28 lists x, dx, v).
    arg_indices = {args->FieldIndex("x"), args->FieldIndex("dx"), args->FieldIndex("v")};
    learning_rate_ = args->learning_rate;
    mu_ = args->mu;
    const TensorView& x = args->x->tensor;
    if (cv->device.device_type() != DevType::kROCM())
      error_msgs.push_back("raf.op.hip.sgd: device is not rocm");
    // The reference's compute is written in x's dtype (python/raf/_tvm_op/sgd.py:18-19): all three
    // tensors share one floating-point type.
    dtype_ = IsF32(x.dtype) ? RAFHIP_F32 : IsF16(x.dtype) ? RAFHIP_F16 : IsBF16(x.dtype) ? RAFHIP_BF16
             : (x.dtype.code == kDLFloat && x.dtype.bits == 64) ? RAFHIP_F64 : -1;
    auto same = [&](const DType& t) { return t.code == x.dtype.code && t.bits == x.dtype.bits; };
    if (dtype_ < 0 || !same(args->dx->tensor.dtype) || !same(args->v->tensor.dtype))
      error_msgs.push_back("raf.op.hip.sgd: x, dx and v must share one of float32, float64, float16, bfloat16");
    if (error_msgs.empty() && rafhip_device_count() <= 0)
      error_msgs.push_back("raf.op.hip.sgd: no HIP device is visible");
  }

  std::string name() const override { return name_; }

  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::SgdArgs>();
    RAF_CHECK(args != nullptr, "raf.op.hip.sgd expects SgdArgs");
    Execute(std::vector<Value>{args->x, args->dx, args->v}, cv->out);
  }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    RAF_CHECK(inputs.size() == 3, "raf.op.hip.sgd takes x, dx, v");
    const TensorView& x = AsTensor(inputs[0])->tensor;
    const TensorView& dx = AsTensor(inputs[1])->tensor;
    const TensorView& v = AsTensor(inputs[2])->tensor;
    auto out = AsTuple(output);
    RAF_CHECK(out->fields.size() == 2, "raf.op.hip.sgd produces (v1, x1)");
    const TensorView& v1 = AsTensor(out->fields[0])->tensor;  // declare/optimizer.cc:42: (v1, x1)
    const TensorView& x1 = AsTensor(out->fields[1])->tensor;
    const int64_t n = dx.numel();
    RAF_CHECK(x.numel() == n && v.numel() == n && v1.numel() == n && x1.numel() == n,
              "raf.op.hip.sgd: tensor sizes differ");
    void* stream = DeviceAPI::Get(DevType::kROCM())->GetStream();
    int st = rafhip_sgd(x.data, dx.data, v.data, v1.data, x1.data, n, dtype_, learning_rate_, mu_, stream);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_sgd", st));
  }

  void SetLearningRate(double learning_rate) override { learning_rate_ = learning_rate; }
  double GetLearningRate() const override { return learning_rate_; }

  static OpEnv* make(const CallValues& cv) { return new SgdHipEnv(cv); }

 private:
  double learning_rate_ = 0.0;
  double mu_ = 0.0;
  int32_t dtype_ = RAFHIP_F32;
  std::string name_ = TruncateName(GetUniqueName("raf.op.hip.sgd"));
};

// ---------------------------------------------------------------------- multi-tensor SGD
// Extension ops raf.op.sgd_multi / raf.op.sgd_multi_mixed: what the reference's traced optimizer
// emits per parameter as cast, multiply, add(out=), multiply, subtract(out=), cast, add(out=)
// (python/raf/optim/sgd.py:187-215), as one in-place launch over the whole list.
class SgdMultiHipEnv : public OpEnv, public HasLearningRate {
 public:
  SgdMultiHipEnv(const CallValues& cv, bool mixed)
      : blocks_(mixed ? 4 : 3),
        op_(mixed ? "raf.op.hip.sgd_multi_mixed" : "raf.op.hip.sgd_multi"),
        name_(TruncateName(GetUniqueName(op_))) {
    const auto* args = cv->args_as<schema::SgdMultiArgs>();
    if (!args) {
      error_msgs.push_back(op_ + ": call does not carry SgdMultiArgs");
      return;
    }
    arg_indices = {args->FieldIndex("tensor_list")};
    learning_rate_ = args->learning_rate;
    mu_ = args->mu;
    const size_t total = args->tensor_list.size();
    if (total % (size_t)blocks_ != 0) {
      error_msgs.push_back(op_ + ": tensor_list must hold " + std::to_string(blocks_) + "n tensors");
      return;
    }
    n_ = (int32_t)(total / (size_t)blocks_);
    if (cv->device.device_type() != DevType::kROCM()) error_msgs.push_back(op_ + ": device is not rocm");
    int32_t grad_dtype = RAFHIP_F32;
    std::vector<int64_t> numels;
    for (int32_t i = 0; i < n_ && error_msgs.empty(); ++i) {
      const TensorView& x = args->tensor_list[i]->tensor;
      const TensorView& dx = args->tensor_list[n_ + i]->tensor;
      const TensorView& v = args->tensor_list[2 * n_ + i]->tensor;
      if (!IsF32(x.dtype) || !IsF32(v.dtype))
        error_msgs.push_back(op_ + ": weights and velocities must be float32");
      const int32_t gd = KernelDType(dx.dtype);
      if (gd < 0 || (i > 0 && gd != grad_dtype))
        error_msgs.push_back(op_ + ": gradients must all be float32, all float16 or all bfloat16");
      grad_dtype = gd;
      if (blocks_ == 4) {
        const int32_t pd = KernelDType(args->tensor_list[3 * n_ + i]->tensor.dtype);
        if (pd != RAFHIP_F16 && pd != RAFHIP_BF16)
          error_msgs.push_back(op_ + ": model parameters must be float16 or bfloat16");
        else if (i > 0 && pd != copy_dtype_)
          error_msgs.push_back(op_ + ": model parameters must share one dtype");
        copy_dtype_ = pd;
      }
      numels.push_back(x.numel());
    }
    if (!error_msgs.empty()) return;
    if (rafhip_device_count() <= 0) {
      error_msgs.push_back(op_ + ": no HIP device is visible");
      return;
    }
    int st = rafhip_sgd_plan_create(n_, numels.data(), grad_dtype, &plan_);
    if (st != RAFHIP_OK) error_msgs.push_back(KernelError("rafhip_sgd_plan_create", st));
  }

  ~SgdMultiHipEnv() override {
    if (plan_) rafhip_sgd_plan_destroy(plan_);
  }

  std::string name() const override { return name_; }

  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::SgdMultiArgs>();
    RAF_CHECK(args != nullptr, op_ + " expects SgdMultiArgs");
    std::vector<Value> fields(args->tensor_list.begin(), args->tensor_list.end());
    Execute(std::vector<Value>{value::MakeTuple(std::move(fields))}, cv->out);
  }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    (void)output;  // aliases the inputs: the update is in place
    RAF_CHECK(inputs.size() == 1, op_ + " takes (tensor_list)");
    auto tuple = AsTuple(inputs[0]);
    RAF_CHECK((int64_t)tuple->fields.size() == (int64_t)blocks_ * (int64_t)n_,
              op_ + ": tensor_list length changed since the OpEnv was made");
    ptrs_.resize(tuple->fields.size());
    CollectDataPointers(tuple->fields, ptrs_.data(), op_);
    void** p = ptrs_.data();
    void* stream = DeviceAPI::Get(DevType::kROCM())->GetStream();
    int st = rafhip_sgd_multi_step(plan_, reinterpret_cast<float* const*>(p),
                                   reinterpret_cast<const void* const*>(p + n_),
                                   reinterpret_cast<float* const*>(p + 2 * n_),
                                   blocks_ == 4 ? p + 3 * n_ : nullptr, copy_dtype_, learning_rate_,
                                   mu_, stream);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_sgd_multi_step", st));
  }

  void SetLearningRate(double learning_rate) override { learning_rate_ = learning_rate; }
  double GetLearningRate() const override { return learning_rate_; }

  static OpEnv* make(const CallValues& cv) { return new SgdMultiHipEnv(cv, false); }
  static OpEnv* make_mixed(const CallValues& cv) { return new SgdMultiHipEnv(cv, true); }

 private:
  int blocks_;
  std::string op_;
  std::string name_;
  double learning_rate_ = 0.0;
  double mu_ = 0.0;
  int32_t n_ = 0;
  int32_t copy_dtype_ = RAFHIP_F16;
  rafhip_sgd_plan* plan_ = nullptr;
  std::vector<void*> ptrs_;  // this call's addresses (kept: no allocation per call)
};

// ---------------------------------------------------------------------------------------- LANS
// One class serves raf.op.lans (tensor_list = g, w, m, v blocks) and the extension op
// raf.op.lans_mixed (a fifth block p: the model's float16 / bfloat16 parameters, which receive the
// new weights narrowed to 16 bits -- what the reference's traced optimizer does with a cast and a
// copy after the op, python/raf/optim/lans.py:289-291, :303-305).  Half gradients are accepted by
// both and widened in the kernel, replacing the group_cast in front of the op (lans.py:261-265).
class LansHipEnv : public OpEnv, public HasLearningRate, public HasGradScaling {
 public:
  LansHipEnv(const CallValues& cv, bool mixed)
      : blocks_(mixed ? 5 : 4),
        op_(mixed ? "raf.op.hip.lans_mixed" : "raf.op.hip.lans"),
        name_(TruncateName(GetUniqueName(op_))) {
    const auto* args = cv->args_as<schema::LansArgs>();
    if (!args) {
      error_msgs.push_back(op_ + ": call does not carry LansArgs");
      return;
    }
    arg_indices = {args->FieldIndex("tensor_list"), args->FieldIndex("step")};  // lans.cc:32-35
    rafhip_lans_default_hparams(&hp_);
    hp_.learning_rate = args->learning_rate;
    hp_.beta1 = args->beta1;
    hp_.beta2 = args->beta2;
    hp_.eps = args->eps;
    hp_.bias_correction = args->bias_correction;
    hp_.weight_decay = args->weight_decay;
    hp_.grad_averaging = args->grad_averaging;
    hp_.mode = args->mode;
    hp_.normalize_grad = args->normalize_grad ? 1 : 0;
    hp_.grad_unscale = 1.0f;  // see HasGradScaling

    const size_t total = args->tensor_list.size();
    if (total % (size_t)blocks_ != 0) {  // lans.cc:53
      error_msgs.push_back(op_ + ": tensor_list must hold " + std::to_string(blocks_) + "n tensors");
      return;
    }
    n_ = (int32_t)(total / (size_t)blocks_);
    if (cv->device.device_type() != DevType::kROCM())
      error_msgs.push_back(op_ + ": device is not rocm");
    if (hp_.mode != 0 && hp_.mode != 1)
      error_msgs.push_back(op_ + ": mode must be 0 (L2) or 1 (decoupled weight decay)");
    int32_t grad_dtype = RAFHIP_F32;
    std::vector<int64_t> numels;
    for (int32_t i = 0; i < n_; ++i) {
      const TensorView& g = args->tensor_list[i]->tensor;
      const int32_t gd = KernelDType(g.dtype);
      if (gd < 0 || (i > 0 && gd != grad_dtype)) {
        error_msgs.push_back(op_ + ": gradients must all be float32, all float16 or all bfloat16");
        break;
      }
      grad_dtype = gd;
      numels.push_back(g.numel());
      for (int q = 1; q < 4; ++q) {  // w, m, v: fp32 (lans.cc:37-40) and as large as g
        const TensorView& t = args->tensor_list[q * n_ + i]->tensor;
        if (!IsF32(t.dtype)) error_msgs.push_back(op_ + ": LANS only takes FP32 weights and state");
        if (t.numel() != g.numel())
          error_msgs.push_back(op_ + ": g, w, m, v of one parameter differ in size");
      }
      if (blocks_ == 5) {  // p: 16-bit, one dtype for the whole list, as large as g
        const TensorView& t = args->tensor_list[4 * n_ + i]->tensor;
        const int32_t pd = KernelDType(t.dtype);
        if (pd != RAFHIP_F16 && pd != RAFHIP_BF16)
          error_msgs.push_back(op_ + ": model parameters must be float16 or bfloat16");
        else if (i > 0 && pd != copy_dtype_)
          error_msgs.push_back(op_ + ": model parameters must share one dtype");
        copy_dtype_ = pd;
        if (t.numel() != g.numel())
          error_msgs.push_back(op_ + ": model parameter and gradient differ in size");
      }
      if (!error_msgs.empty()) break;
    }
    if (!error_msgs.empty()) return;
    if (rafhip_device_count() <= 0) {
      error_msgs.push_back(op_ + ": no HIP device is visible");
      return;
    }
    int st = rafhip_lans_plan_create(n_, numels.data(), grad_dtype, &plan_);
    if (st != RAFHIP_OK) {
      error_msgs.push_back(KernelError("rafhip_lans_plan_create", st));
      return;
    }
    RequestWorkspace(&workspace_, cv->device, rafhip_lans_workspace_bytes(plan_));
    workspace_bytes_ = rafhip_lans_workspace_bytes(plan_);
  }

  ~LansHipEnv() override {
    if (plan_) rafhip_lans_plan_destroy(plan_);
  }

  std::string name() const override { return name_; }

  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::LansArgs>();
    RAF_CHECK(args != nullptr, "raf.op.hip.lans expects LansArgs");
    std::vector<Value> fields(args->tensor_list.begin(), args->tensor_list.end());
    Execute(std::vector<Value>{value::MakeTuple(std::move(fields)), args->step}, cv->out);
  }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    (void)output;  // aliases the inputs (declare/optimizer.cc:53-57); the update is in place
    RAF_CHECK(inputs.size() == 2, "raf.op.hip.lans takes (tensor_list, step)");
    auto tuple = AsTuple(inputs[0]);
    RAF_CHECK((int64_t)tuple->fields.size() == (int64_t)blocks_ * (int64_t)n_,
              op_ + ": tensor_list length changed since the OpEnv was made");
    const TensorView& step = AsTensor(inputs[1])->tensor;
    RAF_CHECK(step.ndim() == 0, "step must be a 0-d tensor");  // lans.cc:96
    RAF_CHECK(IsF32(step.dtype), "step must be float32");
    RAF_CHECK(workspace_ != nullptr || workspace_bytes_ == 0,
              "raf.op.hip.lans: the executor did not provide the requested workspace");
    // Executors hand over a new TupleValue at every call (the VM allocates one per iteration,
    // src/impl/vm/vm.cc:764-769; the interpreter overload above makes one too) and a tuple's
    // fields and a tensor's storage may be replaced between calls, so nothing is concluded from
    // the identity of the tuple: its fields are walked, one pointer read each, and the plan is
    // bound afresh only when an address differs from the last call's.
    now_.resize(tuple->fields.size());
    CollectDataPointers(tuple->fields, now_.data(), op_);
    if (!bound_ || std::memcmp(now_.data(), ptrs_.data(), sizeof(void*) * now_.size()) != 0) {
      bound_ = false;
      ptrs_.swap(now_);
      void** p = ptrs_.data();
      int st = rafhip_lans_plan_bind(plan_, reinterpret_cast<const void* const*>(p),
                                     reinterpret_cast<float* const*>(p + n_),
                                     reinterpret_cast<float* const*>(p + 2 * n_),
                                     reinterpret_cast<float* const*>(p + 3 * n_),
                                     blocks_ == 5 ? p + 4 * n_ : nullptr, copy_dtype_);
      if (st != RAFHIP_OK) throw Error(KernelError("rafhip_lans_plan_bind", st));
      bound_ = true;
    }
    void* stream = DeviceAPI::Get(DevType::kROCM())->GetStream();
    int st = rafhip_lans_step_bound(plan_, static_cast<const float*>(step.data), 0, &hp_, workspace_,
                                    workspace_bytes_, stream);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_lans_step_bound", st));
  }

  void SetLearningRate(double learning_rate) override { hp_.learning_rate = (float)learning_rate; }
  double GetLearningRate() const override { return hp_.learning_rate; }

  void SetGradUnscale(float factor) override { hp_.grad_unscale = factor; }
  void SetDynamicScale(const float* grad_unscale_dev, const float* found_inf_dev) override {
    int st = rafhip_lans_plan_set_dynamic_scale(plan_, grad_unscale_dev, found_inf_dev);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_lans_plan_set_dynamic_scale", st));
  }

  static OpEnv* make(const CallValues& cv) { return new LansHipEnv(cv, false); }
  static OpEnv* make_mixed(const CallValues& cv) { return new LansHipEnv(cv, true); }

 private:
  int blocks_;  // 4: g, w, m, v; 5: and the 16-bit model parameters
  std::string op_;
  std::string name_;
  rafhip_lans_hparams hp_{};
  int32_t n_ = 0;
  int32_t copy_dtype_ = RAFHIP_F16;
  rafhip_lans_plan* plan_ = nullptr;
  void* workspace_ = nullptr;  // bound by the executor around each Execute
  int64_t workspace_bytes_ = 0;
  std::vector<void*> ptrs_;  // the addresses the plan is bound to (g, w, m, v[, p] blocks)
  std::vector<void*> now_;   // this call's addresses
  bool bound_ = false;
};

// -------------------------------------------------------------------------------------- l2norm
class L2NormHipEnv : public OpEnv {
 public:
  explicit L2NormHipEnv(const CallValues& cv) {
    const auto* args = cv->args_as<schema::L2NormArgs>();
    if (!args) {
      error_msgs.push_back("raf.op.hip.l2norm: call does not carry L2NormArgs");
      return;
    }
    arg_indices = {args->FieldIndex("x")};  // l2_norm.cc:38-40
    const TensorView& x = args->x->tensor;
    n_ = x.numel();
    dtype_ = x.dtype.code == kDLFloat && x.dtype.bits == 64 ? (int32_t)RAFHIP_F64 : KernelDType(x.dtype);
    if (cv->device.device_type() != DevType::kROCM())
      error_msgs.push_back("raf.op.hip.l2norm: device is not rocm");
    if (dtype_ < 0) error_msgs.push_back("raf.op.hip.l2norm: Unsupported output dtype");  // l2_norm.cc:73
    if (error_msgs.empty() && rafhip_device_count() <= 0)
      error_msgs.push_back("raf.op.hip.l2norm: no HIP device is visible");
    if (!error_msgs.empty()) return;
    workspace_bytes_ = rafhip_l2norm_workspace_bytes(n_);
    if (workspace_bytes_ > 0) RequestWorkspace(&workspace_, cv->device, workspace_bytes_);
  }

  std::string name() const override { return name_; }

  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::L2NormArgs>();
    RAF_CHECK(args != nullptr, "raf.op.hip.l2norm expects L2NormArgs");
    Execute(std::vector<Value>{args->x}, cv->out);
  }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    RAF_CHECK(inputs.size() == 1, "raf.op.hip.l2norm takes x");
    const TensorView& x = AsTensor(inputs[0])->tensor;
    const TensorView& out = AsTensor(output)->tensor;
    RAF_CHECK(x.numel() == n_, "raf.op.hip.l2norm: element count changed since the OpEnv was made");
    void* stream = DeviceAPI::Get(DevType::kROCM())->GetStream();
    int st = rafhip_l2norm(x.data, dtype_, n_, out.data, workspace_, workspace_bytes_, stream);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_l2norm", st));
  }

  static OpEnv* make(const CallValues& cv) { return new L2NormHipEnv(cv); }

 private:
  int64_t n_ = 0;
  int32_t dtype_ = -1;
  void* workspace_ = nullptr;
  int64_t workspace_bytes_ = 0;
  std::string name_ = TruncateName(GetUniqueName("raf.op.hip.l2norm"));
};

// ------------------------------------------------------------------------- fuse / defuse tensor
// Both hold a plan made from the tensors' byte sizes, which the reference's constructors record
// too (memory.cc:37-43, :99-103), and both request a copy stream with the reference's tags
// (RequestStream, memory.cc:34, :89).  An executor that serves the request gets the single launch
// on that stream (and owns the ordering against the compute stream, as in the reference); one
// that leaves it unserved gets it on the current compute stream, which is the right place when
// nothing else could run beside the copy.
class FuseBase : public OpEnv {
 public:
  ~FuseBase() override {
    if (plan_) rafhip_fuse_plan_destroy(plan_);
  }
  std::string name() const override { return name_; }

 protected:
  FuseBase(const char* op, const CallValues& cv, int stream_tag)
      : op_(op), name_(TruncateName(GetUniqueName(op))) {
    if (cv->device.device_type() != DevType::kROCM()) error_msgs.push_back(op_ + ": device is not rocm");
    RequestStream(&stream_, cv->device, stream_tag);
  }
  void* LaunchStream() const {
    return stream_ ? stream_ : DeviceAPI::Get(DevType::kROCM())->GetStream();
  }
  void MakePlan(const std::vector<int64_t>& nbytes) {
    if (!error_msgs.empty()) return;
    if (rafhip_device_count() <= 0) {
      error_msgs.push_back(op_ + ": no HIP device is visible");
      return;
    }
    int st = rafhip_fuse_plan_create((int32_t)nbytes.size(), nbytes.data(), &plan_);
    if (st != RAFHIP_OK) error_msgs.push_back(KernelError("rafhip_fuse_plan_create", st));
    n_ = nbytes.size();
  }
  std::vector<void*> Pointers(const value::TupleValue& tuple) const {
    RAF_CHECK(tuple->fields.size() == n_, op_ + ": tensor count changed since the OpEnv was made");
    std::vector<void*> ptrs(n_);
    for (size_t i = 0; i < n_; ++i) ptrs[i] = AsTensor(tuple->fields[i])->tensor.data;
    return ptrs;
  }
  std::string op_, name_;
  rafhip_fuse_plan* plan_ = nullptr;
  size_t n_ = 0;
  void* stream_ = nullptr;  // bound by the executor around Execute, or left null
};

class FuseTensorHipEnv : public FuseBase {
 public:
  explicit FuseTensorHipEnv(const CallValues& cv)
      : FuseBase("raf.op.hip.fuse_tensor", cv, stream_pool::kMemCpyCudaToCuda1) {
    const auto* args = cv->args_as<schema::FuseTensorArgs>();
    if (!args) {
      error_msgs.push_back(op_ + ": call does not carry FuseTensorArgs");
      return;
    }
    arg_indices = {args->FieldIndex("data")};  // memory.cc:31
    std::vector<int64_t> nbytes;
    for (const auto& t : args->data) nbytes.push_back(t->tensor.numel() * ((t->tensor.dtype.bits + 7) / 8));
    MakePlan(nbytes);
  }
  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::FuseTensorArgs>();
    RAF_CHECK(args != nullptr, op_ + " expects FuseTensorArgs");
    std::vector<Value> fields(args->data.begin(), args->data.end());
    Execute(std::vector<Value>{value::MakeTuple(std::move(fields))}, cv->out);
  }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    RAF_CHECK(inputs.size() == 1, op_ + " takes (data)");
    std::vector<void*> ptrs = Pointers(AsTuple(inputs[0]));
    void* stream = LaunchStream();
    int st = rafhip_fuse_tensors(plan_, ptrs.data(), AsTensor(output)->tensor.data, stream);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_fuse_tensors", st));
  }
  static OpEnv* make(const CallValues& cv) { return new FuseTensorHipEnv(cv); }
};

class DefuseTensorHipEnv : public FuseBase {
 public:
  explicit DefuseTensorHipEnv(const CallValues& cv)
      : FuseBase("raf.op.hip.defuse_tensor", cv, stream_pool::kMemCpyCudaToCuda2) {
    const auto* args = cv->args_as<schema::DefuseTensorArgs>();
    if (!args) {
      error_msgs.push_back(op_ + ": call does not carry DefuseTensorArgs");
      return;
    }
    arg_indices = {args->FieldIndex("data")};  // memory.cc:92
    const int64_t eb = (args->data->tensor.dtype.bits + 7) / 8;  // memory.cc:97-102
    std::vector<int64_t> nbytes;
    for (int64_t s : args->sizes) nbytes.push_back(s * eb);
    MakePlan(nbytes);
  }
  void Execute(const CallValues& cv) override {
    const auto* args = cv->args_as<schema::DefuseTensorArgs>();
    RAF_CHECK(args != nullptr, op_ + " expects DefuseTensorArgs");
    Execute(std::vector<Value>{args->data}, cv->out);
  }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    RAF_CHECK(inputs.size() == 1, op_ + " takes (data)");
    std::vector<void*> ptrs = Pointers(AsTuple(output));
    void* stream = LaunchStream();
    int st = rafhip_defuse_tensor(plan_, AsTensor(inputs[0])->tensor.data, ptrs.data(), stream);
    if (st != RAFHIP_OK) throw Error(KernelError("rafhip_defuse_tensor", st));
  }
  static OpEnv* make(const CallValues& cv) { return new DefuseTensorHipEnv(cv); }
};

RAF_REGISTER_DIALECT("hip").set_enable(DevType::kROCM());
// plevels above the reference's own backends (cuda lans = 20, tvm sgd = 10).
RAF_REGISTER_DIALECT_OP(hip, lans, 30);
RAF_OP_ENV_MAKER("raf.op.hip.lans", LansHipEnv::make);
RAF_REGISTER_DIALECT_OP(hip, lans_mixed, 30);
RAF_OP_ENV_MAKER("raf.op.hip.lans_mixed", LansHipEnv::make_mixed);
RAF_REGISTER_DIALECT_OP(hip, sgd, 30);
RAF_OP_ENV_MAKER("raf.op.hip.sgd", SgdHipEnv::make);
RAF_REGISTER_DIALECT_OP(hip, sgd_multi, 30);
RAF_OP_ENV_MAKER("raf.op.hip.sgd_multi", SgdMultiHipEnv::make);
RAF_REGISTER_DIALECT_OP(hip, sgd_multi_mixed, 30);
RAF_OP_ENV_MAKER("raf.op.hip.sgd_multi_mixed", SgdMultiHipEnv::make_mixed);
// cublas l2norm is plevel 15, tvm 10; cuda fuse_tensor / defuse_tensor are plevel 10.
RAF_REGISTER_DIALECT_OP(hip, l2norm, 30);
RAF_OP_ENV_MAKER("raf.op.hip.l2norm", L2NormHipEnv::make);
RAF_REGISTER_DIALECT_OP(hip, fuse_tensor, 30);
RAF_OP_ENV_MAKER("raf.op.hip.fuse_tensor", FuseTensorHipEnv::make);
RAF_REGISTER_DIALECT_OP(hip, defuse_tensor, 30);
RAF_OP_ENV_MAKER("raf.op.hip.defuse_tensor", DefuseTensorHipEnv::make);

}  // namespace hip
}  // namespace op
}  // namespace raf

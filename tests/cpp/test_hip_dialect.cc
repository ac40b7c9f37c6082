// Host-side checks of the dialect registry mirror and of the `hip` dialect's registration, in the
// manner of the reference's tests/cpp/test_op_dialect.cc:27-108 (two fake dialects on CPU with
// plevels 10 and 12, dispatch-list order, IsDialectOp / GetDialect, maker lookup), extended with
// the dispatcher's fall-through on error_msgs and the declare checks.  Plain asserts; prints the
// name of each check so a failure names itself.  Runs without a GPU.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "memory_pool.h"
#include "raf_iface.h"

using namespace raf;
using namespace raf::op;

#define EXPECT(cond)                                                      \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                       \
    }                                                                     \
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

class FakeEnv : public OpEnv {
 public:
  explicit FakeEnv(int type, bool refuse = false) : type(type) {
    if (refuse) error_msgs.push_back("fake backend " + std::to_string(type) + " refuses");
  }
  int type;
  std::string name() const override { return "cpptest.sgd"; }
  void Execute(const CallValues&) override {}
  void Execute(const std::vector<value::Value>&, value::Value) override {}
};

static bool g_refuse_high = false;

RAF_REGISTER_DIALECT("mklShallowNN").set_enable(DevType::kCPU());
RAF_REGISTER_DIALECT_OP(mklShallowNN, sgd, 10);
RAF_OP_ENV_MAKER("raf.op.mklShallowNN.sgd", [](const CallValues&) -> OpEnv* { return new FakeEnv(0); });

RAF_REGISTER_DIALECT("sshadow").set_enable(DevType::kCPU());
RAF_REGISTER_DIALECT_OP(sshadow, sgd, 12);
RAF_OP_ENV_MAKER("raf.op.sshadow.sgd",
                 [](const CallValues&) -> OpEnv* { return new FakeEnv(1, g_refuse_high); });

static value::TensorValue T(std::vector<int64_t> shape, DevType dev, int bits = 32) {
  TensorView t;
  t.shape = std::move(shape);
  t.device = Device(dev, 0);
  t.dtype.bits = bits;
  return value::MakeTensor(t);
}

static CallValues SgdCall(DevType dev, std::vector<int64_t> xs = {4, 4},
                          std::vector<int64_t> ds = {4, 4}) {
  auto a = std::make_shared<schema::SgdArgs>();
  a->x = T(xs, dev);
  a->dx = T(ds, dev);
  a->v = T(ds, dev);
  a->learning_rate = 0.1;
  a->mu = 0.9;
  return MakeCall("raf.op.sgd", a);
}

// The rocm pool's constructor makes its device current, which needs a GPU.
static bool DeviceAPI_count_is_zero() {
  return device_api::DeviceAPI::Get(DevType::kROCM())->GetDeviceCount() == 0;
}

int main() {
  std::puts("dispatch list is plevel-descending and filtered by device type");
  auto cpu = OpDialect::GetDispatchList("raf.op.sgd", DevType::kCPU());
  EXPECT(cpu.size() == 2);
  EXPECT(cpu.front().dialect == "sshadow" && cpu.front().plevel == 12);
  EXPECT(cpu.back().dialect == "mklShallowNN" && cpu.back().dialect_op == "raf.op.mklShallowNN.sgd");
  auto rocm = OpDialect::GetDispatchList("raf.op.sgd", DevType::kROCM());
  EXPECT(rocm.size() == 1 && rocm.front().dialect == "hip" && rocm.front().plevel == 30);
  auto lans = OpDialect::GetDispatchList("raf.op.lans", DevType::kROCM());
  EXPECT(lans.size() == 1 && lans.front().dialect_op == "raf.op.hip.lans" && lans.front().plevel == 30);
  EXPECT(OpDialect::GetDispatchList("raf.op.lans", DevType::kCUDA()).empty());
  EXPECT(OpDialect::Dispatch("raf.op.sgd", DevType::kCPU()) == "raf.op.sshadow.sgd");
  EXPECT(OpDialect::Dispatch("raf.op.sgd", DevType::kCPU(), {"sshadow"}) == "raf.op.mklShallowNN.sgd");

  std::puts("dialect-op attributes and makers");
  for (const auto& e : cpu) {
    EXPECT(IsDialectOp(e.dialect_op));
    EXPECT(GetDialect(e.dialect_op) == e.dialect);
    EXPECT(GetBaseOp(e.dialect_op) == "raf.op.sgd");
    EXPECT(OpEnvMaker::Get(e.dialect_op) != nullptr);
  }
  EXPECT(!IsDialectOp("raf.op.sgd"));
  EXPECT(OpEnvMaker::Get("raf.op.hip.lans") != nullptr && OpEnvMaker::Get("raf.op.nope") == nullptr);
  EXPECT(Dialect::IsEnabled("hip", DevType::kROCM()) && !Dialect::IsEnabled("hip", DevType::kCPU()));
  EXPECT(!Raises([] { Dialect::IsEnabled("nope", DevType::kCPU()); }).empty());

  std::puts("duplicate dialect or duplicate plevel on one base op is refused");
  EXPECT(Raises([] {
           OpDialect::RegisterOrGet("raf.op.sgd").add_dialect("sshadow", "raf.op.sshadow.sgd2", 99);
         }).find("already has a registration on dialect sshadow") != std::string::npos);
  Dialect::RegisterOrGet("third").set_name("third").set_enable(DevType::kCPU());
  EXPECT(Raises([] {
           OpDialect::RegisterOrGet("raf.op.sgd").add_dialect("third", "raf.op.third.sgd", 12);
         }).find("same plevel=12") != std::string::npos);

  std::puts("dispatch picks the highest plevel, falls through on error_msgs, reports when none fits");
  auto call = SgdCall(DevType::kCPU());
  RunDeclare(call);
  std::string picked;
  auto env = DispatchSingleOp(call, &picked);
  EXPECT(static_cast<FakeEnv*>(env.get())->type == 1 && picked == "raf.op.sshadow.sgd");
  g_refuse_high = true;
  env = DispatchSingleOp(call, &picked);
  EXPECT(static_cast<FakeEnv*>(env.get())->type == 0 && picked == "raf.op.mklShallowNN.sgd");
  {
    DialectPreference only({"sshadow"});
    std::string msg = Raises([&] { DispatchSingleOp(call); });
    EXPECT(msg.find("Cannot find a valid dispatch for op raf.op.sgd:") == 0);
    EXPECT(msg.find("fake backend 1 refuses") != std::string::npos);
  }
  g_refuse_high = false;
  {
    DialectPreference order({"mklShallowNN", "sshadow"});  // preference order beats plevel
    env = DispatchSingleOp(call, &picked);
    EXPECT(picked == "raf.op.mklShallowNN.sgd");
  }
  EXPECT(DialectPreference::Current() == nullptr);

  std::puts("hip OpEnvs report unsupported calls through error_msgs instead of throwing");
  {
    auto c = SgdCall(DevType::kCPU());
    RunDeclare(c);
    OpEnvPtr e((*OpEnvMaker::Get("raf.op.hip.sgd"))(c));
    EXPECT(e->HasError() && e->error_msgs[0].find("not rocm") != std::string::npos);
    EXPECT((e->arg_indices == std::vector<int>{0, 1, 2}));
    EXPECT(e->name().find("raf_op_hip_sgd") == 0);
    auto l = std::make_shared<schema::LansArgs>();
    for (int i = 0; i < 4; ++i) l->tensor_list.push_back(T({8}, DevType::kROCM(), i == 1 ? 64 : 32));
    l->step = T({}, DevType::kROCM());
    l->mode = 1;
    auto lc = MakeCall("raf.op.lans", l);
    RunDeclare(lc);
    EXPECT(value::AsTuple(lc->out)->fields.size() == 4 && lc->device.device_type() == DevType::kROCM());
    EXPECT(value::AsTuple(lc->out)->fields[2] == l->tensor_list[2]);  // output aliases the inputs
    OpEnvPtr le((*OpEnvMaker::Get("raf.op.hip.lans"))(lc));
    EXPECT(le->HasError() && le->error_msgs[0].find("FP32") != std::string::npos);
    EXPECT(le->stream_requests().empty());  // the optimizer steps run on the compute stream
    EXPECT((le->arg_indices == std::vector<int>{0, 1}));
  }

  std::puts("declare checks");
  EXPECT(Raises([] { RunDeclare(SgdCall(DevType::kCPU(), {4, 4}, {4, 5})); }).find("differ in shape") !=
         std::string::npos);
  EXPECT(Raises([] { RunDeclare(SgdCall(DevType::kCPU(), {4, 4}, {16})); }).find("differ in rank") !=
         std::string::npos);
  {
    auto c = SgdCall(DevType::kCPU(), {2, 3}, {2, 3});
    RunDeclare(c);
    auto out = value::AsTuple(c->out);
    EXPECT(out->fields.size() == 2);  // (v1, x1)
    EXPECT(value::AsTensor(out->fields[0])->tensor.shape == (std::vector<int64_t>{2, 3}));
    auto l = std::make_shared<schema::LansArgs>();
    for (int i = 0; i < 6; ++i) l->tensor_list.push_back(T({8}, DevType::kROCM()));
    l->step = T({}, DevType::kROCM());
    EXPECT(Raises([&] { RunDeclare(MakeCall("raf.op.lans", l)); }).find("4n tensors") != std::string::npos);
    EXPECT(Raises([&] { RunDeclare(MakeCall("raf.op.lans_mixed", l)); }).find("5n tensors") != std::string::npos);
  }

  std::puts("l2norm, fuse_tensor, defuse_tensor: declares and dialect ops");
  {
    for (const char* name : {"l2norm", "fuse_tensor", "defuse_tensor"}) {
      auto l = OpDialect::GetDispatchList(std::string("raf.op.") + name, DevType::kROCM());
      EXPECT(l.size() == 1 && l.front().dialect_op == std::string("raf.op.hip.") + name && l.front().plevel == 30);
    }
    auto n = std::make_shared<schema::L2NormArgs>();
    n->x = T({2, 3, 4}, DevType::kROCM(), 64);
    auto nc = MakeCall("raf.op.l2norm", n);
    RunDeclare(nc);
    const TensorView& no = value::AsTensor(nc->out)->tensor;
    EXPECT(no.ndim() == 0 && no.dtype.bits == 64 && nc->device.device_type() == DevType::kROCM());

    auto f = std::make_shared<schema::FuseTensorArgs>();
    f->data = {T({3, 5}, DevType::kROCM()), T({7}, DevType::kROCM()), T({}, DevType::kROCM())};
    auto fc = MakeCall("raf.op.fuse_tensor", f);
    RunDeclare(fc);
    EXPECT(value::AsTensor(fc->out)->tensor.shape == (std::vector<int64_t>{23}));
    auto fe = MakeCall("raf.op.fuse_tensor", std::make_shared<schema::FuseTensorArgs>());
    RunDeclare(fe);
    EXPECT(fe->callee.empty() && !fe->out);  // empty list: no callee, no output

    auto d = std::make_shared<schema::DefuseTensorArgs>();
    d->data = T({23}, DevType::kROCM());
    d->sizes = {15, 7, 1};
    d->shapes = {3, 5, 7};
    d->shape_indices = {2, 3, 3};
    auto dc = MakeCall("raf.op.defuse_tensor", d);
    RunDeclare(dc);
    auto outs = value::AsTuple(dc->out)->fields;
    EXPECT(outs.size() == 3);
    EXPECT(value::AsTensor(outs[0])->tensor.shape == (std::vector<int64_t>{3, 5}));
    EXPECT(value::AsTensor(outs[2])->tensor.ndim() == 0);
    d->sizes = {15, 7, 2};
    EXPECT(Raises([&] { RunDeclare(MakeCall("raf.op.defuse_tensor", d)); })
               .find("Input tensor size should be 24, got 23.") != std::string::npos);
    d->sizes = {15, 7, 1};
    OpEnvPtr de((*OpEnvMaker::Get("raf.op.hip.defuse_tensor"))(dc));
    EXPECT((de->arg_indices == std::vector<int>{0}));
    // the copy streams the reference's fuse / defuse OpEnvs request (cuda/memory.cc:34, :89)
    OpEnvPtr fe2((*OpEnvMaker::Get("raf.op.hip.fuse_tensor"))(fc));
    EXPECT(fe2->stream_requests().size() == 1 && fe2->stream_requests()[0].tag_idx == stream_pool::kMemCpyCudaToCuda1);
    EXPECT(de->stream_requests().size() == 1 && de->stream_requests()[0].tag_idx == stream_pool::kMemCpyCudaToCuda2 &&
           de->stream_requests()[0].stream_idx == 0 && de->stream_requests()[0].dest != nullptr);
    auto cpu = std::make_shared<schema::L2NormArgs>();
    cpu->x = T({4}, DevType::kCPU());
    auto cc = MakeCall("raf.op.l2norm", cpu);
    RunDeclare(cc);
    OpEnvPtr ce((*OpEnvMaker::Get("raf.op.hip.l2norm"))(cc));
    EXPECT(ce->HasError() && ce->error_msgs[0].find("not rocm") != std::string::npos);
  }

  std::puts("extension op lans_mixed: five blocks, 16-bit parameters");
  {
    auto mixed = OpDialect::GetDispatchList("raf.op.lans_mixed", DevType::kROCM());
    EXPECT(mixed.size() == 1 && mixed.front().dialect_op == "raf.op.hip.lans_mixed");
    auto l = std::make_shared<schema::LansArgs>();
    for (int i = 0; i < 5; ++i) l->tensor_list.push_back(T({8}, DevType::kROCM(), 32));  // p is fp32: refused
    l->step = T({}, DevType::kROCM());
    l->mode = 1;
    auto lc = MakeCall("raf.op.lans_mixed", l);
    RunDeclare(lc);
    EXPECT(value::AsTuple(lc->out)->fields.size() == 5);
    EXPECT(value::AsTuple(lc->out)->fields[4] == l->tensor_list[4]);
    OpEnvPtr le((*OpEnvMaker::Get("raf.op.hip.lans_mixed"))(lc));
    EXPECT(le->HasError() && le->error_msgs[0].find("float16 or bfloat16") != std::string::npos);
    EXPECT(le->name().find("raf_op_hip_lans_mixed") == 0);
  }

  std::puts("unique and truncated OpEnv names");
  std::string a = GetUniqueName("raf.op.hip.zzz"), b = GetUniqueName("raf.op.hip.zzz");
  EXPECT(a == "raf_op_hip_zzz" && b == "raf_op_hip_zzz_1");
  EXPECT(TruncateName(std::string(200, 'x')).size() < 120);

  std::puts("schema field indices");
  schema::LansArgs la;
  EXPECT(la.FieldIndex("tensor_list") == 0 && la.FieldIndex("step") == 1 && la.FieldIndex("normalize_grad") == 10);
  EXPECT(!Raises([&] { la.FieldIndex("nope"); }).empty());

  std::puts("stream plumbing");
  int dummy = 0;
  OpEnv::SetStreamForAllBackends(Device(DevType::kROCM(), 0), &dummy);
  EXPECT(device_api::DeviceAPI::Get(DevType::kROCM())->GetStream() == &dummy);
  EXPECT(device_api::DeviceAPI::Get(DevType::kCPU())->GetStream() == nullptr);
  OpEnv::SetStreamForAllBackends(Device(DevType::kROCM(), 0), nullptr);

  std::puts("device APIs: registration, the cpu API, rocm without a device");
  {
    using device_api::DeviceAPI;
    EXPECT(DeviceAPI::Get(DevType::kCPU()) == DeviceAPI::Get(DevType::kCPU()));  // one instance per type
    EXPECT(Raises([] { DeviceAPI::Get(DevType::kCUDA()); }).find("raf.device_api._make.cuda") != std::string::npos);
    auto cpu = DeviceAPI::Get(DevType::kCPU());
    EXPECT(cpu->GetDeviceCount() >= 1);
    void* a = cpu->AllocMemory(1000, 256);
    EXPECT(a != nullptr && reinterpret_cast<uintptr_t>(a) % 256 == 0);
    TensorView from, to;
    std::vector<float> src(250, 1.5f);
    from.data = src.data();
    from.shape = {250};
    from.device = Device(DevType::kCPU(), 0);
    to = from;
    to.data = a;
    cpu->CopyDataFromTo(from, to, nullptr);
    EXPECT(static_cast<float*>(a)[249] == 1.5f);
    to.shape = {249};
    EXPECT(!Raises([&] { cpu->CopyDataFromTo(from, to, nullptr); }).empty());
    cpu->FreeMemory(a);
    EXPECT(Raises([&] { cpu->CreateStream(Device(DevType::kCPU(), 0)); }).find("no CreateStream") != std::string::npos);
    EXPECT(cpu->GetPoolSize() == (std::pair<int64_t, int64_t>{0, 0}));
    auto rocm = DeviceAPI::Get(DevType::kROCM());
    if (rocm->GetDeviceCount() == 0) {  // no GPU in this process: runtime calls fail as raf::Error
      EXPECT(Raises([&] { rocm->AllocMemory(64, 64); }).find("failed with status") != std::string::npos);
      EXPECT(!Raises([&] { rocm->WaitEvent(nullptr); }).empty());
    }
    EXPECT(!Raises([&] { rocm->CreateStream(Device(DevType::kCPU(), 0)); }).empty());
  }

  std::puts("memory pools on the cpu device API");
  {
    using memory_pool::Memory;
    const Device cpu(DevType::kCPU(), 0);
    EXPECT(Memory::GetPool(cpu)->GetName() == "page_unit_pool");  // the default for cpu
    EXPECT(Memory::GetAllocBytes(cpu, 1) == 4096 && Memory::GetAllocBytes(cpu, 4096) == 4096 &&
           Memory::GetAllocBytes(cpu, 4097) == 8192 && Memory::GetAllocBytes(cpu, 0) == 0);
    auto m1 = Memory::Alloc(cpu, 5000);
    void* p1 = m1->data;
    EXPECT(p1 != nullptr && reinterpret_cast<uintptr_t>(p1) % 64 == 0);
    auto sz = Memory::GetPoolSize(cpu);
    EXPECT(sz.first == 8192.f / 1048576.f && sz.second == sz.first);
    auto m2 = Memory::Alloc(cpu, 6000);  // same page count, the first chunk is busy: a second chunk
    EXPECT(m2->data != p1);
    m1.reset();                          // idle now: the next request of that size gets it back
    auto m3 = Memory::Alloc(cpu, 8000);
    EXPECT(m3->data == p1);
    sz = Memory::GetPoolSize(cpu);
    EXPECT(sz.first == sz.second && sz.second == 16384.f / 1048576.f);
    m2.reset();
    sz = Memory::GetPoolSize(cpu);
    EXPECT(sz.first == 8192.f / 1048576.f && sz.second == 16384.f / 1048576.f);
    EXPECT(Memory::Alloc(cpu, 0)->data == nullptr);
    EXPECT(Raises([&] { Memory::Alloc(cpu, 64, 48); }).find("is not aligned to 64") != std::string::npos);
    EXPECT(Raises([&] { Memory::AllocAsync(cpu, 64, nullptr); }).find("Please use NoPool") != std::string::npos);
    auto batch = Memory::AllocBatch(cpu, {100, 200, 0});
    EXPECT(batch.size() == 3 && batch[0]->data != batch[1]->data && batch[2]->data == nullptr);
    // a removed pool stops serving, its chunks live on with their users; reset keeps the kind
    memory_pool::RemovePool(cpu);
    std::memset(m3->data, 7, 8000);
    memory_pool::InitPool(cpu, "no_pool");
    EXPECT(Memory::GetPool(cpu)->GetName() == "no_pool" && Memory::GetAllocBytes(cpu, 5) == 5);
    auto n1 = Memory::Alloc(cpu, 5000);
    EXPECT(n1->data != nullptr && n1->device.device_type() == DevType::kCPU());
    EXPECT(Raises([&] { Memory::AllocAsync(cpu, 64, nullptr); }).find("no AllocMemoryAsync") != std::string::npos);
    memory_pool::ResetPool(cpu);
    EXPECT(Memory::GetPool(cpu)->GetName() == "no_pool");
    EXPECT(Raises([&] { memory_pool::InitPool(cpu, "nope"); }).find("raf.memory_pool._make.nope") != std::string::npos);
    // a size limit: what the pool holds, idle and in use together, may not outgrow it; the idle
    // blocks go back to the device when a new block would
    setenv("RAF_MEMORY_POOL_SIZE_LIMIT", "20000", 1);
    memory_pool::InitPool(cpu, "page_unit_pool");
    unsetenv("RAF_MEMORY_POOL_SIZE_LIMIT");
    {
      auto a = Memory::Alloc(cpu, 8192);
      a.reset();
      auto held = Memory::GetPoolSize(cpu);
      EXPECT(held.first == 0.f && held.second == 8192.f / 1048576.f);  // kept for the next request
      auto b = Memory::Alloc(cpu, 12288);  // 8192 idle + 12288 > 20000: the idle block is released
      held = Memory::GetPoolSize(cpu);
      EXPECT(held.first == 12288.f / 1048576.f && held.second == held.first);
      auto c = Memory::Alloc(cpu, 4096);   // within the limit again: nothing to release, nothing refused
      held = Memory::GetPoolSize(cpu);
      EXPECT(held.second == 16384.f / 1048576.f);
      memory_pool::RemovePool(cpu);        // b and c outlive their pool and free themselves
      std::memset(b->data, 1, 12288);
    }
    memory_pool::InitPool(cpu, "page_unit_pool");
    if (DeviceAPI_count_is_zero())  // the rocm pool makes its device current: a raf::Error without a GPU
      EXPECT(Raises([] { Memory::GetPool(Device(DevType::kROCM(), 0)); }).find("hipSetDevice") != std::string::npos);
    else
      EXPECT(Memory::GetPool(Device(DevType::kROCM(), 0))->GetName() == "no_pool");
  }

  std::puts("ALL OK");
  return 0;
}

// LansHipEnv and SgdMultiHipEnv against a recording stand-in for the kernel library: what reaches
// rafhip_lans_plan_bind / rafhip_lans_step_bound when an executor hands Execute the same tuple
// again, a new tuple over the same tensors (the VM's pattern), a tuple one of whose fields was
// replaced, or the same tuple after a tensor's storage moved.  No GPU, no HIP.
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "raf_iface.h"
#include "rafhip_optim.h"

using namespace raf;
using namespace raf::op;

#define EXPECT(cond)                                                      \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
      return 1;                                                           \
    }                                                                     \
  } while (0)

// ------------------------------------------------------------- the recording kernel library
struct rafhip_lans_plan {
  int32_t n;
};
struct rafhip_sgd_plan {
  int32_t n;
};
static int g_binds = 0, g_steps = 0, g_sgd_steps = 0;
static std::vector<const void*> g_bound;  // g, w, m, v blocks as last bound
static std::vector<const void*> g_sgd_last;

extern "C" {
int rafhip_device_count(void) { return 1; }
const char* rafhip_last_error(void) { return "recording stand-in"; }
void rafhip_lans_default_hparams(rafhip_lans_hparams* hp) { std::memset(hp, 0, sizeof(*hp)); }
int rafhip_lans_plan_create(int32_t n, const int64_t*, int32_t, rafhip_lans_plan** out) {
  *out = new rafhip_lans_plan{n};
  return RAFHIP_OK;
}
int rafhip_lans_plan_destroy(rafhip_lans_plan* p) {
  delete p;
  return RAFHIP_OK;
}
int64_t rafhip_lans_workspace_bytes(const rafhip_lans_plan*) { return 512; }
int rafhip_lans_plan_bind(rafhip_lans_plan* plan, const void* const* g, float* const* w, float* const* m,
                          float* const* v, void* const*, int32_t) {
  ++g_binds;
  g_bound.clear();
  for (int32_t i = 0; i < plan->n; ++i) g_bound.push_back(g[i]);
  for (int32_t i = 0; i < plan->n; ++i) g_bound.push_back(w[i]);
  for (int32_t i = 0; i < plan->n; ++i) g_bound.push_back(m[i]);
  for (int32_t i = 0; i < plan->n; ++i) g_bound.push_back(v[i]);
  return RAFHIP_OK;
}
int rafhip_lans_step_bound(rafhip_lans_plan*, const float*, int32_t, const rafhip_lans_hparams*, void*, int64_t,
                           void*) {
  ++g_steps;
  return RAFHIP_OK;
}
int rafhip_sgd_plan_create(int32_t n, const int64_t*, int32_t, rafhip_sgd_plan** out) {
  *out = new rafhip_sgd_plan{n};
  return RAFHIP_OK;
}
int rafhip_sgd_plan_destroy(rafhip_sgd_plan* p) {
  delete p;
  return RAFHIP_OK;
}
int rafhip_sgd_multi_step(rafhip_sgd_plan* plan, float* const* x, const void* const* dx, float* const* v,
                          void* const*, int32_t, double, double, void*) {
  ++g_sgd_steps;
  g_sgd_last.clear();
  for (int32_t i = 0; i < plan->n; ++i) g_sgd_last.push_back(x[i]);
  for (int32_t i = 0; i < plan->n; ++i) g_sgd_last.push_back(dx[i]);
  for (int32_t i = 0; i < plan->n; ++i) g_sgd_last.push_back(v[i]);
  return RAFHIP_OK;
}
}  // extern "C"

static float g_memory[64];

static value::TensorValue T(int slot, std::vector<int64_t> shape = {8}) {
  TensorView t;
  t.data = &g_memory[slot];
  t.shape = std::move(shape);
  t.device = Device(DevType::kROCM(), 0);
  return value::MakeTensor(t);
}

int main() {
  auto args = std::make_shared<schema::LansArgs>();
  const int n = 3;
  for (int i = 0; i < 4 * n; ++i) args->tensor_list.push_back(T(i));
  args->step = T(40, {});
  args->mode = 1;
  auto call = MakeCall("raf.op.lans", args);
  RunDeclare(call);
  OpEnvPtr env((*OpEnvMaker::Get("raf.op.hip.lans"))(call));
  EXPECT(!env->HasError());
  char workspace[512];
  for (const auto& r : env->workspace_requests()) *r.dest = workspace;  // what an executor does around Execute

  std::puts("the same tuple twice: bound once");
  std::vector<value::Value> fields(args->tensor_list.begin(), args->tensor_list.end());
  auto tuple = value::MakeTuple(fields);
  env->Execute({tuple, args->step}, tuple);
  env->Execute({tuple, args->step}, tuple);
  EXPECT(g_binds == 1 && g_steps == 2);
  EXPECT(g_bound.size() == 12 && g_bound[0] == &g_memory[0] && g_bound[11] == &g_memory[11]);

  std::puts("a new tuple over the same tensor values (the VM's pattern): not bound again");
  for (int i = 0; i < 3; ++i) {
    auto fresh = value::MakeTuple(fields);
    env->Execute({fresh, args->step}, fresh);
  }
  EXPECT(g_binds == 1 && g_steps == 5);

  std::puts("the interpreter overload makes its own tuple: not bound again either");
  env->Execute(call);
  EXPECT(g_binds == 1 && g_steps == 6);

  std::puts("a field of the SAME tuple object replaced: bound afresh, to the new address");
  tuple->fields[1] = T(50);
  env->Execute({tuple, args->step}, tuple);
  EXPECT(g_binds == 2 && g_steps == 7 && g_bound[1] == &g_memory[50]);

  std::puts("a tensor's storage moved under the same tuple and the same tensor value: bound afresh");
  value::AsTensor(tuple->fields[4])->tensor.data = &g_memory[51];
  env->Execute({tuple, args->step}, tuple);
  EXPECT(g_binds == 3 && g_bound[4] == &g_memory[51]);
  env->Execute({tuple, args->step}, tuple);
  EXPECT(g_binds == 3 && g_steps == 9);

  std::puts("gradients alternating between two allocations: one bind per change, right addresses");
  auto other = fields;
  for (int i = 0; i < n; ++i) other[i] = T(20 + i);
  for (int s = 0; s < 4; ++s) {
    auto t = value::MakeTuple(s % 2 ? fields : other);
    env->Execute({t, args->step}, t);
    EXPECT(g_bound[0] == (s % 2 ? (const void*)&g_memory[0] : (const void*)&g_memory[20]));
  }
  EXPECT(g_binds == 7);

  std::puts("a field that is no tensor, a list of another length");
  auto bad = value::MakeTuple(fields);
  bad->fields[2] = value::MakeTuple({});
  bool raised = false;
  try {
    env->Execute({bad, args->step}, bad);
  } catch (const Error& e) {
    raised = std::string(e.what()).find("field 2 of tensor_list is not a tensor") != std::string::npos;
  }
  EXPECT(raised);
  raised = false;
  try {
    auto shorter = value::MakeTuple(std::vector<value::Value>(fields.begin(), fields.begin() + 8));
    env->Execute({shorter, args->step}, shorter);
  } catch (const Error& e) {
    raised = std::string(e.what()).find("length changed") != std::string::npos;
  }
  EXPECT(raised);

  std::puts("sgd_multi reads the addresses at every call");
  auto sargs = std::make_shared<schema::SgdMultiArgs>();
  for (int i = 0; i < 3 * n; ++i) sargs->tensor_list.push_back(T(i));
  sargs->learning_rate = 0.1;
  sargs->mu = 0.9;
  auto scall = MakeCall("raf.op.sgd_multi", sargs);
  RunDeclare(scall);
  OpEnvPtr senv((*OpEnvMaker::Get("raf.op.hip.sgd_multi"))(scall));
  EXPECT(!senv->HasError());
  std::vector<value::Value> sfields(sargs->tensor_list.begin(), sargs->tensor_list.end());
  auto st = value::MakeTuple(sfields);
  senv->Execute({st}, st);
  EXPECT(g_sgd_steps == 1 && g_sgd_last[3] == &g_memory[3]);
  value::AsTensor(st->fields[3])->tensor.data = &g_memory[33];
  senv->Execute({st}, st);
  EXPECT(g_sgd_steps == 2 && g_sgd_last[3] == &g_memory[33]);

  std::puts("ALL OK");
  return 0;
}

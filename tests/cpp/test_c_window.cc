// The C entry points of rafhip_dialect.h driven the way the Python front end drives them, on a
// host without a GPU: operator makes that must fail cleanly for want of a device, whole traced
// optimizers that are built, fused and printed (and then refuse to dispatch), the cpu device API
// and its memory pool.  Meant to be run under AddressSanitizer / UndefinedBehaviorSanitizer.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "rafhip_dialect.h"

#define EXPECT(cond)                                                         \
  do {                                                                       \
    if (!(cond)) {                                                           \
      std::fprintf(stderr, "FAILED %s:%d: %s\n  last error: %s\n", __FILE__, __LINE__, #cond, \
                   rafhip_raf_last_error());                                 \
      std::exit(1);                                                          \
    }                                                                        \
  } while (0)

static bool Contains(const std::string& s, const char* what) { return s.find(what) != std::string::npos; }

struct Tensors {
  std::vector<std::vector<int64_t>> shapes;
  std::vector<rafhip_tensor_desc> descs;
  Tensors(const std::vector<std::vector<int64_t>>& shp, int device_type, int code, int bits) : shapes(shp) {
    for (auto& s : shapes) {
      rafhip_tensor_desc d;
      d.data = reinterpret_cast<void*>(0x1000);  // never dereferenced: nothing runs without a device
      d.device_type = device_type;
      d.device_id = 0;
      d.dtype_code = code;
      d.dtype_bits = bits;
      d.ndim = (int32_t)s.size();
      d.shape = s.data();
      descs.push_back(d);
    }
  }
};

int main() {
  const int kCpu = 1, kRocm = 10, kFloat = 2;
  const std::vector<std::vector<int64_t>> shapes = {{64, 32}, {32}, {7, 3, 5}};

  std::puts("dispatch lists and dialect preference");
  {
    char buf[256];
    EXPECT(rafhip_raf_dispatch_list("raf.op.lans", kRocm, buf, sizeof(buf)) == 0);
    EXPECT(std::string(buf) == "hip:raf.op.hip.lans:30");
    EXPECT(rafhip_raf_dispatch_list("raf.op.lans", kCpu, buf, sizeof(buf)) == 0 && std::string(buf).empty());
    EXPECT(rafhip_raf_set_dialect_preference("tvm") == 0);
    EXPECT(rafhip_raf_dispatch_list("raf.op.lans", kRocm, buf, sizeof(buf)) == 0 && std::string(buf).empty());
    EXPECT(rafhip_raf_set_dialect_preference(nullptr) == 0);
    EXPECT(rafhip_raf_dispatch_list(nullptr, kRocm, buf, sizeof(buf)) != 0);
  }

  std::puts("operator makes fail cleanly without a device");
  {
    Tensors f32(shapes, kRocm, kFloat, 32);
    rafhip_raf_env* env = reinterpret_cast<rafhip_raf_env*>(1);
    EXPECT(rafhip_raf_sgd_make(&f32.descs[0], &f32.descs[0], &f32.descs[0], 0.01, 0.9, &env) != 0);
    EXPECT(env == nullptr && Contains(rafhip_raf_last_error(), "Cannot find a valid dispatch for op raf.op.sgd"));
    EXPECT(Contains(rafhip_raf_last_error(), "no HIP device is visible"));
    std::vector<rafhip_tensor_desc> list;
    for (int q = 0; q < 4; ++q) list.insert(list.end(), f32.descs.begin(), f32.descs.end());
    std::vector<int64_t> none;
    rafhip_tensor_desc step = {reinterpret_cast<void*>(0x1000), kRocm, 0, kFloat, 32, 0, none.data()};
    EXPECT(rafhip_raf_lans_make((int32_t)list.size(), list.data(), &step, 1e-3f, 0.9f, 0.999f, 1e-6f, 1, 0.01f, 1, 1, 1,
                                &env) != 0);
    EXPECT(env == nullptr && Contains(rafhip_raf_last_error(), "raf.op.lans"));
    // a list that is not 4n long is refused by the op's declare function
    EXPECT(rafhip_raf_lans_make(3, list.data(), &step, 1e-3f, 0.9f, 0.999f, 1e-6f, 1, 0.01f, 1, 1, 1, &env) != 0);
    EXPECT(rafhip_raf_l2norm_make(&f32.descs[0], &env) != 0 && env == nullptr);
    EXPECT(rafhip_raf_fuse_tensor_make(3, f32.descs.data(), &env) != 0 && env == nullptr);
    // an empty list is declared as a no-op: an env without an OpEnv
    EXPECT(rafhip_raf_fuse_tensor_make(0, nullptr, &env) == 0 && env != nullptr);
    EXPECT(rafhip_raf_env_num_outputs(env) == 0 && rafhip_raf_env_workspace_bytes(env) == 0);
    EXPECT(rafhip_raf_env_set_learning_rate(env, 0.1) == 0);
    EXPECT(rafhip_raf_env_destroy(env) == 0);
    EXPECT(rafhip_raf_env_set_grad_unscale(nullptr, 1.f) != 0);
  }

  std::puts("traced optimizers: built, fused, printed; dispatch refuses without a device");
  for (int kind = 0; kind < 2; ++kind) {
    for (int zero_is_constant = 0; zero_is_constant < 2; ++zero_is_constant) {
      Tensors g(shapes, kRocm, kFloat, 16), w(shapes, kRocm, kFloat, 32), m(shapes, kRocm, kFloat, 32),
          v(shapes, kRocm, kFloat, 32), p(shapes, kRocm, kFloat, 16);
      std::vector<int64_t> none;
      rafhip_tensor_desc step = {reinterpret_cast<void*>(0x1000), kRocm, 0, kFloat, 32, 0, none.data()};
      const double sgd_hyper[2] = {0.01, 0.9};
      const double lans_hyper[9] = {1e-3, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, 1};
      rafhip_raf_env* env = nullptr;
      int st = rafhip_raf_traced_optimizer_make(kind, 3, g.descs.data(), w.descs.data(), m.descs.data(),
                                                v.descs.data(), p.descs.data(), &step, zero_is_constant,
                                                kind == 0 ? sgd_hyper : lans_hyper, kind == 0 ? 2 : 9, 1, &env);
      EXPECT(st != 0 && env != nullptr);  // the graphs exist, the dispatch of the fused call failed
      EXPECT(Contains(rafhip_raf_last_error(), "no HIP device is visible"));
      std::vector<char> buf(1 << 16);
      EXPECT(rafhip_raf_env_ir_text(env, 0, buf.data(), (int32_t)buf.size()) == 0);
      const std::string before(buf.data());
      EXPECT(rafhip_raf_env_ir_text(env, 1, buf.data(), (int32_t)buf.size()) == 0);
      const std::string after(buf.data());
      EXPECT(!Contains(before, "hip") && Contains(before, kind == 0 ? "raf.op.subtract(" : "raf.op.group_cast("));
      if (kind == 0)
        EXPECT(Contains(after, zero_is_constant ? "raf.op.hip.sgd_multi_mixed(" : "raf.op.hip.sgd_multi("));
      else
        EXPECT(Contains(after, zero_is_constant ? "raf.op.hip.lans_mixed(" : "raf.op.hip.lans("));
      EXPECT(Contains(after, "raf.op.cast(") == (zero_is_constant == 0));
      EXPECT(rafhip_raf_env_ir_text(env, 1, buf.data(), 8) != 0);  // buffer too small
      EXPECT(rafhip_raf_traced_optimizer_execute(env, 3, g.descs.data(), w.descs.data(), m.descs.data(),
                                                 v.descs.data(), p.descs.data(), &step, 1, nullptr, 0, nullptr) != 0);
      EXPECT(rafhip_raf_env_destroy(env) == 0);
    }
  }
  {
    // on the cpu device nothing fuses and nothing dispatches; bad arguments are refused
    Tensors w(shapes, kCpu, kFloat, 32);
    const double hyper[2] = {0.01, 0.9};
    rafhip_raf_env* env = nullptr;
    EXPECT(rafhip_raf_traced_optimizer_make(0, 3, w.descs.data(), w.descs.data(), nullptr, w.descs.data(), nullptr,
                                            nullptr, 1, hyper, 2, 0, &env) != 0);
    EXPECT(env != nullptr && Contains(rafhip_raf_last_error(), "Cannot find a valid dispatch for op raf.op.multiply"));
    EXPECT(rafhip_raf_env_destroy(env) == 0);
    env = nullptr;
    EXPECT(rafhip_raf_traced_optimizer_make(2, 3, w.descs.data(), w.descs.data(), nullptr, w.descs.data(), nullptr,
                                            nullptr, 1, hyper, 2, 0, &env) != 0 && env == nullptr);
    EXPECT(rafhip_raf_traced_optimizer_make(1, 3, w.descs.data(), w.descs.data(), nullptr, w.descs.data(), nullptr,
                                            nullptr, 1, hyper, 2, 0, &env) != 0 && env == nullptr);
    EXPECT(rafhip_raf_traced_sgd_make(&w.descs[0], &w.descs[0], &w.descs[0], 0.01, 0.9, &env) != 0);
    EXPECT(Contains(rafhip_raf_last_error(), "no fuse pattern matched on device type cpu"));
    if (env) EXPECT(rafhip_raf_env_destroy(env) == 0);
  }

  std::puts("cpu device API and memory pool");
  {
    int32_t count = -1;
    EXPECT(rafhip_raf_device_count(kCpu, &count) == 0 && count >= 1);
    EXPECT(rafhip_raf_device_count(kRocm, &count) != 0 || count == 0);  // no device behind the stub
    rafhip_raf_memory* mem = nullptr;
    EXPECT(rafhip_raf_memory_alloc(kCpu, 0, 1000, 64, 0, nullptr, &mem) == 0 && mem != nullptr);
    char* data = static_cast<char*>(rafhip_raf_memory_data(mem));
    EXPECT(data != nullptr && reinterpret_cast<uintptr_t>(data) % 64 == 0);
    std::memset(data, 7, 1000);
    char name[64];
    float used = 0, pool = 0;
    EXPECT(rafhip_raf_pool_info(kCpu, 0, name, sizeof(name), &used, &pool) == 0 && std::string(name) == "page_unit_pool");
    EXPECT(rafhip_raf_pool_alloc_bytes(kCpu, 0, 1000) >= 1000);
    std::vector<int64_t> shape = {250};
    rafhip_tensor_desc src = {data, kCpu, 0, kFloat, 32, 1, shape.data()};
    rafhip_raf_memory* mem2 = nullptr;
    EXPECT(rafhip_raf_memory_alloc(kCpu, 0, 1000, 0, 0, nullptr, &mem2) == 0);
    rafhip_tensor_desc dst = {rafhip_raf_memory_data(mem2), kCpu, 0, kFloat, 32, 1, shape.data()};
    EXPECT(rafhip_raf_device_copy(&src, &dst, nullptr) == 0);
    EXPECT(std::memcmp(data, rafhip_raf_memory_data(mem2), 1000) == 0);
    EXPECT(rafhip_raf_memory_free(mem) == 0 && rafhip_raf_memory_free(mem2) == 0);
    EXPECT(rafhip_raf_pool_reset(kCpu, 0) == 0);
    EXPECT(rafhip_raf_pool_init(kCpu, 0, "no_pool") == 0);
    EXPECT(rafhip_raf_memory_alloc(kCpu, 0, 128, 64, 0, nullptr, &mem) == 0 && rafhip_raf_memory_free(mem) == 0);
    EXPECT(rafhip_raf_pool_init(kCpu, 0, "no_such_pool") != 0);
    EXPECT(rafhip_raf_pool_init(kCpu, 0, "page_unit_pool") == 0);
    EXPECT(rafhip_raf_memory_alloc(kRocm, 0, 128, 64, 0, nullptr, &mem) != 0);  // no device behind the stub
    void* stream = nullptr;
    EXPECT(rafhip_raf_stream_create(kCpu, 0, &stream) == 0 || Contains(rafhip_raf_last_error(), "cpu"));
  }

  std::puts("ALL OK");
  return 0;
}

// Device APIs behind the DeviceAPI interface of raf_iface.h.
//
//   ROCMDeviceAPI  the ROCm counterpart of the reference's CUDADeviceAPI
//                  (src/device_api/cuda/cuda.cc:25-248): what RAF lacks to place tensors on
//                  DevType::kROCM.  Every method is one call into the C ABI of rafhip_device.h, so
//                  this file needs no HIP headers and compiles with the host compiler.
//   CPUDeviceAPI   src/device_api/cpu/cpu.cc:18-131: aligned host memory, memcpy, and errors for
//                  everything that needs a stream or an event.
//   DeviceAPI::Get / RegisterMaker   src/impl/device_api.cc:18-50.
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <thread>

#include "raf_iface.h"
#include "rafhip_device.h"
#include "rafhip_optim.h"

namespace raf {
namespace device_api {

namespace {

std::mutex& Mu() {
  static std::mutex m;
  return m;
}
std::map<std::string, DeviceAPI::Maker>& Makers() {
  static std::map<std::string, DeviceAPI::Maker> m;
  return m;
}
std::map<int, std::shared_ptr<DeviceAPI>>& Instances() {
  static std::map<int, std::shared_ptr<DeviceAPI>> m;
  return m;
}

int64_t ByteSize(const TensorView& t) { return t.numel() * ((t.dtype.bits + 7) / 8); }

// A failed runtime call becomes a raf::Error, like CUDA_CALL's LOG(FATAL)
// (src/common/cuda_utils.h:10-14).
void Try(int status, const char* what) {
  if (status != RAFHIP_OK)
    throw Error(std::string(what) + " failed with status " + std::to_string(status) + ": " +
                rafhip_last_error());
}

class CPUDeviceAPI final : public DeviceAPI {
 public:
  int GetDeviceCount() override { return (int)std::thread::hardware_concurrency(); }
  void* AllocMemory(int64_t nbytes, int64_t alignment) override {
    void* ptr = nullptr;
    if (posix_memalign(&ptr, (size_t)alignment, (size_t)nbytes) != 0) throw std::bad_alloc();
    return ptr;
  }
  void* AllocMemoryAsync(int64_t, void*, int64_t) override { Unsupported("AllocMemoryAsync"); }
  void FreeMemory(void* ptr) override { free(ptr); }
  void FreeMemoryAsync(void*, void*) override { Unsupported("FreeMemoryAsync"); }
  void CopyDataFromTo(const TensorView& from, const TensorView& to, void*) override {
    RAF_CHECK(ByteSize(from) == ByteSize(to), "CopyDataFromTo: sizes differ");
    std::memcpy(to.data, from.data, (size_t)ByteSize(from));
  }
  void SetDevice(const int) override { Unsupported("SetDevice"); }
  void* CreateStream(const Device&) override { Unsupported("CreateStream"); }
  void FreeStream(const Device&, void*) override { Unsupported("FreeStream"); }
  void SetStream(const Device&, void*) override { Unsupported("SetStream"); }
  void* GetStream() override { return nullptr; }
  void* CreateEvent(const Device&, uint32_t) override { Unsupported("CreateEvent"); }
  void FreeEvent(const Device&, void*) override { Unsupported("FreeEvent"); }
  float EventElapsedTimeInMilliSeconds(void*, void*) override { Unsupported("EventElapsedTimeInMilliSeconds"); }
  void EventRecordOnStream(void*, void*) override { Unsupported("EventRecordOnStream"); }
  void StreamWaitEvent(void*, void*) override { Unsupported("StreamWaitEvent"); }
  void WaitDevice(const Device&) override {}
  void WaitStream(void*) override { Unsupported("WaitStream"); }
  void WaitEvent(void*) override { Unsupported("WaitEvent"); }
  static DeviceAPI* make() { return new CPUDeviceAPI(); }

 private:
  [[noreturn]] static void Unsupported(const char* what) {
    throw Error(std::string("the cpu device API has no ") + what);
  }
};

class ROCMDeviceAPI final : public DeviceAPI {
 public:
  int GetDeviceCount() override { return rafhip_device_count(); }

  void* AllocMemory(int64_t nbytes, int64_t alignment) override {
    RAF_CHECK(alignment <= 256, "hipMalloc guarantees 256-byte alignment, not more");
    Try(rafhip_dev_set(device_id_), "hipSetDevice");
    void* ptr = nullptr;
    Try(rafhip_dev_alloc(nbytes, &ptr), "hipMalloc");
    return ptr;
  }
  void FreeMemory(void* ptr) override { Try(rafhip_dev_free(ptr), "hipFree"); }

  void* AllocMemoryAsync(int64_t nbytes, void* stream, int64_t alignment) override {
    RAF_CHECK(alignment <= 256, "the HIP memory pool guarantees 256-byte alignment, not more");
    void* ptr = nullptr;
    Try(rafhip_dev_alloc_async(device_id_, nbytes, stream, &ptr), "hipMallocFromPoolAsync");
    return ptr;
  }
  void FreeMemoryAsync(void* ptr, void* stream) override {
    Try(rafhip_dev_free_async(ptr, stream), "hipFreeAsync");
  }

  std::pair<int64_t, int64_t> GetPoolSize() override {
    int64_t used = 0, reserved = 0;
    Try(rafhip_dev_pool_size(device_id_, &used, &reserved), "hipMemPoolGetAttribute");
    return {used, reserved};
  }

  void SetDevice(const int device_id) override {
    device_id_ = device_id;
    Try(rafhip_dev_set(device_id), "hipSetDevice");
  }

  void CopyDataFromTo(const TensorView& from, const TensorView& to, void* stream) override {
    const int64_t nbytes = ByteSize(from);
    RAF_CHECK(nbytes == ByteSize(to), "CopyDataFromTo: sizes differ");
    const bool from_dev = from.device.device_type() == DevType::kROCM();
    const bool to_dev = to.device.device_type() == DevType::kROCM();
    if (!from_dev && !to_dev) {  // host to host (cuda.cc:126-129)
      Try(rafhip_dev_memcpy(to.data, from.data, nbytes, RAFHIP_COPY_H2H, nullptr), "memcpy");
      return;
    }
    const int current = device_id_;
    if (from_dev && to_dev) {
      SetDevice(from.device.device_id());
      if (from.device.device_id() == to.device.device_id())
        Try(rafhip_dev_memcpy(to.data, from.data, nbytes, RAFHIP_COPY_D2D, stream), "hipMemcpy");
      else
        Try(rafhip_dev_memcpy_peer(to.data, to.device.device_id(), from.data,
                                   from.device.device_id(), nbytes, stream),
            "hipMemcpyPeerAsync");
    } else if (from_dev) {
      SetDevice(from.device.device_id());
      Try(rafhip_dev_memcpy(to.data, from.data, nbytes, RAFHIP_COPY_D2H, stream), "hipMemcpy");
    } else {
      SetDevice(to.device.device_id());
      Try(rafhip_dev_memcpy(to.data, from.data, nbytes, RAFHIP_COPY_H2D, stream), "hipMemcpy");
    }
    SetDevice(current);
  }

  void* CreateStream(const Device& dev) override {
    RAF_CHECK(dev.device_type() == DevType::kROCM(), "not a rocm device");
    void* s = nullptr;
    Try(rafhip_dev_stream_create(dev.device_id(), &s), "hipStreamCreate");
    return s;
  }
  void FreeStream(const Device& dev, void* stream) override {
    RAF_CHECK(dev.device_type() == DevType::kROCM(), "not a rocm device");
    Try(rafhip_dev_stream_destroy(dev.device_id(), stream), "hipStreamDestroy");
  }
  // The reference also forwards the stream to TVM, cuDNN and cuBLAS (cuda.cc:173-178); the hip
  // dialect's OpEnvs read it from here at Execute time.
  void SetStream(const Device&, void* stream) override { stream_ = stream; }
  void* GetStream() override { return stream_; }

  void* CreateEvent(const Device& dev, uint32_t flags) override {
    RAF_CHECK(dev.device_type() == DevType::kROCM(), "not a rocm device");
    void* e = nullptr;
    Try(rafhip_dev_event_create(dev.device_id(), flags, &e), "hipEventCreateWithFlags");
    return e;
  }
  void FreeEvent(const Device& dev, void* event) override {
    RAF_CHECK(dev.device_type() == DevType::kROCM(), "not a rocm device");
    Try(rafhip_dev_event_destroy(dev.device_id(), event), "hipEventDestroy");
  }
  float EventElapsedTimeInMilliSeconds(void* start_event, void* end_event) override {
    float ms = 0.f;
    Try(rafhip_dev_event_elapsed_ms(start_event, end_event, &ms), "hipEventElapsedTime");
    return ms;
  }
  void EventRecordOnStream(void* event, void* stream) override {
    Try(rafhip_dev_event_record(event, stream), "hipEventRecord");
  }
  void StreamWaitEvent(void* stream, void* event) override {
    Try(rafhip_dev_stream_wait_event(stream, event), "hipStreamWaitEvent");
  }
  void WaitDevice(const Device& dev) override {
    RAF_CHECK(dev.device_type() == DevType::kROCM(), "not a rocm device");
    Try(rafhip_dev_sync_device(dev.device_id()), "hipDeviceSynchronize");
  }
  void WaitStream(void* stream) override { Try(rafhip_dev_sync_stream(stream), "hipStreamSynchronize"); }
  void WaitEvent(void* event) override {
    RAF_CHECK(event != nullptr, "Cannot sync a null event");
    Try(rafhip_dev_sync_event(event), "hipEventSynchronize");
  }
  static DeviceAPI* make() { return new ROCMDeviceAPI(); }

 private:
  int device_id_ = 0;
  void* stream_ = nullptr;  // the default stream unless the executor sets one
};

const bool kCpuRegistered = DeviceAPI::RegisterMaker("cpu", CPUDeviceAPI::make);
const bool kRocmRegistered = DeviceAPI::RegisterMaker("rocm", ROCMDeviceAPI::make);

}  // namespace

bool DeviceAPI::RegisterMaker(const std::string& devtype_name, Maker maker) {
  std::lock_guard<std::mutex> lock(Mu());
  Makers()[devtype_name] = maker;
  return true;
}

std::shared_ptr<DeviceAPI> DeviceAPI::Get(DevType device_type) {
  std::lock_guard<std::mutex> lock(Mu());
  auto& slot = Instances()[(int)device_type];
  if (!slot) {
    auto it = Makers().find(device_type.c_str());
    if (it == Makers().end())
      throw Error(std::string("no device API registered as raf.device_api._make.") +
                  device_type.c_str());
    slot.reset(it->second());
  }
  return slot;
}

}  // namespace device_api
}  // namespace raf

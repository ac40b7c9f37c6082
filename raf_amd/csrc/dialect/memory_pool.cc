// Pool manager and the two pool strategies declared in memory_pool.h.
#include "memory_pool.h"

#include <cstdio>
#include <cstdlib>
#include <list>
#include <map>
#include <mutex>
#include <unordered_map>

namespace raf {
namespace memory_pool {

using device_api::DeviceAPI;

namespace {

// ------------------------------------------------------------------------------- the manager
std::mutex& Mu() {
  static std::mutex m;
  return m;
}
std::map<std::string, MemoryPool::Maker>& Makers() {
  static std::map<std::string, MemoryPool::Maker> m;
  return m;
}
std::map<std::pair<int, int>, std::shared_ptr<MemoryPool>>& Pools() {
  static std::map<std::pair<int, int>, std::shared_ptr<MemoryPool>> m;
  return m;
}

// src/impl/memory_pool.cc:28-36, plus the rocm entry.  The HIP runtime has stream-ordered
// allocation, so rocm goes the way cuda >= 11.3 does.
std::string DefaultStrategy(DevType t) {
  if (t == DevType::kROCM()) return "no_pool";
  if (t == DevType::kCUDA()) return "no_pool";
  return "page_unit_pool";
}

MemoryPool* PoolOf(const Device& dev, const std::string& name) {
  std::lock_guard<std::mutex> lock(Mu());
  auto& slot = Pools()[{(int)dev.device_type(), dev.device_id()}];
  if (!slot) {
    const std::string pool_name = name.empty() ? DefaultStrategy(dev.device_type()) : name;
    auto it = Makers().find(pool_name);
    if (it == Makers().end()) throw Error("no memory pool registered as raf.memory_pool._make." + pool_name);
    slot.reset(it->second(dev));
  }
  return slot.get();
}

void CheckAlignment(int64_t alignment) {  // src/impl/memory_pool.cc:83-87
  RAF_CHECK(alignment % kDefaultMemoryAlignment == 0,
            "Requested memory with alignment " + std::to_string(alignment) + " is not aligned to " +
                std::to_string(kDefaultMemoryAlignment));
}

bool IsGpu(DevType t) { return t == DevType::kCUDA() || t == DevType::kROCM(); }

// A destructor must not throw: a failed release (the device API reports failures as raf::Error)
// is written to stderr and otherwise dropped.
template <typename F>
void Release(F&& free_it) noexcept {
  try {
    free_it();
  } catch (const std::exception& e) {
    std::fprintf(stderr, "raf memory pool: releasing memory failed: %s\n", e.what());
  } catch (...) {
    std::fprintf(stderr, "raf memory pool: releasing memory failed\n");
  }
}

// ---------------------------------------------------------------------------------- chunks
// Memory returned to the device API when the last reference goes.
class NonOwnedMemory final : public Memory {
 public:
  NonOwnedMemory(void* ptr, const Device& dev, std::shared_ptr<DeviceAPI> api) : api_(std::move(api)) {
    data = ptr;
    device = dev;
  }
  ~NonOwnedMemory() override {
    if (data != nullptr) Release([&] { api_->FreeMemory(data); });
  }

 private:
  std::shared_ptr<DeviceAPI> api_;
};

// Stream-ordered: freed on the stream it was allocated on.
class NonOwnedAsyncMemory final : public Memory {
 public:
  NonOwnedAsyncMemory(void* ptr, void* stream, const Device& dev, std::shared_ptr<DeviceAPI> api)
      : api_(std::move(api)), stream_(stream) {
    data = ptr;
    device = dev;
  }
  ~NonOwnedAsyncMemory() override {
    if (data != nullptr) Release([&] { api_->FreeMemoryAsync(data, stream_); });
  }

 private:
  std::shared_ptr<DeviceAPI> api_;
  void* stream_;
};

// ----------------------------------------------------------------------------------- no_pool
// Every request goes straight to the device API (no_pool.cc:60-121).
class NoPool final : public MemoryPool {
 public:
  explicit NoPool(const Device& dev) : device_(dev), api_(DeviceAPI::Get(dev.device_type())) {
    if (IsGpu(dev.device_type())) api_->SetDevice(dev.device_id());
  }
  std::string GetName() override { return "no_pool"; }
  int64_t GetAllocBytes(int64_t nbytes) override { return nbytes; }

  std::shared_ptr<Memory> Alloc(int64_t nbytes, int64_t alignment) override {
    RAF_CHECK(nbytes >= 0, "negative allocation size");
    void* ptr = nbytes > 0 ? api_->AllocMemory(nbytes, alignment) : nullptr;
    return std::make_shared<NonOwnedMemory>(ptr, device_, api_);
  }
  std::shared_ptr<Memory> AllocAsync(int64_t nbytes, void* stream, int64_t alignment) override {
    RAF_CHECK(nbytes >= 0, "negative allocation size");
    void* ptr = nbytes > 0 ? api_->AllocMemoryAsync(nbytes, stream, alignment) : nullptr;
    return std::make_shared<NonOwnedAsyncMemory>(ptr, stream, device_, api_);
  }
  std::vector<std::shared_ptr<Memory>> AllocBatch(const std::vector<int64_t>& nbytes,
                                                  int64_t alignment) override {
    std::vector<std::shared_ptr<Memory>> ret;
    ret.reserve(nbytes.size());
    for (int64_t b : nbytes) ret.push_back(Alloc(b, alignment));
    return ret;
  }
  std::pair<float, float> GetPoolSize() override {
    auto sz = api_->GetPoolSize();
    return {BytesToMegaBytes((float)sz.first), BytesToMegaBytes((float)sz.second)};
  }
  static MemoryPool* make(const Device& dev) { return new NoPool(dev); }

 private:
  Device device_;
  std::shared_ptr<DeviceAPI> api_;
};

// ---------------------------------------------------------------------------- page_unit_pool
// Requests are rounded up to 4 KiB pages and chunks are kept, grouped by size, after their users
// let go; a request takes an idle chunk of its size if there is one.  When the device runs out of
// memory, or the pool outgrows RAF_MEMORY_POOL_SIZE_LIMIT, idle chunks are released and the
// allocation is tried once more (page_unit_pool.cc:64-231).
class PageUnitPool final : public MemoryPool {
 public:
  PageUnitPool(const Device& dev, int64_t limit)
      : device_(dev), max_pool_size_(limit), api_(DeviceAPI::Get(dev.device_type())) {
    if (IsGpu(dev.device_type())) api_->SetDevice(dev.device_id());
  }
  std::string GetName() override { return "page_unit_pool"; }
  int64_t GetAllocBytes(int64_t nbytes) override {
    return (nbytes + kPage - 1) / kPage * kPage;
  }

  std::shared_ptr<Memory> Alloc(int64_t nbytes, int64_t alignment) override {
    RAF_CHECK(nbytes >= 0, "negative allocation size");
    nbytes = GetAllocBytes(nbytes);
    if (nbytes == 0) return std::make_shared<NonOwnedMemory>(nullptr, device_, api_);
    std::lock_guard<std::mutex> lock(mu_);
    auto& chunks = pool_[nbytes];
    for (const auto& c : chunks)  // the pool's own reference is the only one: the chunk is idle
      if (c.use_count() == 1 && reinterpret_cast<uintptr_t>(c->data) % (uintptr_t)alignment == 0) return c;
    void* ptr = TryDevice(nbytes, alignment);
    if (ptr == nullptr || (max_pool_size_ > 0 && pool_bytes_ >= max_pool_size_)) {
      const int64_t freed = FreeIdleChunks();
      if (ptr == nullptr && freed > 0) ptr = TryDevice(nbytes, alignment);
    }
    if (ptr == nullptr) {
      auto sz = SizesLocked();
      throw Error("Out-Of-Memory. Tried to allocate " + std::to_string(BytesToMegaBytes((float)nbytes)) +
                  " MBs; Already allocated " + std::to_string(sz.second) + " MBs and used " +
                  std::to_string(sz.first) + " MBs");
    }
    pool_bytes_ += nbytes;
    auto mem = std::make_shared<NonOwnedMemory>(ptr, device_, api_);
    pool_[nbytes].push_back(mem);
    return mem;
  }
  std::shared_ptr<Memory> AllocAsync(int64_t, void*, int64_t) override {
    throw Error("Please use NoPool to use AllocAsync.");
  }
  std::vector<std::shared_ptr<Memory>> AllocBatch(const std::vector<int64_t>& nbytes,
                                                  int64_t alignment) override {
    std::vector<std::shared_ptr<Memory>> ret;
    ret.reserve(nbytes.size());
    for (int64_t b : nbytes) ret.push_back(Alloc(b, alignment));
    return ret;
  }
  std::pair<float, float> GetPoolSize() override {
    auto dev = api_->GetPoolSize();  // a device-side pool's own numbers win if it has any
    if (dev.first != 0 || dev.second != 0)
      return {BytesToMegaBytes((float)dev.first), BytesToMegaBytes((float)dev.second)};
    std::lock_guard<std::mutex> lock(mu_);
    return SizesLocked();
  }
  static MemoryPool* make(const Device& dev) {
    int64_t limit = 0;
    if (const char* v = std::getenv("RAF_MEMORY_POOL_SIZE_LIMIT")) limit = std::atoll(v);
    return new PageUnitPool(dev, limit);
  }

 private:
  static constexpr int64_t kPage = 4096;

  void* TryDevice(int64_t nbytes, int64_t alignment) {
    try {
      return api_->AllocMemory(nbytes, alignment);
    } catch (const std::exception&) {
      return nullptr;
    }
  }
  int64_t FreeIdleChunks() {
    int64_t freed = 0;
    pool_bytes_ = 0;
    for (auto& kv : pool_) {
      const size_t before = kv.second.size();
      kv.second.remove_if([](const std::shared_ptr<Memory>& m) { return m.use_count() == 1; });
      freed += kv.first * (int64_t)(before - kv.second.size());
      pool_bytes_ += kv.first * (int64_t)kv.second.size();
    }
    return freed;
  }
  std::pair<float, float> SizesLocked() {
    float used = 0.f, total = 0.f;
    for (auto& kv : pool_) {
      size_t busy = 0;
      for (const auto& c : kv.second) busy += c.use_count() > 1 ? 1 : 0;
      used += BytesToMegaBytes((float)(kv.first * (int64_t)busy));
      total += BytesToMegaBytes((float)(kv.first * (int64_t)kv.second.size()));
    }
    return {used, total};
  }

  Device device_;
  int64_t pool_bytes_ = 0;
  int64_t max_pool_size_ = 0;  // 0 = no limit
  std::shared_ptr<DeviceAPI> api_;
  std::mutex mu_;
  std::unordered_map<int64_t, std::list<std::shared_ptr<Memory>>> pool_;
};

const bool kNoPoolRegistered = MemoryPool::RegisterMaker("no_pool", NoPool::make);
const bool kPageUnitRegistered = MemoryPool::RegisterMaker("page_unit_pool", PageUnitPool::make);

}  // namespace

bool MemoryPool::RegisterMaker(const std::string& pool_name, Maker maker) {
  std::lock_guard<std::mutex> lock(Mu());
  Makers()[pool_name] = maker;
  return true;
}

int64_t Memory::GetAllocBytes(const Device& dev, int64_t nbytes) {
  return PoolOf(dev, "")->GetAllocBytes(nbytes);
}
std::shared_ptr<Memory> Memory::Alloc(const Device& dev, int64_t nbytes, int64_t alignment) {
  CheckAlignment(alignment);
  return PoolOf(dev, "")->Alloc(nbytes, alignment);
}
std::shared_ptr<Memory> Memory::AllocAsync(const Device& dev, int64_t nbytes, void* stream,
                                           int64_t alignment) {
  CheckAlignment(alignment);
  return PoolOf(dev, "")->AllocAsync(nbytes, stream, alignment);
}
std::vector<std::shared_ptr<Memory>> Memory::AllocBatch(const Device& dev,
                                                        const std::vector<int64_t>& nbytes,
                                                        int64_t alignment) {
  CheckAlignment(alignment);
  return PoolOf(dev, "")->AllocBatch(nbytes, alignment);
}
std::pair<float, float> Memory::GetPoolSize(const Device& dev) { return PoolOf(dev, "")->GetPoolSize(); }

void Memory::RemovePool(const Device& dev) {
  std::lock_guard<std::mutex> lock(Mu());
  Pools().erase({(int)dev.device_type(), dev.device_id()});
}
MemoryPool* Memory::ResetPool(const Device& dev) {
  const std::string name = PoolOf(dev, "")->GetName();
  RemovePool(dev);
  return PoolOf(dev, name);
}
MemoryPool* Memory::GetPool(const Device& dev) { return PoolOf(dev, ""); }
MemoryPool* Memory::InitPool(const Device& dev, const std::string& name) { return PoolOf(dev, name); }

void InitPool(const Device& dev, const std::string& pool_name) {
  Memory::RemovePool(dev);  // src/impl/memory_pool.cc:160-163
  Memory::InitPool(dev, pool_name);
}
void RemovePool(const Device& dev) { Memory::RemovePool(dev); }
void ResetPool(const Device& dev) { Memory::ResetPool(dev); }

}  // namespace memory_pool
}  // namespace raf

// Pool manager and the two pool strategies declared in memory_pool.h.
#include "memory_pool.h"

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <vector>

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
// The reference's caching strategy (page_unit_pool.cc:64-231): requests are rounded up to 4 KiB
// pages, a block whose users have let go is kept for the next request of its size, and when the
// device runs out of memory, or the pool outgrows RAF_MEMORY_POOL_SIZE_LIMIT, the idle blocks
// go back to the device and the allocation is tried once more.
//
// Bookkeeping here: a block handed out is a `Lease` whose destructor returns the block to a
// per-size free list, so taking and returning a block are O(1) and the pool never scans for
// blocks that have become idle.  The free lists live in a `Ledger` that the leases share with
// the pool: a lease that outlives its pool (RemovePool while tensors are alive) finds the ledger
// closed and hands its block straight back to the device.
class PageUnitPool final : public MemoryPool {
  struct Ledger {
    std::mutex mu;
    std::shared_ptr<DeviceAPI> api;
    std::map<int64_t, std::vector<void*>> idle;  // page-rounded size -> blocks nobody holds
    int64_t idle_bytes = 0;
    int64_t leased_bytes = 0;
    bool closed = false;

    // Returns every idle block to the device; the number of bytes that freed.
    int64_t DrainLocked() {
      const int64_t freed = idle_bytes;
      for (auto& bucket : idle)
        for (void* block : bucket.second) Release([&] { api->FreeMemory(block); });
      idle.clear();
      idle_bytes = 0;
      return freed;
    }
  };

  class Lease final : public Memory {
   public:
    Lease(void* ptr, int64_t nbytes, const Device& dev, std::shared_ptr<Ledger> ledger)
        : nbytes_(nbytes), ledger_(std::move(ledger)) {
      data = ptr;
      device = dev;
    }
    ~Lease() override {
      if (data == nullptr) return;
      std::lock_guard<std::mutex> lock(ledger_->mu);
      ledger_->leased_bytes -= nbytes_;
      if (ledger_->closed) {
        Release([&] { ledger_->api->FreeMemory(data); });
        return;
      }
      ledger_->idle[nbytes_].push_back(data);
      ledger_->idle_bytes += nbytes_;
    }

   private:
    int64_t nbytes_;
    std::shared_ptr<Ledger> ledger_;
  };

 public:
  PageUnitPool(const Device& dev, int64_t limit)
      : device_(dev), size_limit_(limit), ledger_(std::make_shared<Ledger>()) {
    ledger_->api = DeviceAPI::Get(dev.device_type());
    if (IsGpu(dev.device_type())) ledger_->api->SetDevice(dev.device_id());
  }
  ~PageUnitPool() override {
    std::lock_guard<std::mutex> lock(ledger_->mu);
    ledger_->closed = true;
    ledger_->DrainLocked();
  }
  std::string GetName() override { return "page_unit_pool"; }
  int64_t GetAllocBytes(int64_t nbytes) override { return (nbytes + kPage - 1) / kPage * kPage; }

  std::shared_ptr<Memory> Alloc(int64_t nbytes, int64_t alignment) override {
    RAF_CHECK(nbytes >= 0, "negative allocation size");
    nbytes = GetAllocBytes(nbytes);
    if (nbytes == 0) return std::make_shared<Lease>(nullptr, 0, device_, ledger_);
    std::lock_guard<std::mutex> lock(ledger_->mu);
    void* block = TakeIdleLocked(nbytes, alignment);
    if (block == nullptr) {
      block = TryDevice(nbytes, alignment);
      const bool over_limit =
          size_limit_ > 0 && ledger_->idle_bytes + ledger_->leased_bytes + (block ? nbytes : 0) > size_limit_;
      if (block == nullptr || over_limit) {
        const int64_t freed = ledger_->DrainLocked();
        if (block == nullptr && freed > 0) block = TryDevice(nbytes, alignment);
      }
      if (block == nullptr) {
        // the reference's message (page_unit_pool.cc:112-117): its tests match on it
        throw Error("Out-Of-Memory. Tried to allocate " + std::to_string(BytesToMegaBytes((float)nbytes)) +
                    " MBs; Already allocated " +
                    std::to_string(BytesToMegaBytes((float)(ledger_->idle_bytes + ledger_->leased_bytes))) +
                    " MBs and used " + std::to_string(BytesToMegaBytes((float)ledger_->leased_bytes)) + " MBs");
      }
    }
    ledger_->leased_bytes += nbytes;
    return std::make_shared<Lease>(block, nbytes, device_, ledger_);
  }
  std::shared_ptr<Memory> AllocAsync(int64_t, void*, int64_t) override {
    throw Error("Please use NoPool to use AllocAsync.");  // page_unit_pool.cc:127
  }
  std::vector<std::shared_ptr<Memory>> AllocBatch(const std::vector<int64_t>& nbytes,
                                                  int64_t alignment) override {
    std::vector<std::shared_ptr<Memory>> blocks(nbytes.size());
    for (size_t i = 0; i < nbytes.size(); ++i) blocks[i] = Alloc(nbytes[i], alignment);
    return blocks;
  }
  std::pair<float, float> GetPoolSize() override {
    auto dev = ledger_->api->GetPoolSize();  // a device-side pool's own numbers win if it has any
    if (dev.first != 0 || dev.second != 0)
      return {BytesToMegaBytes((float)dev.first), BytesToMegaBytes((float)dev.second)};
    std::lock_guard<std::mutex> lock(ledger_->mu);
    return {BytesToMegaBytes((float)ledger_->leased_bytes),
            BytesToMegaBytes((float)(ledger_->leased_bytes + ledger_->idle_bytes))};
  }
  static MemoryPool* make(const Device& dev) {
    int64_t limit = 0;
    if (const char* v = std::getenv("RAF_MEMORY_POOL_SIZE_LIMIT")) limit = std::atoll(v);
    return new PageUnitPool(dev, limit);
  }

 private:
  static constexpr int64_t kPage = 4096;

  // The most recently returned idle block of this size that satisfies the alignment, if any.
  void* TakeIdleLocked(int64_t nbytes, int64_t alignment) {
    auto bucket = ledger_->idle.find(nbytes);
    if (bucket == ledger_->idle.end()) return nullptr;
    std::vector<void*>& blocks = bucket->second;
    for (size_t i = blocks.size(); i-- > 0;) {
      if (reinterpret_cast<uintptr_t>(blocks[i]) % (uintptr_t)alignment != 0) continue;
      void* block = blocks[i];
      blocks.erase(blocks.begin() + (std::ptrdiff_t)i);
      if (blocks.empty()) ledger_->idle.erase(bucket);
      ledger_->idle_bytes -= nbytes;
      return block;
    }
    return nullptr;
  }
  void* TryDevice(int64_t nbytes, int64_t alignment) {
    try {
      return ledger_->api->AllocMemory(nbytes, alignment);
    } catch (const std::exception&) {
      return nullptr;
    }
  }

  Device device_;
  int64_t size_limit_ = 0;  // bytes the pool may hold, idle and leased together; 0 = no limit
  std::shared_ptr<Ledger> ledger_;
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

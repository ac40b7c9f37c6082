// Restatement of the reference's memory-pool interface (include/raf/memory_pool.h:16-130) and of
// the two pools that ship with it, so that the `rocm` DeviceAPI can be exercised the way RAF's
// executors use a device: through Memory::Alloc / AllocAsync on a per-device pool.
//
//   Memory, MemoryPool ..... include/raf/memory_pool.h:28-127
//   pool manager ........... src/impl/memory_pool.cc:36-142; the default strategy per device type
//                            (:28-36) gains the entry RAF lacks: rocm -> "no_pool", whose
//                            AllocAsync is stream-ordered allocation from the HIP memory pool
//   NoPool ................. src/memory_pool/no_pool/no_pool.cc:60-121
//   PageUnitPool ........... src/memory_pool/page_unit_pool/page_unit_pool.cc:64-231
#pragma once

#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "raf_iface.h"

namespace raf {
namespace memory_pool {

class MemoryPool;

// A chunk of device memory; what frees it when the last reference goes depends on the pool.
class Memory {
 public:
  virtual ~Memory() = default;

  static int64_t GetAllocBytes(const Device& dev, int64_t nbytes);
  static std::shared_ptr<Memory> Alloc(const Device& dev, int64_t nbytes,
                                       int64_t alignment = kDefaultMemoryAlignment);
  static std::shared_ptr<Memory> AllocAsync(const Device& dev, int64_t nbytes, void* stream,
                                            int64_t alignment = kDefaultMemoryAlignment);
  static std::vector<std::shared_ptr<Memory>> AllocBatch(const Device& dev,
                                                         const std::vector<int64_t>& nbytes,
                                                         int64_t alignment = kDefaultMemoryAlignment);
  // <used, pool> in MB.
  static std::pair<float, float> GetPoolSize(const Device& dev);
  // The device's pool stops serving new requests; its chunks live on until their users let go.
  static void RemovePool(const Device& dev);
  // A fresh pool of the current pool's kind.
  static MemoryPool* ResetPool(const Device& dev);
  static MemoryPool* GetPool(const Device& dev);
  // The device's pool, created as `name` if the device has none yet (an existing pool wins).
  static MemoryPool* InitPool(const Device& dev, const std::string& name);

  void* data = nullptr;
  Device device{};
};

class MemoryPool {
 public:
  virtual ~MemoryPool() = default;
  virtual std::string GetName() = 0;
  // Bytes actually taken for a request of nbytes (page rounding etc.).
  virtual int64_t GetAllocBytes(int64_t nbytes) = 0;
  virtual std::shared_ptr<Memory> Alloc(int64_t nbytes, int64_t alignment = kDefaultMemoryAlignment) = 0;
  virtual std::shared_ptr<Memory> AllocAsync(int64_t nbytes, void* stream,
                                             int64_t alignment = kDefaultMemoryAlignment) = 0;
  virtual std::vector<std::shared_ptr<Memory>> AllocBatch(const std::vector<int64_t>& nbytes,
                                                          int64_t alignment = kDefaultMemoryAlignment) = 0;
  virtual std::pair<float, float> GetPoolSize() = 0;
  static float BytesToMegaBytes(float nbytes) { return nbytes / 1048576.0f; }

  using Maker = MemoryPool* (*)(const Device& dev);
  static bool RegisterMaker(const std::string& pool_name, Maker maker);
};

// The functions the reference exports as raf.memory_pool.{InitPool, RemovePool, ResetPool}
// (src/impl/memory_pool.cc:144-180): InitPool first removes the current pool.
void InitPool(const Device& dev, const std::string& pool_name);
void RemovePool(const Device& dev);
void ResetPool(const Device& dev);

}  // namespace memory_pool
}  // namespace raf

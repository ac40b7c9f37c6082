// Tensor fusion and defusion for gfx950: the HIP stand-ins for `raf.op.fuse_tensor` (a list of
// tensors packed back to back into one flat buffer) and `raf.op.defuse_tensor` (the reverse),
// which the reference runs as one cudaMemcpyAsync per tensor
// (src/op/dialect/cuda/memory.cc:55-68 and :120-134; offsets are running sums of the tensors'
// byte sizes, :61-66).
//
// Here one launch moves the whole list.  A plan fixes the byte sizes, like the reference's
// constructors do (memory.cc:33-43, :95-103), and holds a device table of segments (pointer, offset
// in the flat buffer, size) plus a work list of (segment, 8 KiB chunk) items, one workgroup per
// item, so a list of hundreds of small tensors costs one launch instead of
// hundreds of copies, and a list of a few huge tensors still fills the chip.
//
// Bytes are moved 16 per lane whenever source and destination allow it: the destination is
// brought to 16-byte alignment with a byte-wise head, and the source then only needs 4-byte
// alignment (gfx950 vector memory loads need no more than dword alignment).  Segments whose
// offsets differ by an odd number of bytes modulo 4 fall back to byte copies.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <new>
#include <vector>

#include "device_table.h"
#include "status.h"

namespace rafhip {
namespace {

#define RAFHIP_GLOBAL __attribute__((address_space(1)))
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));  // a 16-byte access that is only dword-aligned

constexpr int kCopyBlock = 256;
// One workgroup per work item, and an item is one trip: two 16-byte accesses per lane in flight,
// then the stores, then the workgroup ends.  Measured on the BERT-large list (1.34 GB): 6.3 TB/s,
// against 6.1-6.2 for items of 16-32 KiB and 5.5 for 4 KiB items or for a grid-stride loop over
// CUs x 8 workgroups.
constexpr int64_t kCopyChunk = 8 * 1024;  // bytes per work item
constexpr int kCopyInFlight = 2;          // 16-byte accesses in flight per lane per trip

struct Segment {  // 32 bytes, one per tensor
  char* part;     // the tensor
  int64_t offset; // where it sits in the flat buffer
  int64_t nbytes;
  int64_t reserved;
};

struct CopyItem {
  int32_t segment;
  int32_t chunk;
};

template <bool kNT>
__device__ __forceinline__ void copy_bytes(char* dst, const char* src, int64_t n) {
  // head: bring dst to a 16-byte boundary
  int64_t head = (int64_t)((16u - (unsigned)(reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u);
  if (head > n) head = n;
  if ((int64_t)threadIdx.x < head) dst[threadIdx.x] = src[threadIdx.x];
  dst += head;
  src += head;
  n -= head;
  int64_t done = 0;
  if ((reinterpret_cast<uintptr_t>(src) & 3u) == 0) {
    const int64_t nv = n >> 4;
    RAFHIP_GLOBAL u32x4* d = (RAFHIP_GLOBAL u32x4*)dst;
    const RAFHIP_GLOBAL u32x4_a4* s = (const RAFHIP_GLOBAL u32x4_a4*)src;
    for (int64_t i0 = threadIdx.x; i0 < nv; i0 += kCopyBlock * kCopyInFlight) {
      u32x4 r[kCopyInFlight];
#pragma unroll
      for (int u = 0; u < kCopyInFlight; ++u) {
        const int64_t i = i0 + u * kCopyBlock;
        if (i < nv) {
          if constexpr (kNT)
            r[u] = __builtin_nontemporal_load(s + i);
          else
            r[u] = s[i];
        }
      }
#pragma unroll
      for (int u = 0; u < kCopyInFlight; ++u) {
        const int64_t i = i0 + u * kCopyBlock;
        if (i < nv) {
          if constexpr (kNT)
            __builtin_nontemporal_store(r[u], d + i);
          else
            d[i] = r[u];
        }
      }
    }
    done = nv << 4;
  }
  for (int64_t i = done + threadIdx.x; i < n; i += kCopyBlock) dst[i] = src[i];
}

// gather != 0: parts -> flat buffer (fuse); gather == 0: flat buffer -> parts (defuse).
template <bool kNT>
__global__ __launch_bounds__(kCopyBlock) void fuse_copy(const Segment* segments,
                                                        const CopyItem* items, int64_t n_items,
                                                        char* flat, int gather) {
  for (int64_t it = blockIdx.x; it < n_items; it += gridDim.x) {
    const CopyItem item = items[it];
    const Segment seg = segments[item.segment];
    const int64_t begin = (int64_t)item.chunk * kCopyChunk;
    const int64_t rest = seg.nbytes - begin;
    const int64_t len = rest < kCopyChunk ? rest : kCopyChunk;
    char* in_part = seg.part + begin;
    char* in_flat = flat + seg.offset + begin;
    if (gather)
      copy_bytes<kNT>(in_flat, in_part, len);
    else
      copy_bytes<kNT>(in_part, in_flat, len);
  }
}

constexpr int64_t kStreamFromBytes = 96LL << 20;  // source + destination beyond the Infinity Cache

}  // namespace
}  // namespace rafhip

using namespace rafhip;

struct rafhip_fuse_plan {
  int32_t n = 0;
  int device = 0;
  std::vector<int64_t> nbytes, offset;
  int64_t total_bytes = 0;
  int64_t n_items = 0;
  void* d_tables = nullptr;
  CopyItem* d_items = nullptr;
  RecordTables<Segment> tables;  // device segment tables that follow the caller's pointers
  std::vector<Segment> segs;     // this call's segments, built in place: a call allocates nothing
};

namespace {

void free_plan(rafhip_fuse_plan* p) {
  if (!p) return;
  p->tables.release();
  if (p->d_tables) (void)hipFree(p->d_tables);
  delete p;
}

int run(rafhip_fuse_plan* plan, const char* what, void* const* parts, void* flat, bool gather,
        void* stream) {
  clear_error();
  if (!plan) return fail(RAFHIP_ERR_INVALID_ARG, "%s: plan is NULL", what);
  if (plan->n_items == 0) return RAFHIP_OK;  // nothing to move
  if (int st = check_plan_device(what, plan->device)) return st;
  if (!parts || !flat) return fail(RAFHIP_ERR_INVALID_ARG, "%s: null pointer argument", what);
  return guarded(what, [&]() -> int {
    std::vector<Segment>& segs = plan->segs;  // already n long
    for (int32_t i = 0; i < plan->n; ++i) {
      if (plan->nbytes[i] > 0 && !parts[i])
        return fail(RAFHIP_ERR_INVALID_ARG, "%s: tensor %d has a null data pointer", what, i);
      segs[i] = Segment{static_cast<char*>(parts[i]), plan->offset[i], plan->nbytes[i], 0};
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Segment* table = nullptr;
    if (int st = sync_tables(what, plan->tables, segs, s, &table)) return st;
    // One workgroup per item; the kernel strides over what a launch cannot hold.
    const unsigned grid = (unsigned)(plan->n_items < kMaxGridBlocks ? plan->n_items : kMaxGridBlocks);
    auto go = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(kCopyBlock), 0, s, table, plan->d_items,
                         plan->n_items, static_cast<char*>(flat), gather ? 1 : 0);
    };
    if (plan->total_bytes > kStreamFromBytes)
      go(fuse_copy<true>);
    else
      go(fuse_copy<false>);
    RAFHIP_HIP_TRY(hipGetLastError());
    return RAFHIP_OK;
  });
}

}  // namespace

extern "C" {

int rafhip_fuse_plan_create(int32_t n_tensors, const int64_t* nbytes, rafhip_fuse_plan** out_plan) {
  clear_error();
  if (!out_plan) return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_fuse_plan_create: out_plan is NULL");
  *out_plan = nullptr;
  if (n_tensors < 0 || (n_tensors > 0 && !nbytes))
    return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_fuse_plan_create: bad tensor list");
  return guarded("rafhip_fuse_plan_create", [&]() -> int {
    std::unique_ptr<rafhip_fuse_plan, void (*)(rafhip_fuse_plan*)> p(new rafhip_fuse_plan(), free_plan);
    p->n = n_tensors;
    std::vector<CopyItem> items;
    for (int32_t i = 0; i < n_tensors; ++i) {
      if (nbytes[i] < 0)
        return fail(RAFHIP_ERR_INVALID_ARG, "rafhip_fuse_plan_create: nbytes[%d] = %lld < 0", i,
                    (long long)nbytes[i]);
      const int64_t chunks = (nbytes[i] + kCopyChunk - 1) / kCopyChunk;
      if (chunks > INT32_MAX)
        return fail(RAFHIP_ERR_UNSUPPORTED, "rafhip_fuse_plan_create: tensor %d is too large", i);
      p->nbytes.push_back(nbytes[i]);
      p->offset.push_back(p->total_bytes);
      p->total_bytes += nbytes[i];
      for (int64_t c = 0; c < chunks; ++c) items.push_back(CopyItem{i, (int32_t)c});
    }
    p->n_items = (int64_t)items.size();
    if (p->n_items == 0) {  // an empty list or only empty tensors: valid, nothing to launch
      *out_plan = p.release();
      return RAFHIP_OK;
    }
    if (hipGetDevice(&p->device) != hipSuccess) {
      (void)hipGetLastError();
      return fail(RAFHIP_ERR_NO_DEVICE, "rafhip_fuse_plan_create: no HIP device available");
    }
    p->segs.resize((size_t)n_tensors);
    hipError_t e = hipMalloc(&p->d_tables, sizeof(CopyItem) * items.size());
    if (e == hipSuccess) {
      p->d_items = static_cast<CopyItem*>(p->d_tables);
      e = p->tables.init((size_t)n_tensors);
    }
    if (e == hipSuccess) {
      e = hipMemcpy(p->d_items, items.data(), sizeof(CopyItem) * items.size(), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) return fail(RAFHIP_ERR_HIP, "rafhip_fuse_plan_create: %s", hipGetErrorString(e));
    *out_plan = p.release();
    return RAFHIP_OK;
  });
}

int rafhip_fuse_plan_destroy(rafhip_fuse_plan* plan) {
  clear_error();
  free_plan(plan);
  return RAFHIP_OK;
}

int64_t rafhip_fuse_plan_total_bytes(const rafhip_fuse_plan* plan) {
  return plan ? plan->total_bytes : -1;
}

int rafhip_fuse_tensors(rafhip_fuse_plan* plan, const void* const* parts, void* fused,
                        void* stream) {
  return run(plan, "rafhip_fuse_tensors", const_cast<void* const*>(parts), fused, true, stream);
}

int rafhip_defuse_tensor(rafhip_fuse_plan* plan, const void* fused, void* const* parts,
                         void* stream) {
  return run(plan, "rafhip_defuse_tensor", parts, const_cast<void*>(fused), false, stream);
}

}  // extern "C"

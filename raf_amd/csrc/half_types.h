// 16-bit floating-point helpers shared by the kernels: native vector types for 16-byte (and
// 8-byte) lane accesses, exact widening, and round-to-nearest-even narrowing.
#pragma once
#include <hip/hip_runtime.h>

namespace rafhip {

// Global-address-space qualifier: tensor pointers come out of tables in memory, so without it the
// compiler falls back to flat (generic) loads and stores.
#define RAFHIP_GLOBAL __attribute__((address_space(1)))

// Native vectors (HIP's float4 etc. are classes and cannot be used with address spaces or the
// non-temporal builtins).
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));

// Element type tag for bfloat16 data (two bytes, like the data); values travel as bit patterns.
struct Bf16 {
  unsigned short bits;
};

// bfloat16 is the upper half of the fp32 word: widening is a shift, and exact.
__device__ __forceinline__ float bf16_widen(unsigned short b) {
  return __uint_as_float((unsigned)b << 16);
}

// fp32 -> bfloat16, round to nearest even by add-and-shift on the bit pattern; NaN stays a quiet
// NaN with its sign.
__device__ __forceinline__ unsigned short bf16_narrow(float x) {
  const unsigned u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x0040u);
  return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// fp32 -> binary16 (the hardware conversion, round to nearest even, overflow to infinity) or
// bfloat16, as a bit pattern.
__device__ __forceinline__ unsigned short narrow16(float x, bool bf16) {
  if (bf16) return bf16_narrow(x);
  const _Float16 h = (_Float16)x;
  return __builtin_bit_cast(unsigned short, h);
}

template <bool kNT, typename T>
__device__ __forceinline__ T ldg(const RAFHIP_GLOBAL T* p) {
  if constexpr (kNT)
    return __builtin_nontemporal_load(p);
  else
    return *p;
}
template <bool kNT, typename T>
__device__ __forceinline__ void stg(RAFHIP_GLOBAL T* p, T v) {
  if constexpr (kNT)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// Gradients of any supported dtype as fp32, already multiplied by an unscale factor (one fp32
// rounding, exact for power-of-two loss scales; pass 1.0f for none: x * 1.0f is exact).
template <typename G>
struct GradIO;

template <>
struct GradIO<float> {
  static constexpr int kWide = 4;  // elements per 16-byte lane access
  template <bool kNT>
  static __device__ __forceinline__ void load_wide(const void* g, int iw, float us,
                                                   float (&out)[kWide]) {
    const f32x4 r = ldg<kNT>((const RAFHIP_GLOBAL f32x4*)g + iw);
#pragma unroll
    for (int j = 0; j < kWide; ++j) out[j] = r[j] * us;
  }
  // The wide access in two steps, so that many loads can be in flight before any is widened.
  typedef f32x4 RawWide;
  template <bool kNT>
  static __device__ __forceinline__ RawWide load_raw_wide(const void* g, int iw) {
    return ldg<kNT>((const RAFHIP_GLOBAL f32x4*)g + iw);
  }
  static __device__ __forceinline__ void widen_wide(const RawWide& r, float us, float (&out)[kWide]) {
#pragma unroll
    for (int j = 0; j < kWide; ++j) out[j] = r[j] * us;
  }
  template <bool kNT>
  static __device__ __forceinline__ f32x4 load4(const void* g, int64_t i4, float us) {
    const f32x4 r = ldg<kNT>((const RAFHIP_GLOBAL f32x4*)g + i4);
    return f32x4{r.x * us, r.y * us, r.z * us, r.w * us};
  }
  static __device__ __forceinline__ float load1(const void* g, int64_t i, float us) {
    return ((const RAFHIP_GLOBAL float*)g)[i] * us;
  }
  // The same split in two, so that a load can be issued well before its value is needed.
  typedef f32x4 Raw4;
  template <bool kNT>
  static __device__ __forceinline__ Raw4 load_raw4(const void* g, int64_t i4) {
    return ldg<kNT>((const RAFHIP_GLOBAL f32x4*)g + i4);
  }
  static __device__ __forceinline__ f32x4 widen4(const Raw4& r, float us) {
    return f32x4{r.x * us, r.y * us, r.z * us, r.w * us};
  }
};

template <>
struct GradIO<_Float16> {
  static constexpr int kWide = 8;
  template <bool kNT>
  static __device__ __forceinline__ void load_wide(const void* g, int iw, float us,
                                                   float (&out)[kWide]) {
    const f16x8 r = ldg<kNT>((const RAFHIP_GLOBAL f16x8*)g + iw);
#pragma unroll
    for (int j = 0; j < kWide; ++j) out[j] = (float)r[j] * us;
  }
  typedef f16x8 RawWide;
  template <bool kNT>
  static __device__ __forceinline__ RawWide load_raw_wide(const void* g, int iw) {
    return ldg<kNT>((const RAFHIP_GLOBAL f16x8*)g + iw);
  }
  static __device__ __forceinline__ void widen_wide(const RawWide& r, float us, float (&out)[kWide]) {
#pragma unroll
    for (int j = 0; j < kWide; ++j) out[j] = (float)r[j] * us;
  }
  template <bool kNT>
  static __device__ __forceinline__ f32x4 load4(const void* g, int64_t i4, float us) {
    const f16x4 r = ldg<kNT>((const RAFHIP_GLOBAL f16x4*)g + i4);
    return f32x4{(float)r.x * us, (float)r.y * us, (float)r.z * us, (float)r.w * us};
  }
  static __device__ __forceinline__ float load1(const void* g, int64_t i, float us) {
    return (float)((const RAFHIP_GLOBAL _Float16*)g)[i] * us;
  }
  typedef f16x4 Raw4;
  template <bool kNT>
  static __device__ __forceinline__ Raw4 load_raw4(const void* g, int64_t i4) {
    return ldg<kNT>((const RAFHIP_GLOBAL f16x4*)g + i4);
  }
  static __device__ __forceinline__ f32x4 widen4(const Raw4& r, float us) {
    return f32x4{(float)r.x * us, (float)r.y * us, (float)r.z * us, (float)r.w * us};
  }
};

template <>
struct GradIO<Bf16> {
  static constexpr int kWide = 8;
  template <bool kNT>
  static __device__ __forceinline__ void load_wide(const void* g, int iw, float us,
                                                   float (&out)[kWide]) {
    const u16x8 r = ldg<kNT>((const RAFHIP_GLOBAL u16x8*)g + iw);
#pragma unroll
    for (int j = 0; j < kWide; ++j) out[j] = bf16_widen(r[j]) * us;
  }
  typedef u16x8 RawWide;
  template <bool kNT>
  static __device__ __forceinline__ RawWide load_raw_wide(const void* g, int iw) {
    return ldg<kNT>((const RAFHIP_GLOBAL u16x8*)g + iw);
  }
  static __device__ __forceinline__ void widen_wide(const RawWide& r, float us, float (&out)[kWide]) {
#pragma unroll
    for (int j = 0; j < kWide; ++j) out[j] = bf16_widen(r[j]) * us;
  }
  template <bool kNT>
  static __device__ __forceinline__ f32x4 load4(const void* g, int64_t i4, float us) {
    const u16x4 r = ldg<kNT>((const RAFHIP_GLOBAL u16x4*)g + i4);
    return f32x4{bf16_widen(r.x) * us, bf16_widen(r.y) * us, bf16_widen(r.z) * us,
                 bf16_widen(r.w) * us};
  }
  static __device__ __forceinline__ float load1(const void* g, int64_t i, float us) {
    return bf16_widen(((const RAFHIP_GLOBAL unsigned short*)g)[i]) * us;
  }
  typedef u16x4 Raw4;
  template <bool kNT>
  static __device__ __forceinline__ Raw4 load_raw4(const void* g, int64_t i4) {
    return ldg<kNT>((const RAFHIP_GLOBAL u16x4*)g + i4);
  }
  static __device__ __forceinline__ f32x4 widen4(const Raw4& r, float us) {
    return f32x4{bf16_widen(r.x) * us, bf16_widen(r.y) * us, bf16_widen(r.z) * us,
                 bf16_widen(r.w) * us};
  }
};

}  // namespace rafhip

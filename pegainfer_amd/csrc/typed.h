// Storage-type helpers for kernels that exist in a bf16 and a true-fp32 instance: activations and weights are read through
// ld() and written through st(); all arithmetic in between is fp32.  dtype codes of the C ABI: 0 = bf16 bits, 1 = float.
#pragma once

#include "common.h"

namespace pk {

constexpr int kDtBf16 = 0, kDtF32 = 1;

__device__ __forceinline__ float ld(const uint16_t* p) { return bf2f(*p); }
__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ void st(uint16_t* p, float v) { *p = f2bf(v); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }

// run `fn(tag)` with a null pointer of the storage type that `dtype` names
template <typename F>
inline bool by_dtype(int dtype, F&& fn) {
  if (dtype == kDtBf16) { fn(static_cast<uint16_t*>(nullptr)); return true; }
  if (dtype == kDtF32) { fn(static_cast<float*>(nullptr)); return true; }
  return false;
}

// eight consecutive stored values widened to fp32 (16-byte aligned for bf16, 32-byte span for fp32)
template <typename T>
struct Vec8;
template <>
struct Vec8<uint16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const uint16_t* p, float* o) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(p);
    o[0] = bf_lo(v.x); o[1] = bf_hi(v.x); o[2] = bf_lo(v.y); o[3] = bf_hi(v.y);
    o[4] = bf_lo(v.z); o[5] = bf_hi(v.z); o[6] = bf_lo(v.w); o[7] = bf_hi(v.w);
  }
};
template <>
struct Vec8<float> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
};
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

}  // namespace pk

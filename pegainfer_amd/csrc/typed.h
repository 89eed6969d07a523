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

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

}  // namespace pk

// Dynamic-Tanh normalisation over an fp32 residual stream (beside the RMSNorm family of norm.hip):
//   dyt(x) = tanh(alpha * x) * w + b        - elementwise: no mean, no variance, no reduction, so no row-wide barrier.
// Three forms, all one pass over the row, fp32 arithmetic, storage type of the activations / weights a template parameter:
//   embed_f32          token rows of the embedding table widened into the fp32 stream
//   dyt_norm           out = dyt(x)
//   dyt_add_norm       x += dyt_post(y); out = dyt_next(x)   (post-norm + residual sum + the next sublayer's pre-norm:
//                      the sublayer boundary costs one launch and one read of y, one read-modify-write of x)
// Memory-bound: 4 B read + 2-4 B written per element; a thread handles 4 consecutive elements.
#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

template <typename A>
__global__ __launch_bounds__(256) void embed_f32_kernel(const A* __restrict__ embed, const uint32_t* __restrict__ ids,
                                                        float* __restrict__ out, int width) {
  const A* src = embed + (size_t)ids[blockIdx.x] * width;
  float* dst = out + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += 256) dst[i] = ld(src + i);
}

template <typename A>
__global__ __launch_bounds__(256) void dyt_norm_kernel(const float* __restrict__ x, const A* __restrict__ alpha,
                                                       const A* __restrict__ w, const A* __restrict__ b,
                                                       A* __restrict__ out, int d, long n) {
  const float a = ld(alpha);
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const int c = (int)(i % d);
    st(out + i, tanhf(a * x[i]) * ld(w + c) + ld(b + c));
  }
}

template <typename A, bool NEXT>
__global__ __launch_bounds__(256) void dyt_add_norm_kernel(float* __restrict__ x, const A* __restrict__ y,
                                                           const A* __restrict__ pa, const A* __restrict__ pw,
                                                           const A* __restrict__ pb, const A* __restrict__ na,
                                                           const A* __restrict__ nw, const A* __restrict__ nb,
                                                           A* __restrict__ out, int d, long n) {
  const float a = ld(pa);
  const float a2 = NEXT ? ld(na) : 0.f;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const int c = (int)(i % d);
    const float v = x[i] + (tanhf(a * ld(y + i)) * ld(pw + c) + ld(pb + c));
    x[i] = v;
    if (NEXT) st(out + i, tanhf(a2 * v) * ld(nw + c) + ld(nb + c));
  }
}

__global__ __launch_bounds__(256) void gather_rows_f32_kernel(const float* __restrict__ x, const int32_t* __restrict__ idx,
                                                              float* __restrict__ out, int d) {
  const float* src = x + (size_t)idx[blockIdx.x] * d;
  float* dst = out + (size_t)blockIdx.x * d;
  for (int i = threadIdx.x; i < d; i += 256) dst[i] = src[i];
}

template <typename A>
__global__ __launch_bounds__(256) void relu_sq_kernel(const A* __restrict__ x, A* __restrict__ out, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float v = fmaxf(ld(x + i), 0.f);
    st(out + i, v * v);
  }
}

template <typename A>
__global__ __launch_bounds__(256) void silu_mul_rows_kernel(const A* __restrict__ gu, A* __restrict__ out, int I, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const long row = i / I;
    const int c = (int)(i % I);
    const float g = ld(gu + row * 2 * I + c), u = ld(gu + row * 2 * I + I + c);
    st(out + i, g * sigmoid_f(g) * u);
  }
}

static inline int grid_for(long n) { return (int)std::min<long>((n + 255) / 256, 8192); }

}  // namespace pk

extern "C" {
using namespace pk;

pegainfer_status_t pegainfer_embed_f32(const void* embed, const uint32_t* token_ids, float* out, int32_t width,
                                       int32_t n_tokens, int32_t dtype, pegainfer_stream_t stream) {
  if (n_tokens <= 0) return 0;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        embed_f32_kernel<A><<<n_tokens, 256, 0, as_stream(stream)>>>(static_cast<const A*>(embed), token_ids, out, width);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_dyt_norm(const float* x, const void* alpha, const void* w, const void* b, void* out,
                                      int32_t d, int32_t rows, int32_t dtype, pegainfer_stream_t stream) {
  const long n = (long)d * rows;
  if (n <= 0) return 0;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        dyt_norm_kernel<A><<<grid_for(n), 256, 0, as_stream(stream)>>>(x, static_cast<const A*>(alpha), static_cast<const A*>(w),
                                                                       static_cast<const A*>(b), static_cast<A*>(out), d, n);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_dyt_add_norm(float* x, const void* y, const void* post_alpha, const void* post_w,
                                          const void* post_b, const void* next_alpha, const void* next_w,
                                          const void* next_b, void* out, int32_t d, int32_t rows, int32_t dtype,
                                          pegainfer_stream_t stream) {
  const long n = (long)d * rows;
  if (n <= 0) return 0;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        auto c = [](const void* p) { return static_cast<const A*>(p); };
        if (next_w)
          dyt_add_norm_kernel<A, true><<<grid_for(n), 256, 0, as_stream(stream)>>>(
              x, c(y), c(post_alpha), c(post_w), c(post_b), c(next_alpha), c(next_w), c(next_b), static_cast<A*>(out), d, n);
        else
          dyt_add_norm_kernel<A, false><<<grid_for(n), 256, 0, as_stream(stream)>>>(
              x, c(y), c(post_alpha), c(post_w), c(post_b), nullptr, nullptr, nullptr, nullptr, d, n);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_gather_rows_f32(const float* x, const int32_t* rows_index, float* out, int32_t d,
                                             int32_t n_rows, pegainfer_stream_t stream) {
  if (n_rows <= 0) return 0;
  gather_rows_f32_kernel<<<n_rows, 256, 0, as_stream(stream)>>>(x, rows_index, out, d);
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_relu_sq(const void* x, void* out, int64_t n, int32_t dtype, pegainfer_stream_t stream) {
  if (n <= 0) return 0;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        relu_sq_kernel<A><<<grid_for(n), 256, 0, as_stream(stream)>>>(static_cast<const A*>(x), static_cast<A*>(out), n);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_silu_mul_rows(const void* gate_up, void* out, int32_t I, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream) {
  const long n = (long)I * rows;
  if (n <= 0) return 0;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        silu_mul_rows_kernel<A><<<grid_for(n), 256, 0, as_stream(stream)>>>(static_cast<const A*>(gate_up), static_cast<A*>(out), I, n);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

}  // extern "C"

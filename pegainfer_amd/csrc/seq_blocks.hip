// Blocks around a sequence model's sublayers, each in a bf16 and an fp32 storage instance with fp32 arithmetic:
//   time_conv_kernel        causal per-channel convolution over time on a ragged batch; the inputs before an entry's first
//                           row come from the request's state (its last taps - 1 inputs)
//   time_conv_commit_kernel moves that state on by the entry's rows (one thread per (entry, channel) shifts in place,
//                           oldest first, so it never reads what it has already written)
//   group_rms_add_kernel    RMS norm in equal consecutive groups of a sublayer's OUTPUT, the residual sum, and a weighted
//                           sum over the streams of earlier layers (depth-weighted averaging) in one pass over the row
//   clamp_glu_rows_kernel   g = min(gate, L), u = clamp(up, -L, L):  g sigmoid(alpha g) (u + 1)
//   head_rms_gate_kernel    per-head RMS norm of a read-out * weight * silu / sigmoid gate * constant
#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

template <typename I, typename W, typename O>
__global__ __launch_bounds__(256) void time_conv_kernel(const I* __restrict__ in, int64_t in_stride, const W* __restrict__ w,
                                                        const float* __restrict__ state, int64_t slot_stride,
                                                        O* __restrict__ out, int64_t out_stride, int C, int K, int mode,
                                                        const int32_t* __restrict__ row_entry,
                                                        const int32_t* __restrict__ entry_row0,
                                                        const int32_t* __restrict__ entry_slot) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int e = row_entry[row], r0 = entry_row0[e];
  const int local = row - r0;
  const float* tail = state + (int64_t)entry_slot[e] * slot_stride;
  float acc = 0.f;
  for (int j = 0; j < K; ++j) {
    const int src = local - (K - 1) + j;   // row of the entry this tap reads; negative = carried from earlier steps
    const float v = src >= 0 ? ld(in + (int64_t)(r0 + src) * in_stride + c) : tail[(int64_t)(K - 1 + src) * C + c];
    acc = fmaf(ld(w + (int64_t)c * K + j), v, acc);
  }
  if (mode & 1) acc += ld(in + (int64_t)row * in_stride + c);
  if (mode & 2) acc = silu_f(acc);
  st(out + (int64_t)row * out_stride + c, acc);
}

template <typename I>
__global__ __launch_bounds__(256) void time_conv_commit_kernel(const I* __restrict__ in, int64_t in_stride,
                                                               float* __restrict__ state, int64_t slot_stride, int C, int K,
                                                               const int32_t* __restrict__ entry_row0,
                                                               const int32_t* __restrict__ entry_slot) {
  const int e = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = entry_row0[e], len = entry_row0[e + 1] - r0;
  float* tail = state + (int64_t)entry_slot[e] * slot_stride;
  for (int s = 0; s < K - 1; ++s) {
    const int idx = len + s;   // position in [old state (K - 1) ; this step's inputs (len)]
    tail[(int64_t)s * C + c] = idx < K - 1 ? tail[(int64_t)idx * C + c] : ld(in + (int64_t)(r0 + idx - (K - 1)) * in_stride + c);
  }
}

template <typename Y, typename A>
__global__ __launch_bounds__(256) void group_rms_add_kernel(const float* __restrict__ x_in, const Y* __restrict__ y,
                                                            const A* __restrict__ w, int groups, float eps,
                                                            float* __restrict__ x_out, A* __restrict__ xb_out, int d,
                                                            const float* __restrict__ stack, int64_t stack_stride,
                                                            const A* __restrict__ coef, int n_mix,
                                                            float* __restrict__ mix_out, A* __restrict__ mixb_out) {
  extern __shared__ float inv[];   // [groups]
  const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int gs = d / groups;
  const Y* yr = y + (int64_t)row * d;
  for (int g = wave; g < groups; g += 4) {
    float ss = 0.f;
    for (int i = lane; i < gs; i += 64) {
      const float v = ld(yr + g * gs + i);
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < d; i += 256) {
    const int64_t at = (int64_t)row * d + i;
    float r = ld(yr + i) * inv[i / gs] * ld(w + i);
    if (x_in) r += x_in[at];
    if (x_out) x_out[at] = r;
    if (xb_out) st(xb_out + at, r);
    if (n_mix > 0) {
      float m = 0.f;
      for (int j = 0; j < n_mix - 1; ++j) m = fmaf(ld(coef + j), stack[(int64_t)j * stack_stride + at], m);
      m = fmaf(ld(coef + n_mix - 1), r, m);
      if (mix_out) mix_out[at] = m;
      if (mixb_out) st(mixb_out + at, m);
    }
  }
}

template <typename A>
__global__ __launch_bounds__(256) void clamp_glu_rows_kernel(const A* __restrict__ gu, A* __restrict__ out, int I, float limit,
                                                             float alpha) {
  const int row = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= I) return;
  const float g = fminf(ld(gu + (int64_t)row * 2 * I + i), limit);
  const float u = fminf(fmaxf(ld(gu + (int64_t)row * 2 * I + I + i), -limit), limit);
  st(out + (int64_t)row * I + i, g * sigmoid_f(alpha * g) * (u + 1.0f));
}

// one wave per (row, head)
template <typename A>
__global__ __launch_bounds__(256) void head_rms_gate_kernel(const float* __restrict__ o, const A* __restrict__ w, int w_per_head,
                                                            const A* __restrict__ gate, int64_t gate_stride, int gate_kind,
                                                            float factor, float eps, A* __restrict__ out, int64_t out_stride,
                                                            int heads, int vdim, int rows) {
  const int64_t rh = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (rh >= (int64_t)rows * heads) return;
  const int row = (int)(rh / heads), h = (int)(rh % heads);
  const float* p = o + ((int64_t)row * heads + h) * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += 64) ss = fmaf(p[i], p[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int i = lane; i < vdim; i += 64) {
    const float z = ld(gate + (int64_t)row * gate_stride + h * vdim + i);
    const float a = gate_kind == 0 ? silu_f(z) : sigmoid_f(z);
    st(out + (int64_t)row * out_stride + h * vdim + i, p[i] * inv * ld(w + (w_per_head ? h * vdim : 0) + i) * a * factor);
  }
}

}  // namespace pk

extern "C" {
using namespace pk;

#define PK_BAD ((pegainfer_status_t)hipErrorInvalidValue)

pegainfer_status_t pegainfer_time_conv(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                       const float* state, int64_t slot_stride, void* out, int32_t out_dtype,
                                       int64_t out_row_stride, int32_t channels, int32_t taps, int32_t mode,
                                       const int32_t* row_entry, const int32_t* entry_row0, const int32_t* entry_slot,
                                       int32_t n_rows, pegainfer_stream_t stream) {
  if (n_rows <= 0) return 0;
  if (channels <= 0 || taps < 1) return PK_BAD;
  const dim3 grid(n_rows, ceil_div(channels, 256));
  bool ok = true;
  const bool known = by_dtype(in_dtype, [&](auto* ti) {
    using I = std::remove_pointer_t<decltype(ti)>;
    ok = by_dtype(w_dtype, [&](auto* tw) {
           using W = std::remove_pointer_t<decltype(tw)>;
           ok = by_dtype(out_dtype, [&](auto* to) {
                  using O = std::remove_pointer_t<decltype(to)>;
                  time_conv_kernel<I, W, O><<<grid, 256, 0, as_stream(stream)>>>(
                      static_cast<const I*>(in), in_row_stride, static_cast<const W*>(w), state, slot_stride,
                      static_cast<O*>(out), out_row_stride, channels, taps, mode, row_entry, entry_row0, entry_slot);
                }) && ok;
         }) && ok;
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_time_conv_commit(const void* in, int32_t in_dtype, int64_t in_row_stride, float* state,
                                              int64_t slot_stride, int32_t channels, int32_t taps, const int32_t* entry_row0,
                                              const int32_t* entry_slot, int32_t n_entries, pegainfer_stream_t stream) {
  if (n_entries <= 0 || taps <= 1) return 0;
  const dim3 grid(ceil_div(channels, 256), n_entries);
  if (!by_dtype(in_dtype, [&](auto* ti) {
        using I = std::remove_pointer_t<decltype(ti)>;
        time_conv_commit_kernel<I><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const I*>(in), in_row_stride, state,
                                                                        slot_stride, channels, taps, entry_row0, entry_slot);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_group_rms_add(const float* x_in, const void* y, int32_t y_dtype, const void* w, int32_t groups,
                                           float eps, float* x_out, void* xb_out, int32_t d, int32_t rows, int32_t dtype,
                                           const float* stack, int64_t stack_stride, const void* coef, int32_t n_mix,
                                           float* mix_out, void* mixb_out, pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (groups < 1 || d <= 0 || d % groups || groups > 8192 || (n_mix > 0 && !coef) || (n_mix > 1 && !stack)) return PK_BAD;
  bool ok = true;
  const bool known = by_dtype(y_dtype, [&](auto* ty) {
    using Y = std::remove_pointer_t<decltype(ty)>;
    ok = by_dtype(dtype, [&](auto* ta) {
      using A = std::remove_pointer_t<decltype(ta)>;
      group_rms_add_kernel<Y, A><<<rows, 256, (size_t)groups * sizeof(float), as_stream(stream)>>>(
          x_in, static_cast<const Y*>(y), static_cast<const A*>(w), groups, eps, x_out, static_cast<A*>(xb_out), d, stack,
          stack_stride, static_cast<const A*>(coef), n_mix, mix_out, static_cast<A*>(mixb_out));
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_clamp_glu_rows(const void* gate_up, void* out, int32_t I, int32_t rows, float limit, float alpha,
                                            int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0 || I <= 0) return 0;
  const dim3 grid(rows, ceil_div(I, 256));
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        clamp_glu_rows_kernel<A><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const A*>(gate_up), static_cast<A*>(out), I,
                                                                      limit, alpha);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_head_rms_gate(const float* o, const void* w, int32_t w_per_head, const void* gate,
                                           int64_t gate_stride, int32_t gate_kind, float factor, float eps, void* out,
                                           int64_t out_stride, int32_t heads, int32_t vdim, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || vdim <= 0) return PK_BAD;
  const int blocks = ceil_div((long)rows * heads, 4);
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        head_rms_gate_kernel<A><<<blocks, 256, 0, as_stream(stream)>>>(o, static_cast<const A*>(w), w_per_head,
                                                                       static_cast<const A*>(gate), gate_stride, gate_kind,
                                                                       factor, eps, static_cast<A*>(out), out_stride, heads,
                                                                       vdim, rows);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

}  // extern "C"

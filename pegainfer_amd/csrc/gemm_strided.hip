// Strided / batched / grouped GEMM for the shapes the weight-streaming and 128/256-tile kernels of linear.hip do not take:
// per-head products over slices of a wider row (latent-attention absorb and value up-projection), expert-grouped rows
// gathered through an index (routed feed-forward), and every product of a model served in true fp32.
//
//   y[row, g, m] = sum_k x[row, g, k] * w[g, m, k]
//
// 64 x 64 output tile per 256-thread workgroup, K in slices of 16 staged through LDS as fp32, each thread a 4 x 4 block
// of fp32 accumulators, k strictly ascending: an output's value depends on its own row and weights only (never on the
// tile it lands in, the batch or the group sizes).  Operand storage (bf16 or fp32) is a template parameter, so the bf16
// instance multiplies exact fp32 images of bf16 values and the fp32 instance is plain fp32 FMA - no reduced-precision
// matrix mode.
#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

constexpr int GT = 64, GM = 64, GK = 16;

template <typename TX, typename TW, typename TY, typename TG>
__global__ __launch_bounds__(256) void gemm_strided_kernel(pegainfer_gemm_desc d) {
  __shared__ float xs[GK][GT + 4];
  __shared__ float ws[GK][GM + 4];
  __shared__ int xrow[GT], yrow[GT];
  int g, row0, nrows;
  if (d.tile_group) {
    if ((int)blockIdx.x >= *d.n_tiles) return;
    g = d.tile_group[blockIdx.x];
    row0 = d.tile_row0[blockIdx.x];
    nrows = d.tile_rows[blockIdx.x];
  } else {
    g = blockIdx.z;
    row0 = blockIdx.x * GT;
    nrows = min(GT, d.rows - row0);
  }
  const int m0 = blockIdx.y * GM;
  const int tid = threadIdx.x;
  if (tid < GT) {
    const int p = row0 + tid;
    xrow[tid] = tid < nrows ? (d.x_row_index ? d.x_row_index[p] : p) : -1;
    yrow[tid] = tid < nrows ? (d.y_row_index ? d.y_row_index[p] : p) : -1;
  }
  __syncthreads();
  const TX* X = static_cast<const TX*>(d.x) + (int64_t)g * d.x_group_stride;
  const TW* W = static_cast<const TW*>(d.w) + (int64_t)g * d.w_group_stride;
  const int tr = (tid >> 4) * 4, tm = (tid & 15) * 4;   // this thread's 4 rows x 4 outputs
  float acc[4][4] = {};
  const bool w_k_fast = d.w_k_stride == 1;
  for (int k0 = 0; k0 < d.k; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      {
        const int r = idx >> 4, kk = idx & 15;
        const int src = xrow[r];
        xs[kk][r] = (src >= 0 && k0 + kk < d.k) ? ld(X + (int64_t)src * d.x_row_stride + k0 + kk) : 0.f;
      }
      {
        const int mm = w_k_fast ? idx >> 4 : idx & 63, kk = w_k_fast ? idx & 15 : idx >> 6;
        ws[kk][mm] = (m0 + mm < d.m && k0 + kk < d.k)
                         ? ld(W + (int64_t)(m0 + mm) * d.w_m_stride + (int64_t)(k0 + kk) * d.w_k_stride) : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = xs[kk][tr + i]; b[i] = ws[kk][tm + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  TY* Y = static_cast<TY*>(d.y) + (int64_t)g * d.y_group_stride;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int dst = yrow[tr + i];
    if (dst < 0) continue;
    float scale = 1.f;
    if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE)
      scale = sigmoid_f(ld(static_cast<const TG*>(d.gate) + (int64_t)xrow[tr + i] * d.gate_row_stride + g));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (m0 + tm + j >= d.m) continue;
      float v = acc[i][j];
      if (d.epilogue == PEGAINFER_EPI_RELU_SQ) { v = fmaxf(v, 0.f); v *= v; }
      else if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE) v *= scale;
      st(Y + (int64_t)dst * d.y_row_stride + m0 + tm + j, v);
    }
  }
}

template <typename TX, typename TW, typename TY>
static void gemm_strided_launch(const pegainfer_gemm_desc& d, hipStream_t s) {
  dim3 grid(d.tile_group ? d.max_tiles : ceil_div(d.rows, GT), ceil_div(d.m, GM), d.tile_group ? 1 : d.groups);
  if (d.gate_dtype == kDtF32) gemm_strided_kernel<TX, TW, TY, float><<<grid, 256, 0, s>>>(d);
  else gemm_strided_kernel<TX, TW, TY, uint16_t><<<grid, 256, 0, s>>>(d);
}

}  // namespace pk

extern "C" pegainfer_status_t pegainfer_gemm_strided(const pegainfer_gemm_desc* dp, pegainfer_stream_t stream) {
  using namespace pk;
  const pegainfer_gemm_desc& d = *dp;
  if (d.m <= 0 || d.k <= 0) return 0;
  if (d.tile_group ? d.max_tiles <= 0 : (d.rows <= 0 || d.groups <= 0)) return 0;
  hipStream_t s = as_stream(stream);
  const int key = (d.x_dtype << 2) | (d.w_dtype << 1) | d.y_dtype;
  switch (key) {
    case 0: gemm_strided_launch<uint16_t, uint16_t, uint16_t>(d, s); break;
    case 1: gemm_strided_launch<uint16_t, uint16_t, float>(d, s); break;
    case 4: gemm_strided_launch<float, uint16_t, uint16_t>(d, s); break;
    case 5: gemm_strided_launch<float, uint16_t, float>(d, s); break;
    case 7: gemm_strided_launch<float, float, float>(d, s); break;
    default: return (pegainfer_status_t)hipErrorInvalidValue;
  }
  return (pegainfer_status_t)hipGetLastError();
}

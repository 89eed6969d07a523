// Recurrent matrix memories over ragged batches, fp32 state and fp32 arithmetic throughout.
//
// Both kernels share one shape.  A workgroup of four waves owns 16 value columns of one (entry, head); a column's state
// S[:, col] is spread over the sixteen lanes of a DPP row (lane = 16 * column + r holds the rows d = r + 16 i), so a token
// costs each lane dim / 16 multiply-adds per product and a four-step DPP sum inside the row: the recurrence is a chain of
// dependent steps, so the work of one step is spread as wide as the wave allows and many small workgroups fill the chip.
// The state stays in registers from the entry's first row to its last and touches HBM once on either side.  The tokens'
// keys, queries, values and gates are staged 16 tokens at a time through LDS: the next round's global loads are issued
// before the current round is consumed and land in LDS after it; norms and gate functions are computed once per token there.
//   delta_rule_kernel      S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q   (q, k made unit vectors at staging)
//   matrix_memory_kernel   m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n likewise;  o = S^T q / (max(|n.q|, e^-m') + 1e-6)
// A row's result depends only on the rows before it in its own request: the token order is fixed, and cutting a prompt into
// steps only moves where the state passes through HBM (exactly, it is fp32 either way).
#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

constexpr int kRecTokens = 16;   // tokens staged per round
constexpr int kRecCols = 16;     // value columns per workgroup (four per wave)
constexpr int kRecSlices = 16;   // lanes that share one column

__device__ __forceinline__ float softplus_f(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoid_f(float x) { return fminf(x, 0.0f) - log1pf(expf(-fabsf(x))); }

// One round's q | k | v values, fetched into registers (issue) and put into LDS later (land).  Element e of the round:
// token e / per_tok, then within the token [q: DP | k: DP | v: kRecCols].
template <int NS>
struct RoundFetch {
  static constexpr int DP = kRecSlices * NS;
  static constexpr int PER_TOK = 2 * DP + kRecCols;
  static constexpr int N = (kRecTokens * PER_TOK + 255) / 256;
  float r[N];
  template <typename Load>
  __device__ __forceinline__ void issue(int tc, int tid, Load&& load) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int e = tid + 256 * j;
      const int tt = e / PER_TOK, w = e % PER_TOK;
      r[j] = tt < tc ? load(tt, w) : 0.f;
    }
  }
  __device__ __forceinline__ void land(int tid, float (*s_q)[DP], float (*s_k)[DP], float (*s_v)[kRecCols]) {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int e = tid + 256 * j;
      const int tt = e / PER_TOK, w = e % PER_TOK;
      if (tt < kRecTokens) {
        if (w < DP) s_q[tt][w] = r[j];
        else if (w < 2 * DP) s_k[tt][w - DP] = r[j];
        else s_v[tt][w - 2 * DP] = r[j];
      }
    }
  }
};

template <int NS, typename A>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ qkv, int64_t qkv_stride,
                                                         const A* __restrict__ proj, int64_t proj_stride, int64_t b_off,
                                                         int64_t a_off, const A* __restrict__ A_log,
                                                         const A* __restrict__ dt_bias, float* __restrict__ state,
                                                         int64_t slot_stride, float* __restrict__ o, int H, int G, int dim,
                                                         int vdim, const int32_t* __restrict__ entry_row0,
                                                         const int32_t* __restrict__ entry_slot) {
  constexpr int DP = kRecSlices * NS;
  __shared__ float s_k[kRecTokens][DP], s_q[kRecTokens][DP], s_v[kRecTokens][kRecCols], s_g[kRecTokens], s_b[kRecTokens];
  const int e = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * kRecCols;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, cl = wave * 4 + (lane >> 4);
  const int col = col0 + cl;
  const int g0 = h / (H / G);
  const int row0 = entry_row0[e], len = entry_row0[e + 1] - row0;
  float* S_g = state + (int64_t)entry_slot[e] * slot_stride + (int64_t)h * dim * vdim;
  float S[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int d = r + kRecSlices * i;
    S[i] = d < dim && col < vdim ? S_g[(int64_t)d * vdim + col] : 0.f;
  }
  const float neg_a = -expf(ld(A_log + h)), dtb = ld(dt_bias + h), qs = 1.0f / sqrtf((float)dim);
  RoundFetch<NS> nxt;
  auto load = [&](int t0) {
    return [=](int tt, int w) -> float {
      const float* rowp = qkv + (int64_t)(row0 + t0 + tt) * qkv_stride;
      if (w < DP) return w < dim ? rowp[(int64_t)g0 * dim + w] : 0.f;
      if (w < 2 * DP) return w - DP < dim ? rowp[(int64_t)(G + g0) * dim + (w - DP)] : 0.f;
      const int c = w - 2 * DP;
      return col0 + c < vdim ? rowp[(int64_t)2 * G * dim + (int64_t)h * vdim + col0 + c] : 0.f;
    };
  };
  nxt.issue(min(kRecTokens, len), tid, load(0));
  for (int t0 = 0; t0 < len; t0 += kRecTokens) {
    const int tc = min(kRecTokens, len - t0);
    __syncthreads();
    nxt.land(tid, s_q, s_k, s_v);
    if (tid < tc) {
      const A* pr = proj + (int64_t)(row0 + t0 + tid) * proj_stride;
      s_b[tid] = sigmoid_f(ld(pr + b_off + h));
      s_g[tid] = expf(neg_a * softplus_f(ld(pr + a_off + h) + dtb));
    }
    __syncthreads();
    if (t0 + kRecTokens < len) nxt.issue(min(kRecTokens, len - t0 - kRecTokens), tid, load(t0 + kRecTokens));
    for (int tt = wave; tt < tc; tt += 4) {   // unit vectors: x / sqrt(sum(x^2) + 1e-6); the query also carries dim^-1/2
      float sq = 0.f, sk = 0.f;
      for (int d = lane; d < dim; d += 64) {
        sq = fmaf(s_q[tt][d], s_q[tt][d], sq);
        sk = fmaf(s_k[tt][d], s_k[tt][d], sk);
      }
      sq = qs / sqrtf(wave_sum(sq) + 1e-6f);
      sk = 1.0f / sqrtf(wave_sum(sk) + 1e-6f);
      for (int d = lane; d < dim; d += 64) {
        s_q[tt][d] *= sq;
        s_k[tt][d] *= sk;
      }
    }
    __syncthreads();
#pragma unroll 2
    for (int tt = 0; tt < tc; ++tt) {
      const float g = s_g[tt], beta = s_b[tt], v = s_v[tt][cl];
      float kk[NS], a0 = 0.f, a1 = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        kk[i] = s_k[tt][r + kRecSlices * i];
        S[i] *= g;
        if (i & 1) a1 = fmaf(S[i], kk[i], a1); else a0 = fmaf(S[i], kk[i], a0);
      }
      const float u = beta * (v - row16_sum(a0 + a1));
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        S[i] = fmaf(kk[i], u, S[i]);
        const float qq = s_q[tt][r + kRecSlices * i];
        if (i & 1) o1 = fmaf(S[i], qq, o1); else o0 = fmaf(S[i], qq, o0);
      }
      const float oa = row16_sum(o0 + o1);
      if (r == 0 && col < vdim) o[(int64_t)(row0 + t0 + tt) * ((int64_t)H * vdim) + (int64_t)h * vdim + col] = oa;
    }
  }
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int d = r + kRecSlices * i;
    if (d < dim && col < vdim) S_g[(int64_t)d * vdim + col] = S[i];
  }
}

template <int NS, typename A>
__global__ __launch_bounds__(256) void matrix_memory_kernel(const A* __restrict__ proj, int64_t proj_stride, int64_t q_off,
                                                            int64_t k_off, int64_t v_off, int64_t i_off, int64_t f_off,
                                                            const A* __restrict__ i_bias, const A* __restrict__ f_bias,
                                                            float cap, float* __restrict__ state, int64_t slot_stride,
                                                            float* __restrict__ o, int H, int dim, int vdim,
                                                            const int32_t* __restrict__ entry_row0,
                                                            const int32_t* __restrict__ entry_slot) {
  constexpr int DP = kRecSlices * NS;
  __shared__ float s_k[kRecTokens][DP], s_q[kRecTokens][DP], s_v[kRecTokens][kRecCols], s_i[kRecTokens], s_f[kRecTokens];
  const int e = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * kRecCols;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, cl = wave * 4 + (lane >> 4);
  const int col = col0 + cl;
  const int row0 = entry_row0[e], len = entry_row0[e + 1] - row0;
  float* base = state + (int64_t)entry_slot[e] * slot_stride;
  float* S_g = base + (int64_t)h * dim * vdim;
  float* n_g = base + (int64_t)H * dim * vdim + (int64_t)h * dim;
  float* m_g = base + (int64_t)H * dim * vdim + (int64_t)H * dim + h;
  float S[NS], n[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int d = r + kRecSlices * i;
    S[i] = d < dim && col < vdim ? S_g[(int64_t)d * vdim + col] : 0.f;
    n[i] = d < dim ? n_g[d] : 0.f;
  }
  float m = *m_g;
  const float ib = ld(i_bias + h), fb = ld(f_bias + h), qs = 1.0f / sqrtf((float)dim);
  RoundFetch<NS> nxt;
  auto load = [&](int t0) {
    return [=](int tt, int w) -> float {
      const A* pr = proj + (int64_t)(row0 + t0 + tt) * proj_stride;
      if (w < DP) return w < dim ? ld(pr + q_off + (int64_t)h * dim + w) * qs : 0.f;
      if (w < 2 * DP) return w - DP < dim ? ld(pr + k_off + (int64_t)h * dim + (w - DP)) : 0.f;
      const int c = w - 2 * DP;
      return col0 + c < vdim ? ld(pr + v_off + (int64_t)h * vdim + col0 + c) : 0.f;
    };
  };
  nxt.issue(min(kRecTokens, len), tid, load(0));
  for (int t0 = 0; t0 < len; t0 += kRecTokens) {
    const int tc = min(kRecTokens, len - t0);
    __syncthreads();
    nxt.land(tid, s_q, s_k, s_v);
    if (tid < tc) {
      const A* pr = proj + (int64_t)(row0 + t0 + tid) * proj_stride;
      s_i[tid] = cap * tanhf((ld(pr + i_off + h) + ib) / cap);
      s_f[tid] = logsigmoid_f(cap * tanhf((ld(pr + f_off + h) + fb) / cap));
    }
    __syncthreads();
    if (t0 + kRecTokens < len) nxt.issue(min(kRecTokens, len - t0 - kRecTokens), tid, load(t0 + kRecTokens));
#pragma unroll 2
    for (int tt = 0; tt < tc; ++tt) {
      const float ig = s_i[tt], fg = s_f[tt];
      const float m_new = fmaxf(fg + m, ig);
      const float a = expf(fg + m - m_new), b = expf(ig - m_new);
      m = m_new;
      const float bv = b * s_v[tt][cl];
      float num0 = 0.f, num1 = 0.f, nq0 = 0.f, nq1 = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const float kk = s_k[tt][r + kRecSlices * i], qq = s_q[tt][r + kRecSlices * i];
        S[i] = fmaf(bv, kk, a * S[i]);
        n[i] = fmaf(b, kk, a * n[i]);
        if (i & 1) { num1 = fmaf(S[i], qq, num1); nq1 = fmaf(n[i], qq, nq1); }
        else { num0 = fmaf(S[i], qq, num0); nq0 = fmaf(n[i], qq, nq0); }
      }
      const float num = row16_sum(num0 + num1), nq = row16_sum(nq0 + nq1);
      const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
      if (r == 0 && col < vdim) o[(int64_t)(row0 + t0 + tt) * ((int64_t)H * vdim) + (int64_t)h * vdim + col] = num / den;
    }
  }
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    const int d = r + kRecSlices * i;
    if (d < dim && col < vdim) S_g[(int64_t)d * vdim + col] = S[i];
    if (blockIdx.x == 0 && tid < kRecSlices && d < dim) n_g[d] = n[i];
  }
  if (blockIdx.x == 0 && tid == 0) *m_g = m;
}

template <typename F>
inline bool by_slices(int dim, F&& fn) {
  if (dim <= 16) fn(std::integral_constant<int, 1>());
  else if (dim <= 32) fn(std::integral_constant<int, 2>());
  else if (dim <= 64) fn(std::integral_constant<int, 4>());
  else if (dim <= 128) fn(std::integral_constant<int, 8>());
  else if (dim <= 256) fn(std::integral_constant<int, 16>());
  else return false;
  return true;
}

}  // namespace pk

extern "C" {
using namespace pk;

#define PK_BAD ((pegainfer_status_t)hipErrorInvalidValue)

pegainfer_status_t pegainfer_delta_rule(const float* qkv, int64_t qkv_stride, const void* proj, int64_t proj_stride,
                                        int64_t b_off, int64_t a_off, const void* A_log, const void* dt_bias, float* state,
                                        int64_t slot_stride, float* o, int32_t heads, int32_t kv_heads, int32_t dim,
                                        int32_t vdim, const int32_t* entry_row0, const int32_t* entry_slot, int32_t n_entries,
                                        int32_t dtype, pegainfer_stream_t stream) {
  if (n_entries <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || dim > 256 || vdim <= 0 || heads > 65535 || n_entries > 65535)
    return PK_BAD;
  const dim3 grid(ceil_div(vdim, kRecCols), heads, n_entries);
  bool ok = true;
  const bool known = by_dtype(dtype, [&](auto* t) {
    using A = std::remove_pointer_t<decltype(t)>;
    ok = by_slices(dim, [&](auto ns) {
      delta_rule_kernel<decltype(ns)::value, A><<<grid, 256, 0, as_stream(stream)>>>(
          qkv, qkv_stride, static_cast<const A*>(proj), proj_stride, b_off, a_off, static_cast<const A*>(A_log),
          static_cast<const A*>(dt_bias), state, slot_stride, o, heads, kv_heads, dim, vdim, entry_row0, entry_slot);
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_gated_matrix_memory(const void* proj, int64_t proj_stride, int64_t q_off, int64_t k_off,
                                                 int64_t v_off, int64_t i_off, int64_t f_off, const void* i_bias,
                                                 const void* f_bias, float cap, float* state, int64_t slot_stride, float* o,
                                                 int32_t heads, int32_t dim, int32_t vdim, const int32_t* entry_row0,
                                                 const int32_t* entry_slot, int32_t n_entries, int32_t dtype,
                                                 pegainfer_stream_t stream) {
  if (n_entries <= 0) return 0;
  if (heads <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || heads > 65535 || n_entries > 65535 || !(cap > 0.f)) return PK_BAD;
  const dim3 grid(ceil_div(vdim, kRecCols), heads, n_entries);
  bool ok = true;
  const bool known = by_dtype(dtype, [&](auto* t) {
    using A = std::remove_pointer_t<decltype(t)>;
    ok = by_slices(dim, [&](auto ns) {
      matrix_memory_kernel<decltype(ns)::value, A><<<grid, 256, 0, as_stream(stream)>>>(
          static_cast<const A*>(proj), proj_stride, q_off, k_off, v_off, i_off, f_off, static_cast<const A*>(i_bias),
          static_cast<const A*>(f_bias), cap, state, slot_stride, o, heads, dim, vdim, entry_row0, entry_slot);
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

}  // extern "C"

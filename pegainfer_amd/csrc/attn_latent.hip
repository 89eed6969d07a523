// Attention over a paged LATENT cache (beside the paged K/V attention of attn_prefill.hip / attn_decode.hip).
//
// A token's cache entry in a layer is ONE vector shared by all heads: [c (rank) | kr (rot)] - the normalised compressed
// key/value latent and the rotated key part.  The per-head key up-projection is folded into the query
// (qc[t, h, :rank] = Wuk_h^T q_nope[t, h], the "absorb" GEMM) and the value up-projection is applied to the attention
// output (o[t, h] = Wuv_h o_lat[t, h]), so the kernel works on the cache as stored:
//     score_j = (qc[t, h, :] . entry_j) * scale,   o_lat[t, h, :] = sum_j softmax(score)_j entry_j[:rank].
// Every head of a token reads the same entries, and the rows of a step (prompt portions and single decoded tokens of
// several requests) differ only in (request, position): one kernel serves prefill, decode and mixed steps.
// Scores, softmax weights, running maxima / sums and the output accumulators are fp32; the fp32 instance reads an fp32
// cache, the bf16 instance widens bf16 entries exactly.
//
//   latent_prep_kernel        RMS-norm of the latent, rotation of the shared key part and of the query's rotated part,
//                             cache write (one workgroup per token row)
//   latent_attn_kernel        one workgroup per (token, head, key split): 256 keys per round, scores by one thread per
//                             key, online softmax, value accumulation by one thread per latent dimension
//   latent_attn_merge_kernel  combines the key splits of a row (log-sum-exp weights), fixed split order
// A row's result depends on its own query, position and cache entries only: the split count is a function of the row's
// key count alone, so batch composition and portion boundaries change nothing.
#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

constexpr int kLatKeys = 256;        // keys per round = threads per workgroup
constexpr int kLatAcc = 4;           // latent dims per thread: rank <= 1024
constexpr int kLatSplitKeys = 1024;  // keys per split of a row

__device__ __forceinline__ float block_max256(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

template <typename A>
__device__ __forceinline__ const A* latent_entry(const A* cache, int64_t page_stride, int64_t layer_off, int page_size,
                                                 const int32_t* pages, int j, int E) {
  return cache + (int64_t)pages[j / page_size] * page_stride + layer_off + (int64_t)(j % page_size) * E;
}

template <typename A>
__global__ __launch_bounds__(256) void latent_prep_kernel(const A* __restrict__ proj, int64_t row_stride, int64_t dkv_off,
                                                          const A* __restrict__ cw, float eps,
                                                          const float* __restrict__ inv_freq, int rot_dims,
                                                          const int32_t* __restrict__ positions,
                                                          const int32_t* __restrict__ token_req,
                                                          const int32_t* __restrict__ page_indptr,
                                                          const int32_t* __restrict__ page_ids, A* __restrict__ cache,
                                                          int64_t page_stride, int64_t layer_off, int page_size,
                                                          float* __restrict__ qc, int H, int dn, int dr, int r) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const A* row = proj + (int64_t)t * row_stride;
  const A* dkv = row + dkv_off;
  const int pos = positions[t], req = token_req[t];
  const int E = r + dr;
  A* entry = cache + (int64_t)page_ids[page_indptr[req] + pos / page_size] * page_stride + layer_off +
             (int64_t)(pos % page_size) * E;
  float ss = 0.f;
  for (int i = tid; i < r; i += 256) { const float v = ld(dkv + i); ss += v * v; }
  ss = block_sum<4>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)r + eps);
  for (int i = tid; i < r; i += 256) st(entry + i, ld(dkv + i) * inv * ld(cw + i));
  const int half = rot_dims >> 1;
  const float fpos = (float)pos;
  // vector 0 = the shared key part (-> cache), vectors 1 .. H = the heads' rotated query parts (-> qc, fp32)
  for (int w = tid; w < (H + 1) * dr; w += 256) {
    const int vec = w / dr, i = w % dr;
    const A* src = vec == 0 ? dkv + r : row + (int64_t)(vec - 1) * (dn + dr) + dn;
    float out;
    if (i < half) {
      float sn, cs;
      sincosf(fpos * inv_freq[i], &sn, &cs);
      out = ld(src + i) * cs - ld(src + i + half) * sn;
    } else if (i < rot_dims) {
      float sn, cs;
      sincosf(fpos * inv_freq[i - half], &sn, &cs);
      out = ld(src + i) * cs + ld(src + i - half) * sn;
    } else {
      out = ld(src + i);
    }
    if (vec == 0) st(entry + r + i, out);
    else qc[((int64_t)t * H + (vec - 1)) * E + r + i] = out;
  }
}

// partial layout per (row = t * H + h, split): [m, l, acc[rank]] fp32
template <typename A>
__global__ __launch_bounds__(256) void latent_attn_kernel(const float* __restrict__ qc, float* __restrict__ o_lat,
                                                          const A* __restrict__ cache, int64_t page_stride,
                                                          int64_t layer_off, int page_size,
                                                          const int32_t* __restrict__ positions,
                                                          const int32_t* __restrict__ token_req,
                                                          const int32_t* __restrict__ page_indptr,
                                                          const int32_t* __restrict__ page_ids, int H, int r, int dr,
                                                          float scale, float* __restrict__ partial, int max_splits) {
  extern __shared__ float smem[];
  __shared__ float red[4];
  const int t = blockIdx.x, h = blockIdx.y, split = blockIdx.z, tid = threadIdx.x;
  const int E = r + dr;
  const int n_keys = positions[t] + 1;
  const int n_splits = (n_keys + kLatSplitKeys - 1) / kLatSplitKeys;
  if (split >= n_splits) return;
  const int j_lo = split * kLatSplitKeys, j_hi = min(n_keys, j_lo + kLatSplitKeys);
  float* q = smem;            // [E]
  float* p = smem + E;        // [kLatKeys]
  const float* qrow = qc + ((int64_t)t * H + h) * E;
  for (int i = tid; i < E; i += 256) q[i] = qrow[i];
  const int32_t* pages = page_ids + page_indptr[token_req[t]];
  float m = -INFINITY, l = 0.f, acc[kLatAcc] = {};
  __syncthreads();
  for (int j0 = j_lo; j0 < j_hi; j0 += kLatKeys) {
    const int j = j0 + tid;
    float s = -INFINITY;
    if (j < j_hi) {
      const A* e = latent_entry(cache, page_stride, layer_off, page_size, pages, j, E);
      float a = 0.f;
      for (int i = 0; i < E; ++i) a = fmaf(q[i], ld(e + i), a);
      s = a * scale;
    }
    const float m_new = fmaxf(m, block_max256(s, red));
    const float corr = expf(m - m_new);      // m = -inf on the first round: exp(-inf) = 0
    const float pj = j < j_hi ? expf(s - m_new) : 0.f;
    p[tid] = pj;
    l = l * corr + block_sum<4>(pj, red);    // its barriers also publish p[]
    m = m_new;
    const int cnt = min(kLatKeys, j_hi - j0);
#pragma unroll
    for (int k = 0; k < kLatAcc; ++k) {
      const int d = tid + k * 256;
      if (d >= r) break;
      float a = acc[k] * corr;
      for (int i = 0; i < cnt; ++i)
        a = fmaf(p[i], ld(latent_entry(cache, page_stride, layer_off, page_size, pages, j0 + i, E) + d), a);
      acc[k] = a;
    }
    __syncthreads();
  }
  if (n_splits == 1) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int k = 0; k < kLatAcc; ++k) {
      const int d = tid + k * 256;
      if (d < r) o_lat[((int64_t)t * H + h) * r + d] = acc[k] * inv;
    }
  } else {
    float* part = partial + (((int64_t)t * H + h) * max_splits + split) * (r + 2);
    if (tid == 0) { part[0] = m; part[1] = l; }
#pragma unroll
    for (int k = 0; k < kLatAcc; ++k) {
      const int d = tid + k * 256;
      if (d < r) part[2 + d] = acc[k];
    }
  }
}

__global__ __launch_bounds__(256) void latent_attn_merge_kernel(float* __restrict__ o_lat, const float* __restrict__ partial,
                                                                const int32_t* __restrict__ positions, int H, int r,
                                                                int max_splits) {
  const int t = blockIdx.x, h = blockIdx.y;
  const int n_splits = (positions[t] + 1 + kLatSplitKeys - 1) / kLatSplitKeys;
  if (n_splits <= 1) return;
  const float* part = partial + ((int64_t)t * H + h) * max_splits * (r + 2);
  float m = -INFINITY;
  for (int s = 0; s < n_splits; ++s) m = fmaxf(m, part[(int64_t)s * (r + 2)]);
  float l = 0.f;
  for (int s = 0; s < n_splits; ++s) l += part[(int64_t)s * (r + 2) + 1] * expf(part[(int64_t)s * (r + 2)] - m);
  for (int d = threadIdx.x; d < r; d += 256) {
    float a = 0.f;
    for (int s = 0; s < n_splits; ++s) a += part[(int64_t)s * (r + 2) + 2 + d] * expf(part[(int64_t)s * (r + 2)] - m);
    o_lat[((int64_t)t * H + h) * r + d] = a / l;
  }
}

static inline int latent_max_splits(int max_kv_len) { return std::max(1, (max_kv_len + kLatSplitKeys - 1) / kLatSplitKeys); }

}  // namespace pk

extern "C" {
using namespace pk;

pegainfer_status_t pegainfer_latent_prep(const void* proj, int64_t proj_row_stride, int64_t dkv_offset,
                                         const void* c_norm_w, float eps, const float* inv_freq, int32_t rot_dims,
                                         const int32_t* positions, const int32_t* token_req, const int32_t* page_indptr,
                                         const int32_t* page_ids, void* cache, int64_t page_stride, int64_t layer_off,
                                         int32_t page_size, float* qc, int32_t heads, int32_t nope, int32_t rot,
                                         int32_t rank, int32_t n_tokens, int32_t dtype, pegainfer_stream_t stream) {
  if (n_tokens <= 0) return 0;
  if (rot_dims < 0 || rot_dims > rot || (rot_dims & 1) || rank <= 0 || page_size <= 0)
    return (pegainfer_status_t)hipErrorInvalidValue;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        latent_prep_kernel<A><<<n_tokens, 256, 0, as_stream(stream)>>>(
            static_cast<const A*>(proj), proj_row_stride, dkv_offset, static_cast<const A*>(c_norm_w), eps, inv_freq, rot_dims,
            positions, token_req, page_indptr, page_ids, static_cast<A*>(cache), page_stride, layer_off, page_size, qc,
            heads, nope, rot, rank);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

int64_t pegainfer_latent_attention_workspace(int32_t n_tokens, int32_t heads, int32_t rank, int32_t max_kv_len) {
  const int sp = latent_max_splits(max_kv_len);
  return sp <= 1 ? 0 : (int64_t)n_tokens * heads * sp * (rank + 2);
}

pegainfer_status_t pegainfer_latent_attention(const float* qc, float* o_lat, const void* cache, int64_t page_stride,
                                              int64_t layer_off, int32_t page_size, const int32_t* positions,
                                              const int32_t* token_req, const int32_t* page_indptr,
                                              const int32_t* page_ids, int32_t heads, int32_t rank, int32_t rot,
                                              float scale, int32_t n_tokens, int32_t max_kv_len, float* workspace,
                                              int32_t dtype, pegainfer_stream_t stream) {
  if (n_tokens <= 0 || heads <= 0) return 0;
  const int sp = latent_max_splits(max_kv_len);
  if (rank > kLatAcc * 256 || (sp > 1 && !workspace)) return (pegainfer_status_t)hipErrorInvalidValue;
  const size_t smem = (size_t)(rank + rot + kLatKeys) * sizeof(float);
  if (smem > 60000) return (pegainfer_status_t)hipErrorInvalidValue;
  dim3 grid(n_tokens, heads, sp);
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        latent_attn_kernel<A><<<grid, 256, smem, as_stream(stream)>>>(qc, o_lat, static_cast<const A*>(cache), page_stride,
                                                                       layer_off, page_size, positions, token_req, page_indptr,
                                                                       page_ids, heads, rank, rot, scale, workspace, sp);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  if (sp > 1)
    latent_attn_merge_kernel<<<dim3(n_tokens, heads), 256, 0, as_stream(stream)>>>(o_lat, workspace, positions, heads, rank, sp);
  return (pegainfer_status_t)hipGetLastError();
}

}  // extern "C"

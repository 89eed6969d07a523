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
constexpr int kLatSplitKeys = 1024;  // default keys per split of a row

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
                                                          float scale, float* __restrict__ partial, int max_splits, int split_keys) {
  extern __shared__ float smem[];
  __shared__ float red[4];
  const int t = blockIdx.x, h = blockIdx.y, split = blockIdx.z, tid = threadIdx.x;
  const int E = r + dr;
  const int n_keys = positions[t] + 1;
  const int n_splits = (n_keys + split_keys - 1) / split_keys;
  if (split >= n_splits) return;
  const int j_lo = split * split_keys, j_hi = min(n_keys, j_lo + split_keys);
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
                                                                int max_splits, int split_keys) {
  extern __shared__ float wsm[];   // [n_splits] weights exp(m_s - m) / l
  __shared__ float red[4];
  const int t = blockIdx.x, h = blockIdx.y;
  const int n_splits = (positions[t] + split_keys) / split_keys;
  if (n_splits <= 1) return;
  const float* part = partial + ((int64_t)t * H + h) * max_splits * (r + 2);
  // the splits' maxima and sums are read in parallel (one thread each), combined in split order
  float mloc = -INFINITY;
  for (int s = threadIdx.x; s < n_splits; s += 256) mloc = fmaxf(mloc, part[(int64_t)s * (r + 2)]);
  const float m = block_max256(mloc, red);
  for (int s = threadIdx.x; s < n_splits; s += 256) wsm[s] = expf(part[(int64_t)s * (r + 2)] - m);
  __syncthreads();
  float l = 0.f;
  for (int s = 0; s < n_splits; ++s) l += part[(int64_t)s * (r + 2) + 1] * wsm[s];
  const float inv = 1.0f / l;
  for (int d = threadIdx.x; d < r; d += 256) {
    float a = 0.f;
#pragma unroll 4
    for (int s = 0; s < n_splits; ++s) a = fmaf(part[(int64_t)s * (r + 2) + 2 + d], wsm[s], a);
    o_lat[((int64_t)t * H + h) * r + d] = a * inv;
  }
}

// ------------------------------------------------------------------ MFMA form (bf16 cache)
// One workgroup = 64 consecutive (token, head) rows of ONE request (4 waves x 16 rows) against key tiles of 32 cache entries,
// v_mfma_f32_16x16x32_bf16 for both products:
//   scores^T [32 keys x 16 rows]  = entries [32 x E] . q^T          A = entry rows from LDS, B = the wave's q rows (bf16 in LDS)
//   out^T    [16 dims x 16 rows] += c^T [16 x 32 keys] . p^T        A = the SAME row-major tile read transposed, B = the lane's own p
// The score MFMA leaves lane (row l15, group g) with the scores of keys 4g..4g+3 and 16+4g..16+4g+3 of its row - exactly the
// eight values the second product wants from that lane as its B operand when the reduction index is numbered
// kidx = 8g + i  <->  key (i < 4 ? 4g + i : 16 + 4g + i - 4): the weights never move between lanes.  The matching A fragment
// (dim l15 of those eight keys) comes from two ds_read_b64_tr_b16: inside a 16-lane group lane 4j + c gives the address of
// dims 4c..4c+3 of key row j, and lane i receives dim i of the four rows - so the latent tile is staged once, row-major, and
// serves both products.  Every head of a token reads the same entries, so a tile of 64 rows (8 tokens x 8 heads, or one
// decoded token's heads) shares each staged key tile.  The next key tile's global loads are issued into registers before the
// current tile's products and written to LDS after them.  Softmax state (max, sum) and the output accumulators are fp32; q and
// the weights are rounded to bf16 where they enter the matrix cores.  Keys are split over blockIdx.y like the plain form.
constexpr int kTileRows = 64, kTileKeys = 32;
constexpr int kLatPrefetch = 10;     // 16-byte chunks per thread and key tile: 32 keys x (E / 8) <= 2560 chunks, E <= 640

template <int ND>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(const float* __restrict__ qc, float* __restrict__ o_lat,
                                                               const uint16_t* __restrict__ cache, int64_t page_stride,
                                                               int64_t layer_off, int page_size,
                                                               const int32_t* __restrict__ positions,
                                                               const int32_t* __restrict__ token_req,
                                                               const int32_t* __restrict__ page_indptr,
                                                               const int32_t* __restrict__ page_ids,
                                                               const int32_t* __restrict__ tile_row0,
                                                               const int32_t* __restrict__ tile_rows, int H, int r, int dr,
                                                               float scale, float* __restrict__ partial, int max_splits,
                                                               int split_keys) {
  extern __shared__ __align__(16) uint8_t lat_smem[];
  typedef short v4s_t __attribute__((ext_vector_type(4)));
  const int E = r + dr, Epad = (E + 31) & ~31;
  const int qs = Epad + 8, cs = Epad + 8;                          // LDS row strides (bf16 elements), 16-byte multiples
  uint16_t* Qs = reinterpret_cast<uint16_t*>(lat_smem);            // [64][qs]
  uint16_t* Ck = Qs + kTileRows * qs;                              // [32][cs]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l15 = lane & 15, g = lane >> 4;
  const int row0 = tile_row0[blockIdx.x], cnt = tile_rows[blockIdx.x], split = blockIdx.y;
  const int t_first = row0 / H, t_last = (row0 + cnt - 1) / H;
  const int pmax = positions[t_last];
  const int j_lo = split * split_keys;
  if (j_lo > pmax) return;
  const int j_hi = min(pmax + 1, j_lo + split_keys);
  const int32_t* pages = page_ids + page_indptr[token_req[t_first]];
  const int nchunk = E >> 3, tile_chunks = kTileKeys * nchunk;
  // this thread's chunks of a key tile: key kk, element offset ch * 8 - fixed for the whole loop, so the integer divisions
  // happen once (a wave64 VALU instruction costs four cycles; an emulated division about forty of them)
  u32x4 pre[kLatPrefetch];
  int ck_kk[kLatPrefetch], ck_el[kLatPrefetch];
#pragma unroll
  for (int i = 0; i < kLatPrefetch; ++i) {
    const int c = tid + i * 256;
    const int kk = c < tile_chunks ? c / nchunk : -1;
    ck_kk[i] = kk;
    ck_el[i] = kk < 0 ? 0 : (c - kk * nchunk) * 8;
  }
  const int pshift = (page_size & (page_size - 1)) == 0 ? __ffs(page_size) - 1 : -1;
  auto fetch = [&](int j0) {
#pragma unroll
    for (int i = 0; i < kLatPrefetch; ++i) {
      if (ck_kk[i] >= 0) {
        const int j = min(j0 + ck_kk[i], j_hi - 1);
        const int pg = pshift >= 0 ? j >> pshift : j / page_size;
        const int slot = pshift >= 0 ? j & (page_size - 1) : j - pg * page_size;
        pre[i] = *reinterpret_cast<const u32x4*>(cache + (int64_t)pages[pg] * page_stride + layer_off + (int64_t)slot * E + ck_el[i]);
      }
    }
  };
  fetch(j_lo);
  {  // q rows -> bf16 in LDS, eight values per step; only the 16-row blocks that hold rows are staged
    const int qchunks = Epad >> 3, rows_staged = min(kTileRows, (cnt + 15) & ~15);
    for (int c = tid; c < rows_staged * qchunks; c += 256) {
      const int row = c / qchunks, k = (c - row * qchunks) * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row < cnt && k < E) {
        const float* src = qc + (int64_t)(row0 + row) * E + k;
        const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
        v = u32x4{pack_bf2(a.x, a.y), pack_bf2(a.z, a.w), pack_bf2(b.x, b.y), pack_bf2(b.z, b.w)};
      }
      *reinterpret_cast<u32x4*>(Qs + row * qs + k) = v;
    }
  }
  for (int i = tid; i < kTileKeys * (Epad - E); i += 256) Ck[(i / (Epad - E)) * cs + E + i % (Epad - E)] = 0;
  const int my_row = wave * 16 + l15;
  const int pq = my_row < cnt ? positions[(row0 + my_row) / H] : -1;
  const bool wave_live = wave * 16 < cnt;                            // a wave without rows only helps staging
  f32x4 o[ND];
#pragma unroll
  for (int d = 0; d < ND; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  // per-lane element offset of the transposed reads inside the key tile: key row 4g + (l15 >> 2), dims 4 (l15 & 3) ..
  const int tr_off = (4 * g + (l15 >> 2)) * cs + 4 * (l15 & 3);
  for (int j0 = j_lo; j0 < j_hi; j0 += kTileKeys) {
    __syncthreads();                                                 // the previous tile's reads are done
#pragma unroll
    for (int i = 0; i < kLatPrefetch; ++i)
      if (ck_kk[i] >= 0) *reinterpret_cast<u32x4*>(Ck + ck_kk[i] * cs + ck_el[i]) = pre[i];
    __syncthreads();
    if (j0 + kTileKeys < j_hi) fetch(j0 + kTileKeys);
    if (!wave_live) continue;
    // two independent accumulator pairs over alternating k slices: with one wave per SIMD the LDS read -> MFMA -> MFMA chain
    // of a single pair would run at its latency
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f}, s2 = {0.f, 0.f, 0.f, 0.f}, s3 = {0.f, 0.f, 0.f, 0.f};
    const uint16_t* qp = Qs + my_row * qs + g * 8;
    const uint16_t* kp0 = Ck + l15 * cs + g * 8;
    const uint16_t* kp1 = Ck + (16 + l15) * cs + g * 8;
    int kb = 0;
#pragma unroll 2
    for (; kb + 64 <= Epad; kb += 64) {
      const bf16x8_t qa = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(qp + kb));
      const bf16x8_t qb = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(qp + kb + 32));
      const bf16x8_t a0 = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(kp0 + kb));
      const bf16x8_t a1 = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(kp1 + kb));
      const bf16x8_t b0 = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(kp0 + kb + 32));
      const bf16x8_t b1 = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(kp1 + kb + 32));
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qa, s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qa, s1, 0, 0, 0);
      s2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b0, qb, s2, 0, 0, 0);
      s3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b1, qb, s3, 0, 0, 0);
    }
    if (kb < Epad) {
      const bf16x8_t qa = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(qp + kb));
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(kp0 + kb)), qa, s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(kp1 + kb)), qa, s1, 0, 0, 0);
    }
    s0 += s2;
    s1 += s3;
    float sc[8];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = j0 + (i < 4 ? 4 * g + i : 16 + 4 * g + i - 4);
      const float v = (i < 4 ? s0[i] : s1[i - 4]) * scale;
      sc[i] = (j <= pq && j < j_hi) ? v : -INFINITY;
      mx = fmaxf(mx, sc[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __expf(m - m_use);
    float ps[8], lsum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      ps[i] = bf16_round_f(__expf(sc[i] - m_use));   // the sum uses the weights as the matrix core sees them
      lsum += ps[i];
    }
    lsum += __shfl_xor(lsum, 16, kWave);
    lsum += __shfl_xor(lsum, 32, kWave);
    l = l * corr + lsum;
    m = m_new;
    const u32x4 pw = {pack_bf2(ps[0], ps[1]), pack_bf2(ps[2], ps[3]), pack_bf2(ps[4], ps[5]), pack_bf2(ps[6], ps[7])};
    const bf16x8_t pv = __builtin_bit_cast(bf16x8_t, pw);
    const __attribute__((address_space(3))) uint16_t* ck3 =
        (const __attribute__((address_space(3))) uint16_t*)(Ck) + tr_off;
    // the running maximum of most rows stops moving after the first tiles: rescale only when some row of the wave needs it
    if (__any(corr != 1.0f)) {
#pragma unroll
      for (int d = 0; d < ND; ++d) o[d] *= corr;
    }
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      if (d * 16 >= r) break;
      const v4s_t a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s_t __attribute__((address_space(3)))*)(ck3 + d * 16));
      const v4s_t a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s_t __attribute__((address_space(3)))*)(ck3 + d * 16 + 16 * cs));
      const u32x2 w0 = __builtin_bit_cast(u32x2, a0), w1 = __builtin_bit_cast(u32x2, a1);
      const bf16x8_t cv = __builtin_bit_cast(bf16x8_t, u32x4{w0.x, w0.y, w1.x, w1.y});
      o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cv, pv, o[d], 0, 0, 0);
    }
  }
  if (my_row >= cnt) return;
  const int own_splits = (pq + split_keys) / split_keys;
  const int64_t grow = row0 + my_row;
  if (own_splits == 1) {
    if (split != 0) return;
    const float inv = 1.0f / l;
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      const int dd = d * 16 + 4 * g;
      if (dd < r) *reinterpret_cast<f32x4*>(o_lat + grow * r + dd) = o[d] * inv;
    }
  } else if (split < own_splits) {
    float* part = partial + (grow * max_splits + split) * (r + 2);
    if (g == 0) { part[0] = m; part[1] = l; }
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      const int dd = d * 16 + 4 * g;
      if (dd < r) { part[2 + dd] = o[d][0]; part[3 + dd] = o[d][1]; part[4 + dd] = o[d][2]; part[5 + dd] = o[d][3]; }
    }
  }
}

template <int ND>
static void latent_attn_mfma_launch(const float* qc, float* o_lat, const uint16_t* cache, int64_t page_stride, int64_t layer_off,
                                    int page_size, const int32_t* positions, const int32_t* token_req,
                                    const int32_t* page_indptr, const int32_t* page_ids, const int32_t* tile_row0,
                                    const int32_t* tile_rows, int n_tiles, int H, int r, int dr, float scale, float* ws, int sp,
                                    int split_keys, hipStream_t s) {
  const int Epad = (r + dr + 31) & ~31;
  const int lds = (kTileRows + kTileKeys) * (Epad + 8) * 2;
  auto kern = &latent_attn_mfma_kernel<ND>;
  static const bool once = (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                160 * 1024), true);
  (void)once;
  kern<<<dim3(n_tiles, sp), 256, lds, s>>>(qc, o_lat, cache, page_stride, layer_off, page_size, positions, token_req, page_indptr,
                                           page_ids, tile_row0, tile_rows, H, r, dr, scale, ws, sp, split_keys);
}

static inline int latent_split_keys(int split_keys) { return split_keys > 0 ? split_keys : kLatSplitKeys; }
static inline int latent_max_splits(int max_kv_len, int split_keys) {
  const int sk = latent_split_keys(split_keys);
  return std::max(1, (max_kv_len + sk - 1) / sk);
}

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

int64_t pegainfer_latent_attention_workspace(int32_t n_tokens, int32_t heads, int32_t rank, int32_t max_kv_len,
                                             int32_t split_keys) {
  const int sp = latent_max_splits(max_kv_len, split_keys);
  return sp <= 1 ? 0 : (int64_t)n_tokens * heads * sp * (rank + 2);
}

int32_t pegainfer_latent_attention_tiled_ok(int32_t rank, int32_t rot, int64_t page_stride, int64_t layer_off, int32_t dtype) {
  const int Epad = (rank + rot + 31) & ~31;
  return dtype == kDtBf16 && rank % 16 == 0 && rank <= 512 && rot % 8 == 0 && page_stride % 8 == 0 && layer_off % 8 == 0 &&
         kTileKeys * ((rank + rot) / 8) <= kLatPrefetch * 256 && (kTileRows + kTileKeys) * (Epad + 8) * 2 <= 160 * 1024;
}

pegainfer_status_t pegainfer_latent_attention(const float* qc, float* o_lat, const void* cache, int64_t page_stride,
                                              int64_t layer_off, int32_t page_size, const int32_t* positions,
                                              const int32_t* token_req, const int32_t* page_indptr,
                                              const int32_t* page_ids, int32_t heads, int32_t rank, int32_t rot,
                                              float scale, int32_t n_tokens, int32_t max_kv_len, int32_t split_keys,
                                              float* workspace, const int32_t* tile_row0, const int32_t* tile_rows,
                                              int32_t n_tiles, int32_t dtype, pegainfer_stream_t stream) {
  if (n_tokens <= 0 || heads <= 0) return 0;
  const int sk = latent_split_keys(split_keys), sp = latent_max_splits(max_kv_len, split_keys);
  if (sp > 1 && !workspace) return (pegainfer_status_t)hipErrorInvalidValue;
  hipStream_t s = as_stream(stream);
  if (tile_row0) {
    if (!tile_rows || n_tiles <= 0 || !pegainfer_latent_attention_tiled_ok(rank, rot, page_stride, layer_off, dtype) ||
        (reinterpret_cast<uintptr_t>(cache) & 15u))
      return (pegainfer_status_t)hipErrorInvalidValue;
    const uint16_t* c = static_cast<const uint16_t*>(cache);
#define LAT_LAUNCH(ND) latent_attn_mfma_launch<ND>(qc, o_lat, c, page_stride, layer_off, page_size, positions, token_req, page_indptr, \
                                                   page_ids, tile_row0, tile_rows, n_tiles, heads, rank, rot, scale, workspace, sp, sk, s)
    if (rank <= 64) LAT_LAUNCH(4);
    else if (rank <= 128) LAT_LAUNCH(8);
    else if (rank <= 256) LAT_LAUNCH(16);
    else LAT_LAUNCH(32);
#undef LAT_LAUNCH
  } else {
    if (rank > kLatAcc * 256) return (pegainfer_status_t)hipErrorInvalidValue;
    const size_t smem = (size_t)(rank + rot + kLatKeys) * sizeof(float);
    if (smem > 60000) return (pegainfer_status_t)hipErrorInvalidValue;
    dim3 grid(n_tokens, heads, sp);
    if (!by_dtype(dtype, [&](auto* t) {
          using A = std::remove_pointer_t<decltype(t)>;
          latent_attn_kernel<A><<<grid, 256, smem, s>>>(qc, o_lat, static_cast<const A*>(cache), page_stride, layer_off, page_size,
                                                        positions, token_req, page_indptr, page_ids, heads, rank, rot, scale,
                                                        workspace, sp, sk);
        }))
      return (pegainfer_status_t)hipErrorInvalidValue;
  }
  if (sp > 1) latent_attn_merge_kernel<<<dim3(n_tokens, heads), 256, (size_t)sp * sizeof(float), s>>>(o_lat, workspace, positions, heads, rank, sp, sk);
  return (pegainfer_status_t)hipGetLastError();
}

}  // extern "C"

// C++ host runtime of the Feruzen decoder on MI355X (include/pegainfer_feruzen.h).  Same shape as the runtimes next to it:
// one model = one device + one in-order HIP stream, requests are KvState slots over the shared PagePool (kv_pool.h) plus a
// region of the fp32 state arena (seq_state.h), a step's metadata is ONE pinned block and ONE hipMemcpyAsync, every op goes
// through the kernel library's C ABI (pegainfer_kernels.h: tuned bf16 GEMM routes, samplers; pegainfer_kernels_blocks.h:
// everything else).
//
// What a step does per layer (T = all token rows of the step, prompts' portions and single tokens alike; x = fp32 stream):
//   hb     = x + time_conv(x; canon1)                       input convolution, tail of taps - 1 inputs per request
//   proj   = Wstack hb                                      ONE GEMM over all projections of the mixer, stacked by rows
//   delta    : time_conv + silu on the q | k | v columns -> gated delta rule over the request's matrix state -> per-head
//              RMS norm * weight * silu(gate)
//   parallel : left  q/k RMS norm + pair rotation -> paged cache -> causal softmax attention (* left factor)
//              right exponentially gated matrix memory -> per-head RMS norm * weight * sigmoid(gate) (* right factor)
//              both write into ONE row [left | right], so the two output projections are one GEMM over [Wo_l | Wo_r]
//   y      = Wo mix;   x += grms(y; norm1)                  norm on the OUTPUT, residual sum, bf16 image of x for the ff
//   ff     : [gate ; up] GEMM -> clamp-GLU -> down           dense, or routed (softmax router -> sort by expert -> grouped
//            GEMMs -> weighted sum + shared expert)
//   X_next = x + grms(ff; norm2);  x = sum_j dwa[j] X_j     one launch: norm, residual, depth-weighted sum over the layers
// Key/value cache: page-first [page][attention layer][k: slot, kv head, dim | v: slot, kv head, vdim].
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "kv_pool.h"
#include "seq_state.h"
#include "safetensors_loader.h"
#include "pegainfer_kernels.h"
#include "pegainfer_kernels_blocks.h"
#include "pegainfer_kernels_ext.h"
#include "pegainfer_qwen3.h"     // pegainfer_logprobs_from_logits (pure host)
#include "pegainfer_duguzen.h"   // PEGAINFER_DTYPE_*
#include "pegainfer_feruzen.h"

namespace pfz {

using pq::KvState;
using pq::PagePool;
using pst::Json;

#define FZ_HIP(expr)                                                   \
  do {                                                                 \
    hipError_t e_ = (expr);                                            \
    if (e_ != hipSuccess) {                                            \
      set_error(std::string(#expr) + ": " + hipGetErrorString(e_));    \
      return -1;                                                       \
    }                                                                  \
  } while (0)
#define FZ_K(expr)                                                     \
  do {                                                                 \
    if ((expr) != 0) {                                                 \
      set_error(std::string(#expr) + " failed");                       \
      return -1;                                                       \
    }                                                                  \
  } while (0)

static inline uint16_t host_f2bf(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}
static inline float host_bf2f(uint16_t h) {
  const uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

constexpr int kPageSize = 16;        // tokens per cache page, as in the other runtimes
constexpr float kGluAlpha = 1.702f;  // the clamp-GLU's sigmoid slope, fixed by the design
constexpr int kAttRows = 16;         // (token, query head) rows of one attention workgroup

enum { kDelta = 1, kParallel = 2 };
struct AttnCfg { int heads = 0, kv = 0, dim = 0, vdim = 0, rot_dims = 0; double base = 10000.0; float scale = 1.f; };
struct MemCfg { int heads = 0, dim = 0, vdim = 0; float cap = 1.f; };
struct DeltaCfg { int heads = 0, kv = 0, dim = 0, vdim = 0, taps = 0; };
struct GluCfg { int ff = 0; float limit = 0.f; };
struct MlpCfg { int kind = 0 /* 0 none, 1 dense, 2 routed */; GluCfg glu; int experts = 0, top = 0; bool has_shared = false; GluCfg shared; };
struct LayerCfg {
  int type = 0;
  DeltaCfg dl;
  AttnCfg at;
  MemCfg mm;
  float left_scale = 1.f, right_scale = 1.f;
  MlpCfg mlp;
  // columns of the stacked projection
  int o_q = 0, o_k = 0, o_v = 0, o_g = 0, o_b = 0, o_a = 0;           // delta
  int o_rq = 0, o_rk = 0, o_rv = 0, o_rg = 0, o_ri = 0, o_rf = 0;     // parallel, right (left uses o_q / o_k / o_v)
  int proj_rows = 0, mix_cols = 0, conv_ch = 0;
  // state and cache
  int64_t st_canon = 0, st_conv = 0, st_mem = 0;
  int64_t k_off = 0, v_off = 0;
  int tile_set = -1;
  int fast_hd = 0;   // 128 / 256: the matrix-core attention kernels of pegainfer_kernels.h fit this layer (bf16, dim == vdim)
};
struct LayerW {
  void *norm1 = nullptr, *norm2 = nullptr, *canon = nullptr, *dwa = nullptr, *proj = nullptr, *o = nullptr;
  void *conv = nullptr, *A_log = nullptr, *dt_bias = nullptr, *onorm = nullptr;                  // delta
  void *q_norm = nullptr, *k_norm = nullptr, *rnorm = nullptr, *i_bias = nullptr, *f_bias = nullptr;   // parallel
  float* inv_freq = nullptr;
  void *gate_up = nullptr, *down = nullptr;                                           // dense, or the shared expert
  void *router = nullptr, *gate_up_e = nullptr, *down_e = nullptr;                    // routed
};

struct Model {
  int device = 0, dtype = 0, D = 0, V = 0, max_requests = 0, num_pages = 0, groups = 1, canon_taps = 1;
  float eps = 1e-5f;
  bool plain_kernels = false, finalized = false;
  std::string err;
  std::vector<LayerCfg> layers;
  std::vector<LayerW> weights;
  void *embed = nullptr, *final_norm = nullptr;
  std::map<std::string, std::vector<uint16_t>> staged;
  std::vector<void*> owned;
  int64_t weight_bytes = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  float last_step_ms = 0.f;
  // cache and state
  int64_t page_stride = 0;
  void* cache = nullptr;
  PagePool pool{0};
  std::vector<KvState> requests;
  pq::StateLayout state_layout;
  float* state = nullptr;
  struct TileSet { int per = 1, fast_hd = 0, heads = 0, kv = 0; };
  std::vector<TileSet> tile_sets;   // distinct (query heads per kv head, attention form) of the attention layers
  // step buffers
  size_t cap_rows = 0, cap_want = 0, cap_meta = 0;
  std::vector<void*> step_owned, want_owned;
  float *gates32 = nullptr;
  int mx_dheads = 0;
  float *x = nullptr, *xs = nullptr, *qkv32 = nullptr, *q32 = nullptr, *o32 = nullptr, *ypairs = nullptr, *route_w = nullptr, *route_logits = nullptr;
  Half* split_tmp_v = nullptr;   // partials of the partition decode attention
  float* split_tmp_s = nullptr;
  void *q16 = nullptr, *attn16 = nullptr;   // stored-type queries and contiguous output of the matrix-core attention
  void *hb = nullptr, *xb = nullptr, *proj = nullptr, *mix = nullptr, *y = nullptr, *gu = nullptr, *act = nullptr, *ys = nullptr,
       *gu_e = nullptr, *act_e = nullptr;
  int32_t *route_e = nullptr, *pos_pair = nullptr, *pos_row = nullptr, *tiles = nullptr;
  int max_tiles = 0;
  float *xw = nullptr, *logits32 = nullptr;
  void *hw = nullptr, *logits = nullptr;
  Half* logits16 = nullptr;
  int32_t* tokens_d = nullptr;
  uint8_t* top1_state = nullptr;
  uint8_t *meta_host = nullptr, *meta_dev = nullptr;
  float* probs_scratch = nullptr;
  Half* top1_value = nullptr;
  uint8_t *row_states = nullptr, *valid_scratch = nullptr;
  int32_t* sample_out_d = nullptr;
  int last_rows = 0;
  std::vector<float> lp_row;
  bool tap_on = false;
  float* tap = nullptr;
  size_t tap_cap = 0;
  int tap_rows = 0;
  int mx_proj = 0, mx_mix = 0, mx_conv = 0, mx_q = 0, mx_o = 0, mx_ff = 0, mx_top = 0, mx_gu_e = 0, mx_experts = 0;

  struct GraphKey {
    int n, want; bool tokens, plain; int split;
    bool operator==(const GraphKey& o) const { return n == o.n && want == o.want && tokens == o.tokens && plain == o.plain && split == o.split; }
  };
  std::vector<std::pair<GraphKey, hipGraphExec_t>> graphs;   // captured decode steps, one per shape
  bool graphs_on = [] { const char* e = getenv("PEGAINFER_FERUZEN_GRAPH"); return !(e && e[0] == '0'); }();
  void drop_graphs() {   // the buffers a graph was recorded over are about to move
    for (auto& g : graphs) (void)hipGraphExecDestroy(g.second);
    graphs.clear();
  }

  int set_error(const std::string& e) { err = e; return -1; }
  size_t esize() const { return dtype == PEGAINFER_DTYPE_F32 ? 4 : 2; }
  pegainfer_stream_t S() const { return reinterpret_cast<pegainfer_stream_t>(stream); }
  void* at(void* p, size_t elems) const { return static_cast<uint8_t*>(p) + elems * esize(); }
  const void* at(const void* p, size_t elems) const { return static_cast<const uint8_t*>(p) + elems * esize(); }
  static int pad8(int n) { return (n + 7) & ~7; }

  // ------------------------------------------------------------------ configuration
  static int geti(const Json* j, const char* k, int d) { return j ? (int)j->number_or(k, d) : d; }
  static float getf(const Json* j, const char* k, double d) { return j ? (float)j->number_or(k, d) : (float)d; }
  int parse_glu(const Json* j, GluCfg* g, const std::string& where) {
    if (!j || j->kind != Json::Obj) return set_error("config: " + where + " without sizes");
    g->ff = geti(j, "ff", 0);
    g->limit = getf(j, "limit", 0.0);
    if (g->ff <= 0 || !(g->limit > 0.f)) return set_error("config: " + where + " needs ff and a positive limit");
    return 0;
  }
  int parse_config(const std::string& text) {
    Json j;
    if (!pst::JsonParser(text.data(), text.size()).parse(&j) || j.kind != Json::Obj) return set_error("config: not a JSON object");
    const Json* arch = j.get("architecture");
    if (!arch || arch->str != "Feruzen") return set_error("config: architecture is not Feruzen");
    D = geti(&j, "width", 0);
    V = geti(&j, "vocab", 0);
    if (const Json* n = j.get("norm")) {
      eps = (float)n->number_or("eps", 1e-5);
      groups = geti(n, "groups", 1);
    }
    canon_taps = geti(j.get("canon"), "taps", 1);
    const Json* ls = j.get("layers");
    if (D <= 0 || V <= 0 || !ls || ls->kind != Json::Arr || ls->arr.empty()) return set_error("config: width / vocab / layers missing");
    if (groups < 1 || D % groups) return set_error("config: norm.groups does not divide the width");
    if (canon_taps < 1 || canon_taps > 64) return set_error("config: canon.taps outside 1 .. 64");
    int64_t off = 0;
    for (size_t i = 0; i < ls->arr.size(); ++i) {
      const Json& l = ls->arr[i];
      const std::string li = std::to_string(i);
      LayerCfg c;
      const Json* ty = l.get("type");
      const Json* mx = l.get("mixer");
      if (!ty || !mx || mx->kind != Json::Obj) return set_error("config: layer " + li + " without type / mixer");
      c.st_canon = state_layout.reserve("l" + li + ".canon", (int64_t)(canon_taps - 1) * D);
      if (ty->str == "delta") {
        c.type = kDelta;
        DeltaCfg& d = c.dl;
        d.heads = geti(mx, "heads", 0);
        d.kv = geti(mx, "kv_heads", d.heads);
        d.dim = geti(mx, "dim", 0);
        d.vdim = geti(mx, "vdim", 0);
        d.taps = geti(mx, "conv", 1);
        if (d.heads <= 0 || d.kv <= 0 || d.heads % d.kv || d.dim <= 0 || d.dim > 256 || d.vdim <= 0 || d.taps < 1 || d.taps > 64)
          return set_error("config: unsupported delta mixer sizes in layer " + li);
        c.o_q = 0;
        c.o_k = d.kv * d.dim;
        c.o_v = 2 * d.kv * d.dim;
        c.conv_ch = c.o_v + d.heads * d.vdim;
        c.o_g = c.conv_ch;
        c.o_b = c.o_g + d.heads * d.vdim;
        c.o_a = c.o_b + d.heads;
        c.proj_rows = pad8(c.o_a + d.heads);
        c.mix_cols = d.heads * d.vdim;
        c.st_conv = state_layout.reserve("l" + li + ".conv", (int64_t)(d.taps - 1) * c.conv_ch);
        c.st_mem = state_layout.reserve("l" + li + ".memory", (int64_t)d.heads * d.dim * d.vdim);
      } else if (ty->str == "parallel") {
        c.type = kParallel;
        const Json *lf = mx->get("left"), *rt = mx->get("right");
        if (!lf || !rt) return set_error("config: parallel mixer without left / right in layer " + li);
        AttnCfg& a = c.at;
        a.heads = geti(lf, "heads", 0);
        a.kv = geti(lf, "kv_heads", a.heads);
        a.dim = geti(lf, "dim", 0);
        a.vdim = geti(lf, "vdim", a.dim);
        a.scale = getf(lf, "scale", 1.0 / std::sqrt((double)std::max(1, a.dim)));
        const Json* rot = lf->get("rot");
        a.rot_dims = rot ? geti(rot, "dims", a.dim) : 0;
        a.base = rot ? rot->number_or("base", 10000.0) : 10000.0;
        MemCfg& m = c.mm;
        m.heads = geti(rt, "heads", 0);
        m.dim = geti(rt, "dim", 0);
        m.vdim = geti(rt, "vdim", 0);
        m.cap = getf(rt, "gate_cap", 0.0);
        c.left_scale = getf(mx, "left_scale", 1.0);
        c.right_scale = getf(mx, "right_scale", 1.0);
        if (a.heads <= 0 || a.kv <= 0 || a.heads % a.kv || a.dim <= 0 || a.dim > 256 || a.vdim <= 0 || a.vdim > 256 ||
            a.rot_dims < 0 || a.rot_dims > a.dim || (a.rot_dims & 1))
          return set_error("config: unsupported attention sizes in layer " + li);
        if (m.heads <= 0 || m.dim <= 0 || m.dim > 256 || m.vdim <= 0 || !(m.cap > 0.f))
          return set_error("config: unsupported matrix-memory sizes in layer " + li);
        c.o_q = 0;
        c.o_k = a.heads * a.dim;
        c.o_v = c.o_k + a.kv * a.dim;
        c.o_rq = c.o_v + a.kv * a.vdim;
        c.o_rk = c.o_rq + m.heads * m.dim;
        c.o_rv = c.o_rk + m.heads * m.dim;
        c.o_rg = c.o_rv + m.heads * m.vdim;
        c.o_ri = c.o_rg + m.heads * m.vdim;
        c.o_rf = c.o_ri + m.heads;
        c.proj_rows = pad8(c.o_rf + m.heads);
        c.mix_cols = a.heads * a.vdim + m.heads * m.vdim;
        c.st_mem = state_layout.reserve("l" + li + ".memory", (int64_t)m.heads * m.dim * m.vdim + (int64_t)m.heads * m.dim + m.heads);
        c.k_off = off;
        c.v_off = off + (int64_t)kPageSize * a.kv * a.dim;
        off = c.v_off + (int64_t)kPageSize * a.kv * a.vdim;
        // matrix-core attention (the kernels Qwen3 / Qwen3.5 run): bf16, equal key and value size 128 or 256, 16-byte
        // aligned cache parts; page_stride's own alignment is checked once all layers are known
        if (dtype == PEGAINFER_DTYPE_BF16 && a.dim == a.vdim && (a.dim == 128 || a.dim == 256) && c.k_off % 8 == 0 && c.v_off % 8 == 0)
          c.fast_hd = a.dim;
      } else {
        return set_error("config: layer " + li + " has an unknown mixer type");
      }
      const Json* mlp = l.get("mlp");
      if (mlp && mlp->kind == Json::Obj) {
        const Json* kind = mlp->get("kind");
        if (kind && kind->str == "dense") {
          c.mlp.kind = 1;
          if (parse_glu(mlp, &c.mlp.glu, "dense feed-forward of layer " + li)) return -1;
        } else if (kind && kind->str == "moe") {
          c.mlp.kind = 2;
          if (parse_glu(mlp->get("expert"), &c.mlp.glu, "experts of layer " + li)) return -1;
          const Json* rt = mlp->get("router");
          c.mlp.experts = geti(rt, "experts", 0);
          c.mlp.top = geti(rt, "top", 0);
          if (c.mlp.experts <= 0 || c.mlp.top <= 0 || c.mlp.top > c.mlp.experts || c.mlp.experts > 7000)
            return set_error("config: unsupported router in layer " + li);
          const Json* sh = mlp->get("shared");
          if (sh && sh->kind == Json::Obj) {
            c.mlp.has_shared = true;
            if (parse_glu(sh, &c.mlp.shared, "shared expert of layer " + li)) return -1;
          }
        } else {
          return set_error("config: unknown feed-forward kind in layer " + li);
        }
      }
      layers.push_back(c);
    }
    page_stride = std::max<int64_t>(off, 1);
    for (auto& c : layers) {
      if (c.type != kParallel) continue;
      if (page_stride % 8) c.fast_hd = 0;
      const int per = c.at.heads / c.at.kv;
      size_t k = 0;
      while (k < tile_sets.size() && !(tile_sets[k].per == per && tile_sets[k].fast_hd == c.fast_hd &&
                                       (!c.fast_hd || (tile_sets[k].heads == c.at.heads && tile_sets[k].kv == c.at.kv))))
        ++k;
      if (k == tile_sets.size()) tile_sets.push_back({per, c.fast_hd, c.at.heads, c.at.kv});
      c.tile_set = (int)k;
    }
    weights.resize(layers.size());
    for (auto& c : layers) {
      mx_proj = std::max(mx_proj, c.proj_rows);
      mx_mix = std::max(mx_mix, c.mix_cols);
      mx_conv = std::max(mx_conv, c.conv_ch);
      if (c.type == kDelta) mx_o = std::max(mx_o, c.dl.heads * c.dl.vdim);
      if (c.type == kDelta) mx_dheads = std::max(mx_dheads, c.dl.heads);
      if (c.type == kParallel) {
        mx_q = std::max(mx_q, c.at.heads * c.at.dim);
        mx_o = std::max(mx_o, c.mm.heads * c.mm.vdim);
      }
      if (c.mlp.kind == 1) mx_ff = std::max(mx_ff, c.mlp.glu.ff);
      if (c.mlp.kind == 2) {
        mx_top = std::max(mx_top, c.mlp.top);
        mx_gu_e = std::max(mx_gu_e, c.mlp.top * 2 * c.mlp.glu.ff);
        mx_experts = std::max(mx_experts, c.mlp.experts);
        if (c.mlp.has_shared) mx_ff = std::max(mx_ff, c.mlp.shared.ff);
      }
    }
    return 0;
  }

  // ------------------------------------------------------------------ device memory
  template <typename T>
  int dalloc(T** p, size_t count, std::vector<void*>* into = nullptr) {
    void* raw = nullptr;
    FZ_HIP(hipMalloc(&raw, std::max<size_t>(count, 1) * sizeof(T)));
    FZ_HIP(hipMemset(raw, 0, std::max<size_t>(count, 1) * sizeof(T)));
    (into ? into : &owned)->push_back(raw);
    *p = static_cast<T*>(raw);
    return 0;
  }
  int dalloc_a(void** p, size_t count, std::vector<void*>* into = nullptr) {
    uint8_t* raw = nullptr;
    if (dalloc(&raw, count * esize(), into)) return -1;
    *p = raw;
    return 0;
  }
  static void free_all(std::vector<void*>* v) {
    for (void* p : *v) (void)hipFree(p);
    v->clear();
  }

  int init(int max_tokens) {
    FZ_HIP(hipSetDevice(device));
    cublas_init();
    FZ_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    FZ_HIP(hipEventCreate(&ev0));
    FZ_HIP(hipEventCreate(&ev1));
    num_pages = std::max(1, (max_tokens + kPageSize - 1) / kPageSize);
    pool = PagePool(num_pages);
    requests.assign((size_t)max_requests, KvState());
    if (dalloc_a(&cache, (size_t)num_pages * (size_t)page_stride)) return -1;
    if (dalloc(&state, (size_t)max_requests * (size_t)state_layout.floats_per_slot())) return -1;
    bool any_fast = false;
    for (auto& c : layers) any_fast = any_fast || c.fast_hd != 0;
    if (any_fast && (dalloc(&split_tmp_v, (size_t)max_requests * pq::kSplitMaxChunksPerRequest * (size_t)std::max(1, mx_q)) ||
                     dalloc(&split_tmp_s, (size_t)max_requests * pq::kSplitMaxChunksPerRequest * (size_t)std::max(1, mx_q))))
      return -1;
    if (dalloc(&probs_scratch, (size_t)V) || dalloc(&top1_value, 1) || dalloc(&row_states, 1024 * 1024) ||
        dalloc(&valid_scratch, 1) || dalloc(&sample_out_d, 1))
      return -1;
    return 0;
  }

  // ------------------------------------------------------------------ weights
  typedef std::vector<std::pair<std::string, std::vector<int64_t>>> TensorList;
  static void glu_tensors(TensorList* out, const std::string& p, const GluCfg& g, int D) {
    out->push_back({p + ".gate", {g.ff, D}});
    out->push_back({p + ".up", {g.ff, D}});
    out->push_back({p + ".down", {D, g.ff}});
  }
  TensorList tensor_list() const {
    TensorList out;
    out.push_back({"embed", {V, D}});
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      const std::string p = "l" + std::to_string(i), m = p + ".mix";
      out.push_back({p + ".norm1", {D}});
      if (c.mlp.kind) out.push_back({p + ".norm2", {D}});
      out.push_back({p + ".canon1", {D, canon_taps}});
      out.push_back({p + ".dwa", {(int64_t)i + 2}});
      if (c.type == kDelta) {
        const DeltaCfg& d = c.dl;
        for (const char* n : {".q", ".k"}) {
          out.push_back({m + n, {d.kv * d.dim, D}});
          out.push_back({m + n + ".conv", {d.kv * d.dim, d.taps}});
        }
        out.push_back({m + ".v", {d.heads * d.vdim, D}});
        out.push_back({m + ".v.conv", {d.heads * d.vdim, d.taps}});
        out.push_back({m + ".b", {d.heads, D}});
        out.push_back({m + ".a", {d.heads, D}});
        out.push_back({m + ".A_log", {d.heads}});
        out.push_back({m + ".dt_bias", {d.heads}});
        out.push_back({m + ".norm", {d.vdim}});
        out.push_back({m + ".g", {d.heads * d.vdim, D}});
        out.push_back({m + ".o", {D, d.heads * d.vdim}});
      } else {
        const AttnCfg& a = c.at;
        const MemCfg& r = c.mm;
        out.push_back({m + ".left.q", {a.heads * a.dim, D}});
        out.push_back({m + ".left.k", {a.kv * a.dim, D}});
        out.push_back({m + ".left.v", {a.kv * a.vdim, D}});
        out.push_back({m + ".left.q.norm", {a.dim}});
        out.push_back({m + ".left.k.norm", {a.dim}});
        out.push_back({m + ".left.o", {D, a.heads * a.vdim}});
        out.push_back({m + ".right.q", {r.heads * r.dim, D}});
        out.push_back({m + ".right.k", {r.heads * r.dim, D}});
        out.push_back({m + ".right.v", {r.heads * r.vdim, D}});
        out.push_back({m + ".right.g", {r.heads * r.vdim, D}});
        out.push_back({m + ".right.o", {D, r.heads * r.vdim}});
        out.push_back({m + ".right.norm", {r.heads * r.vdim}});
        out.push_back({m + ".right.i", {r.heads, D}});
        out.push_back({m + ".right.i.b", {r.heads}});
        out.push_back({m + ".right.f", {r.heads, D}});
        out.push_back({m + ".right.f.b", {r.heads}});
      }
      if (c.mlp.kind == 1) {
        glu_tensors(&out, p + ".mlp", c.mlp.glu, D);
      } else if (c.mlp.kind == 2) {
        for (int e = 0; e < c.mlp.experts; ++e) glu_tensors(&out, p + ".mlp.e" + std::to_string(e), c.mlp.glu, D);
        out.push_back({p + ".mlp.router", {c.mlp.experts, D}});
        if (c.mlp.has_shared) glu_tensors(&out, p + ".mlp.shared", c.mlp.shared, D);
      }
    }
    out.push_back({"final.norm", {D}});
    return out;
  }
  static int64_t numel(const std::vector<int64_t>& s) { int64_t n = 1; for (int64_t d : s) n *= d; return n; }
  static bool ends_with(const std::string& s, const char* suf) {
    const size_t n = std::strlen(suf);
    return s.size() >= n && s.compare(s.size() - n, n, suf) == 0;
  }

  int load_tensor(const std::string& name, const uint16_t* bits, int64_t n) {
    if (finalized) return set_error("load_tensor after finalize");
    staged[name].assign(bits, bits + n);
    return 0;
  }
  int fill_synthetic(uint64_t seed, float std) {
    uint64_t state64 = seed * 0x9E3779B97F4A7C15ull + 0x7654321ull;
    auto g = [&state64]() {   // splitmix64; a unit-variance value = four uniforms summed, centred and scaled
      state64 += 0x9E3779B97F4A7C15ull;
      uint64_t z = state64;
      z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
      z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
      z ^= z >> 31;
      const float u = (float)(z & 0xFFFF) + (float)((z >> 16) & 0xFFFF) + (float)((z >> 32) & 0xFFFF) + (float)(z >> 48);
      return (u * (1.0f / 65536.0f) - 2.0f) * 1.7320508f;
    };
    for (auto& t : tensor_list()) {
      const std::string& n = t.first;
      std::vector<uint16_t>& v = staged[n];
      v.resize((size_t)numel(t.second));
      const bool is_dwa = ends_with(n, ".dwa"), is_conv = ends_with(n, ".conv") || ends_with(n, ".canon1");
      const bool is_bias = ends_with(n, ".b") && t.second.size() == 1;
      const bool is_norm = t.second.size() == 1 && !is_dwa && !is_bias && !ends_with(n, ".A_log") && !ends_with(n, ".dt_bias");
      for (size_t k = 0; k < v.size(); ++k) {
        const float z = g();
        float val = std * z;
        if (is_dwa) val = (k + 1 == v.size() ? 0.8f : 0.2f / (float)(v.size() - 1)) + 0.02f * z;
        else if (is_conv) val = 0.3f * z;
        else if (is_norm) val = 1.0f + 0.1f * z;
        else if (is_bias) val = ends_with(n, ".f.b") ? 3.0f + 0.5f * z : 0.5f * z;
        else if (ends_with(n, ".A_log")) val = -1.0f + 0.5f * z;
        else if (ends_with(n, ".dt_bias")) val = 0.3f * z;
        v[k] = host_f2bf(val);
      }
    }
    return 0;
  }
  int upload(void** out, const uint16_t* bits, size_t n) {
    if (dalloc_a(out, n)) return -1;
    if (dtype == PEGAINFER_DTYPE_BF16) {
      FZ_HIP(hipMemcpy(*out, bits, n * 2, hipMemcpyHostToDevice));
    } else {
      std::vector<float> f(n);
      for (size_t i = 0; i < n; ++i) f[i] = host_bf2f(bits[i]);
      FZ_HIP(hipMemcpy(*out, f.data(), n * 4, hipMemcpyHostToDevice));
    }
    weight_bytes += (int64_t)(n * esize());
    return 0;
  }
  const std::vector<uint16_t>* need(const std::string& name, int64_t n) {
    auto it = staged.find(name);
    if (it == staged.end()) { set_error("missing tensor " + name); return nullptr; }
    if ((int64_t)it->second.size() != n) { set_error("tensor " + name + " has the wrong number of elements"); return nullptr; }
    return &it->second;
  }
  int up(void** out, const std::string& name, int64_t n) {
    const auto* v = need(name, n);
    return v ? upload(out, v->data(), v->size()) : -1;
  }
  // several [rows_i, cols] tensors stacked by rows, zero rows appended up to pad_rows
  int up_stacked(void** out, const std::vector<std::pair<std::string, int64_t>>& parts, int64_t cols, int64_t pad_rows) {
    std::vector<uint16_t> st;
    for (auto& p : parts) {
      const auto* v = need(p.first, p.second * cols);
      if (!v) return -1;
      st.insert(st.end(), v->begin(), v->end());
    }
    if (pad_rows > 0) st.resize((size_t)(pad_rows * cols), 0);
    return upload(out, st.data(), st.size());
  }
  int up_glu(void** gate_up, void** down, const std::string& p, const GluCfg& g) {
    return (up_stacked(gate_up, {{p + ".gate", g.ff}, {p + ".up", g.ff}}, D, 0) || up(down, p + ".down", (int64_t)D * g.ff)) ? -1 : 0;
  }
  int finalize() {
    if (finalized) return 0;
    if (up(&embed, "embed", (int64_t)V * D) || up(&final_norm, "final.norm", D)) return -1;
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      LayerW& w = weights[i];
      const std::string p = "l" + std::to_string(i), m = p + ".mix";
      if (up(&w.norm1, p + ".norm1", D) || (c.mlp.kind && up(&w.norm2, p + ".norm2", D)) ||
          up(&w.canon, p + ".canon1", (int64_t)D * canon_taps) || up(&w.dwa, p + ".dwa", (int64_t)i + 2))
        return -1;
      if (c.type == kDelta) {
        const DeltaCfg& d = c.dl;
        const int64_t qk = (int64_t)d.kv * d.dim, hv = (int64_t)d.heads * d.vdim;
        if (up_stacked(&w.proj, {{m + ".q", qk}, {m + ".k", qk}, {m + ".v", hv}, {m + ".g", hv}, {m + ".b", d.heads}, {m + ".a", d.heads}},
                       D, c.proj_rows) ||
            up_stacked(&w.conv, {{m + ".q.conv", qk}, {m + ".k.conv", qk}, {m + ".v.conv", hv}}, d.taps, 0) ||
            up(&w.A_log, m + ".A_log", d.heads) || up(&w.dt_bias, m + ".dt_bias", d.heads) || up(&w.onorm, m + ".norm", d.vdim) ||
            up(&w.o, m + ".o", (int64_t)D * hv))
          return -1;
      } else {
        const AttnCfg& a = c.at;
        const MemCfg& r = c.mm;
        const int64_t rq = (int64_t)r.heads * r.dim, rv = (int64_t)r.heads * r.vdim, lo = (int64_t)a.heads * a.vdim;
        if (up_stacked(&w.proj,
                       {{m + ".left.q", (int64_t)a.heads * a.dim}, {m + ".left.k", (int64_t)a.kv * a.dim}, {m + ".left.v", (int64_t)a.kv * a.vdim},
                        {m + ".right.q", rq}, {m + ".right.k", rq}, {m + ".right.v", rv}, {m + ".right.g", rv},
                        {m + ".right.i", r.heads}, {m + ".right.f", r.heads}},
                       D, c.proj_rows))
          return -1;
        {  // the two output projections side by side: row m = [left.o[m, :] | right.o[m, :]]
          const auto *ol = need(m + ".left.o", (int64_t)D * lo), *orr = need(m + ".right.o", (int64_t)D * rv);
          if (!ol || !orr) return -1;
          std::vector<uint16_t> st((size_t)D * (lo + rv));
          for (int64_t row = 0; row < D; ++row) {
            std::memcpy(&st[(size_t)(row * (lo + rv))], &(*ol)[(size_t)(row * lo)], (size_t)lo * 2);
            std::memcpy(&st[(size_t)(row * (lo + rv) + lo)], &(*orr)[(size_t)(row * rv)], (size_t)rv * 2);
          }
          if (upload(&w.o, st.data(), st.size())) return -1;
        }
        if (up(&w.q_norm, m + ".left.q.norm", a.dim) || up(&w.k_norm, m + ".left.k.norm", a.dim) ||
            up(&w.rnorm, m + ".right.norm", rv) || up(&w.i_bias, m + ".right.i.b", r.heads) || up(&w.f_bias, m + ".right.f.b", r.heads))
          return -1;
        const int half = a.rot_dims / 2;   // rotation frequencies base^(-2i/dims), rounded once to fp32
        std::vector<float> f((size_t)std::max(1, half));
        for (int k = 0; k < half; ++k) f[k] = (float)std::pow(a.base, -2.0 * k / (double)a.rot_dims);
        if (dalloc(&w.inv_freq, f.size())) return -1;
        FZ_HIP(hipMemcpy(w.inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice));
      }
      if (c.mlp.kind == 1) {
        if (up_glu(&w.gate_up, &w.down, p + ".mlp", c.mlp.glu)) return -1;
      } else if (c.mlp.kind == 2) {
        std::vector<uint16_t> gu, dn;
        const GluCfg& g = c.mlp.glu;
        for (int e = 0; e < c.mlp.experts; ++e) {
          const std::string pe = p + ".mlp.e" + std::to_string(e);
          const auto *ga = need(pe + ".gate", (int64_t)g.ff * D), *u = need(pe + ".up", (int64_t)g.ff * D),
                     *d = need(pe + ".down", (int64_t)D * g.ff);
          if (!ga || !u || !d) return -1;
          gu.insert(gu.end(), ga->begin(), ga->end());
          gu.insert(gu.end(), u->begin(), u->end());
          dn.insert(dn.end(), d->begin(), d->end());
        }
        if (upload(&w.gate_up_e, gu.data(), gu.size()) || upload(&w.down_e, dn.data(), dn.size()) ||
            up(&w.router, p + ".mlp.router", (int64_t)c.mlp.experts * D))
          return -1;
        if (c.mlp.has_shared && up_glu(&w.gate_up, &w.down, p + ".mlp.shared", c.mlp.shared)) return -1;
      }
    }
    staged.clear();
    finalized = true;
    return 0;
  }
  int load_checkpoint(const std::string& path) {
    pst::Checkpoint ck;
    std::string e;
    if (!ck.open(path, &e)) return set_error(e);
    for (auto& t : tensor_list()) {
      const pst::TensorView* v = ck.find(t.first);
      if (!v) return set_error("checkpoint has no tensor " + t.first);
      if (v->numel() != numel(t.second)) return set_error("checkpoint tensor " + t.first + " has another shape than config.json gives");
      std::vector<uint16_t>& dst = staged[t.first];
      dst.resize((size_t)v->numel());
      if (v->dtype == "BF16") {
        std::memcpy(dst.data(), v->data, dst.size() * 2);
      } else if (v->dtype == "F32") {
        const float* f = reinterpret_cast<const float*>(v->data);
        for (size_t i = 0; i < dst.size(); ++i) dst[i] = host_f2bf(f[i]);
      } else {
        return set_error("checkpoint tensor " + t.first + " has dtype " + v->dtype + " (bf16 expected)");
      }
    }
    return finalize();
  }

  // ------------------------------------------------------------------ requests
  int new_request() {
    for (size_t i = 0; i < requests.size(); ++i)
      if (!requests[i].live) {
        const size_t n = (size_t)state_layout.floats_per_slot();
        // the slot's state region starts from zero: empty convolution tails, empty memories, running maximum 0
        if (n) FZ_HIP(hipMemsetAsync(state + i * n, 0, n * sizeof(float), stream));
        requests[i].live = true;
        requests[i].seq_len = 0;
        return (int)i;
      }
    return set_error("no free request slot");
  }
  int drop_request(int id) {
    if (id < 0 || id >= (int)requests.size() || !requests[id].live) return set_error("drop_request: unknown request");
    requests[id].reset(&pool);
    requests[id].live = false;
    return 0;
  }

  // ------------------------------------------------------------------ step
  int ensure_rows(size_t T) {
    if (T <= cap_rows) return 0;
    FZ_HIP(hipStreamSynchronize(stream));
    drop_graphs();
    free_all(&step_owned);
    cap_rows = 0;
    size_t n = 64;
    while (n < T) n *= 2;
    auto* so = &step_owned;
    const size_t P = n * (size_t)std::max(1, mx_top);
    max_tiles = (int)((P + 63) / 64) + std::max(1, mx_experts);
    if (dalloc(&x, n * D, so) || dalloc(&xs, (layers.size() + 1) * n * D, so) || dalloc(&qkv32, n * std::max(1, mx_conv), so) ||
        dalloc(&q32, n * std::max(1, mx_q), so) || dalloc(&gates32, n * (size_t)std::max(1, 2 * mx_dheads), so) || dalloc(&o32, n * std::max(1, mx_o), so) || dalloc_a(&hb, n * D, so) ||
        dalloc_a(&xb, n * D, so) || dalloc_a(&proj, n * mx_proj, so) || dalloc_a(&mix, n * mx_mix, so) || dalloc_a(&y, n * D, so) ||
        dalloc_a(&gu, n * (size_t)std::max(1, 2 * mx_ff), so) || dalloc_a(&act, n * (size_t)std::max(1, mx_ff), so) ||
        dalloc_a(&ys, n * D, so) || dalloc_a(&q16, n * (size_t)std::max(1, mx_q), so) ||
        dalloc_a(&attn16, n * (size_t)std::max(1, mx_q), so))
      return -1;
    if (mx_top > 0 && (dalloc(&ypairs, P * D, so) || dalloc(&route_w, P, so) || dalloc(&route_logits, n * (size_t)std::max(1, mx_experts), so) || dalloc(&route_e, P, so) || dalloc(&pos_pair, P, so) ||
                       dalloc(&pos_row, P, so) || dalloc(&tiles, (size_t)3 * max_tiles + 1, so) || dalloc_a(&gu_e, n * mx_gu_e, so) ||
                       dalloc_a(&act_e, n * (size_t)(mx_gu_e / 2), so)))
      return -1;
    cap_rows = n;
    return 0;
  }
  int ensure_want(size_t n) {
    if (n <= cap_want) return 0;
    FZ_HIP(hipStreamSynchronize(stream));
    drop_graphs();
    free_all(&want_owned);
    cap_want = 0;
    size_t c = 16;
    while (c < n) c *= 2;
    auto* wo = &want_owned;
    if (dalloc(&xw, c * D, wo) || dalloc_a(&hw, c * D, wo) || dalloc_a(&logits, c * V, wo) || dalloc(&logits32, c * V, wo) ||
        dalloc(&logits16, c * V, wo) || dalloc(&tokens_d, c, wo) || dalloc(&top1_state, c * 16, wo))
      return -1;
    cap_want = c;
    return 0;
  }
  // Y[T, M] = X[T, K] W[M, K]^T in the model's storage type
  int linear(const void* W, const void* X, void* Y, int M, int T, int K) {
    if (dtype == PEGAINFER_DTYPE_BF16 && !plain_kernels) {
      gemm_cuda(static_cast<const Half*>(W), static_cast<const Half*>(X), static_cast<Half*>(Y), M, T, K, S());
      return 0;
    }
    pegainfer_gemm_desc d{};
    d.x = X; d.w = W; d.y = Y;
    d.x_dtype = d.w_dtype = d.y_dtype = dtype;
    d.m = M; d.k = K; d.rows = T; d.groups = 1;
    d.x_row_stride = K; d.w_m_stride = K; d.w_k_stride = 1; d.y_row_stride = M;
    d.plain = plain_kernels;
    FZ_K(pegainfer_gemm_strided(&d, S()));
    return 0;
  }
  // out = Wdown clamp_glu([Wgate ; Wup] in)
  int glu(const void* gate_up, const void* down, const GluCfg& g, const void* in, void* out, int T) {
    if (linear(gate_up, in, gu, 2 * g.ff, T, D)) return -1;
    FZ_K(pegainfer_clamp_glu_rows(gu, act, g.ff, T, g.limit, kGluAlpha, dtype, S()));
    return linear(down, act, out, D, T, g.ff);
  }

  int step(int n, const int32_t* ids, const int32_t* lens, const uint32_t* tokens, int n_want, const int32_t* want_rows,
           float* out_logits, int32_t* out_tokens) {
    if (!finalized) return set_error("step before finalize");
    if (n <= 0 || n > max_requests) return set_error("step: batch size outside 1 .. max_requests");
    // ---- validate everything before anything changes
    size_t T = 0;
    int need_pages = 0;
    for (int i = 0; i < n; ++i) {
      if (ids[i] < 0 || ids[i] >= (int)requests.size() || !requests[ids[i]].live) return set_error("step: unknown request");
      for (int k = 0; k < i; ++k)
        if (ids[k] == ids[i]) return set_error("step: a request is listed twice");
      if (lens[i] <= 0) return set_error("step: an entry without tokens");
      const KvState& st = requests[ids[i]];
      need_pages += st.pages_short(st.seq_len + lens[i], kPageSize);
      T += (size_t)lens[i];
    }
    if (need_pages > pool.available()) return set_error("step: not enough free cache pages");
    for (size_t t = 0; t < T; ++t)
      if (tokens[t] >= (uint32_t)V) return set_error("step: token outside the vocabulary");
    std::vector<int32_t> want;
    if (n_want < 0) {
      size_t off = 0;
      for (int i = 0; i < n; ++i) { off += (size_t)lens[i]; want.push_back((int32_t)off - 1); }
    } else {
      for (int i = 0; i < n_want; ++i) {
        if (want_rows[i] < 0 || (size_t)want_rows[i] >= T) return set_error("step: wanted row outside the step");
        want.push_back(want_rows[i]);
      }
    }
    const int W = (int)want.size();
    if (ensure_rows(T) || ensure_want((size_t)std::max(1, W))) return -1;
    size_t total_pages = 0;
    for (int i = 0; i < n; ++i) {
      KvState& st = requests[ids[i]];
      if (!st.ensure_capacity(&pool, st.seq_len + lens[i], kPageSize)) return set_error("step: page pool ran dry");
      total_pages += st.pages.size();
    }
    // ---- the packed metadata block:
    //   tokens | positions | row_entry | entry_row0 | entry_slot | page_indptr | want | page_ids | attention tile sets
    // An attention tile is a run of token rows of one entry times a run of the query heads of one key/value head, at most
    // 16 rows in all; one set of tiles per distinct heads-per-kv-head value of the model's attention layers.
    bool single = true;   // every entry brings one token: decoding
    for (int i = 0; i < n && single; ++i) single = lens[i] == 1;
    const size_t o_tok = 0, o_pos = o_tok + T, o_ent = o_pos + T, o_row0 = o_ent + T, o_slot = o_row0 + (size_t)n + 1,
                 o_ind = o_slot + (size_t)n, o_lpl = o_ind + (size_t)n + 1, o_kvlen = o_lpl + (size_t)n, o_rows = o_kvlen + (size_t)n,
                 o_want = o_rows + 1;
    size_t words = o_want + (size_t)std::max(1, W);   // the page lists come last: everything before them sits at offsets that
                                                      // depend on the step's shape only, which a captured graph relies on
    // plain sets: [row0 | ntok | qh0 | nqh] per tile.  matrix-core sets: [request | tile of the request | 0] per tile of
    // `cta` packed (token, query head) rows, the plan batch_prefill_paged_cuda reads
    // matrix-core sets of a decoding step: the partition plan of the framework's decode attention instead (kv_pool.h
    // make_split_plan: every request's keys cut into chunks that run as workgroups of their own, merged afterwards),
    //   [request per slot | chunk per slot | chunk size | output indptr | zeros (n) | valid bytes per slot]
    std::vector<size_t> tile_off(tile_sets.size()), tile_cnt(tile_sets.size());
    std::vector<int> tile_cta(tile_sets.size(), 0);
    std::vector<pq::SplitPlan> dplan(tile_sets.size());
    int split_mask = 0;
    for (size_t k = 0; k < tile_sets.size(); ++k) {
      const TileSet& ts = tile_sets[k];
      const int per = ts.per;
      size_t cnt = 0;
      if (ts.fast_hd && !plain_kernels && single) {
        std::vector<int> kv_lens(n);
        for (int i = 0; i < n; ++i) kv_lens[i] = requests[ids[i]].seq_len + 1;
        dplan[k] = pq::make_split_plan(1, kv_lens, n, ts.kv, false);
        if (dplan[k].use_split) split_mask |= 1 << (k & 30);
        tile_cta[k] = -1;
        tile_off[k] = words;
        tile_cnt[k] = (size_t)dplan[k].slots;
        words += 2 * tile_cnt[k] + 1 + (size_t)n + 1 + (size_t)n + (tile_cnt[k] + 3) / 4;
        continue;
      }
      if (ts.fast_hd && !plain_kernels) {
        tile_cta[k] = batch_prefill_cta_tile_q((int)T, ts.heads, ts.kv, ts.fast_hd);
        for (int i = 0; i < n; ++i) cnt += ((size_t)lens[i] * per + tile_cta[k] - 1) / tile_cta[k];
      } else {
        for (int i = 0; i < n; ++i)
          cnt += per <= kAttRows ? ((size_t)lens[i] + (kAttRows / per) - 1) / (kAttRows / per) : (size_t)lens[i] * ((per + kAttRows - 1) / kAttRows);
      }
      tile_off[k] = words;
      tile_cnt[k] = cnt;
      words += 4 * cnt;
    }
    const size_t o_pages = words;
    words += total_pages;
    if (words > cap_meta) {
      FZ_HIP(hipStreamSynchronize(stream));
      if (meta_host) (void)hipHostFree(meta_host);
      if (meta_dev) (void)hipFree(meta_dev);
      meta_host = meta_dev = nullptr;
      cap_meta = 0;
      size_t c = 4096;
      while (c < words) c *= 2;
      FZ_HIP(hipHostMalloc(reinterpret_cast<void**>(&meta_host), c * 4, hipHostMallocDefault));
      FZ_HIP(hipMalloc(reinterpret_cast<void**>(&meta_dev), c * 4));
      cap_meta = c;
      drop_graphs();
    }
    int32_t* mh = reinterpret_cast<int32_t*>(meta_host);
    {
      size_t t = 0, pg = 0;
      for (int i = 0; i < n; ++i) {
        const KvState& st = requests[ids[i]];
        mh[o_row0 + i] = (int32_t)t;
        mh[o_slot + i] = ids[i];
        mh[o_ind + i] = (int32_t)pg;
        const int kv_len = st.seq_len + lens[i];
        mh[o_kvlen + i] = kv_len;
        mh[o_lpl + i] = kv_len % kPageSize == 0 ? kPageSize : kv_len % kPageSize;
        for (int32_t p : st.pages) mh[o_pages + pg++] = p;
        for (int k = 0; k < lens[i]; ++k, ++t) {
          mh[o_tok + t] = (int32_t)tokens[t];
          mh[o_pos + t] = st.seq_len + k;
          mh[o_ent + t] = i;
        }
      }
      mh[o_row0 + n] = (int32_t)t;
      mh[o_ind + n] = (int32_t)pg;
      mh[o_rows] = (int32_t)T;
      for (int i = 0; i < W; ++i) mh[o_want + i] = want[i];
      for (size_t k = 0; k < tile_sets.size(); ++k) {
        const int per = tile_sets[k].per;
        int32_t *t_row0 = mh + tile_off[k], *t_ntok = t_row0 + tile_cnt[k], *t_qh0 = t_ntok + tile_cnt[k], *t_nqh = t_qh0 + tile_cnt[k];
        size_t at_ = 0, r0 = 0;
        if (tile_cta[k] < 0) {
          const pq::SplitPlan& pl = dplan[k];
          const size_t sl = tile_cnt[k];
          int32_t* b = mh + tile_off[k];
          std::memcpy(b, pl.request_indices.data(), sl * 4);
          std::memcpy(b + sl, pl.kv_tile_indices.data(), sl * 4);
          b[2 * sl] = pl.chunk;
          std::memcpy(b + 2 * sl + 1, pl.o_indptr.data(), (size_t)(n + 1) * 4);
          std::memset(b + 2 * sl + 1 + n + 1, 0, (size_t)n * 4);
          std::memcpy(b + 2 * sl + 1 + n + 1 + n, pl.valid.data(), sl);
          continue;
        }
        if (tile_cta[k]) {
          for (int i = 0; i < n; ++i) {
            const int tiles_i = (lens[i] * per + tile_cta[k] - 1) / tile_cta[k];
            for (int t = 0; t < tiles_i; ++t, ++at_) { t_row0[at_] = i; t_ntok[at_] = t; t_qh0[at_] = 0; }
          }
          continue;
        }
        for (int i = 0; i < n; ++i) {
          if (per <= kAttRows) {
            const int tpt = kAttRows / per;
            for (int t0 = 0; t0 < lens[i]; t0 += tpt, ++at_) {
              t_row0[at_] = (int32_t)r0 + t0; t_ntok[at_] = std::min(tpt, lens[i] - t0); t_qh0[at_] = 0; t_nqh[at_] = per;
            }
          } else {
            for (int t0 = 0; t0 < lens[i]; ++t0)
              for (int q0 = 0; q0 < per; q0 += kAttRows, ++at_) {
                t_row0[at_] = (int32_t)r0 + t0; t_ntok[at_] = 1; t_qh0[at_] = q0; t_nqh[at_] = std::min(kAttRows, per - q0);
              }
          }
          r0 += (size_t)lens[i];
        }
      }
    }
    FZ_HIP(hipEventRecord(ev0, stream));
    FZ_HIP(hipMemcpyAsync(meta_dev, meta_host, words * 4, hipMemcpyHostToDevice, stream));
    const int32_t* md = reinterpret_cast<const int32_t*>(meta_dev);
    const uint32_t* d_tok = reinterpret_cast<const uint32_t*>(md + o_tok);
    const int32_t *d_pos = md + o_pos, *d_ent = md + o_ent, *d_row0 = md + o_row0, *d_slot = md + o_slot, *d_ind = md + o_ind,
                  *d_want = md + o_want, *d_pages = md + o_pages, *d_lpl = md + o_lpl, *d_kvlen = md + o_kvlen;
    const int Ti = (int)T;
    const int64_t slot_stride = state_layout.floats_per_slot(), xs_stride = (int64_t)cap_rows * D;
    if (tap_on) {
      const size_t needf = layers.size() * T * D;
      if (needf > tap_cap) {
        FZ_HIP(hipStreamSynchronize(stream));
        if (tap) (void)hipFree(tap);
        tap = nullptr;
        tap_cap = 0;
        FZ_HIP(hipMalloc(reinterpret_cast<void**>(&tap), needf * 4));
        tap_cap = needf;
      }
      tap_rows = Ti;
    }
    // ---- the layers (everything below reads the step's shape from its arguments and the step's contents from the metadata
    //      block, so a launch sequence recorded for one decode step serves every later step of the same shape)
    auto run_layers = [&]() -> int {
    FZ_K(pegainfer_embed_f32(embed, d_tok, xs, D, Ti, dtype, S()));
    FZ_K(pegainfer_embed_f32(embed, d_tok, x, D, Ti, dtype, S()));
    for (size_t li = 0; li < layers.size(); ++li) {
      const LayerCfg& c = layers[li];
      const LayerW& w = weights[li];
      const int Mp = c.proj_rows;
      // input convolution: hb = x + conv(x), then the tail moves on
      if (single) {
        FZ_K(pegainfer_time_conv_step(x, PEGAINFER_DTYPE_F32, D, w.canon, dtype, state + c.st_canon, slot_stride, hb, dtype, D, D,
                                      canon_taps, 1, d_slot, n, S()));
      } else {
        FZ_K(pegainfer_time_conv(x, PEGAINFER_DTYPE_F32, D, w.canon, dtype, state + c.st_canon, slot_stride, hb, dtype, D, D,
                                 canon_taps, 1, d_ent, d_row0, d_slot, Ti, S()));
        FZ_K(pegainfer_time_conv_commit(x, PEGAINFER_DTYPE_F32, D, state + c.st_canon, slot_stride, D, canon_taps, d_row0, d_slot, n, S()));
      }
      if (linear(w.proj, hb, proj, Mp, Ti, D)) return -1;
      if (c.type == kDelta) {
        const DeltaCfg& d = c.dl;
        if (single) {
          FZ_K(pegainfer_time_conv_step(proj, dtype, Mp, w.conv, dtype, state + c.st_conv, slot_stride, qkv32, PEGAINFER_DTYPE_F32,
                                        c.conv_ch, c.conv_ch, d.taps, 2, d_slot, n, S()));
        } else {
          FZ_K(pegainfer_time_conv(proj, dtype, Mp, w.conv, dtype, state + c.st_conv, slot_stride, qkv32, PEGAINFER_DTYPE_F32,
                                   c.conv_ch, c.conv_ch, d.taps, 2, d_ent, d_row0, d_slot, Ti, S()));
          FZ_K(pegainfer_time_conv_commit(proj, dtype, Mp, state + c.st_conv, slot_stride, c.conv_ch, d.taps, d_row0, d_slot, n, S()));
        }
        FZ_K(pegainfer_delta_rule(qkv32, c.conv_ch, proj, Mp, c.o_b, c.o_a, w.A_log, w.dt_bias, gates32, state + c.st_mem, slot_stride,
                                  o32, d.heads, d.kv, d.dim, d.vdim, Ti, d_row0, d_slot, n, dtype, S()));
        FZ_K(pegainfer_head_rms_gate(o32, w.onorm, 0, at(proj, (size_t)c.o_g), Mp, 0, 1.0f, eps, mix, c.mix_cols, d.heads, d.vdim,
                                     Ti, dtype, S()));
      } else {
        const AttnCfg& a = c.at;
        const MemCfg& r = c.mm;
        const size_t ts = (size_t)c.tile_set;
        const int32_t* tb = md + tile_off[ts];
        const bool fast = tile_cta[ts] != 0, fast_decode = tile_cta[ts] < 0;
        FZ_K(pegainfer_qk_norm_rope_paged(proj, Mp, c.o_q, c.o_k, c.o_v, a.heads, a.kv, a.dim, a.vdim, w.q_norm, w.k_norm, eps,
                                          w.inv_freq, a.rot_dims, d_pos, d_ent, d_ind, d_pages, cache, page_stride, c.k_off, c.v_off,
                                          kPageSize, q32, fast ? q16 : nullptr, Ti, dtype, S()));
        if (fast_decode) {
          // decoding: one query row per request; long contexts are cut into chunks that run side by side (partials in bf16)
          const size_t sl = tile_cnt[ts];
          const int32_t *sri = tb, *skt = tb + sl, *skc = tb + 2 * sl, *soi = skc + 1, *zeros = soi + n + 1;
          const uint8_t* sva = reinterpret_cast<const uint8_t*>(zeros + n);
          const Half *q = static_cast<const Half*>(q16), *kv = static_cast<const Half*>(cache);
          Half* out = static_cast<Half*>(attn16);
          int rc;
          if (dplan[ts].use_split)
            rc = a.dim == 256 ? pegainfer_paged_attention_decode_split_kv_hd256(q, out, kv, c.k_off, c.v_off, d_pages, d_ind, d_lpl, sri, skt, skc, soi, sva,
                                                                                split_tmp_v, split_tmp_s, a.heads, a.kv, a.dim, kPageSize, n, (int)sl,
                                                                                page_stride, a.scale, nullptr, S())
                              : paged_attention_decode_split_kv_cuda(q, out, kv, c.k_off, c.v_off, d_pages, d_ind, d_lpl, sri, skt, skc, soi, sva, split_tmp_v,
                                                                     split_tmp_s, a.heads, a.kv, a.dim, kPageSize, n, (int)sl, page_stride, a.scale, S());
          else
            rc = a.dim == 256 ? paged_attention_decode_cuda_hd256(q, out, kv, c.k_off, c.v_off, d_pages, d_ind, d_lpl, d_ent, zeros, d_kvlen, a.heads, a.kv,
                                                                  a.dim, kPageSize, n, page_stride, a.scale, S())
                              : paged_attention_decode_cuda(q, out, kv, c.k_off, c.v_off, d_pages, d_ind, d_lpl, d_ent, zeros, d_kvlen, a.heads, a.kv, a.dim,
                                                            kPageSize, n, page_stride, a.scale, S());
          if (rc) return set_error("matrix-core decode attention failed");
          FZ_K(pegainfer_scale_rows(attn16, (int64_t)a.heads * a.vdim, mix, c.mix_cols, a.heads * a.vdim, Ti, c.left_scale, dtype, S()));
        } else if (fast) {
          // every entry is a request whose last rows are this step's: the kernel takes a row's position from the request's
          // key count; scores and softmax state in fp32, weights rounded to bf16 where they enter the matrix cores
          auto attn = a.dim == 256 ? batch_prefill_paged_cuda_hd256 : batch_prefill_paged_cuda;
          if (attn(static_cast<const Half*>(q16), static_cast<Half*>(attn16), static_cast<const Half*>(cache), c.k_off, c.v_off, d_pages,
                   d_ind, d_lpl, d_row0, tb, tb + tile_cnt[ts], tb + 2 * tile_cnt[ts], d_kvlen,
                   reinterpret_cast<const uint32_t*>(md + o_rows), a.heads, a.kv, a.dim, kPageSize, Ti, n, (int)tile_cnt[ts],
                   page_stride, a.scale, S()))
            return set_error("matrix-core prefill attention failed");
          FZ_K(pegainfer_scale_rows(attn16, (int64_t)a.heads * a.vdim, mix, c.mix_cols, a.heads * a.vdim, Ti, c.left_scale, dtype, S()));
        } else {
          FZ_K(pegainfer_paged_attention(q32, cache, page_stride, c.k_off, c.v_off, kPageSize, d_pos, d_ent, d_ind, d_pages, a.heads,
                                         a.kv, a.dim, a.vdim, a.scale, c.left_scale, tb, tb + tile_cnt[ts], tb + 2 * tile_cnt[ts],
                                         tb + 3 * tile_cnt[ts], (int)tile_cnt[ts], mix, c.mix_cols, dtype, S()));
        }
        FZ_K(pegainfer_gated_matrix_memory(proj, Mp, c.o_rq, c.o_rk, c.o_rv, c.o_ri, c.o_rf, w.i_bias, w.f_bias, r.cap,
                                           state + c.st_mem, slot_stride, o32, r.heads, r.dim, r.vdim, d_row0, d_slot, n, dtype, S()));
        FZ_K(pegainfer_head_rms_gate(o32, w.rnorm, 1, at(proj, (size_t)c.o_rg), Mp, 1, c.right_scale, eps,
                                     at(mix, (size_t)a.heads * a.vdim), c.mix_cols, r.heads, r.vdim, Ti, dtype, S()));
      }
      if (linear(w.o, mix, y, D, Ti, c.mix_cols)) return -1;
      float* x_next = xs + (li + 1) * xs_stride;
      const int n_mix = (int)li + 2;
      if (c.mlp.kind) {
        FZ_K(pegainfer_group_rms_add(x, y, dtype, w.norm1, groups, eps, x, xb, D, Ti, dtype, nullptr, 0, nullptr, 0, nullptr, nullptr, S()));
        if (c.mlp.kind == 1) {
          if (glu(w.gate_up, w.down, c.mlp.glu, xb, y, Ti)) return -1;
        } else if (routed_ff(c, w, Ti)) {
          return -1;
        }
        FZ_K(pegainfer_group_rms_add(x, y, dtype, w.norm2, groups, eps, x_next, nullptr, D, Ti, dtype, xs, xs_stride, w.dwa, n_mix, x,
                                     nullptr, S()));
      } else {
        FZ_K(pegainfer_group_rms_add(x, y, dtype, w.norm1, groups, eps, x_next, nullptr, D, Ti, dtype, xs, xs_stride, w.dwa, n_mix, x,
                                     nullptr, S()));
      }
      if (tap_on) FZ_HIP(hipMemcpyAsync(tap + li * T * D, x, T * D * 4, hipMemcpyDeviceToDevice, stream));
    }
    // ---- wanted rows: final norm + logits over the embedding table
    if (W > 0) {
      FZ_K(pegainfer_gather_rows_f32(x, d_want, xw, D, W, S()));
      FZ_K(pegainfer_group_rms_add(nullptr, xw, PEGAINFER_DTYPE_F32, final_norm, groups, eps, nullptr, hw, D, W, dtype, nullptr, 0,
                                   nullptr, 0, nullptr, nullptr, S()));
      if (linear(embed, hw, logits, V, W, D)) return -1;
      if (dtype == PEGAINFER_DTYPE_BF16) {
        FZ_K(deepseek_bf16_to_f32_cuda(static_cast<const Half*>(logits), logits32, W * V, S()));
        FZ_HIP(hipMemcpyAsync(logits16, logits, (size_t)W * V * 2, hipMemcpyDeviceToDevice, stream));
      } else {
        FZ_HIP(hipMemcpyAsync(logits32, logits, (size_t)W * V * 4, hipMemcpyDeviceToDevice, stream));
        FZ_K(deepseek_f32_to_bf16_cuda(logits32, logits16, W * V, S()));
      }
      if (out_tokens) FZ_K(pegainfer_batched_top1(logits16, V, W, V, top1_state, tokens_d, S()));
    }
    return 0;
    };
    // a step of single tokens only (decoding) is launch-bound: its launches are captured once per shape as a hipGraph and
    // replayed; steps with prompt portions run eagerly
    if (single && graphs_on && !tap_on) {
      const GraphKey key{n, W, out_tokens != nullptr, plain_kernels, split_mask};
      hipGraphExec_t exec = nullptr;
      for (auto& g : graphs)
        if (g.first == key) exec = g.second;
      if (!exec) {
        hipGraph_t g = nullptr;
        FZ_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        const int rc = run_layers();
        const hipError_t e = hipStreamEndCapture(stream, &g);
        if (rc) return -1;
        if (e != hipSuccess) return set_error("graph capture failed");
        FZ_HIP(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
        FZ_HIP(hipGraphDestroy(g));
        graphs.emplace_back(key, exec);
      }
      FZ_HIP(hipGraphLaunch(exec, stream));
    } else if (run_layers()) {
      return -1;
    }
    last_rows = W;
    FZ_HIP(hipEventRecord(ev1, stream));
    if (W > 0 && out_logits) FZ_HIP(hipMemcpyAsync(out_logits, logits32, (size_t)W * V * 4, hipMemcpyDeviceToHost, stream));
    if (W > 0 && out_tokens) FZ_HIP(hipMemcpyAsync(out_tokens, tokens_d, (size_t)W * 4, hipMemcpyDeviceToHost, stream));
    FZ_HIP(hipStreamSynchronize(stream));
    (void)hipEventElapsedTime(&last_step_ms, ev0, ev1);
    for (int i = 0; i < n; ++i) requests[ids[i]].seq_len += lens[i];
    return 0;
  }

  int routed_ff(const LayerCfg& c, const LayerW& w, int T) {
    const MlpCfg& f = c.mlp;
    const int ff = f.glu.ff, P = T * f.top;
    int32_t *t_group = tiles, *t_row0 = tiles + max_tiles, *t_rows = tiles + 2 * max_tiles, *n_tiles = tiles + 3 * max_tiles;
    if (T > 8 || f.experts > 1024) {   // many rows (or more experts than the selection kernel's four rows hold in LDS): one
                                       // workgroup per row does logits and selection
      FZ_K(pegainfer_route_topk(xb, w.router, nullptr, route_e, route_w, D, f.experts, 1, 1, f.top, T, PEGAINFER_SCORE_SOFTMAX, dtype, S()));
    } else {       // few rows (decoding): the few-rows GEMM streams the router with the whole chip into fp32 logits, then the selection
      pegainfer_gemm_desc r{};
      r.x = xb; r.w = w.router; r.y = route_logits;
      r.x_dtype = r.w_dtype = dtype; r.y_dtype = PEGAINFER_DTYPE_F32;
      r.m = f.experts; r.k = D; r.rows = T; r.groups = 1;
      r.x_row_stride = D; r.w_m_stride = D; r.w_k_stride = 1; r.y_row_stride = f.experts;
      r.plain = plain_kernels;
      FZ_K(pegainfer_gemm_strided(&r, S()));
      FZ_K(pegainfer_route_from_logits(route_logits, nullptr, route_e, route_w, f.experts, 1, 1, f.top, T, PEGAINFER_SCORE_SOFTMAX, dtype, S()));
    }
    const int per_tile = dtype == PEGAINFER_DTYPE_BF16 && !plain_kernels && T > 8 && D % 8 == 0 && ff % 8 == 0 ? 128 : 64;
    FZ_K(pegainfer_route_sort(route_e, P, f.top, f.experts, pos_pair, pos_row, t_group, t_row0, t_rows, n_tiles, max_tiles, per_tile, S()));
    pegainfer_gemm_desc d{};
    d.x = xb; d.w = w.gate_up_e; d.y = gu_e;
    d.x_dtype = d.w_dtype = d.y_dtype = dtype;
    d.m = 2 * ff; d.k = D;
    d.x_row_stride = D; d.w_m_stride = D; d.w_k_stride = 1; d.w_group_stride = (int64_t)2 * ff * D;
    d.y_row_stride = 2 * ff;
    d.tile_group = t_group; d.tile_row0 = t_row0; d.tile_rows = t_rows; d.n_tiles = n_tiles; d.max_tiles = (P + per_tile - 1) / per_tile + f.experts;
    d.tile_rows_cap = per_tile;
    d.x_row_index = pos_row;
    d.max_tile_rows = std::min(T, 64);   // a row chooses distinct experts: an expert never gets more pairs than there are rows
    d.plain = plain_kernels;
    FZ_K(pegainfer_gemm_strided(&d, S()));
    FZ_K(pegainfer_clamp_glu_rows(gu_e, act_e, ff, P, f.glu.limit, kGluAlpha, dtype, S()));
    pegainfer_gemm_desc e{};
    e.x = act_e; e.w = w.down_e; e.y = ypairs;
    e.x_dtype = e.w_dtype = dtype; e.y_dtype = PEGAINFER_DTYPE_F32;
    e.m = D; e.k = ff;
    e.x_row_stride = ff; e.w_m_stride = ff; e.w_k_stride = 1; e.w_group_stride = (int64_t)D * ff;
    e.y_row_stride = D;
    e.tile_group = t_group; e.tile_row0 = t_row0; e.tile_rows = t_rows; e.n_tiles = n_tiles; e.max_tiles = d.max_tiles;
    e.y_row_index = pos_pair;
    e.max_tile_rows = d.max_tile_rows;
    e.tile_rows_cap = per_tile;
    e.plain = plain_kernels;
    FZ_K(pegainfer_gemm_strided(&e, S()));
    if (f.has_shared && glu(w.gate_up, w.down, f.shared, xb, ys, T)) return -1;
    FZ_K(pegainfer_route_combine_add(ypairs, route_w, f.has_shared ? ys : nullptr, y, D, f.top, T, dtype, S()));
    return 0;
  }

  // ------------------------------------------------------------------ sampling over the last step's wanted rows
  int sample(int row, float temperature, int top_k, float top_p, float random_val, int32_t* out) {
    if (row < 0 || row >= last_rows) return set_error("no logits for that row");
    const Half* lg = logits16 + (size_t)row * V;
    if ((temperature <= 0.0f || top_k == 1) && top_p >= 1.0f) {
      flashinfer_top1_cuda(lg, top1_value, row_states, sample_out_d, V, S());
    } else {
      uint32_t bits;
      std::memcpy(&bits, &random_val, 4);
      gpu_sample_flashinfer_cuda(lg, probs_scratch, valid_scratch, sample_out_d, V, 1.0f / temperature, top_k, top_p, (uint64_t)bits, S());
    }
    FZ_HIP(hipStreamSynchronize(stream));
    FZ_HIP(hipMemcpy(out, sample_out_d, 4, hipMemcpyDeviceToHost));
    return 0;
  }
  int logprobs(int row, uint32_t token, int top_k, float* out_lp, uint32_t* top_ids, float* top_lps) {
    if (row < 0 || row >= last_rows) return set_error("no logits for that row");
    if (token >= (uint32_t)V) return set_error("logprobs: token outside the vocabulary");
    lp_row.resize((size_t)V);
    FZ_HIP(hipStreamSynchronize(stream));
    FZ_HIP(hipMemcpy(lp_row.data(), logits32 + (size_t)row * V, (size_t)V * 4, hipMemcpyDeviceToHost));
    return pegainfer_logprobs_from_logits(lp_row.data(), V, token, top_k, out_lp, top_ids, top_lps);
  }
  int debug_hidden(int run, float* out, int max_rows) {
    if (!tap || run < 0 || run >= (int)layers.size()) return set_error("debug_hidden: no tap for that layer");
    const int rows = std::min(max_rows, tap_rows);
    FZ_HIP(hipStreamSynchronize(stream));
    FZ_HIP(hipMemcpy(out, tap + (size_t)run * tap_rows * D, (size_t)rows * D * 4, hipMemcpyDeviceToHost));
    return rows;
  }

  ~Model() {
    if (stream) (void)hipStreamSynchronize(stream);
    drop_graphs();
    free_all(&owned);
    free_all(&step_owned);
    free_all(&want_owned);
    if (tap) (void)hipFree(tap);
    if (meta_dev) (void)hipFree(meta_dev);
    if (meta_host) (void)hipHostFree(meta_host);
    if (ev0) (void)hipEventDestroy(ev0);
    if (ev1) (void)hipEventDestroy(ev1);
    if (stream) (void)hipStreamDestroy(stream);
    cublas_destroy();
  }
};

static thread_local std::string g_create_error;
static Model* M(pegainfer_feruzen_t m) { return static_cast<Model*>(m); }

static Model* create(const std::string& config, int device, int dtype, int max_tokens, int max_requests) {
  if (dtype != PEGAINFER_DTYPE_BF16 && dtype != PEGAINFER_DTYPE_F32) { g_create_error = "dtype must be 0 (bf16) or 1 (f32)"; return nullptr; }
  if (max_tokens <= 0 || max_requests <= 0) { g_create_error = "max_tokens and max_requests must be positive"; return nullptr; }
  Model* m = new Model();
  m->device = device;
  m->dtype = dtype;
  m->max_requests = max_requests;
  if (m->parse_config(config) || m->init(max_tokens)) {
    g_create_error = m->err;
    delete m;
    return nullptr;
  }
  return m;
}

}  // namespace pfz

extern "C" {
using pfz::M;

pegainfer_feruzen_t pegainfer_feruzen_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests) {
  if (!config_json) { pfz::g_create_error = "no configuration"; return nullptr; }
  return pfz::create(config_json, device_ordinal, dtype, max_tokens, max_requests);
}
pegainfer_feruzen_t pegainfer_feruzen_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests) {
  std::string e;
  auto f = pst::MappedFile::open(std::string(model_dir) + "/config.json", &e);
  if (!f) { pfz::g_create_error = e; return nullptr; }
  pfz::Model* m = pfz::create(std::string(reinterpret_cast<const char*>(f->data), f->size), device_ordinal, dtype, max_tokens, max_requests);
  if (!m) return nullptr;
  if (m->load_checkpoint(model_dir)) {
    pfz::g_create_error = m->err;
    delete m;
    return nullptr;
  }
  return m;
}
void pegainfer_feruzen_destroy(pegainfer_feruzen_t m) { delete M(m); }
const char* pegainfer_feruzen_last_error(pegainfer_feruzen_t m) { return m ? M(m)->err.c_str() : pfz::g_create_error.c_str(); }
int32_t pegainfer_feruzen_load_tensor(pegainfer_feruzen_t m, const char* name, const void* host_bf16, int64_t numel) {
  return M(m)->load_tensor(name, static_cast<const uint16_t*>(host_bf16), numel);
}
int32_t pegainfer_feruzen_fill_synthetic(pegainfer_feruzen_t m, uint64_t seed, float std) { return M(m)->fill_synthetic(seed, std); }
int32_t pegainfer_feruzen_finalize(pegainfer_feruzen_t m) { return M(m)->finalize(); }
int32_t pegainfer_feruzen_new_request(pegainfer_feruzen_t m) { return M(m)->new_request(); }
int32_t pegainfer_feruzen_drop_request(pegainfer_feruzen_t m, int32_t id) { return M(m)->drop_request(id); }
int32_t pegainfer_feruzen_request_seq_len(pegainfer_feruzen_t m, int32_t id) {
  if (id < 0 || id >= (int)M(m)->requests.size() || !M(m)->requests[id].live) return -1;
  return M(m)->requests[id].seq_len;
}
int32_t pegainfer_feruzen_available_pages(pegainfer_feruzen_t m) { return M(m)->pool.available(); }
int32_t pegainfer_feruzen_capacity_pages(pegainfer_feruzen_t m) { return M(m)->pool.capacity(); }
int32_t pegainfer_feruzen_page_size(pegainfer_feruzen_t) { return pfz::kPageSize; }
int32_t pegainfer_feruzen_max_batch_size(pegainfer_feruzen_t m) { return M(m)->max_requests; }
int32_t pegainfer_feruzen_vocab_size(pegainfer_feruzen_t m) { return M(m)->V; }
int32_t pegainfer_feruzen_width(pegainfer_feruzen_t m) { return M(m)->D; }
int32_t pegainfer_feruzen_num_layer_runs(pegainfer_feruzen_t m) { return (int32_t)M(m)->layers.size(); }
int32_t pegainfer_feruzen_dtype(pegainfer_feruzen_t m) { return M(m)->dtype; }
int64_t pegainfer_feruzen_state_floats(pegainfer_feruzen_t m) { return M(m)->state_layout.floats_per_slot(); }
int32_t pegainfer_feruzen_step(pegainfer_feruzen_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens) {
  return M(m)->step(n_entries, request_ids, lens, tokens_concat, n_want, want_rows, out_logits_host, out_tokens);
}
int32_t pegainfer_feruzen_sample(pegainfer_feruzen_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token) {
  return M(m)->sample(row, temperature, top_k, top_p, random_val, out_token);
}
int32_t pegainfer_feruzen_logprobs(pegainfer_feruzen_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs) {
  return M(m)->logprobs(row, token, top_k, out_logprob, out_top_ids, out_top_logprobs);
}
int32_t pegainfer_feruzen_debug_hidden_enable(pegainfer_feruzen_t m, int32_t enable) { M(m)->tap_on = enable != 0; return 0; }
int32_t pegainfer_feruzen_debug_hidden(pegainfer_feruzen_t m, int32_t layer_run, float* out_host, int32_t max_rows) {
  return M(m)->debug_hidden(layer_run, out_host, max_rows);
}
float pegainfer_feruzen_last_step_ms(pegainfer_feruzen_t m) { return M(m)->last_step_ms; }
int64_t pegainfer_feruzen_weight_bytes(pegainfer_feruzen_t m) { return M(m)->weight_bytes; }
int32_t pegainfer_feruzen_set_plain_kernels(pegainfer_feruzen_t m, int32_t on) { M(m)->plain_kernels = on != 0; return 0; }

}  // extern "C"

// C++ host runtime of the Duguzen decoder on MI355X (include/pegainfer_duguzen.h).  Same shape as the Qwen3 / Qwen3.5
// runtimes next to it: one model = one device + one in-order HIP stream, requests are KvState slots over the shared
// PagePool (kv_pool.h), a step's metadata is ONE pinned block and ONE hipMemcpyAsync, every op goes through the kernel
// library's C ABI (pegainfer_kernels.h for the tuned bf16 GEMM routes and the samplers, pegainfer_kernels_blocks.h for the
// fp32-stream norms, the latent attention, the strided GEMM and the router).
//
// What a step does per layer run (T = all token rows of the step, prompts' portions and single tokens alike):
//   h      = dyt_1(x)                                   (fused into the previous sublayer's closing launch)
//   proj   = [Wq ; Wdkv ; Wg] h                         one GEMM over the stacked matrix
//   prep   : latent RMS norm + rotation -> cache entry; rotated query parts -> qc
//   absorb : qc[t, h, :rank] = Wuk_h^T q_nope[t, h]     batched per-head GEMM
//   attn   : softmax over the request's cache entries   (fp32 scores / weights)
//   value  : out[t, h] = sigmoid(g[t, h]) * Wuv_h o_lat[t, h]      batched per-head GEMM + gate epilogue
//   y      = Wo out;   x += dyt_1b(y);  h = dyt_2(x)    one launch for post-norm + residual + next pre-norm
//   dense  : y = Wdown relu(Wup h)^2      routed: route -> sort by expert -> grouped gate|up GEMM -> SwiGLU -> grouped
//            down GEMM -> weighted sum;   x += dyt_2b(y);  h = dyt_1(x) of the next layer run
// The cache is page-first [page][layer run][slot][rank + rot]; a layer run that borrows another layer's weights still has
// its own slice of every page.
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
#include "safetensors_loader.h"
#include "pegainfer_kernels.h"
#include "pegainfer_kernels_blocks.h"
#include "pegainfer_kernels_ext.h"
#include "pegainfer_qwen3.h"   // pegainfer_logprobs_from_logits (pure host)
#include "pegainfer_duguzen.h"

namespace pdz {

using pq::KvState;
using pq::PagePool;
using pst::Json;

#define DZ_HIP(expr)                                                   \
  do {                                                                 \
    hipError_t e_ = (expr);                                            \
    if (e_ != hipSuccess) {                                            \
      set_error(std::string(#expr) + ": " + hipGetErrorString(e_));    \
      return -1;                                                       \
    }                                                                  \
  } while (0)
#define DZ_K(expr)                                                     \
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

constexpr int kPageSize = 16;   // tokens per cache page, as in the other runtimes

struct MixerCfg { int heads = 0, nope = 0, rot = 0, vdim = 0, rank = 0, rot_dims = 0; double base = 10000.0; float scale = 1.f; };
struct MlpCfg { int kind = 0 /* 0 none, 1 dense, 2 routed */, ff = 0, experts = 0, top = 0, groups = 1, keep = 1; };
struct LayerCfg {
  MixerCfg mx;
  MlpCfg mlp;
  int owner = 0;
  int64_t cache_off = 0;   // element offset of this layer run's slice inside a page
  int entry() const { return mx.rank + mx.rot; }
  // rows of the stacked projection [q ; dkv ; g], padded with zero rows to a multiple of 8 so that every row of its output
  // starts on a 16-byte boundary
  int proj_rows() const { return (mx.heads * (mx.nope + mx.rot) + mx.rank + mx.rot + mx.heads + 7) & ~7; }
};
struct Norm { void *w = nullptr, *b = nullptr, *alpha = nullptr; };
struct LayerW {
  bool loaded = false;
  Norm n1, n1b, n2, n2b;
  void *proj = nullptr, *cnorm = nullptr, *uk = nullptr, *uv = nullptr, *o = nullptr;
  void *up = nullptr, *down = nullptr;                       // dense
  void *router = nullptr, *corr = nullptr, *gate_up_e = nullptr, *down_e = nullptr;   // routed
  float* inv_freq = nullptr;
};

struct Model {
  int device = 0, dtype = 0, D = 0, V = 0, max_requests = 0, num_pages = 0;
  float eps = 1e-5f;
  bool plain_kernels = false, finalized = false;
  std::string err;
  std::vector<LayerCfg> layers;
  std::vector<LayerW> weights;          // indexed by owner layer
  Norm final_norm;
  void *embed = nullptr, *head = nullptr;
  std::map<std::string, std::vector<uint16_t>> staged;   // checkpoint tensors waiting for finalize()
  std::vector<void*> owned;
  int64_t weight_bytes = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  float last_step_ms = 0.f;
  // cache
  int64_t page_stride = 0;
  void* cache = nullptr;
  PagePool pool{0};
  std::vector<KvState> requests;
  // step buffers (grow-only, sized by token rows / wanted rows)
  size_t cap_rows = 0, cap_want = 0, cap_meta = 0;
  std::vector<void*> step_owned, want_owned;
  float *x = nullptr, *qc = nullptr, *olat = nullptr, *ypairs = nullptr, *route_w = nullptr, *attn_ws = nullptr;
  size_t attn_ws_cap = 0;
  void *h = nullptr, *proj = nullptr, *attn = nullptr, *y = nullptr, *ffb = nullptr, *gu = nullptr, *act = nullptr;
  int32_t *route_e = nullptr, *pos_pair = nullptr, *pos_row = nullptr, *tiles = nullptr;
  int max_tiles = 0;
  float *xw = nullptr, *logits32 = nullptr;
  void *hw = nullptr, *logits = nullptr;
  Half* logits16 = nullptr;      // bf16 image of the wanted rows' logits for the samplers
  int32_t* tokens_d = nullptr;
  uint8_t* top1_state = nullptr;
  uint8_t *meta_host = nullptr, *meta_dev = nullptr;
  // sampling scratch
  float* probs_scratch = nullptr;
  Half* top1_value = nullptr;
  uint8_t *row_states = nullptr, *valid_scratch = nullptr;
  int32_t* sample_out_d = nullptr;
  int last_rows = 0;
  std::vector<float> lp_row;
  // taps
  bool tap_on = false;
  float* tap = nullptr;
  size_t tap_cap = 0;
  int tap_rows = 0;
  // maxima over the layers
  int mx_proj = 0, mx_qc = 0, mx_olat = 0, mx_attn = 0, mx_ff = 0, mx_top = 0, mx_gu = 0, mx_experts = 0, mx_heads = 0, mx_rank = 0;

  int set_error(const std::string& e) { err = e; return -1; }
  size_t esize() const { return dtype == PEGAINFER_DTYPE_F32 ? 4 : 2; }
  pegainfer_stream_t S() const { return reinterpret_cast<pegainfer_stream_t>(stream); }

  // ------------------------------------------------------------------ configuration
  static int geti(const Json* j, const char* k, int d) { return j ? (int)j->number_or(k, d) : d; }
  int parse_config(const std::string& text) {
    Json j;
    if (!pst::JsonParser(text.data(), text.size()).parse(&j) || j.kind != Json::Obj) return set_error("config: not a JSON object");
    const Json* arch = j.get("architecture");
    if (!arch || arch->str != "Duguzen") return set_error("config: architecture is not Duguzen");
    D = geti(&j, "width", 0);
    V = geti(&j, "vocab", 0);
    if (const Json* n = j.get("norm")) eps = (float)n->number_or("eps", 1e-5);
    const Json* ls = j.get("layers");
    if (D <= 0 || V <= 0 || !ls || ls->kind != Json::Arr || ls->arr.empty()) return set_error("config: width / vocab / layers missing");
    int64_t off = 0;
    for (size_t i = 0; i < ls->arr.size(); ++i) {
      const Json& l = ls->arr[i];
      LayerCfg c;
      const Json* ty = l.get("type");
      if (!ty || ty->str != "latent_attention") return set_error("config: layer " + std::to_string(i) + " has an unknown mixer type");
      const Json* mx = l.get("mixer");
      if (!mx || mx->kind != Json::Obj) return set_error("config: layer without mixer sizes");
      c.mx.heads = geti(mx, "heads", 0);
      c.mx.nope = geti(mx, "dim", 0);
      c.mx.rot = geti(mx, "rot_dim", 0);
      c.mx.vdim = geti(mx, "vdim", 0);
      c.mx.rank = geti(mx, "kv_rank", 0);
      c.mx.scale = (float)mx->number_or("scale", 1.0 / std::sqrt((double)std::max(1, c.mx.nope + c.mx.rot)));
      const Json* rot = mx->get("rot");
      c.mx.rot_dims = rot ? geti(rot, "dims", c.mx.rot) : c.mx.rot;
      c.mx.base = rot ? rot->number_or("base", 10000.0) : 10000.0;
      if (c.mx.heads <= 0 || c.mx.nope < 0 || c.mx.rot < 0 || c.mx.vdim <= 0 || c.mx.rank <= 0 || c.mx.rot_dims > c.mx.rot ||
          (c.mx.rot_dims & 1) || c.mx.rank > 1024)
        return set_error("config: unsupported mixer sizes in layer " + std::to_string(i));
      const Json* mlp = l.get("mlp");
      if (mlp && mlp->kind == Json::Obj) {
        const Json* kind = mlp->get("kind");
        if (kind && kind->str == "dense") {
          c.mlp.kind = 1;
          c.mlp.ff = geti(mlp, "ff", 0);
        } else if (kind && kind->str == "moe") {
          c.mlp.kind = 2;
          c.mlp.ff = geti(mlp->get("expert"), "ff", 0);
          const Json* rt = mlp->get("router");
          c.mlp.experts = geti(rt, "experts", 0);
          c.mlp.top = geti(rt, "top", 0);
          const Json* g = rt ? rt->get("groups") : nullptr;
          c.mlp.groups = g ? geti(g, "count", 1) : 1;
          c.mlp.keep = g ? geti(g, "keep", c.mlp.groups) : 1;
          if (c.mlp.groups < 1) c.mlp.groups = 1;
          if (c.mlp.experts <= 0 || c.mlp.top <= 0 || c.mlp.top > c.mlp.experts || c.mlp.experts % c.mlp.groups ||
              c.mlp.keep < 1 || c.mlp.keep > c.mlp.groups)
            return set_error("config: unsupported router in layer " + std::to_string(i));
        } else {
          return set_error("config: unknown feed-forward kind in layer " + std::to_string(i));
        }
        if (c.mlp.ff <= 0) return set_error("config: feed-forward without a size in layer " + std::to_string(i));
      }
      const Json* wo = l.get("weights_of");
      c.owner = wo && wo->kind == Json::Num ? (int)wo->num : (int)i;
      if (c.owner < 0 || c.owner >= (int)ls->arr.size()) return set_error("config: weights_of outside the layer list");
      c.cache_off = off;
      off += (int64_t)kPageSize * c.entry();
      layers.push_back(c);
    }
    for (auto& c : layers) {   // a borrowed layer may itself borrow: follow the chain to the layer that owns tensors
      int o = c.owner, hops = 0;
      while (layers[o].owner != o && hops++ < (int)layers.size()) o = layers[o].owner;
      if (layers[o].owner != o) return set_error("config: weights_of forms a cycle");
      c.owner = o;
    }
    page_stride = off;
    weights.resize(layers.size());
    for (auto& c : layers) {
      mx_proj = std::max(mx_proj, c.proj_rows());
      mx_qc = std::max(mx_qc, c.mx.heads * c.entry());
      mx_olat = std::max(mx_olat, c.mx.heads * c.mx.rank);
      mx_attn = std::max(mx_attn, c.mx.heads * c.mx.vdim);
      mx_heads = std::max(mx_heads, c.mx.heads);
      mx_rank = std::max(mx_rank, c.mx.rank);
      if (c.mlp.kind == 1) mx_ff = std::max(mx_ff, c.mlp.ff);
      if (c.mlp.kind == 2) {
        mx_top = std::max(mx_top, c.mlp.top);
        mx_gu = std::max(mx_gu, c.mlp.top * 2 * c.mlp.ff);
        mx_experts = std::max(mx_experts, c.mlp.experts);
      }
    }
    return 0;
  }

  // ------------------------------------------------------------------ device memory
  template <typename T>
  int dalloc(T** p, size_t count, std::vector<void*>* into = nullptr) {
    void* raw = nullptr;
    DZ_HIP(hipMalloc(&raw, std::max<size_t>(count, 1) * sizeof(T)));
    DZ_HIP(hipMemset(raw, 0, std::max<size_t>(count, 1) * sizeof(T)));
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
    DZ_HIP(hipSetDevice(device));
    cublas_init();
    DZ_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    DZ_HIP(hipEventCreate(&ev0));
    DZ_HIP(hipEventCreate(&ev1));
    num_pages = std::max(1, (max_tokens + kPageSize - 1) / kPageSize);
    pool = PagePool(num_pages);
    requests.assign((size_t)max_requests, KvState());
    if (dalloc_a(&cache, (size_t)num_pages * (size_t)page_stride)) return -1;
    if (dalloc(&probs_scratch, (size_t)V) || dalloc(&top1_value, 1) || dalloc(&row_states, 1024 * 1024) ||
        dalloc(&valid_scratch, 1) || dalloc(&sample_out_d, 1))
      return -1;
    return 0;
  }

  // ------------------------------------------------------------------ weights
  std::vector<std::pair<std::string, std::vector<int64_t>>> tensor_list() const {
    std::vector<std::pair<std::string, std::vector<int64_t>>> out;
    auto norm = [&](const std::string& n, int d) {
      out.push_back({n, {d}});
      out.push_back({n + ".b", {d}});
      out.push_back({n + ".alpha", {}});
    };
    out.push_back({"embed", {V, D}});
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      if (c.owner != (int)i) continue;
      const std::string p = "l" + std::to_string(i);
      norm(p + ".norm1", D);
      norm(p + ".norm1b", D);
      const MixerCfg& m = c.mx;
      out.push_back({p + ".mix.q", {m.heads * (m.nope + m.rot), D}});
      out.push_back({p + ".mix.dkv", {m.rank + m.rot, D}});
      out.push_back({p + ".mix.dkv.norm", {m.rank}});
      out.push_back({p + ".mix.uk", {m.heads * m.nope, m.rank}});
      out.push_back({p + ".mix.uv", {m.heads * m.vdim, m.rank}});
      out.push_back({p + ".mix.g", {m.heads, D}});
      out.push_back({p + ".mix.o", {D, m.heads * m.vdim}});
      if (c.mlp.kind) {
        norm(p + ".norm2", D);
        norm(p + ".norm2b", D);
      }
      if (c.mlp.kind == 1) {
        out.push_back({p + ".mlp.up", {c.mlp.ff, D}});
        out.push_back({p + ".mlp.down", {D, c.mlp.ff}});
      } else if (c.mlp.kind == 2) {
        for (int e = 0; e < c.mlp.experts; ++e) {
          const std::string pe = p + ".mlp.e" + std::to_string(e);
          out.push_back({pe + ".gate", {c.mlp.ff, D}});
          out.push_back({pe + ".up", {c.mlp.ff, D}});
          out.push_back({pe + ".down", {D, c.mlp.ff}});
        }
        out.push_back({p + ".mlp.router", {c.mlp.experts, D}});
        out.push_back({p + ".mlp.correction", {c.mlp.experts}});
      }
    }
    norm("final.norm", D);
    out.push_back({"head", {V, D}});
    return out;
  }
  static int64_t numel(const std::vector<int64_t>& s) { int64_t n = 1; for (int64_t d : s) n *= d; return n; }

  int load_tensor(const std::string& name, const uint16_t* bits, int64_t n) {
    if (finalized) return set_error("load_tensor after finalize");
    staged[name].assign(bits, bits + n);
    return 0;
  }
  int fill_synthetic(uint64_t seed, float std) {
    // splitmix64 stream; a unit-variance value = sum of four uniforms, centred and scaled (cheap, and enough for weights)
    uint64_t state = seed * 0x9E3779B97F4A7C15ull + 0x1234567ull;
    auto g = [&state](int) {
      state += 0x9E3779B97F4A7C15ull;
      uint64_t z = state;
      z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
      z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
      z ^= z >> 31;
      const float u = (float)(z & 0xFFFF) + (float)((z >> 16) & 0xFFFF) + (float)((z >> 32) & 0xFFFF) + (float)(z >> 48);
      return (u * (1.0f / 65536.0f) - 2.0f) * 1.7320508f;
    };
    int rng = 0;
    for (auto& t : tensor_list()) {
      const std::string& n = t.first;
      std::vector<uint16_t>& v = staged[n];
      v.resize((size_t)numel(t.second));
      const bool alpha = n.size() > 6 && n.compare(n.size() - 6, 6, ".alpha") == 0;
      const bool bias = n.size() > 2 && n.compare(n.size() - 2, 2, ".b") == 0;
      const bool normw = t.second.size() == 1 && !bias && n.find("correction") == std::string::npos;
      const bool corr = n.find("correction") != std::string::npos;
      for (auto& x : v) {
        const float z = g(rng);
        x = host_f2bf(alpha ? 0.5f + 0.05f * z : normw ? 1.0f + 0.1f * z : corr ? 0.1f * z : bias ? 0.02f * z : std * z);
      }
    }
    return 0;
  }
  // device image (storage type of the model) of host bf16 bits
  int upload(void** out, const uint16_t* bits, size_t n) {
    if (dalloc_a(out, n)) return -1;
    if (dtype == PEGAINFER_DTYPE_BF16) {
      DZ_HIP(hipMemcpy(*out, bits, n * 2, hipMemcpyHostToDevice));
    } else {
      std::vector<float> f(n);
      for (size_t i = 0; i < n; ++i) f[i] = host_bf2f(bits[i]);
      DZ_HIP(hipMemcpy(*out, f.data(), n * 4, hipMemcpyHostToDevice));
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
  int up_norm(Norm* nm, const std::string& name, int d) {
    return (up(&nm->w, name, d) || up(&nm->b, name + ".b", d) || up(&nm->alpha, name + ".alpha", 1)) ? -1 : 0;
  }
  int finalize() {
    if (finalized) return 0;
    if (up(&embed, "embed", (int64_t)V * D) || up(&head, "head", (int64_t)V * D) || up_norm(&final_norm, "final.norm", D)) return -1;
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      if (c.owner != (int)i) continue;
      LayerW& w = weights[i];
      const MixerCfg& m = c.mx;
      const std::string p = "l" + std::to_string(i);
      if (up_norm(&w.n1, p + ".norm1", D) || up_norm(&w.n1b, p + ".norm1b", D)) return -1;
      if (c.mlp.kind && (up_norm(&w.n2, p + ".norm2", D) || up_norm(&w.n2b, p + ".norm2b", D))) return -1;
      {  // stacked projection [q ; dkv ; g]
        const auto *q = need(p + ".mix.q", (int64_t)m.heads * (m.nope + m.rot) * D),
                   *dkv = need(p + ".mix.dkv", (int64_t)(m.rank + m.rot) * D), *g = need(p + ".mix.g", (int64_t)m.heads * D);
        if (!q || !dkv || !g) return -1;
        std::vector<uint16_t> st(*q);
        st.insert(st.end(), dkv->begin(), dkv->end());
        st.insert(st.end(), g->begin(), g->end());
        st.resize((size_t)c.proj_rows() * D, 0);
        if (upload(&w.proj, st.data(), st.size())) return -1;
      }
      {  // key up-projection stored transposed per head, [heads][rank][nope]: the absorb GEMM reads it with k contiguous
        const auto* uk = need(p + ".mix.uk", (int64_t)m.heads * m.nope * m.rank);
        if (!uk) return -1;
        std::vector<uint16_t> tr(uk->size());
        for (int hh = 0; hh < m.heads; ++hh)
          for (int dd = 0; dd < m.nope; ++dd)
            for (int rr = 0; rr < m.rank; ++rr)
              tr[((size_t)hh * m.rank + rr) * m.nope + dd] = (*uk)[((size_t)hh * m.nope + dd) * m.rank + rr];
        if (upload(&w.uk, tr.data(), tr.size())) return -1;
      }
      if (up(&w.cnorm, p + ".mix.dkv.norm", m.rank) ||
          up(&w.uv, p + ".mix.uv", (int64_t)m.heads * m.vdim * m.rank) || up(&w.o, p + ".mix.o", (int64_t)D * m.heads * m.vdim))
        return -1;
      {  // rotation frequencies base^(-2i/dims), rounded once to fp32
        const int half = m.rot_dims / 2;
        std::vector<float> f((size_t)std::max(1, half));
        for (int k = 0; k < half; ++k) f[k] = (float)std::pow(m.base, -2.0 * k / (double)m.rot_dims);
        if (dalloc(&w.inv_freq, f.size())) return -1;
        DZ_HIP(hipMemcpy(w.inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice));
      }
      if (c.mlp.kind == 1) {
        if (up(&w.up, p + ".mlp.up", (int64_t)c.mlp.ff * D) || up(&w.down, p + ".mlp.down", (int64_t)D * c.mlp.ff)) return -1;
      } else if (c.mlp.kind == 2) {
        std::vector<uint16_t> gu, dn;
        for (int e = 0; e < c.mlp.experts; ++e) {
          const std::string pe = p + ".mlp.e" + std::to_string(e);
          const auto *g = need(pe + ".gate", (int64_t)c.mlp.ff * D), *u = need(pe + ".up", (int64_t)c.mlp.ff * D),
                     *d = need(pe + ".down", (int64_t)D * c.mlp.ff);
          if (!g || !u || !d) return -1;
          gu.insert(gu.end(), g->begin(), g->end());
          gu.insert(gu.end(), u->begin(), u->end());
          dn.insert(dn.end(), d->begin(), d->end());
        }
        if (upload(&w.gate_up_e, gu.data(), gu.size()) || upload(&w.down_e, dn.data(), dn.size())) return -1;
        if (up(&w.router, p + ".mlp.router", (int64_t)c.mlp.experts * D)) return -1;
        if (staged.count(p + ".mlp.correction") && up(&w.corr, p + ".mlp.correction", c.mlp.experts)) return -1;
      }
      w.loaded = true;
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
      if (!v) {
        if (t.first.find(".correction") != std::string::npos) continue;   // a router without correction chooses by its scores
        return set_error("checkpoint has no tensor " + t.first);
      }
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
    DZ_HIP(hipStreamSynchronize(stream));
    free_all(&step_owned);
    cap_rows = 0;
    size_t n = 64;
    while (n < T) n *= 2;
    auto* so = &step_owned;
    const size_t P = n * (size_t)std::max(1, mx_top);
    max_tiles = (int)((P + 63) / 64) + std::max(1, mx_experts);
    if (dalloc(&x, n * D, so) || dalloc(&qc, n * mx_qc, so) || dalloc(&olat, n * mx_olat, so) || dalloc_a(&h, n * D, so) ||
        dalloc_a(&proj, n * mx_proj, so) || dalloc_a(&attn, n * mx_attn, so) || dalloc_a(&y, n * D, so) ||
        dalloc_a(&ffb, n * std::max(1, mx_ff), so))
      return -1;
    if (mx_top > 0 && (dalloc(&ypairs, P * D, so) || dalloc(&route_w, P, so) || dalloc(&route_e, P, so) || dalloc(&pos_pair, P, so) ||
                       dalloc(&pos_row, P, so) || dalloc(&tiles, (size_t)3 * max_tiles + 1, so) || dalloc_a(&gu, n * mx_gu, so) ||
                       dalloc_a(&act, n * (size_t)(mx_gu / 2), so)))
      return -1;
    cap_rows = n;
    return 0;
  }
  int ensure_want(size_t n) {
    if (n <= cap_want) return 0;
    DZ_HIP(hipStreamSynchronize(stream));
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
  int linear(const void* W, const void* X, void* Y, int M, int T, int K, int epilogue = PEGAINFER_EPI_NONE) {
    if (dtype == PEGAINFER_DTYPE_BF16 && !plain_kernels) {
      gemm_cuda(static_cast<const Half*>(W), static_cast<const Half*>(X), static_cast<Half*>(Y), M, T, K, S());
      if (epilogue == PEGAINFER_EPI_RELU_SQ) DZ_K(pegainfer_relu_sq(Y, Y, (int64_t)M * T, dtype, S()));
      return 0;
    }
    pegainfer_gemm_desc d{};
    d.x = X; d.w = W; d.y = Y;
    d.x_dtype = d.w_dtype = d.y_dtype = dtype;
    d.m = M; d.k = K; d.rows = T; d.groups = 1;
    d.x_row_stride = K; d.w_m_stride = K; d.w_k_stride = 1; d.y_row_stride = M;
    d.epilogue = epilogue;
    d.plain = plain_kernels;
    DZ_K(pegainfer_gemm_strided(&d, S()));
    return 0;
  }

  int step(int n, const int32_t* ids, const int32_t* lens, const uint32_t* tokens, int n_want, const int32_t* want_rows,
           float* out_logits, int32_t* out_tokens) {
    if (!finalized) return set_error("step before finalize");
    if (n <= 0 || n > max_requests) return set_error("step: batch size outside 1 .. max_requests");
    // ---- validate everything before anything changes
    size_t T = 0;
    int need_pages = 0, max_kv = 0;
    for (int i = 0; i < n; ++i) {
      if (ids[i] < 0 || ids[i] >= (int)requests.size() || !requests[ids[i]].live) return set_error("step: unknown request");
      for (int k = 0; k < i; ++k)
        if (ids[k] == ids[i]) return set_error("step: a request is listed twice");
      if (lens[i] <= 0) return set_error("step: an entry without tokens");
      const KvState& st = requests[ids[i]];
      need_pages += st.pages_short(st.seq_len + lens[i], kPageSize);
      max_kv = std::max(max_kv, st.seq_len + lens[i]);
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
    // decode-like steps (few rows) cut the keys finely so that one request's context spreads over many workgroups;
    // prompt-sized steps have rows enough and only cut very long contexts
    const int split_keys = T * (size_t)mx_heads <= 1024 ? 32 : 4096;
    const int64_t ws_need = pegainfer_latent_attention_workspace((int)T, mx_heads, mx_rank, max_kv, split_keys);
    if ((size_t)ws_need > attn_ws_cap) {
      DZ_HIP(hipStreamSynchronize(stream));
      if (attn_ws) (void)hipFree(attn_ws);
      attn_ws = nullptr;
      attn_ws_cap = 0;
      DZ_HIP(hipMalloc(reinterpret_cast<void**>(&attn_ws), (size_t)ws_need * 4));
      attn_ws_cap = (size_t)ws_need;
    }
    // ---- pages, then the packed metadata block: tokens | positions | token_req | page_indptr | want | page_ids
    size_t total_pages = 0;
    for (int i = 0; i < n; ++i) {
      KvState& st = requests[ids[i]];
      if (!st.ensure_capacity(&pool, st.seq_len + lens[i], kPageSize)) return set_error("step: page pool ran dry");   // cannot happen after the check above
      total_pages += st.pages.size();
    }
    // row tiles of the matrix-core attention: per distinct head count, the flattened (token, head) rows cut into runs of
    // <= 64 rows that stay inside one entry
    std::vector<int> head_vals;
    for (auto& c : layers)
      if (std::find(head_vals.begin(), head_vals.end(), c.mx.heads) == head_vals.end()) head_vals.push_back(c.mx.heads);
    std::vector<size_t> tile_off(head_vals.size()), tile_cnt(head_vals.size());
    const size_t o_tok = 0, o_pos = o_tok + T, o_req = o_pos + T, o_ind = o_req + T, o_want = o_ind + (size_t)n + 1,
                 o_pages = o_want + (size_t)std::max(1, W);
    size_t words = o_pages + total_pages;
    for (size_t k = 0; k < head_vals.size(); ++k) {
      size_t cnt = 0;
      for (int i = 0; i < n; ++i) cnt += ((size_t)lens[i] * head_vals[k] + 63) / 64;
      tile_off[k] = words;
      tile_cnt[k] = cnt;
      words += 2 * cnt;
    }
    if (words > cap_meta) {
      DZ_HIP(hipStreamSynchronize(stream));
      if (meta_host) (void)hipHostFree(meta_host);
      if (meta_dev) (void)hipFree(meta_dev);
      meta_host = meta_dev = nullptr;
      cap_meta = 0;
      size_t c = 4096;
      while (c < words) c *= 2;
      DZ_HIP(hipHostMalloc(reinterpret_cast<void**>(&meta_host), c * 4, hipHostMallocDefault));
      DZ_HIP(hipMalloc(reinterpret_cast<void**>(&meta_dev), c * 4));
      cap_meta = c;
    }
    int32_t* mh = reinterpret_cast<int32_t*>(meta_host);
    {
      size_t t = 0, pg = 0;
      for (int i = 0; i < n; ++i) {
        const KvState& st = requests[ids[i]];
        mh[o_ind + i] = (int32_t)pg;
        for (int32_t p : st.pages) mh[o_pages + pg++] = p;
        for (int k = 0; k < lens[i]; ++k, ++t) {
          mh[o_tok + t] = (int32_t)tokens[t];
          mh[o_pos + t] = st.seq_len + k;
          mh[o_req + t] = i;
        }
      }
      mh[o_ind + n] = (int32_t)pg;
      for (int i = 0; i < W; ++i) mh[o_want + i] = want[i];
      for (size_t k = 0; k < head_vals.size(); ++k) {
        const int Hk = head_vals[k];
        size_t at = 0, tok0 = 0;
        for (int i = 0; i < n; ++i) {
          const int rows = lens[i] * Hk;
          for (int r0 = 0; r0 < rows; r0 += 64, ++at) {
            mh[tile_off[k] + at] = (int32_t)(tok0 * Hk) + r0;
            mh[tile_off[k] + tile_cnt[k] + at] = std::min(64, rows - r0);
          }
          tok0 += (size_t)lens[i];
        }
      }
    }
    DZ_HIP(hipEventRecord(ev0, stream));
    DZ_HIP(hipMemcpyAsync(meta_dev, meta_host, words * 4, hipMemcpyHostToDevice, stream));
    const int32_t* md = reinterpret_cast<const int32_t*>(meta_dev);
    const uint32_t* d_tok = reinterpret_cast<const uint32_t*>(md + o_tok);
    const int32_t *d_pos = md + o_pos, *d_req = md + o_req, *d_ind = md + o_ind, *d_want = md + o_want, *d_pages = md + o_pages;
    const int Ti = (int)T;
    if (tap_on) {
      const size_t needf = layers.size() * T * D;
      if (needf > tap_cap) {
        DZ_HIP(hipStreamSynchronize(stream));
        if (tap) (void)hipFree(tap);
        tap = nullptr;
        tap_cap = 0;
        DZ_HIP(hipMalloc(reinterpret_cast<void**>(&tap), needf * 4));
        tap_cap = needf;
      }
      tap_rows = Ti;
    }
    // ---- the layers
    DZ_K(pegainfer_embed_f32(embed, d_tok, x, D, Ti, dtype, S()));
    {
      const LayerW& w0 = weights[layers[0].owner];
      DZ_K(pegainfer_dyt_norm(x, w0.n1.alpha, w0.n1.w, w0.n1.b, h, D, Ti, dtype, S()));
    }
    for (size_t li = 0; li < layers.size(); ++li) {
      const LayerCfg& c = layers[li];
      const LayerW& w = weights[c.owner];
      const MixerCfg& m = c.mx;
      const int E = c.entry(), Mp = c.proj_rows(), qrow = m.heads * (m.nope + m.rot);
      const Norm* next_pre = li + 1 < layers.size() ? &weights[layers[li + 1].owner].n1 : nullptr;
      if (linear(w.proj, h, proj, Mp, Ti, D)) return -1;
      DZ_K(pegainfer_latent_prep(proj, Mp, qrow, w.cnorm, eps, w.inv_freq, m.rot_dims, d_pos, d_req, d_ind, d_pages, cache,
                                 page_stride, c.cache_off, kPageSize, qc, m.heads, m.nope, m.rot, m.rank, Ti, dtype, S()));
      if (m.nope > 0) {   // absorb: qc[t, h, :rank] = sum_d q[t, h, d] * Wuk[h * nope + d, :]
        pegainfer_gemm_desc d{};
        d.x = proj; d.w = w.uk; d.y = qc;
        d.x_dtype = d.w_dtype = dtype; d.y_dtype = PEGAINFER_DTYPE_F32;
        d.m = m.rank; d.k = m.nope; d.rows = Ti; d.groups = m.heads;
        d.x_row_stride = Mp; d.x_group_stride = m.nope + m.rot;
        d.w_m_stride = m.nope; d.w_k_stride = 1; d.w_group_stride = (int64_t)m.nope * m.rank;
        d.y_row_stride = (int64_t)m.heads * E; d.y_group_stride = E;
        d.plain = plain_kernels;
        DZ_K(pegainfer_gemm_strided(&d, S()));
      } else {
        DZ_HIP(hipMemsetAsync(qc, 0, T * (size_t)m.heads * E * 4, stream));
      }
      {
        const size_t hk = std::find(head_vals.begin(), head_vals.end(), m.heads) - head_vals.begin();
        const bool tiled = !plain_kernels && pegainfer_latent_attention_tiled_ok(m.rank, m.rot, page_stride, c.cache_off, dtype);
        DZ_K(pegainfer_latent_attention(qc, olat, cache, page_stride, c.cache_off, kPageSize, d_pos, d_req, d_ind, d_pages,
                                        m.heads, m.rank, m.rot, m.scale, Ti, max_kv, split_keys, attn_ws,
                                        tiled ? md + tile_off[hk] : nullptr, tiled ? md + tile_off[hk] + tile_cnt[hk] : nullptr,
                                        (int)tile_cnt[hk], dtype, S()));
      }
      {  // value up-projection per head + sigmoid gate
        pegainfer_gemm_desc d{};
        d.x = olat; d.w = w.uv; d.y = attn;
        d.x_dtype = PEGAINFER_DTYPE_F32; d.w_dtype = d.y_dtype = dtype;
        d.m = m.vdim; d.k = m.rank; d.rows = Ti; d.groups = m.heads;
        d.x_row_stride = (int64_t)m.heads * m.rank; d.x_group_stride = m.rank;
        d.w_m_stride = m.rank; d.w_k_stride = 1; d.w_group_stride = (int64_t)m.vdim * m.rank;
        d.y_row_stride = (int64_t)m.heads * m.vdim; d.y_group_stride = m.vdim;
        d.epilogue = PEGAINFER_EPI_SIGMOID_GATE;
        d.gate = static_cast<const uint8_t*>(proj) + (size_t)(qrow + E) * esize();
        d.gate_dtype = dtype;
        d.gate_row_stride = Mp;
        d.plain = plain_kernels;
        DZ_K(pegainfer_gemm_strided(&d, S()));
      }
      if (linear(w.o, attn, y, D, Ti, m.heads * m.vdim)) return -1;
      if (c.mlp.kind) {
        DZ_K(pegainfer_dyt_add_norm(x, y, w.n1b.alpha, w.n1b.w, w.n1b.b, w.n2.alpha, w.n2.w, w.n2.b, h, D, Ti, dtype, S()));
        if (c.mlp.kind == 1) {
          if (linear(w.up, h, ffb, c.mlp.ff, Ti, D, PEGAINFER_EPI_RELU_SQ) || linear(w.down, ffb, y, D, Ti, c.mlp.ff)) return -1;
        } else if (routed_ff(c, w, Ti)) {
          return -1;
        }
        DZ_K(pegainfer_dyt_add_norm(x, y, w.n2b.alpha, w.n2b.w, w.n2b.b, next_pre ? next_pre->alpha : nullptr,
                                    next_pre ? next_pre->w : nullptr, next_pre ? next_pre->b : nullptr, h, D, Ti, dtype, S()));
      } else {
        DZ_K(pegainfer_dyt_add_norm(x, y, w.n1b.alpha, w.n1b.w, w.n1b.b, next_pre ? next_pre->alpha : nullptr,
                                    next_pre ? next_pre->w : nullptr, next_pre ? next_pre->b : nullptr, h, D, Ti, dtype, S()));
      }
      if (tap_on) DZ_HIP(hipMemcpyAsync(tap + li * T * D, x, T * D * 4, hipMemcpyDeviceToDevice, stream));
    }
    // ---- wanted rows: final norm + head
    if (W > 0) {
      DZ_K(pegainfer_gather_rows_f32(x, d_want, xw, D, W, S()));
      DZ_K(pegainfer_dyt_norm(xw, final_norm.alpha, final_norm.w, final_norm.b, hw, D, W, dtype, S()));
      if (linear(head, hw, logits, V, W, D)) return -1;
      if (dtype == PEGAINFER_DTYPE_BF16) {
        DZ_K(deepseek_bf16_to_f32_cuda(static_cast<const Half*>(logits), logits32, W * V, S()));
        DZ_HIP(hipMemcpyAsync(logits16, logits, (size_t)W * V * 2, hipMemcpyDeviceToDevice, stream));
      } else {
        DZ_HIP(hipMemcpyAsync(logits32, logits, (size_t)W * V * 4, hipMemcpyDeviceToDevice, stream));
        DZ_K(deepseek_f32_to_bf16_cuda(logits32, logits16, W * V, S()));
      }
      if (out_tokens) DZ_K(pegainfer_batched_top1(logits16, V, W, V, top1_state, tokens_d, S()));
    }
    last_rows = W;
    DZ_HIP(hipEventRecord(ev1, stream));
    if (W > 0 && out_logits) DZ_HIP(hipMemcpyAsync(out_logits, logits32, (size_t)W * V * 4, hipMemcpyDeviceToHost, stream));
    if (W > 0 && out_tokens) DZ_HIP(hipMemcpyAsync(out_tokens, tokens_d, (size_t)W * 4, hipMemcpyDeviceToHost, stream));
    DZ_HIP(hipStreamSynchronize(stream));
    (void)hipEventElapsedTime(&last_step_ms, ev0, ev1);
    for (int i = 0; i < n; ++i) requests[ids[i]].seq_len += lens[i];
    return 0;
  }

  int routed_ff(const LayerCfg& c, const LayerW& w, int T) {
    const MlpCfg& f = c.mlp;
    const int P = T * f.top;
    int32_t *t_group = tiles, *t_row0 = tiles + max_tiles, *t_rows = tiles + 2 * max_tiles, *n_tiles = tiles + 3 * max_tiles;
    DZ_K(pegainfer_route_sigmoid_grouped(h, w.router, w.corr, route_e, route_w, D, f.experts, f.groups, f.keep, f.top, T, dtype, S()));
    // 128-row tiles for the matrix-core form (bf16, prompt-sized steps), 64-row tiles otherwise
    const int per_tile = dtype == PEGAINFER_DTYPE_BF16 && !plain_kernels && T > 8 && D % 8 == 0 && f.ff % 8 == 0 ? 128 : 64;
    DZ_K(pegainfer_route_sort(route_e, P, f.top, f.experts, pos_pair, pos_row, t_group, t_row0, t_rows, n_tiles, max_tiles, per_tile, S()));
    pegainfer_gemm_desc d{};
    d.x = h; d.w = w.gate_up_e; d.y = gu;
    d.x_dtype = d.w_dtype = d.y_dtype = dtype;
    d.m = 2 * f.ff; d.k = D;
    d.x_row_stride = D; d.w_m_stride = D; d.w_k_stride = 1; d.w_group_stride = (int64_t)2 * f.ff * D;
    d.y_row_stride = 2 * f.ff;
    d.tile_group = t_group; d.tile_row0 = t_row0; d.tile_rows = t_rows; d.n_tiles = n_tiles; d.max_tiles = (P + per_tile - 1) / per_tile + f.experts;
    d.tile_rows_cap = per_tile;
    d.x_row_index = pos_row;
    d.max_tile_rows = std::min(T, 64);   // a row chooses distinct experts: an expert never gets more pairs than there are rows
    d.plain = plain_kernels;
    DZ_K(pegainfer_gemm_strided(&d, S()));
    DZ_K(pegainfer_silu_mul_rows(gu, act, f.ff, P, dtype, S()));
    pegainfer_gemm_desc e{};
    e.x = act; e.w = w.down_e; e.y = ypairs;
    e.x_dtype = e.w_dtype = dtype; e.y_dtype = PEGAINFER_DTYPE_F32;
    e.m = D; e.k = f.ff;
    e.x_row_stride = f.ff; e.w_m_stride = f.ff; e.w_k_stride = 1; e.w_group_stride = (int64_t)D * f.ff;
    e.y_row_stride = D;
    e.tile_group = t_group; e.tile_row0 = t_row0; e.tile_rows = t_rows; e.n_tiles = n_tiles; e.max_tiles = d.max_tiles;
    e.y_row_index = pos_pair;
    e.max_tile_rows = d.max_tile_rows;
    e.tile_rows_cap = per_tile;
    e.plain = plain_kernels;
    DZ_K(pegainfer_gemm_strided(&e, S()));
    DZ_K(pegainfer_route_combine(ypairs, route_w, y, D, f.top, T, dtype, S()));
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
    DZ_HIP(hipStreamSynchronize(stream));
    DZ_HIP(hipMemcpy(out, sample_out_d, 4, hipMemcpyDeviceToHost));
    return 0;
  }
  int logprobs(int row, uint32_t token, int top_k, float* out_lp, uint32_t* top_ids, float* top_lps) {
    if (row < 0 || row >= last_rows) return set_error("no logits for that row");
    if (token >= (uint32_t)V) return set_error("logprobs: token outside the vocabulary");
    lp_row.resize((size_t)V);
    DZ_HIP(hipStreamSynchronize(stream));
    DZ_HIP(hipMemcpy(lp_row.data(), logits32 + (size_t)row * V, (size_t)V * 4, hipMemcpyDeviceToHost));
    return pegainfer_logprobs_from_logits(lp_row.data(), V, token, top_k, out_lp, top_ids, top_lps);
  }
  int debug_hidden(int run, float* out, int max_rows) {
    if (!tap || run < 0 || run >= (int)layers.size()) return set_error("debug_hidden: no tap for that layer run");
    const int rows = std::min(max_rows, tap_rows);
    DZ_HIP(hipStreamSynchronize(stream));
    DZ_HIP(hipMemcpy(out, tap + (size_t)run * tap_rows * D, (size_t)rows * D * 4, hipMemcpyDeviceToHost));
    return rows;
  }

  ~Model() {
    if (stream) (void)hipStreamSynchronize(stream);
    free_all(&owned);
    free_all(&step_owned);
    free_all(&want_owned);
    if (attn_ws) (void)hipFree(attn_ws);
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
static Model* M(pegainfer_duguzen_t m) { return static_cast<Model*>(m); }

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

}  // namespace pdz

extern "C" {
using pdz::M;

pegainfer_duguzen_t pegainfer_duguzen_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests) {
  if (!config_json) { pdz::g_create_error = "no configuration"; return nullptr; }
  return pdz::create(config_json, device_ordinal, dtype, max_tokens, max_requests);
}
pegainfer_duguzen_t pegainfer_duguzen_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests) {
  std::string e;
  auto f = pst::MappedFile::open(std::string(model_dir) + "/config.json", &e);
  if (!f) { pdz::g_create_error = e; return nullptr; }
  pdz::Model* m = pdz::create(std::string(reinterpret_cast<const char*>(f->data), f->size), device_ordinal, dtype, max_tokens, max_requests);
  if (!m) return nullptr;
  if (m->load_checkpoint(model_dir)) {
    pdz::g_create_error = m->err;
    delete m;
    return nullptr;
  }
  return m;
}
void pegainfer_duguzen_destroy(pegainfer_duguzen_t m) { delete M(m); }
const char* pegainfer_duguzen_last_error(pegainfer_duguzen_t m) { return m ? M(m)->err.c_str() : pdz::g_create_error.c_str(); }
int32_t pegainfer_duguzen_load_tensor(pegainfer_duguzen_t m, const char* name, const void* host_bf16, int64_t numel) {
  return M(m)->load_tensor(name, static_cast<const uint16_t*>(host_bf16), numel);
}
int32_t pegainfer_duguzen_fill_synthetic(pegainfer_duguzen_t m, uint64_t seed, float std) { return M(m)->fill_synthetic(seed, std); }
int32_t pegainfer_duguzen_finalize(pegainfer_duguzen_t m) { return M(m)->finalize(); }
int32_t pegainfer_duguzen_new_request(pegainfer_duguzen_t m) { return M(m)->new_request(); }
int32_t pegainfer_duguzen_drop_request(pegainfer_duguzen_t m, int32_t id) { return M(m)->drop_request(id); }
int32_t pegainfer_duguzen_request_seq_len(pegainfer_duguzen_t m, int32_t id) {
  if (id < 0 || id >= (int)M(m)->requests.size() || !M(m)->requests[id].live) return -1;
  return M(m)->requests[id].seq_len;
}
int32_t pegainfer_duguzen_available_pages(pegainfer_duguzen_t m) { return M(m)->pool.available(); }
int32_t pegainfer_duguzen_capacity_pages(pegainfer_duguzen_t m) { return M(m)->pool.capacity(); }
int32_t pegainfer_duguzen_page_size(pegainfer_duguzen_t) { return pdz::kPageSize; }
int32_t pegainfer_duguzen_max_batch_size(pegainfer_duguzen_t m) { return M(m)->max_requests; }
int32_t pegainfer_duguzen_vocab_size(pegainfer_duguzen_t m) { return M(m)->V; }
int32_t pegainfer_duguzen_width(pegainfer_duguzen_t m) { return M(m)->D; }
int32_t pegainfer_duguzen_num_layer_runs(pegainfer_duguzen_t m) { return (int32_t)M(m)->layers.size(); }
int32_t pegainfer_duguzen_dtype(pegainfer_duguzen_t m) { return M(m)->dtype; }
int32_t pegainfer_duguzen_step(pegainfer_duguzen_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens) {
  return M(m)->step(n_entries, request_ids, lens, tokens_concat, n_want, want_rows, out_logits_host, out_tokens);
}
int32_t pegainfer_duguzen_sample(pegainfer_duguzen_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token) {
  return M(m)->sample(row, temperature, top_k, top_p, random_val, out_token);
}
int32_t pegainfer_duguzen_logprobs(pegainfer_duguzen_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs) {
  return M(m)->logprobs(row, token, top_k, out_logprob, out_top_ids, out_top_logprobs);
}
int32_t pegainfer_duguzen_debug_hidden_enable(pegainfer_duguzen_t m, int32_t enable) { M(m)->tap_on = enable != 0; return 0; }
int32_t pegainfer_duguzen_debug_hidden(pegainfer_duguzen_t m, int32_t layer_run, float* out_host, int32_t max_rows) {
  return M(m)->debug_hidden(layer_run, out_host, max_rows);
}
float pegainfer_duguzen_last_step_ms(pegainfer_duguzen_t m) { return M(m)->last_step_ms; }
int64_t pegainfer_duguzen_weight_bytes(pegainfer_duguzen_t m) { return M(m)->weight_bytes; }
int32_t pegainfer_duguzen_set_plain_kernels(pegainfer_duguzen_t m, int32_t on) { M(m)->plain_kernels = on != 0; return 0; }

}  // extern "C"

// C++ host runtime of the Kukulorn decoder on MI355X (include/pegainfer_kukulorn.h).  Same shape as the runtimes next to it:
// one model = one device + one in-order HIP stream, requests are KvState slots over the shared PagePool (kv_pool.h) plus a
// region of the fp32 state arena (seq_state.h), a step's metadata is ONE pinned block and ONE hipMemcpyAsync, every op goes
// through the kernel library's C ABI (pegainfer_kernels.h: tuned bf16 GEMM routes, samplers; pegainfer_kernels_blocks.h:
// everything else).
//
// The layers of config.json are expanded into LAYER RUNS: the span loop.start .. loop.stop - 1 is walked loop.times times on
// the same weights, every run with its own part of the cache pages and its own state parts.  What a step does per run (T = all
// token rows of the step, prompts' portions and single tokens alike; x = fp32 stream, x0 = the embedding rows):
//   pass start : x <- W_in [x ; x0]                             one GEMM over the fp32 pair of rows, fp32 out
//   h      = x / rms(x) * norm1                                 one launch with the residual sums before it
//   proj   = Wstack h                                           ONE GEMM over everything that reads h: the mixer's projections
//                                                               and the feed-forward's gate | up
//   attention : q | k | v (+ biases) through the time convolution into fp32 (tail of taps - 1 biased inputs per (run, request));
//               rotation of the halves, unit root mean square per head, k / v into the paged cache; causal softmax attention
//               with tanh-capped scores, times sigmoid(g) per value, in the attention launch; Wo
//   parallel  : left  - biases, q / k RMS-normed over the whole projection, k / v into the paged cache; attention over a sliding
//                       window plus the kept first tokens with a bias by distance, times sigmoid(g) per head; Wo
//               right - x | B | C through the time convolution (+ bias, silu) into fp32; the state-space scan over the request's
//                       fp32 state; y * silu(z) normed in groups; Wo
//               both outputs RMS-normed over the width, weighted, averaged - inside the closing launch
//   ff        : relu(gate) * up from proj's columns; Wdown
//   x     += mixer + ff;  h = x / rms(x) * (next run's norm1)   the closing launch
//   logits = cap * tanh(embed (x / rms(x) * final.norm) / cap)  on the wanted rows
// Key/value cache: page-first [page][attention of run r][k: slot, kv head, dim | v: slot, kv head, vdim].
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
#include "pegainfer_kukulorn.h"

namespace pkk {

using pq::KvState;
using pq::PagePool;
using pst::Json;

#define KK_HIP(expr)                                                   \
  do {                                                                 \
    hipError_t e_ = (expr);                                            \
    if (e_ != hipSuccess) {                                            \
      set_error(std::string(#expr) + ": " + hipGetErrorString(e_));    \
      return -1;                                                       \
    }                                                                  \
  } while (0)
#define KK_K(expr)                                                     \
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
constexpr int kAttRows = 16;    // (token, query head) rows of one attention workgroup
constexpr int kSplitGroups = 512;   // most (tile, kv head, key split) workgroups of an attention launch that cuts its keys
constexpr int kMaxSplits = 16;

enum { kAttention = 1, kParallel = 2 };
// softmax attention: the "attention" mixer and the left half of "parallel"
struct AttnCfg {
  int heads = 0, kv = 0, dim = 0, vdim = 0;
  float scale = 1.f, softcap = 0.f;
  int taps = 0;                                   // time convolution on q | k | v (0: none)
  int rot_dims = 0;
  double base = 10000.0;
  bool scaled = false;                            // frequency scaling for long contexts
  double sc_factor = 1.0, sc_low = 1.0, sc_high = 1.0, sc_orig = 0.0;
  int window = 0, keep_first = 0;                 // sliding window that keeps the first tokens
  int bias_max = 0, rel_rows = 0;                 // bias by distance bucket
};
// selective state-space layer: the right half of "parallel"
struct SsmCfg {
  int heads = 0, vdim = 0, state = 0, groups = 1, norm_groups = 1, taps = 1;
  int inner() const { return heads * vdim; }
  int conv_ch() const { return inner() + 2 * groups * state; }
  int in_rows() const { return 2 * inner() + 2 * groups * state + heads; }
};
struct LayerCfg {
  int type = 0;
  AttnCfg at;
  SsmCfg sm;
  int ff = 0;        // 0: no feed-forward
  // columns of the stacked projection
  int o_q = 0, o_k = 0, o_v = 0, o_g = 0, o_in = 0, o_ffg = 0, o_ffu = 0, proj_rows = 0;
  int qkv_ch = 0;    // q | k | v columns
  int tile_set = -1;
};
struct LayerW {
  void *norm1 = nullptr, *proj = nullptr, *o = nullptr, *down = nullptr;
  void *qkv_bias = nullptr, *conv = nullptr;                                   // attention: stacked q | k | v biases and taps
  float* inv_freq = nullptr;
  void *q_norm = nullptr, *k_norm = nullptr, *o_bias = nullptr, *left_out = nullptr, *right_out = nullptr;   // parallel, left
  float* dist_bias = nullptr;
  int n_dist = 0;
  void *sconv = nullptr, *sconv_b = nullptr, *dt_bias = nullptr, *A_log = nullptr, *Dskip = nullptr, *snorm = nullptr, *ro = nullptr;   // right
};
// one walk over one layer: its weights (layer), its own cache part and state parts, and the pass it opens (or -1)
struct Run {
  int layer = 0, pass = -1;
  int64_t st_conv = 0, st_sconv = 0, st_mem = 0;
  int64_t k_off = 0, v_off = 0;
};

struct Model {
  int device = 0, dtype = 0, D = 0, V = 0, max_requests = 0, num_pages = 0;
  int loop_start = 0, loop_stop = 0, loop_times = 1;
  bool has_loop = false;
  float eps = 1e-5f, logit_cap = 0.f;
  bool plain_kernels = false, finalized = false;
  std::string err;
  std::vector<LayerCfg> layers;
  std::vector<LayerW> weights;
  std::vector<Run> runs;
  void *embed = nullptr, *final_norm = nullptr, *loop_in = nullptr;
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
  std::vector<int> tile_sets;   // distinct query-heads-per-kv-head values of the attention layers
  // step buffers
  size_t cap_rows = 0, cap_want = 0, cap_meta = 0;
  std::vector<void*> step_owned, want_owned;
  float *x = nullptr, *emb = nullptr, *xcat = nullptr, *conv32 = nullptr, *q32 = nullptr, *o32 = nullptr;
  void *hb = nullptr, *proj = nullptr, *mix = nullptr, *mixr = nullptr, *y1 = nullptr, *y2 = nullptr, *y3 = nullptr, *act = nullptr;
  float *xw = nullptr, *hw = nullptr, *logits32 = nullptr;
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
  float* att_part = nullptr;   // softmax states of the key splits of an attention launch
  int mx_proj = 0, mx_mix = 0, mx_inner = 0, mx_conv = 0, mx_q = 0, mx_ff = 0, mx_vdim = 0;

  struct GraphKey {
    int n, want; bool tokens, plain;
    bool operator==(const GraphKey& o) const { return n == o.n && want == o.want && tokens == o.tokens && plain == o.plain; }
  };
  std::vector<std::pair<GraphKey, hipGraphExec_t>> graphs;   // captured decode steps, one per shape
  bool graphs_on = [] { const char* e = getenv("PEGAINFER_KUKULORN_GRAPH"); return !(e && e[0] == '0'); }();
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
  // heads, sizes, scale; the options each mixer kind may carry are read where they are named
  int parse_attn(const Json* mx, AttnCfg* a, const std::string& li) {
    a->heads = geti(mx, "heads", 0);
    a->kv = geti(mx, "kv_heads", a->heads);
    a->dim = geti(mx, "dim", 0);
    a->vdim = geti(mx, "vdim", a->dim);
    a->scale = getf(mx, "scale", 1.0 / std::sqrt((double)std::max(1, a->dim)));
    a->softcap = getf(mx, "softcap", 0.0);
    a->taps = geti(mx, "conv", 0);
    if (const Json* rot = mx->get("rot")) {
      if (rot->kind == Json::Obj) {
        a->rot_dims = geti(rot, "dims", a->dim);
        a->base = rot->number_or("base", 10000.0);
        const Json* sc = rot->get("scaling");
        if (sc && sc->kind == Json::Obj) {
          a->scaled = true;
          a->sc_factor = sc->number_or("factor", 1.0);
          a->sc_low = sc->number_or("low", 1.0);
          a->sc_high = sc->number_or("high", 1.0);
          a->sc_orig = sc->number_or("original", 0.0);
          if (!(a->sc_factor > 0.0) || !(a->sc_orig > 0.0) || !(a->sc_high > 0.0) || !(a->sc_low > 0.0))
            return set_error("config: rot.scaling needs positive factor / low / high / original in layer " + li);
        }
      }
    }
    if (const Json* mk = mx->get("mask")) {
      if (mk->kind == Json::Obj) {
        a->window = geti(mk, "size", 0);
        a->keep_first = geti(mk, "keep_first", 0);
        if (a->window < 1 || a->keep_first < 0) return set_error("config: mask.size must be positive in layer " + li);
      }
    }
    a->bias_max = geti(mx, "bias_max", 0);
    a->rel_rows = geti(mx, "rel_rows", 0);
    if (a->heads <= 0 || a->kv <= 0 || a->heads % a->kv || a->dim <= 0 || a->dim > 256 || a->vdim <= 0 || a->vdim > 256 ||
        a->rot_dims < 0 || a->rot_dims > a->dim || (a->rot_dims & 1) || a->taps < 0 || a->taps > 64 || a->softcap < 0.f)
      return set_error("config: unsupported attention sizes in layer " + li);
    const int per = a->heads / a->kv;
    size_t k = 0;
    while (k < tile_sets.size() && tile_sets[k] != per) ++k;
    if (k == tile_sets.size()) tile_sets.push_back(per);
    return (int)k;
  }
  int parse_config(const std::string& text) {
    Json j;
    if (!pst::JsonParser(text.data(), text.size()).parse(&j) || j.kind != Json::Obj) return set_error("config: not a JSON object");
    const Json* arch = j.get("architecture");
    if (!arch || arch->str != "Kukulorn") return set_error("config: architecture is not Kukulorn");
    D = geti(&j, "width", 0);
    V = geti(&j, "vocab", 0);
    eps = getf(j.get("norm"), "eps", 1e-5);
    logit_cap = getf(&j, "logit_softcap", 0.0);
    const Json* ls = j.get("layers");
    if (D <= 0 || V <= 0 || !ls || ls->kind != Json::Arr || ls->arr.empty()) return set_error("config: width / vocab / layers missing");
    if (logit_cap < 0.f) return set_error("config: logit_softcap must not be negative");
    for (size_t i = 0; i < ls->arr.size(); ++i) {
      const Json& l = ls->arr[i];
      const std::string li = std::to_string(i);
      LayerCfg c;
      const Json* ty = l.get("type");
      const Json* mx = l.get("mixer");
      if (!ty || !mx || mx->kind != Json::Obj) return set_error("config: layer " + li + " without type / mixer");
      const Json* mlp = l.get("mlp");
      if (mlp && mlp->kind == Json::Obj) {
        const Json* kind = mlp->get("kind");
        if (kind && kind->str != "dense") return set_error("config: unknown feed-forward kind in layer " + li);
        c.ff = geti(mlp, "ff", 0);
        if (c.ff <= 0) return set_error("config: feed-forward without ff in layer " + li);
      }
      if (ty->str == "attention") {
        c.type = kAttention;
        if ((c.tile_set = parse_attn(mx, &c.at, li)) < 0) return -1;
        const AttnCfg& a = c.at;
        c.o_q = 0;
        c.o_k = a.heads * a.dim;
        c.o_v = c.o_k + a.kv * a.dim;
        c.qkv_ch = c.o_v + a.kv * a.vdim;
        c.o_g = pad8(c.qkv_ch);
        c.o_ffg = pad8(c.o_g + a.heads * a.vdim);
      } else if (ty->str == "parallel") {
        c.type = kParallel;
        const Json *lf = mx->get("left"), *rt = mx->get("right");
        if (!lf || lf->kind != Json::Obj || !rt || rt->kind != Json::Obj) return set_error("config: parallel layer " + li + " without left / right");
        if ((c.tile_set = parse_attn(lf, &c.at, li)) < 0) return -1;
        const AttnCfg& a = c.at;
        if (a.bias_max > 0 && a.rel_rows == 0) c.at.rel_rows = -1;   // known once the bias table's tensor is
        SsmCfg& s = c.sm;
        s.heads = geti(rt, "heads", 0);
        s.vdim = geti(rt, "vdim", 0);
        s.state = geti(rt, "state", 0);
        s.groups = geti(rt, "groups", 1);
        s.norm_groups = geti(rt, "norm_groups", 1);
        s.taps = geti(rt, "conv", 1);
        if (s.heads <= 0 || s.vdim <= 0 || s.state <= 0 || s.state > 256 || s.groups <= 0 || s.heads % s.groups || s.norm_groups <= 0 ||
            s.inner() % s.norm_groups || s.taps < 1 || s.taps > 64)
          return set_error("config: unsupported state-space sizes in layer " + li);
        c.o_q = 0;
        c.o_k = a.heads * a.dim;
        c.o_v = c.o_k + a.kv * a.dim;
        c.qkv_ch = c.o_v + a.kv * a.vdim;
        c.o_g = pad8(c.qkv_ch);
        c.o_in = pad8(c.o_g + a.heads);
        c.o_ffg = pad8(c.o_in + s.in_rows());
      } else {
        return set_error("config: layer " + li + " has an unknown mixer type");
      }
      c.o_ffu = pad8(c.o_ffg + c.ff);
      c.proj_rows = pad8(c.o_ffu + c.ff);
      layers.push_back(c);
    }
    const int L = (int)layers.size();
    if (const Json* lp = j.get("loop")) {
      if (lp->kind == Json::Obj) {
        loop_start = geti(lp, "start", 0);
        loop_stop = geti(lp, "stop", 0);
        loop_times = geti(lp, "times", 1);
        if (loop_start < 0 || loop_stop < loop_start || loop_stop > L || loop_times < 1 || loop_times > 4096)
          return set_error("config: loop outside the layers");
        has_loop = loop_stop > loop_start;
      }
    }
    // layer runs; every run reserves its state parts and its part of a cache page
    int64_t off = 0;
    auto add_run = [&](int layer, int pass) {
      const LayerCfg& c = layers[(size_t)layer];
      Run r;
      r.layer = layer;
      r.pass = pass;
      const std::string tag = "run" + std::to_string(runs.size());
      if (c.type == kAttention && c.at.taps > 1) r.st_conv = state_layout.reserve(tag + ".conv", (int64_t)(c.at.taps - 1) * c.qkv_ch);
      if (c.type == kParallel) {
        r.st_sconv = state_layout.reserve(tag + ".ssm_conv", (int64_t)(c.sm.taps - 1) * c.sm.conv_ch());
        r.st_mem = state_layout.reserve(tag + ".ssm_state", (int64_t)c.sm.heads * c.sm.state * c.sm.vdim);
      }
      r.k_off = off;
      r.v_off = off + (int64_t)kPageSize * c.at.kv * c.at.dim;
      off = r.v_off + (int64_t)kPageSize * c.at.kv * c.at.vdim;
      runs.push_back(r);
    };
    for (int i = 0; i < (has_loop ? loop_start : L); ++i) add_run(i, -1);
    if (has_loop) {
      for (int t = 0; t < loop_times; ++t)
        for (int i = loop_start; i < loop_stop; ++i) add_run(i, i == loop_start ? t : -1);
      for (int i = loop_stop; i < L; ++i) add_run(i, -1);
    }
    page_stride = std::max<int64_t>(off, 1);
    weights.resize(layers.size());
    for (auto& c : layers) {
      mx_proj = std::max(mx_proj, c.proj_rows);
      mx_mix = std::max(mx_mix, c.at.heads * c.at.vdim);
      mx_q = std::max(mx_q, c.at.heads * c.at.dim);
      mx_vdim = std::max(mx_vdim, c.at.vdim);
      mx_ff = std::max(mx_ff, c.ff);
      if (c.type == kAttention) mx_conv = std::max(mx_conv, c.qkv_ch);
      if (c.type == kParallel) {
        mx_conv = std::max(mx_conv, c.sm.conv_ch());
        mx_inner = std::max(mx_inner, c.sm.inner());
      }
    }
    return 0;
  }

  // ------------------------------------------------------------------ device memory
  template <typename T>
  int dalloc(T** p, size_t count, std::vector<void*>* into = nullptr) {
    void* raw = nullptr;
    KK_HIP(hipMalloc(&raw, std::max<size_t>(count, 1) * sizeof(T)));
    KK_HIP(hipMemset(raw, 0, std::max<size_t>(count, 1) * sizeof(T)));
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
    KK_HIP(hipSetDevice(device));
    cublas_init();
    KK_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    KK_HIP(hipEventCreate(&ev0));
    KK_HIP(hipEventCreate(&ev1));
    num_pages = std::max(1, (max_tokens + kPageSize - 1) / kPageSize);
    pool = PagePool(num_pages);
    requests.assign((size_t)max_requests, KvState());
    if (dalloc_a(&cache, (size_t)num_pages * (size_t)page_stride)) return -1;
    if (dalloc(&state, (size_t)max_requests * (size_t)std::max<int64_t>(1, state_layout.floats_per_slot()))) return -1;
    if (dalloc(&probs_scratch, (size_t)V) || dalloc(&top1_value, 1) || dalloc(&row_states, 1024 * 1024) ||
        dalloc(&valid_scratch, 1) || dalloc(&sample_out_d, 1))
      return -1;
    return 0;
  }

  // ------------------------------------------------------------------ weights
  typedef std::vector<std::pair<std::string, std::vector<int64_t>>> TensorList;
  TensorList tensor_list() const {
    TensorList out;
    out.push_back({"embed", {V, D}});
    if (has_loop) out.push_back({"loop.in", {D, 2 * D}});
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      const AttnCfg& a = c.at;
      const std::string p = "l" + std::to_string(i), m = p + ".mix";
      out.push_back({p + ".norm1", {D}});
      const std::string am = c.type == kParallel ? m + ".left" : m;
      out.push_back({am + ".q", {a.heads * a.dim, D}});
      out.push_back({am + ".q.b", {a.heads * a.dim}});
      out.push_back({am + ".k", {a.kv * a.dim, D}});
      out.push_back({am + ".k.b", {a.kv * a.dim}});
      out.push_back({am + ".v", {a.kv * a.vdim, D}});
      out.push_back({am + ".v.b", {a.kv * a.vdim}});
      out.push_back({am + ".o", {D, a.heads * a.vdim}});
      if (c.type == kAttention) {
        if (a.taps > 0) {
          out.push_back({am + ".q.conv", {a.heads * a.dim, a.taps}});
          out.push_back({am + ".k.conv", {a.kv * a.dim, a.taps}});
          out.push_back({am + ".v.conv", {a.kv * a.vdim, a.taps}});
        }
        out.push_back({am + ".g", {a.heads * a.vdim, D}});
      } else {
        const SsmCfg& s = c.sm;
        const std::string r = m + ".right";
        out.push_back({am + ".o.b", {D}});
        out.push_back({am + ".q.norm", {a.heads * a.dim}});
        out.push_back({am + ".k.norm", {a.kv * a.dim}});
        if (a.bias_max > 0) out.push_back({am + ".rel", {a.rel_rows, a.heads}});
        out.push_back({am + ".g", {a.heads, D}});
        out.push_back({r + ".in", {s.in_rows(), D}});
        out.push_back({r + ".conv", {s.conv_ch(), s.taps}});
        out.push_back({r + ".conv.b", {s.conv_ch()}});
        out.push_back({r + ".dt_bias", {s.heads}});
        out.push_back({r + ".A_log", {s.heads}});
        out.push_back({r + ".D", {s.heads}});
        out.push_back({r + ".norm", {s.inner()}});
        out.push_back({r + ".o", {D, s.inner()}});
        out.push_back({m + ".left.out", {D}});
        out.push_back({m + ".right.out", {D}});
      }
      if (c.ff > 0) {
        out.push_back({p + ".mlp.gate", {c.ff, D}});
        out.push_back({p + ".mlp.up", {c.ff, D}});
        out.push_back({p + ".mlp.down", {D, c.ff}});
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
  // bucket counts that the configuration does not name, from the sizes of the staged bias tables ([buckets, heads])
  void rel_rows_from_staged() {
    for (size_t i = 0; i < layers.size(); ++i) {
      AttnCfg& a = layers[i].at;
      if (layers[i].type != kParallel || a.bias_max <= 0 || a.rel_rows > 0) continue;
      auto it = staged.find("l" + std::to_string(i) + ".mix.left.rel");
      if (it != staged.end() && it->second.size() % (size_t)a.heads == 0) a.rel_rows = (int)(it->second.size() / (size_t)a.heads);
    }
  }
  int fill_synthetic(uint64_t seed, float std) {
    for (auto& c : layers)
      if (c.type == kParallel && c.at.bias_max > 0 && c.at.rel_rows <= 0) c.at.rel_rows = 32;
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
      const bool is_conv = ends_with(n, ".conv");
      const bool is_gain = ends_with(n, ".norm1") || ends_with(n, ".norm") || ends_with(n, ".out") || n == "final.norm";
      const bool is_bias = ends_with(n, ".b");
      for (size_t k = 0; k < v.size(); ++k) {
        const float z = g();
        float val = std * z;
        if (is_conv) val = 0.4f * z;
        else if (is_gain) val = 1.0f + 0.1f * z;
        else if (is_bias) val = 0.1f * z;
        else if (ends_with(n, ".rel")) val = 0.5f * z;
        else if (ends_with(n, ".A_log")) val = -0.5f + 0.5f * z;
        else if (ends_with(n, ".dt_bias")) val = -1.0f + 0.5f * z;
        else if (ends_with(n, ".D")) val = 1.0f + 0.2f * z;
        else if (n == "loop.in") val = (k / (size_t)(2 * D) == k % (size_t)(2 * D) ? 1.0f : 0.f) + std * z;   // near [I | 0]
        v[k] = host_f2bf(val);
      }
    }
    return 0;
  }
  int upload(void** out, const uint16_t* bits, size_t n) {
    if (dalloc_a(out, n)) return -1;
    if (dtype == PEGAINFER_DTYPE_BF16) {
      KK_HIP(hipMemcpy(*out, bits, n * 2, hipMemcpyHostToDevice));
    } else {
      std::vector<float> f(n);
      for (size_t i = 0; i < n; ++i) f[i] = host_bf2f(bits[i]);
      KK_HIP(hipMemcpy(*out, f.data(), n * 4, hipMemcpyHostToDevice));
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
  // [rows_i, cols] tensors stacked by rows, each part's first row at the given row of the stack (zero rows between and after)
  struct Part { std::string name; int64_t rows, at; };
  int up_stacked(void** out, const std::vector<Part>& parts, int64_t cols, int64_t total_rows) {
    std::vector<uint16_t> st((size_t)(total_rows * cols), 0);
    for (auto& p : parts) {
      const auto* v = need(p.name, p.rows * cols);
      if (!v) return -1;
      std::memcpy(&st[(size_t)(p.at * cols)], v->data(), v->size() * 2);
    }
    return upload(out, st.data(), st.size());
  }
  // rotation frequencies base^(-2i/dims), with the long-context scaling by wavelength: short waves stay, long waves are
  // slowed by `factor`, those between are blended; rounded once to fp32
  std::vector<float> frequencies(const AttnCfg& a) const {
    const int half = a.rot_dims / 2;
    const double two_pi = 6.283185307179586476925286766559;
    std::vector<float> f((size_t)std::max(1, half));
    for (int k = 0; k < half; ++k) {
      double fk = std::pow(a.base, -2.0 * k / (double)a.rot_dims);
      if (a.scaled) {
        const double wave = two_pi / fk;
        if (wave > a.sc_orig / a.sc_low) {
          fk = fk / a.sc_factor;
        } else if (!(wave < a.sc_orig / a.sc_high)) {
          const double s = (a.sc_orig / wave - a.sc_low) / (a.sc_high - a.sc_low);
          fk = (1.0 - s) * fk / a.sc_factor + s * fk;
        }
      }
      f[k] = (float)fk;
    }
    return f;
  }
  // bucket of a distance: one bucket per distance below half the table, logarithmic steps up to bias_max above it
  static int distance_bucket(int n, int rows, int far) {
    const int hb = rows / 2;
    if (n < hb) return n;
    const double v = std::log((double)n / hb) / std::log((double)far / hb) * (double)(rows - hb);
    return std::min(rows - 1, hb + (int)std::floor(v));
  }
  int finalize() {
    if (finalized) return 0;
    rel_rows_from_staged();
    if (up(&embed, "embed", (int64_t)V * D) || up(&final_norm, "final.norm", D)) return -1;
    if (has_loop && up(&loop_in, "loop.in", (int64_t)2 * D * D)) return -1;
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      const AttnCfg& a = c.at;
      LayerW& w = weights[i];
      const std::string p = "l" + std::to_string(i), m = p + ".mix";
      const std::string am = c.type == kParallel ? m + ".left" : m;
      const int64_t qn = (int64_t)a.heads * a.dim, kn = (int64_t)a.kv * a.dim, vn = (int64_t)a.kv * a.vdim, on = (int64_t)a.heads * a.vdim;
      if (up(&w.norm1, p + ".norm1", D)) return -1;
      std::vector<Part> parts{{am + ".q", qn, c.o_q}, {am + ".k", kn, c.o_k}, {am + ".v", vn, c.o_v}};
      if (c.type == kAttention) {
        parts.push_back({am + ".g", on, c.o_g});
      } else {
        parts.push_back({am + ".g", a.heads, c.o_g});
        parts.push_back({m + ".right.in", c.sm.in_rows(), c.o_in});
      }
      if (c.ff > 0) {
        parts.push_back({p + ".mlp.gate", c.ff, c.o_ffg});
        parts.push_back({p + ".mlp.up", c.ff, c.o_ffu});
      }
      if (up_stacked(&w.proj, parts, D, c.proj_rows) || up(&w.o, am + ".o", (int64_t)D * on)) return -1;
      if (up_stacked(&w.qkv_bias, {{am + ".q.b", qn, c.o_q}, {am + ".k.b", kn, c.o_k}, {am + ".v.b", vn, c.o_v}}, 1, c.qkv_ch)) return -1;
      if (c.ff > 0 && up(&w.down, p + ".mlp.down", (int64_t)D * c.ff)) return -1;
      if (c.type == kAttention) {
        if (a.taps > 0 &&
            up_stacked(&w.conv, {{am + ".q.conv", qn, c.o_q}, {am + ".k.conv", kn, c.o_k}, {am + ".v.conv", vn, c.o_v}}, a.taps, c.qkv_ch))
          return -1;
      } else {
        const SsmCfg& s = c.sm;
        const std::string r = m + ".right";
        if (up(&w.o_bias, am + ".o.b", D) || up(&w.q_norm, am + ".q.norm", qn) || up(&w.k_norm, am + ".k.norm", kn) ||
            up(&w.left_out, m + ".left.out", D) || up(&w.right_out, m + ".right.out", D) ||
            up(&w.sconv, r + ".conv", (int64_t)s.conv_ch() * s.taps) || up(&w.sconv_b, r + ".conv.b", s.conv_ch()) ||
            up(&w.dt_bias, r + ".dt_bias", s.heads) || up(&w.A_log, r + ".A_log", s.heads) || up(&w.Dskip, r + ".D", s.heads) ||
            up(&w.snorm, r + ".norm", s.inner()) || up(&w.ro, r + ".o", (int64_t)D * s.inner()))
          return -1;
        if (a.bias_max > 0) {
          // the learned bias, one row per distance up to the distance from which the bucket no longer changes
          const int rows = a.rel_rows;
          if (rows < 2 || a.bias_max <= rows / 2) return set_error("layer " + std::to_string(i) + ": bias_max must exceed half the bias table's rows");
          const auto* rel = need(am + ".rel", (int64_t)rows * a.heads);
          if (!rel) return -1;
          int nd = 1;
          while (nd < (1 << 24) && distance_bucket(nd - 1, rows, a.bias_max) < rows - 1) ++nd;
          std::vector<float> tab((size_t)nd * a.heads);
          for (int n = 0; n < nd; ++n)
            for (int h = 0; h < a.heads; ++h) tab[(size_t)n * a.heads + h] = host_bf2f((*rel)[(size_t)distance_bucket(n, rows, a.bias_max) * a.heads + h]);
          if (dalloc(&w.dist_bias, tab.size())) return -1;
          KK_HIP(hipMemcpy(w.dist_bias, tab.data(), tab.size() * 4, hipMemcpyHostToDevice));
          w.n_dist = nd;
        }
      }
      if (a.rot_dims > 0) {
        const std::vector<float> f = frequencies(a);
        if (dalloc(&w.inv_freq, f.size())) return -1;
        KK_HIP(hipMemcpy(w.inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice));
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
    for (size_t i = 0; i < layers.size(); ++i) {   // bucket counts = first sizes of the bias tables
      AttnCfg& a = layers[i].at;
      if (layers[i].type != kParallel || a.bias_max <= 0) continue;
      const pst::TensorView* r = ck.find("l" + std::to_string(i) + ".mix.left.rel");
      if (!r || r->shape.size() != 2) return set_error("checkpoint has no bias table for layer " + std::to_string(i));
      a.rel_rows = (int)r->shape[0];
    }
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
        for (size_t k = 0; k < dst.size(); ++k) dst[k] = host_f2bf(f[k]);
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
        // the slot's state region starts from zero: empty convolution tails, empty memories
        if (n) KK_HIP(hipMemsetAsync(state + i * n, 0, n * sizeof(float), stream));
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
    KK_HIP(hipStreamSynchronize(stream));
    drop_graphs();
    free_all(&step_owned);
    cap_rows = 0;
    size_t n = 64;
    while (n < T) n *= 2;
    auto* so = &step_owned;
    if (dalloc(&x, n * D, so) || dalloc(&emb, n * D, so) || dalloc(&xcat, has_loop ? n * 2 * D : 1, so) ||
        dalloc(&conv32, n * (size_t)std::max(1, mx_conv), so) || dalloc(&q32, n * (size_t)std::max(1, mx_q), so) ||
        dalloc(&o32, n * (size_t)std::max(1, mx_inner), so) || dalloc_a(&hb, n * D, so) || dalloc_a(&proj, n * (size_t)mx_proj, so) ||
        dalloc_a(&mix, n * (size_t)mx_mix, so) || dalloc_a(&mixr, n * (size_t)std::max(1, mx_inner), so) || dalloc_a(&y1, n * D, so) ||
        dalloc_a(&y2, n * D, so) || dalloc_a(&y3, n * D, so) || dalloc_a(&act, n * (size_t)std::max(1, mx_ff), so) ||
        dalloc(&att_part, (size_t)kSplitGroups * kAttRows * (size_t)(mx_vdim + 2), so))
      return -1;
    cap_rows = n;
    return 0;
  }
  int ensure_want(size_t n) {
    if (n <= cap_want) return 0;
    KK_HIP(hipStreamSynchronize(stream));
    drop_graphs();
    free_all(&want_owned);
    cap_want = 0;
    size_t c = 16;
    while (c < n) c *= 2;
    auto* wo = &want_owned;
    if (dalloc(&xw, c * D, wo) || dalloc(&hw, c * D, wo) || dalloc(&logits32, c * V, wo) || dalloc(&logits16, c * V, wo) ||
        dalloc(&tokens_d, c, wo) || dalloc(&top1_state, c * 16, wo))
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
    KK_K(pegainfer_gemm_strided(&d, S()));
    return 0;
  }
  // Y[T, M] (y_dtype, row stride M) = X[T, K] (x_dtype, row stride x_stride) W[M, K]^T: the strided GEMM, for operands that are
  // columns of a wider matrix or outputs that stay in fp32
  int linear_strided(const void* W, const void* X, int x_dtype, int64_t x_stride, void* Y, int y_dtype, int M, int T, int K) {
    pegainfer_gemm_desc d{};
    d.x = X; d.w = W; d.y = Y;
    d.x_dtype = x_dtype; d.w_dtype = dtype; d.y_dtype = y_dtype;
    d.m = M; d.k = K; d.rows = T; d.groups = 1;
    d.x_row_stride = x_stride; d.w_m_stride = K; d.w_k_stride = 1; d.y_row_stride = M;
    d.plain = plain_kernels;
    KK_K(pegainfer_gemm_strided(&d, S()));
    return 0;
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
    //   tokens | positions | row_entry | entry_row0 | entry_slot | page_indptr | want | attention tile sets | page_ids
    // An attention tile is a run of token rows of one entry times a run of the query heads of one key/value head, at most
    // 16 rows in all; one set of tiles per distinct heads-per-kv-head value of the model's attention layers.
    bool single = true;   // every entry brings one token: decoding
    for (int i = 0; i < n && single; ++i) single = lens[i] == 1;
    const size_t o_tok = 0, o_pos = o_tok + T, o_ent = o_pos + T, o_row0 = o_ent + T, o_slot = o_row0 + (size_t)n + 1,
                 o_ind = o_slot + (size_t)n, o_want = o_ind + (size_t)n + 1;
    size_t words = o_want + (size_t)std::max(1, W);   // the page lists come last: everything before them sits at offsets that
                                                      // depend on the step's shape only, which a captured graph relies on
    std::vector<size_t> tile_off(tile_sets.size()), tile_cnt(tile_sets.size());
    for (size_t k = 0; k < tile_sets.size(); ++k) {
      const int per = tile_sets[k];
      size_t cnt = 0;
      for (int i = 0; i < n; ++i)
        cnt += per <= kAttRows ? ((size_t)lens[i] + (kAttRows / per) - 1) / (kAttRows / per) : (size_t)lens[i] * ((per + kAttRows - 1) / kAttRows);
      tile_off[k] = words;
      tile_cnt[k] = cnt;
      words += 4 * cnt;
    }
    const size_t o_pages = words;
    words += total_pages;
    if (words > cap_meta) {
      KK_HIP(hipStreamSynchronize(stream));
      if (meta_host) (void)hipHostFree(meta_host);
      if (meta_dev) (void)hipFree(meta_dev);
      meta_host = meta_dev = nullptr;
      cap_meta = 0;
      size_t c = 4096;
      while (c < words) c *= 2;
      KK_HIP(hipHostMalloc(reinterpret_cast<void**>(&meta_host), c * 4, hipHostMallocDefault));
      KK_HIP(hipMalloc(reinterpret_cast<void**>(&meta_dev), c * 4));
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
        for (int32_t p : st.pages) mh[o_pages + pg++] = p;
        for (int k = 0; k < lens[i]; ++k, ++t) {
          mh[o_tok + t] = (int32_t)tokens[t];
          mh[o_pos + t] = st.seq_len + k;
          mh[o_ent + t] = i;
        }
      }
      mh[o_row0 + n] = (int32_t)t;
      mh[o_ind + n] = (int32_t)pg;
      for (int i = 0; i < W; ++i) mh[o_want + i] = want[i];
      for (size_t k = 0; k < tile_sets.size(); ++k) {
        const int per = tile_sets[k];
        int32_t *t_row0 = mh + tile_off[k], *t_ntok = t_row0 + tile_cnt[k], *t_qh0 = t_ntok + tile_cnt[k], *t_nqh = t_qh0 + tile_cnt[k];
        size_t at_ = 0, r0 = 0;
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
    KK_HIP(hipEventRecord(ev0, stream));
    KK_HIP(hipMemcpyAsync(meta_dev, meta_host, words * 4, hipMemcpyHostToDevice, stream));
    const int32_t* md = reinterpret_cast<const int32_t*>(meta_dev);
    const uint32_t* d_tok = reinterpret_cast<const uint32_t*>(md + o_tok);
    const int32_t *d_pos = md + o_pos, *d_ent = md + o_ent, *d_row0 = md + o_row0, *d_slot = md + o_slot, *d_ind = md + o_ind,
                  *d_want = md + o_want, *d_pages = md + o_pages;
    const int Ti = (int)T;
    const int64_t slot_stride = state_layout.floats_per_slot();
    if (tap_on) {
      const size_t needf = runs.size() * T * D;
      if (needf > tap_cap) {
        KK_HIP(hipStreamSynchronize(stream));
        if (tap) (void)hipFree(tap);
        tap = nullptr;
        tap_cap = 0;
        KK_HIP(hipMalloc(reinterpret_cast<void**>(&tap), needf * 4));
        tap_cap = needf;
      }
      tap_rows = Ti;
    }
    // ---- the layer runs (everything below reads the step's shape from its arguments and the step's contents from the
    //      metadata block, so a launch sequence recorded for one decode step serves every later step of the same shape)
    // time convolution of some columns of `proj` into fp32, with the request's tail moved on
    auto conv = [&](const void* in, const void* w, const void* in_bias, const void* out_bias, int64_t st_off, int ch, int taps,
                    int mode) -> int {
      float* tail = state + st_off;   // taps == 1: never touched
      if (single) {
        KK_K(pegainfer_time_conv_step_biased(in, dtype, proj_stride, w, dtype, in_bias, out_bias, tail, slot_stride, conv32,
                                             PEGAINFER_DTYPE_F32, ch, ch, taps, mode, d_slot, n, S()));
        return 0;
      }
      KK_K(pegainfer_time_conv_biased(in, dtype, proj_stride, w, dtype, in_bias, out_bias, tail, slot_stride, conv32, PEGAINFER_DTYPE_F32, ch,
                                      ch, taps, mode, d_ent, d_row0, d_slot, Ti, S()));
      KK_K(pegainfer_time_conv_commit_biased(in, dtype, proj_stride, in_bias, dtype, tail, slot_stride, ch, taps, d_row0, d_slot, n, S()));
      return 0;
    };
    auto attention = [&](const LayerCfg& c, const LayerW& w, const Run& r, const void* gate, int gate_kind) -> int {
      const AttnCfg& a = c.at;
      const size_t ts = (size_t)c.tile_set;
      const int32_t* tb = md + tile_off[ts];
      // a step of few rows (decoding, short portions) cannot fill the chip with one workgroup per (row tile, kv head): its
      // keys are dealt to several workgroups.  The count depends on the step's shape only, never on the contexts' lengths.
      const int wgs = (int)tile_cnt[ts] * a.kv;
      const int nsplit = wgs >= 128 ? 1 : std::max(1, std::min(kMaxSplits, kSplitGroups / wgs));
      KK_K(pegainfer_paged_attention_masked(q32, cache, page_stride, r.k_off, r.v_off, kPageSize, d_pos, d_ent, d_ind, d_pages, a.heads,
                                            a.kv, a.dim, a.vdim, a.scale, 1.0f, tb, tb + tile_cnt[ts], tb + 2 * tile_cnt[ts],
                                            tb + 3 * tile_cnt[ts], (int)tile_cnt[ts], mix, a.heads * a.vdim, 1, 0.f, 0, nullptr, 0, 0.f,
                                            a.softcap, a.window, a.keep_first, w.dist_bias, w.n_dist, gate, proj_stride, gate_kind, nsplit,
                                            att_part, plain_kernels ? 1 : 0, dtype, S()));
      return 0;
    };
    auto run_layers = [&]() -> int {
    KK_K(pegainfer_embed_f32(embed, d_tok, x, D, Ti, dtype, S()));
    if (has_loop) KK_K(pegainfer_scale_rows(x, D, xcat + D, 2 * D, D, Ti, 1.0f, PEGAINFER_DTYPE_F32, S()));
    for (size_t ri = 0; ri < runs.size(); ++ri) {
      const Run& r = runs[ri];
      const LayerCfg& c = layers[(size_t)r.layer];
      const LayerW& w = weights[(size_t)r.layer];
      const AttnCfg& a = c.at;
      proj_stride = c.proj_rows;
      if (r.pass >= 0) {
        // a pass over the repeated span begins: the stream is mixed with the embedding rows again
        KK_K(pegainfer_scale_rows(x, D, xcat, 2 * D, D, Ti, 1.0f, PEGAINFER_DTYPE_F32, S()));
        if (linear_strided(loop_in, xcat, PEGAINFER_DTYPE_F32, 2 * D, x, PEGAINFER_DTYPE_F32, D, Ti, 2 * D)) return -1;
      }
      if (r.pass >= 0 || ri == 0)   // otherwise the launch that closed the run before has left hb
        KK_K(pegainfer_terms_rms_add(x, nullptr, 0, nullptr, w.norm1, eps, hb, dtype, D, Ti, dtype, S()));
      if (linear(w.proj, hb, proj, c.proj_rows, Ti, D)) return -1;
      pegainfer_sum_term terms[3];
      int n_terms = 0;
      if (c.type == kAttention) {
        const void* qkv = proj;
        int qkv_dtype = dtype;
        int64_t qkv_stride = c.proj_rows;
        const void* bias = w.qkv_bias;
        if (a.taps > 0) {   // biases join the inputs of the convolution; what it leaves is fp32
          if (conv(proj, w.conv, w.qkv_bias, nullptr, r.st_conv, c.qkv_ch, a.taps, 0)) return -1;
          qkv = conv32; qkv_dtype = PEGAINFER_DTYPE_F32; qkv_stride = c.qkv_ch; bias = nullptr;
        }
        KK_K(pegainfer_qk_prep_paged_form(qkv, qkv_dtype, qkv_stride, c.o_q, c.o_k, c.o_v, a.heads, a.kv, a.dim, a.vdim, nullptr, nullptr,
                                          PEGAINFER_QKNORM_HEAD_UNIT_AFTER, eps, bias, bias ? at(bias, (size_t)c.o_k) : nullptr,
                                          bias ? at(bias, (size_t)c.o_v) : nullptr, 0.f, 0, w.inv_freq, a.rot_dims, PEGAINFER_ROT_HALVES,
                                          d_pos, d_ent, d_ind, d_pages, cache, page_stride, r.k_off, r.v_off, kPageSize, q32, nullptr, Ti,
                                          dtype, S()));
        if (attention(c, w, r, at(proj, (size_t)c.o_g), PEGAINFER_GATE_PER_VALUE)) return -1;
        if (linear(w.o, mix, y1, D, Ti, a.heads * a.vdim)) return -1;
        terms[n_terms++] = pegainfer_sum_term{y1, D, nullptr, nullptr, 1.0f};
      } else {
        const SsmCfg& s = c.sm;
        // left: attention over a window and the kept first tokens, a bias by distance, a gate per head
        KK_K(pegainfer_qk_prep_paged_form(proj, dtype, c.proj_rows, c.o_q, c.o_k, c.o_v, a.heads, a.kv, a.dim, a.vdim, w.q_norm, w.k_norm,
                                          PEGAINFER_QKNORM_ALL_WEIGHT, eps, w.qkv_bias, at(w.qkv_bias, (size_t)c.o_k),
                                          at(w.qkv_bias, (size_t)c.o_v), 0.f, 0, w.inv_freq, a.rot_dims, PEGAINFER_ROT_HALVES, d_pos, d_ent,
                                          d_ind, d_pages, cache, page_stride, r.k_off, r.v_off, kPageSize, q32, nullptr, Ti, dtype, S()));
        if (attention(c, w, r, at(proj, (size_t)c.o_g), PEGAINFER_GATE_PER_HEAD)) return -1;
        if (linear(w.o, mix, y1, D, Ti, a.heads * a.vdim)) return -1;
        // right: [z | x | B | C | dt] at o_in; x | B | C through the convolution, the scan, y * silu(z) normed in groups
        const int inner = s.inner();
        if (conv(at(proj, (size_t)(c.o_in + inner)), w.sconv, nullptr, w.sconv_b, r.st_sconv, s.conv_ch(), s.taps, 2)) return -1;
        KK_K(pegainfer_ssd_scan(conv32, s.conv_ch(), proj, c.proj_rows, c.o_in + 2 * inner + 2 * s.groups * s.state, w.A_log, w.dt_bias,
                                w.Dskip, state + r.st_mem, slot_stride, o32, s.heads, s.groups, s.state, s.vdim, d_row0, d_slot, n, dtype,
                                S()));
        KK_K(pegainfer_head_gate_rms(o32, w.snorm, 1, at(proj, (size_t)c.o_in), c.proj_rows, 0, 1, 1.0f, eps, mixr, inner, s.norm_groups,
                                     inner / s.norm_groups, Ti, dtype, S()));
        if (linear(w.ro, mixr, y2, D, Ti, inner)) return -1;
        terms[n_terms++] = pegainfer_sum_term{y1, D, w.o_bias, w.left_out, 0.5f};
        terms[n_terms++] = pegainfer_sum_term{y2, D, nullptr, w.right_out, 0.5f};
      }
      if (c.ff > 0) {
        KK_K(pegainfer_glu_rows(at(proj, (size_t)c.o_ffg), at(proj, (size_t)c.o_ffu), c.proj_rows, act, c.ff, c.ff, Ti, PEGAINFER_ACT_RELU,
                                dtype, S()));
        if (linear(w.down, act, y3, D, Ti, c.ff)) return -1;
        terms[n_terms++] = pegainfer_sum_term{y3, D, nullptr, nullptr, 1.0f};
      }
      // the closing launch also norms for the next run, unless that run opens a pass (its input projection comes first) or
      // there is none (the final norm runs on the wanted rows only)
      const bool next_plain = ri + 1 < runs.size() && runs[ri + 1].pass < 0;
      KK_K(pegainfer_terms_rms_add(x, terms, n_terms, x, next_plain ? weights[(size_t)runs[ri + 1].layer].norm1 : nullptr, eps,
                                   next_plain ? hb : nullptr, dtype, D, Ti, dtype, S()));
      if (tap_on) KK_HIP(hipMemcpyAsync(tap + ri * T * D, x, T * D * 4, hipMemcpyDeviceToDevice, stream));
    }
    // ---- wanted rows: final norm, logits over the embedding table in fp32, the soft cap
    if (W > 0) {
      KK_K(pegainfer_gather_rows_f32(x, d_want, xw, D, W, S()));
      KK_K(pegainfer_terms_rms_add(xw, nullptr, 0, nullptr, final_norm, eps, hw, PEGAINFER_DTYPE_F32, D, W, dtype, S()));
      if (linear_strided(embed, hw, PEGAINFER_DTYPE_F32, D, logits32, PEGAINFER_DTYPE_F32, V, W, D)) return -1;
      if (logit_cap > 0.f) KK_K(pegainfer_softcap_rows(logits32, logits32, (int64_t)W * V, logit_cap, S()));
      KK_K(deepseek_f32_to_bf16_cuda(logits32, logits16, W * V, S()));
      if (out_tokens) KK_K(pegainfer_batched_top1(logits16, V, W, V, top1_state, tokens_d, S()));
    }
    return 0;
    };
    // a step of single tokens only (decoding) is launch-bound: its launches are captured once per shape as a hipGraph and
    // replayed; steps with prompt portions run eagerly
    if (single && graphs_on && !tap_on) {
      const GraphKey key{n, W, out_tokens != nullptr, plain_kernels};
      hipGraphExec_t exec = nullptr;
      for (auto& g : graphs)
        if (g.first == key) exec = g.second;
      if (!exec) {
        hipGraph_t g = nullptr;
        KK_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        const int rc = run_layers();
        const hipError_t e = hipStreamEndCapture(stream, &g);
        if (rc) return -1;
        if (e != hipSuccess) return set_error("graph capture failed");
        KK_HIP(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
        KK_HIP(hipGraphDestroy(g));
        graphs.emplace_back(key, exec);
      }
      KK_HIP(hipGraphLaunch(exec, stream));
    } else if (run_layers()) {
      return -1;
    }
    last_rows = W;
    KK_HIP(hipEventRecord(ev1, stream));
    if (W > 0 && out_logits) KK_HIP(hipMemcpyAsync(out_logits, logits32, (size_t)W * V * 4, hipMemcpyDeviceToHost, stream));
    if (W > 0 && out_tokens) KK_HIP(hipMemcpyAsync(out_tokens, tokens_d, (size_t)W * 4, hipMemcpyDeviceToHost, stream));
    KK_HIP(hipStreamSynchronize(stream));
    (void)hipEventElapsedTime(&last_step_ms, ev0, ev1);
    for (int i = 0; i < n; ++i) requests[ids[i]].seq_len += lens[i];
    return 0;
  }
  int64_t proj_stride = 0;   // row stride of `proj` in the layer run at hand

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
    KK_HIP(hipStreamSynchronize(stream));
    KK_HIP(hipMemcpy(out, sample_out_d, 4, hipMemcpyDeviceToHost));
    return 0;
  }
  int logprobs(int row, uint32_t token, int top_k, float* out_lp, uint32_t* top_ids, float* top_lps) {
    if (row < 0 || row >= last_rows) return set_error("no logits for that row");
    if (token >= (uint32_t)V) return set_error("logprobs: token outside the vocabulary");
    lp_row.resize((size_t)V);
    KK_HIP(hipStreamSynchronize(stream));
    KK_HIP(hipMemcpy(lp_row.data(), logits32 + (size_t)row * V, (size_t)V * 4, hipMemcpyDeviceToHost));
    return pegainfer_logprobs_from_logits(lp_row.data(), V, token, top_k, out_lp, top_ids, top_lps);
  }
  int debug_hidden(int run, float* out, int max_rows) {
    if (!tap || run < 0 || run >= (int)runs.size()) return set_error("debug_hidden: no tap for that layer run");
    const int rows = std::min(max_rows, tap_rows);
    KK_HIP(hipStreamSynchronize(stream));
    KK_HIP(hipMemcpy(out, tap + (size_t)run * tap_rows * D, (size_t)rows * D * 4, hipMemcpyDeviceToHost));
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
static Model* M(pegainfer_kukulorn_t m) { return static_cast<Model*>(m); }

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

}  // namespace pkk

extern "C" {
using pkk::M;

pegainfer_kukulorn_t pegainfer_kukulorn_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests) {
  if (!config_json) { pkk::g_create_error = "no configuration"; return nullptr; }
  return pkk::create(config_json, device_ordinal, dtype, max_tokens, max_requests);
}
pegainfer_kukulorn_t pegainfer_kukulorn_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests) {
  std::string e;
  auto f = pst::MappedFile::open(std::string(model_dir) + "/config.json", &e);
  if (!f) { pkk::g_create_error = e; return nullptr; }
  pkk::Model* m = pkk::create(std::string(reinterpret_cast<const char*>(f->data), f->size), device_ordinal, dtype, max_tokens, max_requests);
  if (!m) return nullptr;
  if (m->load_checkpoint(model_dir)) {
    pkk::g_create_error = m->err;
    delete m;
    return nullptr;
  }
  return m;
}
void pegainfer_kukulorn_destroy(pegainfer_kukulorn_t m) { delete M(m); }
const char* pegainfer_kukulorn_last_error(pegainfer_kukulorn_t m) { return m ? M(m)->err.c_str() : pkk::g_create_error.c_str(); }
int32_t pegainfer_kukulorn_load_tensor(pegainfer_kukulorn_t m, const char* name, const void* host_bf16, int64_t numel) {
  return M(m)->load_tensor(name, static_cast<const uint16_t*>(host_bf16), numel);
}
int32_t pegainfer_kukulorn_fill_synthetic(pegainfer_kukulorn_t m, uint64_t seed, float std) { return M(m)->fill_synthetic(seed, std); }
int32_t pegainfer_kukulorn_finalize(pegainfer_kukulorn_t m) { return M(m)->finalize(); }
int32_t pegainfer_kukulorn_new_request(pegainfer_kukulorn_t m) { return M(m)->new_request(); }
int32_t pegainfer_kukulorn_drop_request(pegainfer_kukulorn_t m, int32_t id) { return M(m)->drop_request(id); }
int32_t pegainfer_kukulorn_request_seq_len(pegainfer_kukulorn_t m, int32_t id) {
  if (id < 0 || id >= (int)M(m)->requests.size() || !M(m)->requests[id].live) return -1;
  return M(m)->requests[id].seq_len;
}
int32_t pegainfer_kukulorn_available_pages(pegainfer_kukulorn_t m) { return M(m)->pool.available(); }
int32_t pegainfer_kukulorn_capacity_pages(pegainfer_kukulorn_t m) { return M(m)->pool.capacity(); }
int32_t pegainfer_kukulorn_page_size(pegainfer_kukulorn_t) { return pkk::kPageSize; }
int32_t pegainfer_kukulorn_max_batch_size(pegainfer_kukulorn_t m) { return M(m)->max_requests; }
int32_t pegainfer_kukulorn_vocab_size(pegainfer_kukulorn_t m) { return M(m)->V; }
int32_t pegainfer_kukulorn_width(pegainfer_kukulorn_t m) { return M(m)->D; }
int32_t pegainfer_kukulorn_num_layer_runs(pegainfer_kukulorn_t m) { return (int32_t)M(m)->runs.size(); }
int32_t pegainfer_kukulorn_dtype(pegainfer_kukulorn_t m) { return M(m)->dtype; }
int64_t pegainfer_kukulorn_state_floats(pegainfer_kukulorn_t m) { return M(m)->state_layout.floats_per_slot(); }
int32_t pegainfer_kukulorn_step(pegainfer_kukulorn_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens) {
  return M(m)->step(n_entries, request_ids, lens, tokens_concat, n_want, want_rows, out_logits_host, out_tokens);
}
int32_t pegainfer_kukulorn_sample(pegainfer_kukulorn_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token) {
  return M(m)->sample(row, temperature, top_k, top_p, random_val, out_token);
}
int32_t pegainfer_kukulorn_logprobs(pegainfer_kukulorn_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs) {
  return M(m)->logprobs(row, token, top_k, out_logprob, out_top_ids, out_top_logprobs);
}
int32_t pegainfer_kukulorn_debug_hidden_enable(pegainfer_kukulorn_t m, int32_t enable) { M(m)->tap_on = enable != 0; return 0; }
int32_t pegainfer_kukulorn_debug_hidden(pegainfer_kukulorn_t m, int32_t layer_run, float* out_host, int32_t max_rows) {
  return M(m)->debug_hidden(layer_run, out_host, max_rows);
}
float pegainfer_kukulorn_last_step_ms(pegainfer_kukulorn_t m) { return M(m)->last_step_ms; }
int64_t pegainfer_kukulorn_weight_bytes(pegainfer_kukulorn_t m) { return M(m)->weight_bytes; }
int32_t pegainfer_kukulorn_set_plain_kernels(pegainfer_kukulorn_t m, int32_t on) { M(m)->plain_kernels = on != 0; return 0; }

}  // extern "C"

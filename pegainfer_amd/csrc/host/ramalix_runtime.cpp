// C++ host runtime of the Ramalix decoder on MI355X (include/pegainfer_ramalix.h).  Same shape as the runtimes next to it:
// one model = one device + one in-order HIP stream, requests are KvState slots over the shared PagePool (kv_pool.h) plus a
// region of the fp32 state arena (seq_state.h), a step's metadata is ONE pinned block and ONE hipMemcpyAsync, every op goes
// through the kernel library's C ABI (pegainfer_kernels.h: tuned bf16 GEMM routes, samplers; pegainfer_kernels_blocks.h:
// everything else).
//
// The layers of config.json are expanded into LAYER RUNS: the span loop.start .. loop.stop - 1 is walked loop.times times on
// the same weights, every run with cache pages' part and state parts of its own.  What a step does per run (T = all token rows
// of the step, prompts' portions and single tokens alike; x = fp32 stream, m = residual_mult):
//   pass start : x += embedding rows (from the second pass on) + loop.step[pass]          fused with the norm below
//   n      = x / rms(x) * g1                                  fp32, one launch with the residual sum before it
//   hb     = n + time_conv(n; canon1)                         tail of taps - 1 inputs per (run, request)
//   proj   = Wstack hb                                        ONE GEMM over all first-stage projections of the mixer
//   attention     : [q | k] hold two maps per head; bias, query temperature -> paged cache -> two causal softmax maps over
//                   the same values, map 1 - lambda map 2, RMS norm per head, * (1 - diff)          one attention launch
//   attention_2   : pair rotation of the first rot.dims values -> paged cache -> softmax over the keys of the query's own
//                   block of mask.size positions, with a per-head sink logit in the denominator
//   channel_delta : time_conv + silu on q | k | v; decay inputs and output gate by second-stage GEMMs over the low-rank columns
//                   of proj; gated delta rule with a decay per (head, key channel) over the request's matrix state; per-head
//                   RMS norm * weight * sigmoid(gate)
//   x     += m (Wo mix + bias);  n = x / rms(x) * g2;  hb = n + time_conv(n; canon2)
//   ff     : [router ; shared gate] GEMM into fp32 logits -> softmax, best groups, top experts, renormalised -> sort by expert
//            -> grouped GEMMs (SwiGLU) -> weighted sum + sigmoid(gate) * shared expert
//   x     += m ff;  n = x / rms(x) * (next run's g1)          the same launch
// Key/value cache: page-first [page][attention run][k: slot, kv head, maps * dim | v: slot, kv head, vdim].
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
#include "pegainfer_ramalix.h"

namespace prx {

using pq::KvState;
using pq::PagePool;
using pst::Json;

#define RX_HIP(expr)                                                   \
  do {                                                                 \
    hipError_t e_ = (expr);                                            \
    if (e_ != hipSuccess) {                                            \
      set_error(std::string(#expr) + ": " + hipGetErrorString(e_));    \
      return -1;                                                       \
    }                                                                  \
  } while (0)
#define RX_K(expr)                                                     \
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

enum { kDiffAttn = 1, kBlockAttn = 2, kChannelDelta = 3 };
struct AttnCfg {
  int heads = 0, kv = 0, dim = 0, vdim = 0, maps = 1;
  float scale = 1.f;
  float diff = 0.f, qt_coef = 0.f;   // two-map form
  int qt_every = 0;
  int rot_dims = 0, block = 0;       // one-map form
  double base = 10000.0;
  bool sink = false;
};
struct DeltaCfg { int heads = 0, kv = 0, dim = 0, vdim = 0, taps = 0, a_rank = 0, g_rank = 0; };
struct MlpCfg { int kind = 0 /* 0 none, 2 routed */, ff = 0, experts = 0, top = 0, groups = 1, keep = 1, shared_ff = 0; bool has_shared = false; };
struct LayerCfg {
  int type = 0;
  AttnCfg at;
  DeltaCfg dl;
  MlpCfg mlp;
  // columns of the stacked first-stage projection
  int o_q = 0, o_k = 0, o_v = 0, o_b = 0, o_a1 = 0, o_g1 = 0;
  int proj_rows = 0, mix_cols = 0, conv_ch = 0;
  int tile_set = -1;
};
struct LayerW {
  void *norm1 = nullptr, *norm2 = nullptr, *canon1 = nullptr, *canon2 = nullptr, *proj = nullptr, *o = nullptr;
  void *q_bias = nullptr, *k_bias = nullptr, *v_bias = nullptr, *o_bias = nullptr, *sink = nullptr;   // attention forms
  float lambda = 0.f;
  float* inv_freq = nullptr;
  void *conv = nullptr, *a2 = nullptr, *g2 = nullptr, *A_log = nullptr, *dt_bias = nullptr, *onorm = nullptr;   // channel_delta
  void *router = nullptr, *gate_up_e = nullptr, *down_e = nullptr, *gate_up = nullptr, *down = nullptr;      // feed-forward
};
// one walk over one layer: its weights (layer), its own cache part and state parts, and the pass it opens (or -1)
struct Run {
  int layer = 0, pass = -1;
  int64_t st_canon1 = 0, st_canon2 = 0, st_conv = 0, st_mem = 0;
  int64_t k_off = 0, v_off = 0;
};

struct Model {
  int device = 0, dtype = 0, D = 0, V = 0, max_requests = 0, num_pages = 0, canon_taps = 1;
  int loop_start = 0, loop_stop = 0, loop_times = 1;
  float eps = 1e-5f, mult = 1.f, logit_scale = 1.f;
  bool plain_kernels = false, finalized = false, planned = false;
  std::string err;
  std::vector<LayerCfg> layers;
  std::vector<LayerW> weights;
  std::vector<Run> runs;
  void *embed = nullptr, *head = nullptr, *final_norm = nullptr, *loop_step = nullptr;
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
  float *x = nullptr, *emb = nullptr, *n32 = nullptr, *qkv32 = nullptr, *q32 = nullptr, *o32 = nullptr, *a32 = nullptr,
        *gates32 = nullptr, *ypairs = nullptr, *route_w = nullptr, *route_logits = nullptr;
  void *hb = nullptr, *proj = nullptr, *mix = nullptr, *y = nullptr, *gate_d = nullptr, *gu = nullptr, *act = nullptr, *ys = nullptr,
       *gu_e = nullptr, *act_e = nullptr;
  int32_t *route_e = nullptr, *pos_pair = nullptr, *pos_row = nullptr, *tiles = nullptr;
  int max_tiles = 0;
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
  int mx_vdim = 0;
  int mx_proj = 0, mx_mix = 0, mx_conv = 0, mx_q = 0, mx_o = 0, mx_gates = 0, mx_a = 0, mx_ff = 0, mx_top = 0, mx_gu_e = 0, mx_experts = 0;

  struct GraphKey {
    int n, want; bool tokens, plain;
    bool operator==(const GraphKey& o) const { return n == o.n && want == o.want && tokens == o.tokens && plain == o.plain; }
  };
  std::vector<std::pair<GraphKey, hipGraphExec_t>> graphs;   // captured decode steps, one per shape
  bool graphs_on = [] { const char* e = getenv("PEGAINFER_RAMALIX_GRAPH"); return !(e && e[0] == '0'); }();
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
  int parse_config(const std::string& text) {
    Json j;
    if (!pst::JsonParser(text.data(), text.size()).parse(&j) || j.kind != Json::Obj) return set_error("config: not a JSON object");
    const Json* arch = j.get("architecture");
    if (!arch || arch->str != "Ramalix") return set_error("config: architecture is not Ramalix");
    D = geti(&j, "width", 0);
    V = geti(&j, "vocab", 0);
    eps = getf(j.get("norm"), "eps", 1e-5);
    mult = getf(&j, "residual_mult", 1.0);
    logit_scale = getf(&j, "logit_scale", 1.0);
    canon_taps = geti(j.get("canon"), "taps", 1);
    const Json* ls = j.get("layers");
    if (D <= 0 || V <= 0 || !ls || ls->kind != Json::Arr || ls->arr.empty()) return set_error("config: width / vocab / layers missing");
    if (canon_taps < 1 || canon_taps > 64) return set_error("config: canon.taps outside 1 .. 64");
    for (size_t i = 0; i < ls->arr.size(); ++i) {
      const Json& l = ls->arr[i];
      const std::string li = std::to_string(i);
      LayerCfg c;
      const Json* ty = l.get("type");
      const Json* mx = l.get("mixer");
      if (!ty || !mx || mx->kind != Json::Obj) return set_error("config: layer " + li + " without type / mixer");
      if (ty->str == "attention" || ty->str == "attention_2") {
        AttnCfg& a = c.at;
        a.heads = geti(mx, "heads", 0);
        a.kv = geti(mx, "kv_heads", a.heads);
        a.dim = geti(mx, "dim", 0);
        a.vdim = geti(mx, "vdim", a.dim);
        a.scale = getf(mx, "scale", 1.0 / std::sqrt((double)std::max(1, a.dim)));
        if (ty->str == "attention") {
          c.type = kDiffAttn;
          a.maps = 2;
          a.diff = getf(mx, "diff", 0.0);
          if (const Json* qt = mx->get("q_temp")) {
            a.qt_coef = getf(qt, "coef", 0.0);
            a.qt_every = geti(qt, "every", 0);
            if (a.qt_every < 1) return set_error("config: q_temp.every must be positive in layer " + li);
          }
        } else {
          c.type = kBlockAttn;
          a.sink = true;
          if (const Json* rot = mx->get("rot")) {
            a.rot_dims = geti(rot, "dims", a.dim);
            a.base = rot->number_or("base", 10000.0);
          }
          if (const Json* mk = mx->get("mask")) {
            a.block = geti(mk, "size", 0);
            if (a.block < 1) return set_error("config: mask.size must be positive in layer " + li);
          }
        }
        if (a.heads <= 0 || a.kv <= 0 || a.heads % a.kv || a.dim <= 0 || a.maps * a.dim > 256 || a.vdim <= 0 || a.vdim > 256 ||
            a.rot_dims < 0 || a.rot_dims > a.dim || (a.rot_dims & 1))
          return set_error("config: unsupported attention sizes in layer " + li);
        const int qd = a.maps * a.dim;
        c.o_q = 0;
        c.o_k = a.heads * qd;
        c.o_v = c.o_k + a.kv * qd;
        c.proj_rows = pad8(c.o_v + a.kv * a.vdim);
        c.mix_cols = a.heads * a.vdim;
        const int per = a.heads / a.kv;
        size_t k = 0;
        while (k < tile_sets.size() && tile_sets[k] != per) ++k;
        if (k == tile_sets.size()) tile_sets.push_back(per);
        c.tile_set = (int)k;
      } else if (ty->str == "channel_delta") {
        c.type = kChannelDelta;
        DeltaCfg& d = c.dl;
        d.heads = geti(mx, "heads", 0);
        d.kv = geti(mx, "kv_heads", d.heads);
        d.dim = geti(mx, "dim", 0);
        d.vdim = geti(mx, "vdim", 0);
        d.taps = geti(mx, "conv", 1);
        // the ranks of the two-step projections are tensor shapes: known once the checkpoint is; a configuration used without
        // one (synthetic weights) may name them
        d.a_rank = geti(mx, "a_rank", 0);
        d.g_rank = geti(mx, "g_rank", 0);
        if (d.heads <= 0 || d.kv <= 0 || d.heads % d.kv || d.dim <= 0 || d.dim > 256 || d.vdim <= 0 || d.taps < 1 || d.taps > 64)
          return set_error("config: unsupported channel_delta sizes in layer " + li);
        c.mix_cols = d.heads * d.vdim;
        c.conv_ch = 2 * d.kv * d.dim + d.heads * d.vdim;
      } else {
        return set_error("config: layer " + li + " has an unknown mixer type");
      }
      const Json* mlp = l.get("mlp");
      if (mlp && mlp->kind == Json::Obj) {
        const Json* kind = mlp->get("kind");
        if (!kind || kind->str != "moe") return set_error("config: unknown feed-forward kind in layer " + li);
        MlpCfg& f = c.mlp;
        f.kind = 2;
        f.ff = geti(mlp->get("expert"), "ff", 0);
        const Json* rt = mlp->get("router");
        f.experts = geti(rt, "experts", 0);
        f.top = geti(rt, "top", 0);
        if (const Json* g = rt ? rt->get("groups") : nullptr) {
          f.groups = geti(g, "count", 1);
          f.keep = geti(g, "keep", f.groups);
        }
        if (f.ff <= 0 || f.experts <= 0 || f.top <= 0 || f.top > f.experts || f.experts > 1024 || f.groups < 1 || f.experts % f.groups ||
            f.keep < 1 || f.keep > f.groups || f.top > f.keep * (f.experts / f.groups))
          return set_error("config: unsupported router in layer " + li);
        const Json* sh = mlp->get("shared");
        if (sh && sh->kind == Json::Obj) {
          f.has_shared = true;
          f.shared_ff = geti(sh, "ff", 0);
          if (f.shared_ff <= 0) return set_error("config: shared expert without ff in layer " + li);
        }
      }
      layers.push_back(c);
    }
    const int L = (int)layers.size();
    if (const Json* lp = j.get("loop")) {
      loop_start = geti(lp, "start", 0);
      loop_stop = geti(lp, "stop", 0);
      loop_times = geti(lp, "times", 1);
      if (loop_start < 0 || loop_stop < loop_start || loop_stop > L || loop_times < 1 || loop_times > 4096)
        return set_error("config: loop outside the layers");
    }
    // layer runs; every run reserves its state parts and, for the attention forms, its part of a cache page
    int64_t off = 0;
    auto add_run = [&](int layer, int pass) {
      const LayerCfg& c = layers[(size_t)layer];
      Run r;
      r.layer = layer;
      r.pass = pass;
      const std::string tag = "run" + std::to_string(runs.size());
      r.st_canon1 = state_layout.reserve(tag + ".canon1", (int64_t)(canon_taps - 1) * D);
      if (c.mlp.kind) r.st_canon2 = state_layout.reserve(tag + ".canon2", (int64_t)(canon_taps - 1) * D);
      if (c.type == kChannelDelta) {
        r.st_conv = state_layout.reserve(tag + ".conv", (int64_t)(c.dl.taps - 1) * c.conv_ch);
        r.st_mem = state_layout.reserve(tag + ".memory", (int64_t)c.dl.heads * c.dl.dim * c.dl.vdim);
      } else {
        r.k_off = off;
        r.v_off = off + (int64_t)kPageSize * c.at.kv * c.at.maps * c.at.dim;
        off = r.v_off + (int64_t)kPageSize * c.at.kv * c.at.vdim;
      }
      runs.push_back(r);
    };
    for (int i = 0; i < loop_start; ++i) add_run(i, -1);
    if (loop_stop > loop_start)
      for (int t = 0; t < loop_times; ++t)
        for (int i = loop_start; i < loop_stop; ++i) add_run(i, i == loop_start ? t : -1);
    for (int i = loop_stop; i < L; ++i) add_run(i, -1);
    page_stride = std::max<int64_t>(off, 1);
    weights.resize(layers.size());
    return 0;
  }
  // the stacked projection's columns and the step buffers' widths; needs the ranks of the two-step projections
  int plan_layout() {
    for (size_t i = 0; i < layers.size(); ++i) {
      LayerCfg& c = layers[i];
      if (c.type == kChannelDelta) {
        DeltaCfg& d = c.dl;
        if (d.a_rank <= 0 || d.g_rank <= 0) return set_error("channel_delta layer " + std::to_string(i) + ": the ranks of a1 / g1 are unknown");
        c.o_q = 0;
        c.o_k = d.kv * d.dim;
        c.o_v = 2 * d.kv * d.dim;
        c.o_b = pad8(c.conv_ch);            // the second-stage GEMMs read their columns in 16-byte chunks: starts at multiples of 8
        c.o_a1 = pad8(c.o_b + d.heads);
        c.o_g1 = pad8(c.o_a1 + d.a_rank);
        c.proj_rows = pad8(c.o_g1 + d.g_rank);
      }
    }
    for (auto& c : layers) {
      mx_proj = std::max(mx_proj, c.proj_rows);
      mx_mix = std::max(mx_mix, c.mix_cols);
      if (c.type == kChannelDelta) {
        mx_conv = std::max(mx_conv, c.conv_ch);
        mx_o = std::max(mx_o, c.dl.heads * c.dl.vdim);
        mx_gates = std::max(mx_gates, c.dl.heads * c.dl.dim + c.dl.heads);
        mx_a = std::max(mx_a, c.dl.heads * c.dl.dim);
      } else {
        mx_q = std::max(mx_q, c.at.heads * c.at.maps * c.at.dim);
        mx_vdim = std::max(mx_vdim, c.at.vdim);
      }
      if (c.mlp.kind == 2) {
        mx_top = std::max(mx_top, c.mlp.top);
        mx_gu_e = std::max(mx_gu_e, c.mlp.top * 2 * c.mlp.ff);
        mx_experts = std::max(mx_experts, c.mlp.experts);
        if (c.mlp.has_shared) mx_ff = std::max(mx_ff, c.mlp.shared_ff);
      }
    }
    planned = true;
    return 0;
  }

  // ------------------------------------------------------------------ device memory
  template <typename T>
  int dalloc(T** p, size_t count, std::vector<void*>* into = nullptr) {
    void* raw = nullptr;
    RX_HIP(hipMalloc(&raw, std::max<size_t>(count, 1) * sizeof(T)));
    RX_HIP(hipMemset(raw, 0, std::max<size_t>(count, 1) * sizeof(T)));
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
    RX_HIP(hipSetDevice(device));
    cublas_init();
    RX_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    RX_HIP(hipEventCreate(&ev0));
    RX_HIP(hipEventCreate(&ev1));
    num_pages = std::max(1, (max_tokens + kPageSize - 1) / kPageSize);
    pool = PagePool(num_pages);
    requests.assign((size_t)max_requests, KvState());
    if (dalloc_a(&cache, (size_t)num_pages * (size_t)page_stride)) return -1;
    if (dalloc(&state, (size_t)max_requests * (size_t)state_layout.floats_per_slot())) return -1;
    if (dalloc(&probs_scratch, (size_t)V) || dalloc(&top1_value, 1) || dalloc(&row_states, 1024 * 1024) ||
        dalloc(&valid_scratch, 1) || dalloc(&sample_out_d, 1))
      return -1;
    return 0;
  }

  // ------------------------------------------------------------------ weights
  typedef std::vector<std::pair<std::string, std::vector<int64_t>>> TensorList;
  static void glu_tensors(TensorList* out, const std::string& p, int ff, int D) {
    out->push_back({p + ".gate", {ff, D}});
    out->push_back({p + ".up", {ff, D}});
    out->push_back({p + ".down", {D, ff}});
  }
  TensorList tensor_list() const {
    TensorList out;
    out.push_back({"embed", {V, D}});
    if (loop_stop > loop_start) out.push_back({"loop.step", {loop_times, D}});
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      const std::string p = "l" + std::to_string(i), m = p + ".mix";
      out.push_back({p + ".norm1", {}});
      out.push_back({p + ".canon1", {D, canon_taps}});
      if (c.mlp.kind) {
        out.push_back({p + ".norm2", {}});
        out.push_back({p + ".canon2", {D, canon_taps}});
      }
      if (c.type == kChannelDelta) {
        const DeltaCfg& d = c.dl;
        for (const char* n : {".q", ".k"}) {
          out.push_back({m + n, {d.kv * d.dim, D}});
          out.push_back({m + n + ".conv", {d.kv * d.dim, d.taps}});
        }
        out.push_back({m + ".v", {d.heads * d.vdim, D}});
        out.push_back({m + ".v.conv", {d.heads * d.vdim, d.taps}});
        out.push_back({m + ".b", {d.heads, D}});
        out.push_back({m + ".A_log", {d.heads}});
        out.push_back({m + ".norm", {d.vdim}});
        out.push_back({m + ".a1", {d.a_rank, D}});
        out.push_back({m + ".a2", {d.heads * d.dim, d.a_rank}});
        out.push_back({m + ".dt_bias", {d.heads * d.dim}});
        out.push_back({m + ".g1", {d.g_rank, D}});
        out.push_back({m + ".g2", {d.heads * d.vdim, d.g_rank}});
        out.push_back({m + ".o", {D, d.heads * d.vdim}});
      } else {
        const AttnCfg& a = c.at;
        const int qd = a.maps * a.dim;
        out.push_back({m + ".q", {a.heads * qd, D}});
        out.push_back({m + ".k", {a.kv * qd, D}});
        out.push_back({m + ".v", {a.kv * a.vdim, D}});
        out.push_back({m + ".o", {D, a.heads * a.vdim}});
        if (c.type == kDiffAttn) {
          out.push_back({m + ".q.b", {a.heads * qd}});
          out.push_back({m + ".k.b", {a.kv * qd}});
          out.push_back({m + ".v.b", {a.kv * a.vdim}});
          out.push_back({m + ".o.b", {D}});
          for (const char* n : {".lq1", ".lk1", ".lq2", ".lk2"}) out.push_back({m + n, {a.dim}});
        } else {
          out.push_back({m + ".sink", {a.heads}});
        }
      }
      if (c.mlp.kind == 2) {
        for (int e = 0; e < c.mlp.experts; ++e) glu_tensors(&out, p + ".mlp.e" + std::to_string(e), c.mlp.ff, D);
        out.push_back({p + ".mlp.router", {c.mlp.experts, D}});
        if (c.mlp.has_shared) {
          glu_tensors(&out, p + ".mlp.shared", c.mlp.shared_ff, D);
          out.push_back({p + ".mlp.shared.sg", {1, D}});
        }
      }
    }
    out.push_back({"final.norm", {}});
    out.push_back({"head", {V, D}});
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
  // ranks that the configuration does not name, from the sizes of the staged a1 / g1 tensors ([rank, width])
  void ranks_from_staged() {
    for (size_t i = 0; i < layers.size(); ++i) {
      if (layers[i].type != kChannelDelta) continue;
      const std::string m = "l" + std::to_string(i) + ".mix";
      auto a = staged.find(m + ".a1"), g = staged.find(m + ".g1");
      if (a != staged.end() && a->second.size() % (size_t)D == 0) layers[i].dl.a_rank = (int)(a->second.size() / (size_t)D);
      if (g != staged.end() && g->second.size() % (size_t)D == 0) layers[i].dl.g_rank = (int)(g->second.size() / (size_t)D);
    }
  }
  int fill_synthetic(uint64_t seed, float std) {
    for (auto& c : layers)
      if (c.type == kChannelDelta) {
        if (c.dl.a_rank <= 0) c.dl.a_rank = 32;
        if (c.dl.g_rank <= 0) c.dl.g_rank = 32;
      }
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
      const bool is_conv = ends_with(n, ".conv") || ends_with(n, ".canon1") || ends_with(n, ".canon2");
      const bool is_gain = t.second.empty() || ends_with(n, ".mix.norm");
      const bool is_bias = ends_with(n, ".b") && t.second.size() == 1;
      const bool is_l = ends_with(n, ".lq1") || ends_with(n, ".lk1") || ends_with(n, ".lq2") || ends_with(n, ".lk2");
      for (size_t k = 0; k < v.size(); ++k) {
        const float z = g();
        float val = std * z;
        if (is_conv) val = 0.3f * z;
        else if (is_gain) val = 1.0f + 0.1f * z;
        else if (is_bias) val = 0.1f * z;
        else if (is_l) val = 0.1f * z;
        else if (ends_with(n, ".sink")) val = 0.5f * z;
        else if (ends_with(n, ".A_log")) val = -1.0f + 0.5f * z;
        else if (ends_with(n, ".dt_bias")) val = 0.3f * z;
        else if (n == "loop.step") val = 0.1f * z;
        else if (ends_with(n, ".a2") || ends_with(n, ".g2")) val = 0.2f * z;
        v[k] = host_f2bf(val);
      }
    }
    return 0;
  }
  int upload(void** out, const uint16_t* bits, size_t n) {
    if (dalloc_a(out, n)) return -1;
    if (dtype == PEGAINFER_DTYPE_BF16) {
      RX_HIP(hipMemcpy(*out, bits, n * 2, hipMemcpyHostToDevice));
    } else {
      std::vector<float> f(n);
      for (size_t i = 0; i < n; ++i) f[i] = host_bf2f(bits[i]);
      RX_HIP(hipMemcpy(*out, f.data(), n * 4, hipMemcpyHostToDevice));
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
  int up_glu(void** gate_up, void** down, const std::string& p, int ff) {
    return (up_stacked(gate_up, {{p + ".gate", ff, 0}, {p + ".up", ff, ff}}, D, 2 * (int64_t)ff) || up(down, p + ".down", (int64_t)D * ff)) ? -1 : 0;
  }
  double staged_dot(const std::string& a, const std::string& b, int n) {
    const auto *x = need(a, n), *y = need(b, n);
    if (!x || !y) return NAN;
    double s = 0.0;
    for (int i = 0; i < n; ++i) s += (double)host_bf2f((*x)[i]) * (double)host_bf2f((*y)[i]);
    return s;
  }
  int finalize() {
    if (finalized) return 0;
    ranks_from_staged();
    if (!planned && plan_layout()) return -1;
    if (up(&embed, "embed", (int64_t)V * D) || up(&head, "head", (int64_t)V * D) || up(&final_norm, "final.norm", 1)) return -1;
    if (loop_stop > loop_start && up(&loop_step, "loop.step", (int64_t)loop_times * D)) return -1;
    for (size_t i = 0; i < layers.size(); ++i) {
      const LayerCfg& c = layers[i];
      LayerW& w = weights[i];
      const std::string p = "l" + std::to_string(i), m = p + ".mix";
      if (up(&w.norm1, p + ".norm1", 1) || up(&w.canon1, p + ".canon1", (int64_t)D * canon_taps)) return -1;
      if (c.mlp.kind && (up(&w.norm2, p + ".norm2", 1) || up(&w.canon2, p + ".canon2", (int64_t)D * canon_taps))) return -1;
      if (c.type == kChannelDelta) {
        const DeltaCfg& d = c.dl;
        const int64_t qk = (int64_t)d.kv * d.dim, hv = (int64_t)d.heads * d.vdim;
        if (up_stacked(&w.proj, {{m + ".q", qk, c.o_q}, {m + ".k", qk, c.o_k}, {m + ".v", hv, c.o_v}, {m + ".b", d.heads, c.o_b},
                                 {m + ".a1", d.a_rank, c.o_a1}, {m + ".g1", d.g_rank, c.o_g1}},
                       D, c.proj_rows) ||
            up_stacked(&w.conv, {{m + ".q.conv", qk, 0}, {m + ".k.conv", qk, qk}, {m + ".v.conv", hv, 2 * qk}}, d.taps, 2 * qk + hv) ||
            up(&w.a2, m + ".a2", (int64_t)d.heads * d.dim * d.a_rank) || up(&w.g2, m + ".g2", hv * d.g_rank) ||
            up(&w.A_log, m + ".A_log", d.heads) || up(&w.dt_bias, m + ".dt_bias", (int64_t)d.heads * d.dim) ||
            up(&w.onorm, m + ".norm", d.vdim) || up(&w.o, m + ".o", (int64_t)D * hv))
          return -1;
      } else {
        const AttnCfg& a = c.at;
        const int64_t qd = (int64_t)a.maps * a.dim;
        if (up_stacked(&w.proj, {{m + ".q", a.heads * qd, c.o_q}, {m + ".k", a.kv * qd, c.o_k}, {m + ".v", (int64_t)a.kv * a.vdim, c.o_v}}, D,
                       c.proj_rows) ||
            up(&w.o, m + ".o", (int64_t)D * a.heads * a.vdim))
          return -1;
        if (c.type == kDiffAttn) {
          if (up(&w.q_bias, m + ".q.b", a.heads * qd) || up(&w.k_bias, m + ".k.b", a.kv * qd) ||
              up(&w.v_bias, m + ".v.b", (int64_t)a.kv * a.vdim) || up(&w.o_bias, m + ".o.b", D))
            return -1;
          // one number per layer, from four learned vectors
          const double l1 = staged_dot(m + ".lq1", m + ".lk1", a.dim), l2 = staged_dot(m + ".lq2", m + ".lk2", a.dim);
          if (std::isnan(l1) || std::isnan(l2)) return -1;
          w.lambda = (float)(std::exp(l1) - std::exp(l2) + (double)a.diff);
        } else {
          if (up(&w.sink, m + ".sink", a.heads)) return -1;
          const int half = a.rot_dims / 2;   // rotation frequencies base^(-2i/dims), rounded once to fp32
          std::vector<float> f((size_t)std::max(1, half));
          for (int k = 0; k < half; ++k) f[k] = (float)std::pow(a.base, -2.0 * k / (double)a.rot_dims);
          if (dalloc(&w.inv_freq, f.size())) return -1;
          RX_HIP(hipMemcpy(w.inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice));
        }
      }
      if (c.mlp.kind == 2) {
        std::vector<uint16_t> gu, dn;
        const int ff = c.mlp.ff;
        for (int e = 0; e < c.mlp.experts; ++e) {
          const std::string pe = p + ".mlp.e" + std::to_string(e);
          const auto *ga = need(pe + ".gate", (int64_t)ff * D), *u = need(pe + ".up", (int64_t)ff * D), *d = need(pe + ".down", (int64_t)D * ff);
          if (!ga || !u || !d) return -1;
          gu.insert(gu.end(), ga->begin(), ga->end());
          gu.insert(gu.end(), u->begin(), u->end());
          dn.insert(dn.end(), d->begin(), d->end());
        }
        if (upload(&w.gate_up_e, gu.data(), gu.size()) || upload(&w.down_e, dn.data(), dn.size())) return -1;
        // the router's rows and, after them, the shared expert's gate row: one GEMM gives all of a token's logits
        std::vector<Part> rp{{p + ".mlp.router", c.mlp.experts, 0}};
        if (c.mlp.has_shared) rp.push_back({p + ".mlp.shared.sg", 1, c.mlp.experts});
        if (up_stacked(&w.router, rp, D, c.mlp.experts + 1)) return -1;
        if (c.mlp.has_shared && up_glu(&w.gate_up, &w.down, p + ".mlp.shared", c.mlp.shared_ff)) return -1;
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
    for (size_t i = 0; i < layers.size(); ++i) {   // ranks = first sizes of the a1 / g1 tensors
      if (layers[i].type != kChannelDelta) continue;
      const std::string m = "l" + std::to_string(i) + ".mix";
      const pst::TensorView *a = ck.find(m + ".a1"), *g = ck.find(m + ".g1");
      if (!a || !g || a->shape.size() != 2 || g->shape.size() != 2) return set_error("checkpoint has no two-step projections for " + m);
      layers[i].dl.a_rank = (int)a->shape[0];
      layers[i].dl.g_rank = (int)g->shape[0];
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
        // the slot's state region starts from zero: empty convolution tails, empty memories
        if (n) RX_HIP(hipMemsetAsync(state + i * n, 0, n * sizeof(float), stream));
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
    RX_HIP(hipStreamSynchronize(stream));
    drop_graphs();
    free_all(&step_owned);
    cap_rows = 0;
    size_t n = 64;
    while (n < T) n *= 2;
    auto* so = &step_owned;
    const size_t P = n * (size_t)std::max(1, mx_top);
    max_tiles = (int)((P + 63) / 64) + std::max(1, mx_experts);
    if (dalloc(&x, n * D, so) || dalloc(&emb, n * D, so) || dalloc(&n32, n * D, so) || dalloc(&qkv32, n * (size_t)std::max(1, mx_conv), so) ||
        dalloc(&q32, n * (size_t)std::max(1, mx_q), so) || dalloc(&gates32, n * (size_t)std::max(1, mx_gates), so) ||
        dalloc(&a32, n * (size_t)std::max(1, mx_a), so) || dalloc(&o32, n * (size_t)std::max(1, mx_o), so) || dalloc_a(&hb, n * D, so) ||
        dalloc_a(&proj, n * (size_t)mx_proj, so) || dalloc_a(&mix, n * (size_t)mx_mix, so) || dalloc_a(&y, n * D, so) ||
        dalloc_a(&gate_d, n * (size_t)std::max(1, mx_o), so) || dalloc_a(&gu, n * (size_t)std::max(1, 2 * mx_ff), so) ||
        dalloc_a(&act, n * (size_t)std::max(1, mx_ff), so) || dalloc_a(&ys, n * D, so) ||
        dalloc(&att_part, (size_t)kSplitGroups * kAttRows * 2 * (size_t)(mx_vdim + 2), so))
      return -1;
    if (mx_top > 0 && (dalloc(&ypairs, P * D, so) || dalloc(&route_w, P, so) || dalloc(&route_logits, n * (size_t)(mx_experts + 1), so) ||
                       dalloc(&route_e, P, so) || dalloc(&pos_pair, P, so) || dalloc(&pos_row, P, so) ||
                       dalloc(&tiles, (size_t)3 * max_tiles + 1, so) || dalloc_a(&gu_e, n * (size_t)mx_gu_e, so) ||
                       dalloc_a(&act_e, n * (size_t)(mx_gu_e / 2), so)))
      return -1;
    cap_rows = n;
    return 0;
  }
  int ensure_want(size_t n) {
    if (n <= cap_want) return 0;
    RX_HIP(hipStreamSynchronize(stream));
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
    RX_K(pegainfer_gemm_strided(&d, S()));
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
    RX_K(pegainfer_gemm_strided(&d, S()));
    return 0;
  }
  // out = Wdown (silu(Wgate in) * (Wup in))
  int swiglu(const void* gate_up, const void* down, int ff, const void* in, void* out, int T) {
    // few rows (decoding) in bf16: the framework's GEMV with the SwiGLU in its epilogue, where its shapes allow
    const bool fused = dtype == PEGAINFER_DTYPE_BF16 && !plain_kernels && T <= 16 && D % 8 == 0 &&
                       pegainfer_gemv_fused(static_cast<const Half*>(gate_up), static_cast<const Half*>(in), static_cast<Half*>(act),
                                            2 * ff, T, D, nullptr, nullptr, nullptr, eps, ff, S()) == 0;
    if (!fused) {
      if (linear(gate_up, in, gu, 2 * ff, T, D)) return -1;
      RX_K(pegainfer_silu_mul_rows(gu, act, ff, T, dtype, S()));
    }
    return linear(down, act, out, D, T, ff);
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
      RX_HIP(hipStreamSynchronize(stream));
      if (meta_host) (void)hipHostFree(meta_host);
      if (meta_dev) (void)hipFree(meta_dev);
      meta_host = meta_dev = nullptr;
      cap_meta = 0;
      size_t c = 4096;
      while (c < words) c *= 2;
      RX_HIP(hipHostMalloc(reinterpret_cast<void**>(&meta_host), c * 4, hipHostMallocDefault));
      RX_HIP(hipMalloc(reinterpret_cast<void**>(&meta_dev), c * 4));
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
    RX_HIP(hipEventRecord(ev0, stream));
    RX_HIP(hipMemcpyAsync(meta_dev, meta_host, words * 4, hipMemcpyHostToDevice, stream));
    const int32_t* md = reinterpret_cast<const int32_t*>(meta_dev);
    const uint32_t* d_tok = reinterpret_cast<const uint32_t*>(md + o_tok);
    const int32_t *d_pos = md + o_pos, *d_ent = md + o_ent, *d_row0 = md + o_row0, *d_slot = md + o_slot, *d_ind = md + o_ind,
                  *d_want = md + o_want, *d_pages = md + o_pages;
    const int Ti = (int)T;
    const int64_t slot_stride = state_layout.floats_per_slot();
    if (tap_on) {
      const size_t needf = runs.size() * T * D;
      if (needf > tap_cap) {
        RX_HIP(hipStreamSynchronize(stream));
        if (tap) (void)hipFree(tap);
        tap = nullptr;
        tap_cap = 0;
        RX_HIP(hipMalloc(reinterpret_cast<void**>(&tap), needf * 4));
        tap_cap = needf;
      }
      tap_rows = Ti;
    }
    // ---- the layer runs (everything below reads the step's shape from its arguments and the step's contents from the
    //      metadata block, so a launch sequence recorded for one decode step serves every later step of the same shape)
    // x <- x + mlt (yv + bias) + add_rows + add_vec; with a gain also the norm of the sublayer that follows and its input
    // convolution (hb = n + conv(n), the tail moved on)
    auto open_sublayer = [&](const void* yv, const void* bias, float mlt, const float* add_rows, const void* add_vec, bool write_x,
                             const void* gain, const void* conv_w, int64_t st_off) -> int {
      if (!gain) {
        RX_K(pegainfer_scalar_rms_add(x, yv, dtype, bias, mlt, add_rows, add_vec, x, nullptr, eps, nullptr, D, Ti, dtype, S()));
        return 0;
      }
      RX_K(pegainfer_scalar_rms_add(x, yv, dtype, bias, mlt, add_rows, add_vec, write_x ? x : nullptr, gain, eps, n32, D, Ti, dtype, S()));
      if (single) {   // output and the moved-on tail in one launch (folding it into the norm's launch was measured: one workgroup
                      // per row then walks every channel's tail, 15 us against 5.6 + 4.3)
        RX_K(pegainfer_time_conv_step(n32, PEGAINFER_DTYPE_F32, D, conv_w, dtype, state + st_off, slot_stride, hb, dtype, D, D,
                                      canon_taps, 1, d_slot, n, S()));
        return 0;
      }
      RX_K(pegainfer_time_conv(n32, PEGAINFER_DTYPE_F32, D, conv_w, dtype, state + st_off, slot_stride, hb, dtype, D, D, canon_taps, 1,
                               d_ent, d_row0, d_slot, Ti, S()));
      RX_K(pegainfer_time_conv_commit(n32, PEGAINFER_DTYPE_F32, D, state + st_off, slot_stride, D, canon_taps, d_row0, d_slot, n, S()));
      return 0;
    };
    auto run_layers = [&]() -> int {
    RX_K(pegainfer_embed_f32(embed, d_tok, emb, D, Ti, dtype, S()));
    RX_K(pegainfer_embed_f32(embed, d_tok, x, D, Ti, dtype, S()));
    for (size_t ri = 0; ri < runs.size(); ++ri) {
      const Run& r = runs[ri];
      const LayerCfg& c = layers[(size_t)r.layer];
      const LayerW& w = weights[(size_t)r.layer];
      const int Mp = c.proj_rows;
      if (r.pass >= 0) {
        // a pass over the repeated span begins: the embedding rows again (not before the first pass), this pass's own row,
        // and the first sublayer's norm and input convolution
        if (open_sublayer(nullptr, nullptr, 0.f, r.pass > 0 ? emb : nullptr, at(loop_step, (size_t)r.pass * D), true, w.norm1, w.canon1,
                          r.st_canon1))
          return -1;
      } else if (ri == 0) {
        if (open_sublayer(nullptr, nullptr, 0.f, nullptr, nullptr, false, w.norm1, w.canon1, r.st_canon1)) return -1;
      }   // otherwise the launch that closed the run before has left hb
      if (linear(w.proj, hb, proj, Mp, Ti, D)) return -1;
      if (c.type == kChannelDelta) {
        const DeltaCfg& d = c.dl;
        if (single) {
          RX_K(pegainfer_time_conv_step(proj, dtype, Mp, w.conv, dtype, state + r.st_conv, slot_stride, qkv32, PEGAINFER_DTYPE_F32,
                                        c.conv_ch, c.conv_ch, d.taps, 2, d_slot, n, S()));
        } else {
          RX_K(pegainfer_time_conv(proj, dtype, Mp, w.conv, dtype, state + r.st_conv, slot_stride, qkv32, PEGAINFER_DTYPE_F32,
                                   c.conv_ch, c.conv_ch, d.taps, 2, d_ent, d_row0, d_slot, Ti, S()));
          RX_K(pegainfer_time_conv_commit(proj, dtype, Mp, state + r.st_conv, slot_stride, c.conv_ch, d.taps, d_row0, d_slot, n, S()));
        }
        // second stage of the two-step projections: decay inputs (kept in fp32) and the output gate
        if (linear_strided(w.a2, at(proj, (size_t)c.o_a1), dtype, Mp, a32, PEGAINFER_DTYPE_F32, d.heads * d.dim, Ti, d.a_rank) ||
            linear_strided(w.g2, at(proj, (size_t)c.o_g1), dtype, Mp, gate_d, dtype, d.heads * d.vdim, Ti, d.g_rank))
          return -1;
        RX_K(pegainfer_delta_rule_channel(qkv32, c.conv_ch, proj, Mp, c.o_b, a32, (int64_t)d.heads * d.dim, w.A_log, w.dt_bias, gates32,
                                          state + r.st_mem, slot_stride, o32, d.heads, d.kv, d.dim, d.vdim, Ti, d_row0, d_slot, n, dtype, S()));
        RX_K(pegainfer_head_rms_gate(o32, w.onorm, 0, gate_d, (int64_t)d.heads * d.vdim, 1, 1.0f, eps, mix, c.mix_cols, d.heads, d.vdim,
                                     Ti, dtype, S()));
      } else {
        const AttnCfg& a = c.at;
        const size_t ts = (size_t)c.tile_set;
        const int32_t* tb = md + tile_off[ts];
        const int qd = a.maps * a.dim;
        RX_K(pegainfer_qk_prep_paged(proj, Mp, c.o_q, c.o_k, c.o_v, a.heads, a.kv, qd, a.vdim, nullptr, nullptr, eps, w.q_bias, w.k_bias,
                                     w.v_bias, a.qt_coef, a.qt_every, w.inv_freq, a.rot_dims, d_pos, d_ent, d_ind, d_pages, cache,
                                     page_stride, r.k_off, r.v_off, kPageSize, q32, nullptr, Ti, dtype, S()));
        const bool two = a.maps == 2;
        // a step of few rows (decoding, short portions) cannot fill the chip with one workgroup per (row tile, kv head): its
        // keys are dealt to several workgroups.  The count depends on the step's shape only, never on the contexts' lengths.
        const int wgs = (int)tile_cnt[ts] * a.kv;
        const int nsplit = wgs >= 128 ? 1 : std::max(1, std::min(kMaxSplits, kSplitGroups / wgs));
        RX_K(pegainfer_paged_attention_ex(q32, cache, page_stride, r.k_off, r.v_off, kPageSize, d_pos, d_ent, d_ind, d_pages, a.heads,
                                          a.kv, a.dim, a.vdim, a.scale, two ? 1.0f - a.diff : 1.0f, tb, tb + tile_cnt[ts],
                                          tb + 2 * tile_cnt[ts], tb + 3 * tile_cnt[ts], (int)tile_cnt[ts], mix, c.mix_cols, a.maps,
                                          w.lambda, a.block, w.sink, two ? 1 : 0, eps, nsplit, att_part, plain_kernels ? 1 : 0, dtype, S()));
      }
      if (linear(w.o, mix, y, D, Ti, c.mix_cols)) return -1;
      // what the launch that closes this run norms for: the next run's first sublayer, unless that run opens a pass (its own
      // launch sums first) or there is none (the final norm runs on the wanted rows only)
      const bool next_plain = ri + 1 < runs.size() && runs[ri + 1].pass < 0;
      const LayerW* nw = next_plain ? &weights[(size_t)runs[ri + 1].layer] : nullptr;
      const int64_t next_st = next_plain ? runs[ri + 1].st_canon1 : 0;
      if (c.mlp.kind) {
        if (open_sublayer(y, w.o_bias, mult, nullptr, nullptr, true, w.norm2, w.canon2, r.st_canon2)) return -1;
        if (routed_ff(c, w, Ti)) return -1;
        if (open_sublayer(y, nullptr, mult, nullptr, nullptr, true, nw ? nw->norm1 : nullptr, nw ? nw->canon1 : nullptr, next_st)) return -1;
      } else if (open_sublayer(y, w.o_bias, mult, nullptr, nullptr, true, nw ? nw->norm1 : nullptr, nw ? nw->canon1 : nullptr, next_st)) {
        return -1;
      }
      if (tap_on) RX_HIP(hipMemcpyAsync(tap + ri * T * D, x, T * D * 4, hipMemcpyDeviceToDevice, stream));
    }
    // ---- wanted rows: final norm, logits over the output table in fp32, the constant factor
    if (W > 0) {
      RX_K(pegainfer_gather_rows_f32(x, d_want, xw, D, W, S()));
      RX_K(pegainfer_scalar_rms_add(xw, nullptr, dtype, nullptr, 0.f, nullptr, nullptr, nullptr, final_norm, eps, hw, D, W, dtype, S()));
      if (linear_strided(head, hw, PEGAINFER_DTYPE_F32, D, logits32, PEGAINFER_DTYPE_F32, V, W, D)) return -1;
      if (logit_scale != 1.0f) RX_K(pegainfer_scale_rows(logits32, V, logits32, V, V, W, logit_scale, PEGAINFER_DTYPE_F32, S()));
      RX_K(deepseek_f32_to_bf16_cuda(logits32, logits16, W * V, S()));
      if (out_tokens) RX_K(pegainfer_batched_top1(logits16, V, W, V, top1_state, tokens_d, S()));
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
        RX_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        const int rc = run_layers();
        const hipError_t e = hipStreamEndCapture(stream, &g);
        if (rc) return -1;
        if (e != hipSuccess) return set_error("graph capture failed");
        RX_HIP(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
        RX_HIP(hipGraphDestroy(g));
        graphs.emplace_back(key, exec);
      }
      RX_HIP(hipGraphLaunch(exec, stream));
    } else if (run_layers()) {
      return -1;
    }
    last_rows = W;
    RX_HIP(hipEventRecord(ev1, stream));
    if (W > 0 && out_logits) RX_HIP(hipMemcpyAsync(out_logits, logits32, (size_t)W * V * 4, hipMemcpyDeviceToHost, stream));
    if (W > 0 && out_tokens) RX_HIP(hipMemcpyAsync(out_tokens, tokens_d, (size_t)W * 4, hipMemcpyDeviceToHost, stream));
    RX_HIP(hipStreamSynchronize(stream));
    (void)hipEventElapsedTime(&last_step_ms, ev0, ev1);
    for (int i = 0; i < n; ++i) requests[ids[i]].seq_len += lens[i];
    return 0;
  }

  // hb -> y: router logits and the shared expert's gate logit by one GEMM into fp32, selection, experts, weighted sum
  int routed_ff(const LayerCfg& c, const LayerW& w, int T) {
    const MlpCfg& f = c.mlp;
    const int ff = f.ff, P = T * f.top, E1 = f.experts + 1;
    int32_t *t_group = tiles, *t_row0 = tiles + max_tiles, *t_rows = tiles + 2 * max_tiles, *n_tiles = tiles + 3 * max_tiles;
    if (linear_strided(w.router, hb, dtype, D, route_logits, PEGAINFER_DTYPE_F32, E1, T, D)) return -1;
    RX_K(pegainfer_route_from_logits_ex(route_logits, E1, nullptr, route_e, route_w, f.experts, f.groups, f.keep, f.top, T,
                                        PEGAINFER_SCORE_SOFTMAX, PEGAINFER_GROUP_MAX, 1, dtype, S()));
    const int per_tile = dtype == PEGAINFER_DTYPE_BF16 && !plain_kernels && T > 8 && D % 8 == 0 && ff % 8 == 0 ? 128 : 64;
    RX_K(pegainfer_route_sort(route_e, P, f.top, f.experts, pos_pair, pos_row, t_group, t_row0, t_rows, n_tiles, max_tiles, per_tile, S()));
    pegainfer_gemm_desc d{};
    d.x = hb; d.w = w.gate_up_e; d.y = gu_e;
    d.x_dtype = d.w_dtype = d.y_dtype = dtype;
    d.m = 2 * ff; d.k = D;
    d.x_row_stride = D; d.w_m_stride = D; d.w_k_stride = 1; d.w_group_stride = (int64_t)2 * ff * D;
    d.y_row_stride = 2 * ff;
    d.tile_group = t_group; d.tile_row0 = t_row0; d.tile_rows = t_rows; d.n_tiles = n_tiles; d.max_tiles = (P + per_tile - 1) / per_tile + f.experts;
    d.tile_rows_cap = per_tile;
    d.x_row_index = pos_row;
    d.max_tile_rows = std::min(T, 64);   // a row chooses distinct experts: an expert never gets more pairs than there are rows
    d.plain = plain_kernels;
    RX_K(pegainfer_gemm_strided(&d, S()));
    RX_K(pegainfer_silu_mul_rows(gu_e, act_e, ff, P, dtype, S()));
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
    RX_K(pegainfer_gemm_strided(&e, S()));
    if (f.has_shared && swiglu(w.gate_up, w.down, f.shared_ff, hb, ys, T)) return -1;
    RX_K(pegainfer_route_combine_gated(ypairs, route_w, f.has_shared ? ys : nullptr, f.has_shared ? route_logits + f.experts : nullptr, E1, y,
                                       D, f.top, T, dtype, S()));
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
    RX_HIP(hipStreamSynchronize(stream));
    RX_HIP(hipMemcpy(out, sample_out_d, 4, hipMemcpyDeviceToHost));
    return 0;
  }
  int logprobs(int row, uint32_t token, int top_k, float* out_lp, uint32_t* top_ids, float* top_lps) {
    if (row < 0 || row >= last_rows) return set_error("no logits for that row");
    if (token >= (uint32_t)V) return set_error("logprobs: token outside the vocabulary");
    lp_row.resize((size_t)V);
    RX_HIP(hipStreamSynchronize(stream));
    RX_HIP(hipMemcpy(lp_row.data(), logits32 + (size_t)row * V, (size_t)V * 4, hipMemcpyDeviceToHost));
    return pegainfer_logprobs_from_logits(lp_row.data(), V, token, top_k, out_lp, top_ids, top_lps);
  }
  int debug_hidden(int run, float* out, int max_rows) {
    if (!tap || run < 0 || run >= (int)runs.size()) return set_error("debug_hidden: no tap for that layer run");
    const int rows = std::min(max_rows, tap_rows);
    RX_HIP(hipStreamSynchronize(stream));
    RX_HIP(hipMemcpy(out, tap + (size_t)run * tap_rows * D, (size_t)rows * D * 4, hipMemcpyDeviceToHost));
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
static Model* M(pegainfer_ramalix_t m) { return static_cast<Model*>(m); }

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

}  // namespace prx

extern "C" {
using prx::M;

pegainfer_ramalix_t pegainfer_ramalix_create(const char* config_json, int32_t device_ordinal, int32_t dtype,
                                             int32_t max_tokens, int32_t max_requests) {
  if (!config_json) { prx::g_create_error = "no configuration"; return nullptr; }
  return prx::create(config_json, device_ordinal, dtype, max_tokens, max_requests);
}
pegainfer_ramalix_t pegainfer_ramalix_from_pretrained(const char* model_dir, int32_t device_ordinal, int32_t dtype,
                                                      int32_t max_tokens, int32_t max_requests) {
  std::string e;
  auto f = pst::MappedFile::open(std::string(model_dir) + "/config.json", &e);
  if (!f) { prx::g_create_error = e; return nullptr; }
  prx::Model* m = prx::create(std::string(reinterpret_cast<const char*>(f->data), f->size), device_ordinal, dtype, max_tokens, max_requests);
  if (!m) return nullptr;
  if (m->load_checkpoint(model_dir)) {
    prx::g_create_error = m->err;
    delete m;
    return nullptr;
  }
  return m;
}
void pegainfer_ramalix_destroy(pegainfer_ramalix_t m) { delete M(m); }
const char* pegainfer_ramalix_last_error(pegainfer_ramalix_t m) { return m ? M(m)->err.c_str() : prx::g_create_error.c_str(); }
int32_t pegainfer_ramalix_load_tensor(pegainfer_ramalix_t m, const char* name, const void* host_bf16, int64_t numel) {
  return M(m)->load_tensor(name, static_cast<const uint16_t*>(host_bf16), numel);
}
int32_t pegainfer_ramalix_fill_synthetic(pegainfer_ramalix_t m, uint64_t seed, float std) { return M(m)->fill_synthetic(seed, std); }
int32_t pegainfer_ramalix_finalize(pegainfer_ramalix_t m) { return M(m)->finalize(); }
int32_t pegainfer_ramalix_new_request(pegainfer_ramalix_t m) { return M(m)->new_request(); }
int32_t pegainfer_ramalix_drop_request(pegainfer_ramalix_t m, int32_t id) { return M(m)->drop_request(id); }
int32_t pegainfer_ramalix_request_seq_len(pegainfer_ramalix_t m, int32_t id) {
  if (id < 0 || id >= (int)M(m)->requests.size() || !M(m)->requests[id].live) return -1;
  return M(m)->requests[id].seq_len;
}
int32_t pegainfer_ramalix_available_pages(pegainfer_ramalix_t m) { return M(m)->pool.available(); }
int32_t pegainfer_ramalix_capacity_pages(pegainfer_ramalix_t m) { return M(m)->pool.capacity(); }
int32_t pegainfer_ramalix_page_size(pegainfer_ramalix_t) { return prx::kPageSize; }
int32_t pegainfer_ramalix_max_batch_size(pegainfer_ramalix_t m) { return M(m)->max_requests; }
int32_t pegainfer_ramalix_vocab_size(pegainfer_ramalix_t m) { return M(m)->V; }
int32_t pegainfer_ramalix_width(pegainfer_ramalix_t m) { return M(m)->D; }
int32_t pegainfer_ramalix_num_layer_runs(pegainfer_ramalix_t m) { return (int32_t)M(m)->runs.size(); }
int32_t pegainfer_ramalix_dtype(pegainfer_ramalix_t m) { return M(m)->dtype; }
int64_t pegainfer_ramalix_state_floats(pegainfer_ramalix_t m) { return M(m)->state_layout.floats_per_slot(); }
int32_t pegainfer_ramalix_step(pegainfer_ramalix_t m, int32_t n_entries, const int32_t* request_ids, const int32_t* lens,
                               const uint32_t* tokens_concat, int32_t n_want, const int32_t* want_rows,
                               float* out_logits_host, int32_t* out_tokens) {
  return M(m)->step(n_entries, request_ids, lens, tokens_concat, n_want, want_rows, out_logits_host, out_tokens);
}
int32_t pegainfer_ramalix_sample(pegainfer_ramalix_t m, int32_t row, float temperature, int32_t top_k, float top_p,
                                 float random_val, int32_t* out_token) {
  return M(m)->sample(row, temperature, top_k, top_p, random_val, out_token);
}
int32_t pegainfer_ramalix_logprobs(pegainfer_ramalix_t m, int32_t row, uint32_t token, int32_t top_k, float* out_logprob,
                                   uint32_t* out_top_ids, float* out_top_logprobs) {
  return M(m)->logprobs(row, token, top_k, out_logprob, out_top_ids, out_top_logprobs);
}
int32_t pegainfer_ramalix_debug_hidden_enable(pegainfer_ramalix_t m, int32_t enable) { M(m)->tap_on = enable != 0; return 0; }
int32_t pegainfer_ramalix_debug_hidden(pegainfer_ramalix_t m, int32_t layer_run, float* out_host, int32_t max_rows) {
  return M(m)->debug_hidden(layer_run, out_host, max_rows);
}
float pegainfer_ramalix_last_step_ms(pegainfer_ramalix_t m) { return M(m)->last_step_ms; }
int64_t pegainfer_ramalix_weight_bytes(pegainfer_ramalix_t m) { return M(m)->weight_bytes; }
int32_t pegainfer_ramalix_set_plain_kernels(pegainfer_ramalix_t m, int32_t on) { M(m)->plain_kernels = on != 0; return 0; }

}  // extern "C"

// Softmax attention over a paged key/value cache for any head sizes and grouped key/value heads, in a bf16 and an fp32
// storage instance; norms, angles, scores, softmax state and accumulators are fp32 in both.
//   qk_prep_paged_kernel       one or several workgroups per token row, a wave per head: optional bias, optional RMS norm over the head
//                              (plain weight), optional position-dependent query factor (query temperature), rotation
//                              of neighbouring pairs (2i, 2i + 1) of the first rot_dims values by position * inv_freq[i],
//                              queries to an fp32 buffer, keys and values into the cache entry of (request, position)
//   paged_attention_kernel     one workgroup per (row tile, key/value head): up to 16 (token, query head) rows that share the
//                              key/value head; key and value tiles of 64 positions are staged once in LDS (fp32) for all
//                              rows; a wave owns up to four rows and takes them through a tile together (a key or value
//                              read from LDS serves four products), a lane one key of the tile for the scores and value
//                              columns lane, lane + 64, ... for the output; running maximum / sum per row.  Options
//                              (AttnForm): keys restricted to the query's own run of `block` positions, a per-head sink
//                              logit in the denominator, two softmax maps over the same values combined as
//                              map 1 - lambda * map 2, an RMS norm of the head's output
// Keys are always visited in tiles of 64 from position 0, whatever the step's shape, so a row's arithmetic does not depend on
// how its prompt was cut or on what else runs in the step.
#include <algorithm>

#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

// how qk_prep_paged_kernel norms and rotates
struct PrepForm {
  int norm_kind = 0;    // 0: per head before the rotation, times a weight [dim] (when weights are given); 1: per head AFTER the
                        // rotation, no weight (unit root mean square); 2: over ALL heads of the projection at once before the
                        // rotation, times a weight [heads * dim] / [kv_heads * dim]
  int rot_halves = 0;   // 0: neighbours (2i, 2i + 1) are rotated together; 1: value i with value i + rot_dims / 2
};

// I: type of the projection rows read (the storage type, or float for rows that an fp32 stage such as a convolution left)
template <typename A, typename I>
__global__ __launch_bounds__(256) void qk_prep_paged_kernel(
    const I* __restrict__ proj, int64_t proj_stride, int64_t q_off, int64_t k_off, int64_t v_off, int H, int G, int dim, int vdim,
    const A* __restrict__ q_norm, const A* __restrict__ k_norm, float eps, const float* __restrict__ inv_freq, int rot_dims,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_entry, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ page_ids, A* __restrict__ cache, int64_t page_stride, int64_t k_cache_off, int64_t v_cache_off,
    int page_size, float* __restrict__ q_out, A* __restrict__ q_out_stored, const A* __restrict__ q_bias,
    const A* __restrict__ k_bias, const A* __restrict__ v_bias, float qt_coef, int qt_every, PrepForm pf) {
  extern __shared__ float sm[];   // [4 waves][dim]
  __shared__ float red[4];
  const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = positions[row], e = row_entry[row];
  const int64_t page = page_ids[page_indptr[e] + pos / page_size];
  const int slot = pos % page_size;
  const I* pr = proj + (int64_t)row * proj_stride;
  float* buf = sm + wave * dim;
  // query temperature: a factor on the whole query that grows with the logarithm of the position's block number
  const float qt = qt_every > 0 ? 1.0f + qt_coef * logf((float)((pos + 1) / qt_every) + 1.0f) : 1.0f;
  float inv_all_q = 1.f, inv_all_k = 1.f;
  if (pf.norm_kind == 2) {   // root mean squares over the whole q and the whole k projection
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < H * dim; i += 256) {
      const float v = ld(pr + q_off + i) + (q_bias ? ld(q_bias + i) : 0.f);
      sq = fmaf(v, v, sq);
    }
    for (int i = threadIdx.x; i < G * dim; i += 256) {
      const float v = ld(pr + k_off + i) + (k_bias ? ld(k_bias + i) : 0.f);
      sk = fmaf(v, v, sk);
    }
    inv_all_q = 1.0f / sqrtf(block_sum<4>(sq, red) / (float)(H * dim) + eps);
    inv_all_k = 1.0f / sqrtf(block_sum<4>(sk, red) / (float)(G * dim) + eps);
  }
  const int half = rot_dims >> 1;
  // the row's heads are dealt to the workgroups of its grid column, a wave per head
  for (int hh = blockIdx.y * 4 + wave; hh < H + G; hh += 4 * gridDim.y) {
    const bool is_q = hh < H;
    const int hd = is_q ? hh : hh - H;
    const I* src = is_q ? pr + q_off + (int64_t)hd * dim : pr + k_off + (int64_t)hd * dim;
    const A* nw = is_q ? q_norm : k_norm;
    const A* bs = is_q ? (q_bias ? q_bias + (int64_t)hd * dim : nullptr) : (k_bias ? k_bias + (int64_t)hd * dim : nullptr);
    float ss = 0.f;
    for (int i = lane; i < dim; i += 64) {
      const float v = ld(src + i) + (bs ? ld(bs + i) : 0.f);
      buf[i] = v;
      ss = fmaf(v, v, ss);
    }
    if (pf.norm_kind == 0 && nw) {
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
      for (int i = lane; i < dim; i += 64) buf[i] = buf[i] * inv * ld(nw + i);
    } else if (pf.norm_kind == 2) {
      const float inv = is_q ? inv_all_q : inv_all_k;
      for (int i = lane; i < dim; i += 64) buf[i] = buf[i] * inv * ld(nw + (int64_t)hd * dim + i);
    }
    if (is_q && qt_every > 0)
      for (int i = lane; i < dim; i += 64) buf[i] *= qt;
    __builtin_amdgcn_wave_barrier();
    float keep[4];   // dim <= 256: a lane's values i = lane, lane + 64, ...
    float ss2 = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int i = lane + 64 * c;
      float out = 0.f;
      if (i < dim) {
        out = buf[i];
        if (i < rot_dims) {
          if (pf.rot_halves) {
            const int f = i < half ? i : i - half;
            const float ang = (float)pos * inv_freq[f];
            const float cs = cosf(ang), sn = sinf(ang);
            out = i < half ? buf[i] * cs - buf[i + half] * sn : buf[i] * cs + buf[i - half] * sn;
          } else {
            const float ang = (float)pos * inv_freq[i >> 1];
            const float cs = cosf(ang), sn = sinf(ang);
            out = (i & 1) ? buf[i] * cs + buf[i - 1] * sn : buf[i] * cs - buf[i + 1] * sn;
          }
        }
        ss2 = fmaf(out, out, ss2);
      }
      keep[c] = out;
    }
    const float post = pf.norm_kind == 1 ? 1.0f / sqrtf(wave_sum(ss2) / (float)dim + eps) : 1.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int i = lane + 64 * c;
      if (i >= dim) continue;
      const float out = keep[c] * post;
      if (is_q) {
        if (q_out_stored) st(q_out_stored + ((int64_t)row * H + hh) * dim + i, out);
        else q_out[((int64_t)row * H + hh) * dim + i] = out;
      } else
        st(cache + page * page_stride + k_cache_off + ((int64_t)slot * G + hd) * dim + i, out);
    }
    __builtin_amdgcn_wave_barrier();
  }
  for (int i = blockIdx.y * 256 + threadIdx.x; i < G * vdim; i += 256 * gridDim.y) {
    A* dst = cache + page * page_stride + v_cache_off + (int64_t)slot * G * vdim + i;
    st(dst, ld(pr + v_off + i) + (v_bias ? ld(v_bias + i) : 0.f));
  }
}

constexpr int kAttKeys = 64;    // keys per staged tile
constexpr int kAttRows = 16;    // (token, query head) rows per workgroup
constexpr int kAttRpw = 4;      // rows per wave

// What the general kernel can do beyond plain causal softmax attention; a zeroed struct is the plain form.
struct AttnForm {
  int block = 0;               // > 0: a key is visible only inside the query's own run of `block` positions (runs counted from
                               // position 0 of the sequence), and not after the query
  const void* sink = nullptr;  // [heads] logits (storage type) that join the softmax denominator, unscaled, without a value
  float lambda = 0.f;          // MAPS == 2: out = map 1 - lambda * map 2 (two softmax maps over the same values; a query /
                               // key head holds [map 1 : dim | map 2 : dim])
  int head_norm = 0;           // != 0: out / sqrt(mean(out^2) + norm_eps) over the head's vdim values, before `factor`
  float norm_eps = 0.f;
  float softcap = 0.f;         // > 0: score <- softcap * tanh(score / softcap), after the scale
  int window = 0;              // > 0: a key j is visible to position i only if i - j < window or j < keep_first (kept first
  int keep_first = 0;          // tokens stay visible at their true positions)
  const float* dist_bias = nullptr;   // fp32 [n_dist][heads], added to the (scaled, capped) score of query head h by distance:
  int n_dist = 0;                     // dist_bias[min(i - j, n_dist - 1)][h]
  const void* gate = nullptr;  // output gate logits (storage type), rows at gate_stride: the finished head is multiplied by
  int64_t gate_stride = 0;     // sigmoid(gate[row, h * vdim + c]) (gate_kind 1: one per value) or sigmoid(gate[row, h]) (2: one
  int gate_kind = 0;           // per head)
};

// first position of the run of keys that position `pos` sees (besides the kept first tokens)
__device__ __forceinline__ int attn_row_lo(const AttnForm& form, int pos) {
  int lo = form.block > 0 ? (pos / form.block) * form.block : 0;
  if (form.window > 0) lo = max(lo, pos - form.window + 1);
  return lo;
}
// a raw dot product turned into the score of (query position rpos, key position kp, query head qh)
__device__ __forceinline__ float attn_score(const AttnForm& form, float dot, float scale, int rpos, int kp, int qh, int H) {
  float sc = dot * scale;
  if (form.softcap > 0.f) sc = form.softcap * tanhf(sc / form.softcap);
  if (form.dist_bias) sc += form.dist_bias[(int64_t)min(rpos - kp, form.n_dist - 1) * H + qh];
  return sc;
}

// A row's softmax states (one per map) turned into its output: the sink joins every denominator, the maps are combined, the
// head is normed, `factor` comes last.  The wave holds the row: lane l has columns l, l + 64, ...
template <typename A, int MAPS>
__device__ __forceinline__ void attn_finish_row(float* mrun, float* lrun, float (*acc)[4], const AttnForm& form, int row, int qh,
                                                int vdim, float factor, int lane, A* __restrict__ dst) {
  float res[4];
  if (form.sink) {   // rescale to the larger of the two maxima first
    const float sk = ld(static_cast<const A*>(form.sink) + qh);
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      const float mnew = fmaxf(mrun[m], sk);
      const float corr = mrun[m] == -INFINITY ? 0.f : expf(mrun[m] - mnew);
      lrun[m] = lrun[m] * corr + expf(sk - mnew);
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[m][c] *= corr;
    }
  }
  if constexpr (MAPS == 1) {
    const float invl = 1.0f / lrun[0];
#pragma unroll
    for (int c = 0; c < 4; ++c) res[c] = acc[0][c] * invl;
  } else {
    const float inv0 = 1.0f / lrun[0], inv1 = form.lambda / lrun[MAPS - 1];
#pragma unroll
    for (int c = 0; c < 4; ++c) res[c] = acc[0][c] * inv0 - acc[MAPS - 1][c] * inv1;
  }
  float post = factor;
  if (form.head_norm) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (lane + 64 * c < vdim) ss = fmaf(res[c], res[c], ss);
    post = factor / sqrtf(wave_sum(ss) / (float)vdim + form.norm_eps);
  }
  if (form.gate_kind == 2) post *= sigmoid_f(ld(static_cast<const A*>(form.gate) + (int64_t)row * form.gate_stride + qh));
#pragma unroll
  for (int c = 0; c < 4; ++c)
    if (lane + 64 * c < vdim) {
      float v = res[c] * post;
      if (form.gate_kind == 1)
        v *= sigmoid_f(ld(static_cast<const A*>(form.gate) + (int64_t)row * form.gate_stride + (int64_t)qh * vdim + lane + 64 * c));
      st(dst + lane + 64 * c, v);
    }
}

template <typename A, int MAPS>
__global__ __launch_bounds__(256) void paged_attention_kernel(
    const float* __restrict__ q, const A* __restrict__ cache, int64_t page_stride, int64_t k_cache_off, int64_t v_cache_off,
    int page_size, const int32_t* __restrict__ positions, const int32_t* __restrict__ row_entry,
    const int32_t* __restrict__ page_indptr, const int32_t* __restrict__ page_ids, int H, int G, int dim, int vdim, float scale,
    float factor, const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ tile_ntok,
    const int32_t* __restrict__ tile_qh0, const int32_t* __restrict__ tile_nqh, A* __restrict__ out, int64_t out_stride,
    AttnForm form, int nsplit, float* __restrict__ part) {
  extern __shared__ float sm[];
  const int qd = MAPS * dim;                          // values of one query / key head (all maps)
  const int kd = qd + 1;                              // padded key row: a lane per key reads its row without bank conflicts
  float* s_k = sm;                                    // [64][qd + 1]
  float* s_v = s_k + kAttKeys * kd;                   // [64][vdim]
  float* s_q = s_v + kAttKeys * vdim;                 // [16][qd]
  float* s_p = s_q + kAttRows * qd;                   // [4 waves][MAPS][64 keys][4 rows of the wave]
  // 16-byte loads from the cache: every key / value row of the request starts at a multiple of eight values
  const bool vec_k = (qd & 7) == 0 && (page_stride & 7) == 0 && (k_cache_off & 7) == 0 && aligned16(cache);
  const bool vec_v = (vdim & 7) == 0 && (page_stride & 7) == 0 && (v_cache_off & 7) == 0 && aligned16(cache);
  const int tile = blockIdx.x, g = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int row0 = tile_row0[tile], ntok = tile_ntok[tile], qh0 = tile_qh0[tile], nqh = tile_nqh[tile];
  const int nrows = ntok * nqh, per_group = H / G;
  const int e = row_entry[row0];
  const int32_t* pages = page_ids + page_indptr[e];
  const int kmax = positions[row0 + ntok - 1] + 1;    // keys 0 .. kmax - 1 are visible to the tile's last token
  // the first key any row of the tile sees, rounded down to the 64-key grid that starts at position 0
  const int lo0 = attn_row_lo(form, positions[row0]);   // rows of a tile are in position order: the lowest run start
  const int kfirst = form.keep_first > 0 ? 0 : (lo0 / kAttKeys) * kAttKeys;
  for (int i = tid; i < nrows * qd; i += 256) {
    const int lr = i / qd, d = i % qd;
    const int tok = lr / nqh, qh = g * per_group + qh0 + lr % nqh;
    s_q[lr * qd + d] = q[((int64_t)(row0 + tok) * H + qh) * qd + d];
  }
  float mrun[kAttRpw][MAPS], lrun[kAttRpw][MAPS], acc[kAttRpw][MAPS][4];
  int rpos[kAttRpw], rlo[kAttRpw], rqh[kAttRpw];
#pragma unroll
  for (int i = 0; i < kAttRpw; ++i) {
    const int lr = wave + 4 * i;
    rpos[i] = lr < nrows ? positions[row0 + lr / nqh] : -1;
    rlo[i] = rpos[i] >= 0 ? attn_row_lo(form, rpos[i]) : 0;
    rqh[i] = g * per_group + qh0 + (lr < nrows ? lr % nqh : 0);
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      mrun[i][m] = -INFINITY;
      lrun[i][m] = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[i][m][c] = 0.f;
    }
  }
  // nsplit > 1: workgroup z of the tile takes key tiles z, z + nsplit, ... (the count of splits does not depend on the
  // context's length, so a recorded launch serves every later length) and leaves its softmax state to the merge kernel
  for (int k0 = kfirst + (int)blockIdx.z * kAttKeys; k0 < kmax; k0 += kAttKeys * nsplit) {
    const int nk = min(kAttKeys, kmax - k0);
    // a tile between the kept first tokens and the lowest run start is seen by no row (uniform over the workgroup)
    if (k0 >= form.keep_first && k0 + kAttKeys <= lo0) continue;
    __syncthreads();
    {   // staging: four threads per key; one page lookup per thread and tile, 16-byte loads where the layout allows
      const int j = tid >> 2, sub = tid & 3;
      if (j < nk) {
        const int p = k0 + j;
        const int64_t pg = (int64_t)pages[p / page_size] * page_stride;
        const A* kp = cache + pg + k_cache_off + ((int64_t)(p % page_size) * G + g) * qd;
        const A* vp = cache + pg + v_cache_off + ((int64_t)(p % page_size) * G + g) * vdim;
        float* dk = s_k + j * kd;
        float* dv = s_v + j * vdim;
        if (vec_k) {
          for (int d = sub * 8; d < qd; d += 32) {
            float t[8];
            Vec8<A>::load(kp + d, t);
#pragma unroll
            for (int u = 0; u < 8; ++u) dk[d + u] = t[u];
          }
        } else {
          for (int d = sub; d < qd; d += 4) dk[d] = ld(kp + d);
        }
        if (vec_v) {
          for (int d = sub * 8; d < vdim; d += 32) {
            float t[8];
            Vec8<A>::load(vp + d, t);
#pragma unroll
            for (int u = 0; u < 8; ++u) dv[d + u] = t[u];
          }
        } else {
          for (int d = sub; d < vdim; d += 4) dv[d] = ld(vp + d);
        }
      }
    }
    __syncthreads();
    // the wave's (up to) four rows go through the tile together: a key value read from LDS serves four products
    bool act[kAttRpw];
    int jlo = nk, jhi = 0;
    bool any = false;
#pragma unroll
    for (int i = 0; i < kAttRpw; ++i) {
      const int lr = wave + 4 * i;
      // a row whose position lies before the tile, or whose run of visible keys begins after it, is left as it is
      act[i] = lr < nrows && k0 <= rpos[i] && (k0 + nk > rlo[i] || k0 < form.keep_first);
      if (act[i]) {
        any = true;
        jlo = min(jlo, k0 < form.keep_first ? 0 : max(0, rlo[i] - k0));
        jhi = max(jhi, min(nk, rpos[i] - k0 + 1));
      }
    }
    if (!any) continue;       // uniform over the wave; the barriers are at the head of the loop, which every wave reaches
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      float a[kAttRpw] = {0.f, 0.f, 0.f, 0.f};
      if (lane < nk) {
        const float* kr = s_k + lane * kd + m * dim;
        const float* qb = s_q + wave * qd + m * dim;        // row i of the wave: + 4 * i * qd
        if ((dim & 3) == 0) {
          for (int d = 0; d < dim; d += 4) {
            const float k0v = kr[d], k1v = kr[d + 1], k2v = kr[d + 2], k3v = kr[d + 3];
#pragma unroll
            for (int i = 0; i < kAttRpw; ++i) {
              const f32x4 qv = *reinterpret_cast<const f32x4*>(qb + 4 * i * qd + d);
              a[i] = fmaf(qv.x, k0v, a[i]);
              a[i] = fmaf(qv.y, k1v, a[i]);
              a[i] = fmaf(qv.z, k2v, a[i]);
              a[i] = fmaf(qv.w, k3v, a[i]);
            }
          }
        } else {
          for (int d = 0; d < dim; ++d) {
            const float kv = kr[d];
#pragma unroll
            for (int i = 0; i < kAttRpw; ++i) a[i] = fmaf(qb[4 * i * qd + d], kv, a[i]);
          }
        }
      }
      float* pw = s_p + (wave * MAPS + m) * (64 * kAttRpw);   // [key][row of the wave]
      float corr[kAttRpw];
#pragma unroll
      for (int i = 0; i < kAttRpw; ++i) {
        corr[i] = 1.0f;
        float pv = 0.f;
        if (act[i]) {
          const int kp_ = k0 + lane;
          const bool seen = lane < nk && kp_ <= rpos[i] && (kp_ >= rlo[i] || kp_ < form.keep_first);
          const float sc = seen ? attn_score(form, a[i], scale, rpos[i], kp_, rqh[i], H) : -INFINITY;
          const float mnew = fmaxf(mrun[i][m], wave_max(sc));
          pv = sc == -INFINITY ? 0.f : expf(sc - mnew);
          corr[i] = mrun[i][m] == -INFINITY ? 0.f : expf(mrun[i][m] - mnew);
          lrun[i][m] = lrun[i][m] * corr[i] + wave_sum(pv);
          mrun[i][m] = mnew;
        }
        pw[lane * kAttRpw + i] = pv;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int col = lane + 64 * c;
        if (col < vdim) {
          float o0 = act[0] ? acc[0][m][c] * corr[0] : acc[0][m][c], o1 = act[1] ? acc[1][m][c] * corr[1] : acc[1][m][c],
                o2 = act[2] ? acc[2][m][c] * corr[2] : acc[2][m][c], o3 = act[3] ? acc[3][m][c] * corr[3] : acc[3][m][c];
          for (int j = jlo; j < jhi; ++j) {    // weights outside a row's own range are exact zeros: they add nothing
            const f32x4 pj = *reinterpret_cast<const f32x4*>(pw + j * kAttRpw);
            const float v = s_v[j * vdim + col];
            o0 = fmaf(pj.x, v, o0);
            o1 = fmaf(pj.y, v, o1);
            o2 = fmaf(pj.z, v, o2);
            o3 = fmaf(pj.w, v, o3);
          }
          acc[0][m][c] = o0; acc[1][m][c] = o1; acc[2][m][c] = o2; acc[3][m][c] = o3;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (nsplit > 1) {   // [tile][kv head][split][row][map][vdim values | maximum | sum]
    float* pb = part + (((int64_t)(tile * G + g) * nsplit + blockIdx.z) * kAttRows) * MAPS * (vdim + 2);
#pragma unroll
    for (int i = 0; i < kAttRpw; ++i) {
      const int lr = wave + 4 * i;
      if (lr >= nrows) continue;
#pragma unroll
      for (int m = 0; m < MAPS; ++m) {
        float* pr = pb + ((int64_t)lr * MAPS + m) * (vdim + 2);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (lane + 64 * c < vdim) pr[lane + 64 * c] = acc[i][m][c];
        if (lane == 0) { pr[vdim] = mrun[i][m]; pr[vdim + 1] = lrun[i][m]; }
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < kAttRpw; ++i) {
    const int lr = wave + 4 * i;
    if (lr >= nrows) continue;
    const int tok = lr / nqh, qh = g * per_group + qh0 + lr % nqh;
    attn_finish_row<A, MAPS>(mrun[i], lrun[i], acc[i], form, row0 + tok, qh, vdim, factor, lane,
                             out + (int64_t)(row0 + tok) * out_stride + (int64_t)qh * vdim);
  }
}

// The same attention on the matrix cores, for a bf16 cache (v_mfma_f32_16x16x16_bf16 for both products).  Same tiles: up to 16
// (token, query head) rows of one key/value head per workgroup, key tiles of 64 positions on the grid that starts at position 0.
// Each of the four waves owns 16 keys of a tile and is a softmax stream of its own over them (its own running maximum, sum and
// output block for all 16 rows), so a tile costs no exchange between waves; the four streams are folded once, after the last
// tile, through LDS.  A wave computes S^T = K Q^T: the result leaves lane l with the scores of row l % 16 against keys
// 4 (l / 16) .. + 3 - exactly the A operand (weights, rounded to bf16) the second product P V wants from it; its B operand comes
// from a transposed copy of the value tile in LDS.  Scores, maxima, sums and outputs are fp32; q and the weights are rounded to
// bf16 where they enter the matrix cores, and the row sum is taken over the rounded weights.  dim is padded to a multiple of
// 16 per map, vdim to NCB * 16 columns (zeros).
typedef short v4s_t __attribute__((ext_vector_type(4)));
constexpr int kMfVs = kAttKeys + 4;     // row stride of the transposed value tile (bf16 values; 8-byte aligned rows)

template <int MAPS, int NCB>
__global__ __launch_bounds__(256) void paged_attention_mfma_kernel(
    const float* __restrict__ q, const uint16_t* __restrict__ cache, int64_t page_stride, int64_t k_cache_off, int64_t v_cache_off,
    int page_size, const int32_t* __restrict__ positions, const int32_t* __restrict__ row_entry,
    const int32_t* __restrict__ page_indptr, const int32_t* __restrict__ page_ids, int H, int G, int dim, int vdim, float scale,
    float factor, const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ tile_ntok,
    const int32_t* __restrict__ tile_qh0, const int32_t* __restrict__ tile_nqh, uint16_t* __restrict__ out, int64_t out_stride,
    AttnForm form, int nsplit, float* __restrict__ part) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smraw[];
  constexpr int VP = NCB * 16;
  const int qd = MAPS * dim, dp = (dim + 15) & ~15, ks = MAPS * dp + 4;
  uint16_t* s_k = reinterpret_cast<uint16_t*>(smraw);        // [64][ks]
  uint16_t* s_q = s_k + kAttKeys * ks;                         // [16][ks]
  uint16_t* s_vt = s_q + kAttRows * ks;                        // [VP][kMfVs]: value column major
  float* f_buf = reinterpret_cast<float*>(smraw);              // after the last tile: [2][MAPS][16][VP] partial outputs,
  float* f_st = f_buf + 2 * MAPS * kAttRows * VP;              //   [4 waves][MAPS][16][2] maxima and sums, [MAPS][16][2] folded
  float* f_fin = f_st + 4 * MAPS * kAttRows * 2;
  const int tile = blockIdx.x, g = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lrow = lane & 15, lgrp = lane >> 4;
  const int row0 = tile_row0[tile], ntok = tile_ntok[tile], qh0 = tile_qh0[tile], nqh = tile_nqh[tile];
  const int nrows = ntok * nqh, per_group = H / G;
  const int e = row_entry[row0];
  const int32_t* pages = page_ids + page_indptr[e];
  const int kmax = positions[row0 + ntok - 1] + 1;
  const int lo0 = attn_row_lo(form, positions[row0]);   // rows of a tile are in position order: the lowest run start
  const int kfirst = form.keep_first > 0 ? 0 : (lo0 / kAttKeys) * kAttKeys;
  // zeros everywhere first: padding columns, rows past the tile's, keys past the context's end must multiply as zeros
  {   // (the tiles' bytes are a multiple of 16: ks is a multiple of 4 values, the row counts of 16, VP * kMfVs of 8)
    u32x4* z = reinterpret_cast<u32x4*>(smraw);
    for (int i = tid; i < ((kAttKeys + kAttRows) * ks + VP * kMfVs) / 8; i += 256) z[i] = u32x4{0u, 0u, 0u, 0u};
  }
  __syncthreads();
  for (int i = tid; i < nrows * qd; i += 256) {
    const int lr = i / qd, c = i % qd;
    const int tok = lr / nqh, qh = g * per_group + qh0 + lr % nqh;
    s_q[lr * ks + (c / dim) * dp + c % dim] = f2bf(q[((int64_t)(row0 + tok) * H + qh) * qd + c]);
  }
  const int rpos = lrow < nrows ? positions[row0 + lrow / nqh] : -1;      // this lane's row (as a column of S^T)
  const int rlo = rpos >= 0 ? attn_row_lo(form, rpos) : 0;
  const int lqh = g * per_group + qh0 + (lrow < nrows ? lrow % nqh : 0);
  float mrun[MAPS], lrun[MAPS];
  f32x4 o[MAPS][NCB];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) {
    mrun[m] = -INFINITY;
    lrun[m] = 0.f;
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) o[m][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const bool vec_k = (dim & 7) == 0 && (page_stride & 7) == 0 && (k_cache_off & 7) == 0 && aligned16(cache);
  const bool vec_v = (vdim & 7) == 0 && (page_stride & 7) == 0 && (v_cache_off & 7) == 0 && aligned16(cache);
  for (int k0 = kfirst + (int)blockIdx.z * kAttKeys; k0 < kmax; k0 += kAttKeys * nsplit) {
    const int nk = min(kAttKeys, kmax - k0);
    if (k0 >= form.keep_first && k0 + kAttKeys <= lo0) continue;   // seen by no row of the tile (uniform over the workgroup)
    __syncthreads();
    {   // staging: four threads per key; the value tile is written transposed
      const int j = tid >> 2, sub = tid & 3;
      if (j < nk) {
        const int p = k0 + j;
        const int64_t pg = (int64_t)pages[p / page_size] * page_stride;
        const uint16_t* kp = cache + pg + k_cache_off + ((int64_t)(p % page_size) * G + g) * qd;
        const uint16_t* vp = cache + pg + v_cache_off + ((int64_t)(p % page_size) * G + g) * vdim;
        uint16_t* dk = s_k + j * ks;
        if (vec_k) {
          for (int c = sub * 8; c < qd; c += 32) {
            const u32x4 t = *reinterpret_cast<const u32x4*>(kp + c);
            uint16_t* dst = dk + (c / dim) * dp + c % dim;           // 8-byte aligned (ks * 2 is a multiple of 8 only)
            *reinterpret_cast<u32x2*>(dst) = u32x2{t.x, t.y};
            *reinterpret_cast<u32x2*>(dst + 4) = u32x2{t.z, t.w};
          }
        } else {
          for (int c = sub; c < qd; c += 4) dk[(c / dim) * dp + c % dim] = kp[c];
        }
        if (vec_v) {
          for (int c = sub * 8; c < vdim; c += 32) {
            const u32x4 t = *reinterpret_cast<const u32x4*>(vp + c);
            const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              s_vt[(c + 2 * u) * kMfVs + j] = (uint16_t)(w[u] & 0xFFFFu);
              s_vt[(c + 2 * u + 1) * kMfVs + j] = (uint16_t)(w[u] >> 16);
            }
          }
        } else {
          for (int c = sub; c < vdim; c += 4) s_vt[c * kMfVs + j] = vp[c];
        }
      }
    }
    __syncthreads();
    const int kb = wave * 16;                       // this wave's keys of the tile
    if (k0 + kb >= kmax) continue;                  // uniform over the wave; barriers sit at the loop's head
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
      const uint16_t* ka = s_k + (kb + lrow) * ks + m * dp + 4 * lgrp;
      const uint16_t* qb = s_q + lrow * ks + m * dp + 4 * lgrp;
      for (int kk = 0; kk < dp; kk += 16)
        sc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const v4s_t*>(ka + kk), *reinterpret_cast<const v4s_t*>(qb + kk),
                                                       sc, 0, 0, 0);
      float sv[4] = {sc.x, sc.y, sc.z, sc.w};
      float tmax = -INFINITY;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kp_ = k0 + kb + 4 * lgrp + r;
        sv[r] = (kp_ <= rpos && (kp_ >= rlo || kp_ < form.keep_first)) ? attn_score(form, sv[r], scale, rpos, kp_, lqh, H) : -INFINITY;
        tmax = fmaxf(tmax, sv[r]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float mnew = fmaxf(mrun[m], tmax);
      const float corr = mnew == -INFINITY ? 1.0f : (mrun[m] == -INFINITY ? 0.f : expf(mrun[m] - mnew));
      uint16_t pb[4];
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pb[r] = f2bf(sv[r] == -INFINITY ? 0.f : expf(sv[r] - mnew));
        psum += bf2f(pb[r]);
      }
      psum += __shfl_xor(psum, 16, kWave);
      psum += __shfl_xor(psum, 32, kWave);
      lrun[m] = lrun[m] * corr + psum;
      mrun[m] = mnew;
      // the output block holds rows 4 (l / 16) + r: their factors sit in the lanes of those numbers
      float cr[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, 4 * lgrp + r, kWave);
      v4s_t pa;
      pa.x = (short)pb[0]; pa.y = (short)pb[1]; pa.z = (short)pb[2]; pa.w = (short)pb[3];
      const uint16_t* vb = s_vt + lrow * kMfVs + kb + 4 * lgrp;
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        f32x4 t = o[m][cb];
        t.x *= cr[0]; t.y *= cr[1]; t.z *= cr[2]; t.w *= cr[3];
        o[m][cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa, *reinterpret_cast<const v4s_t*>(vb + cb * 16 * kMfVs), t, 0, 0, 0);
      }
    }
  }
  __syncthreads();                                  // the tiles' LDS is free: the four streams are folded through it
  if (lane < 16) {
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      f_st[((wave * MAPS + m) * kAttRows + lane) * 2] = mrun[m];
      f_st[((wave * MAPS + m) * kAttRows + lane) * 2 + 1] = lrun[m];
    }
  }
  __syncthreads();
#pragma unroll
  for (int m = 0; m < MAPS; ++m) {
    float mall = -INFINITY, lall = 0.f, mine = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) mall = fmaxf(mall, f_st[((w * MAPS + m) * kAttRows + lrow) * 2]);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = f_st[((w * MAPS + m) * kAttRows + lrow) * 2];
      const float sw = mw == -INFINITY ? 0.f : expf(mw - mall);
      lall += f_st[((w * MAPS + m) * kAttRows + lrow) * 2 + 1] * sw;
      if (w == wave) mine = sw;
    }
    if (wave == 0 && lane < 16) {
      f_fin[(m * kAttRows + lane) * 2] = mall;
      f_fin[(m * kAttRows + lane) * 2 + 1] = lall;
    }
    float cr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) cr[r] = __shfl(mine, 4 * lgrp + r, kWave);
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) { o[m][cb].x *= cr[0]; o[m][cb].y *= cr[1]; o[m][cb].z *= cr[2]; o[m][cb].w *= cr[3]; }
  }
  // element (map m, row 4 (l / 16) + r, column 16 cb + l % 16) of a wave's block
  auto slot = [&](int b, int m, int cb, int r) { return f_buf + ((b * MAPS + m) * kAttRows + 4 * lgrp + r) * VP + cb * 16 + lrow; };
  auto put = [&](int b) {
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) { *slot(b, m, cb, 0) = o[m][cb].x; *slot(b, m, cb, 1) = o[m][cb].y; *slot(b, m, cb, 2) = o[m][cb].z; *slot(b, m, cb, 3) = o[m][cb].w; }
  };
  auto take = [&](int b) {
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) { o[m][cb].x += *slot(b, m, cb, 0); o[m][cb].y += *slot(b, m, cb, 1); o[m][cb].z += *slot(b, m, cb, 2); o[m][cb].w += *slot(b, m, cb, 3); }
  };
  if (wave >= 2) put(wave - 2);
  __syncthreads();
  if (wave < 2) take(wave);
  __syncthreads();
  if (wave == 1) put(0);
  __syncthreads();
  if (wave == 0) { take(0); put(0); }
  __syncthreads();
  // rows go back to the layout of the plain kernel: wave w finishes rows w, w + 4, ...; a lane holds columns l, l + 64, ...
  float* pbase = nsplit > 1 ? part + (((int64_t)(tile * G + g) * nsplit + blockIdx.z) * kAttRows) * MAPS * (vdim + 2) : nullptr;
  for (int lr = wave; lr < nrows; lr += 4) {
    float fm[MAPS], fl[MAPS], acc[MAPS][4];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      fm[m] = f_fin[(m * kAttRows + lr) * 2];
      fl[m] = f_fin[(m * kAttRows + lr) * 2 + 1];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[m][c] = lane + 64 * c < vdim ? f_buf[(m * kAttRows + lr) * VP + lane + 64 * c] : 0.f;
    }
    if (nsplit > 1) {
#pragma unroll
      for (int m = 0; m < MAPS; ++m) {
        float* pr = pbase + ((int64_t)lr * MAPS + m) * (vdim + 2);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (lane + 64 * c < vdim) pr[lane + 64 * c] = acc[m][c];
        if (lane == 0) { pr[vdim] = fm[m]; pr[vdim + 1] = fl[m]; }
      }
      continue;
    }
    const int tok = lr / nqh, qh = g * per_group + qh0 + lr % nqh;
    attn_finish_row<uint16_t, MAPS>(fm, fl, acc, form, row0 + tok, qh, vdim, factor, lane, out + (int64_t)(row0 + tok) * out_stride + (int64_t)qh * vdim);
  }
}

// bytes of LDS the matrix-core kernel needs: the tiles while the keys are walked, the fold buffers afterwards
static size_t mfma_attention_lds(int maps, int dim, int ncb) {
  const size_t ks = (size_t)maps * ((dim + 15) & ~15) + 4, vp = (size_t)ncb * 16;
  const size_t tiles = ((kAttKeys + kAttRows) * ks + vp * kMfVs) * sizeof(uint16_t);
  const size_t fold = (2 * maps * kAttRows * vp + 4 * maps * kAttRows * 2 + maps * kAttRows * 2) * sizeof(float);
  return std::max(tiles, fold);
}

// The states that the splits of a tile have left, brought to their common maximum and summed in split order, then finished like
// an unsplit row.
template <typename A, int MAPS>
__global__ __launch_bounds__(256) void paged_attention_merge_kernel(
    const float* __restrict__ part, int nsplit, int H, int G, int vdim, float factor, const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ tile_ntok, const int32_t* __restrict__ tile_qh0, const int32_t* __restrict__ tile_nqh,
    A* __restrict__ out, int64_t out_stride, AttnForm form) {
  const int tile = blockIdx.x, g = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int row0 = tile_row0[tile], ntok = tile_ntok[tile], qh0 = tile_qh0[tile], nqh = tile_nqh[tile];
  const int nrows = ntok * nqh, per_group = H / G;
  for (int lr = wave; lr < nrows; lr += 4) {
    float mrun[MAPS], lrun[MAPS], acc[MAPS][4];
    const int64_t zs = (int64_t)kAttRows * MAPS * (vdim + 2);      // floats between two splits of a row
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      // lane z reads split z's maximum and sum; the common maximum and every split's weight follow without a dependent load,
      // and the value loads of all splits are in flight together (nsplit <= 64)
      const float* pr = part + ((((int64_t)(tile * G + g) * nsplit) * kAttRows + lr) * MAPS + m) * (vdim + 2);
      const float mz = lane < nsplit ? pr[lane * zs + vdim] : -INFINITY;
      const float lz = lane < nsplit ? pr[lane * zs + vdim + 1] : 0.f;
      const float mall = wave_max(mz);
      const float wz = mz == -INFINITY ? 0.f : expf(mz - mall);     // 0: a split that met no visible key
      mrun[m] = mall;
      lrun[m] = wave_sum(lz * wz);
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[m][c] = 0.f;
      for (int z0 = 0; z0 < nsplit; z0 += 8) {      // eight splits' values requested before the first is used
        float val[8][4];
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
          for (int c = 0; c < 4; ++c)
            val[u][c] = z0 + u < nsplit && lane + 64 * c < vdim ? pr[(z0 + u) * zs + lane + 64 * c] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const float w = __shfl(wz, min(z0 + u, 63), kWave);
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[m][c] = fmaf(val[u][c], w, acc[m][c]);
        }
      }
    }
    const int tok = lr / nqh, qh = g * per_group + qh0 + lr % nqh;
    attn_finish_row<A, MAPS>(mrun, lrun, acc, form, row0 + tok, qh, vdim, factor, lane, out + (int64_t)(row0 + tok) * out_stride + (int64_t)qh * vdim);
  }
}

// out[row, :cols] = in[row, :cols] * factor, rows of either side at their own stride
template <typename A>
__global__ __launch_bounds__(256) void scale_rows_kernel(const A* __restrict__ in, int64_t in_stride, A* __restrict__ out,
                                                         int64_t out_stride, int cols, float factor) {
  const int row = blockIdx.x;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < cols; i += gridDim.y * 256)
    st(out + (int64_t)row * out_stride + i, ld(in + (int64_t)row * in_stride + i) * factor);
}

}  // namespace pk

extern "C" {
using namespace pk;

#define PK_BAD ((pegainfer_status_t)hipErrorInvalidValue)

pegainfer_status_t pegainfer_qk_prep_paged(const void* proj, int64_t proj_stride, int64_t q_off, int64_t k_off, int64_t v_off,
                                          int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, const void* q_norm,
                                          const void* k_norm, float eps, const void* q_bias, const void* k_bias,
                                          const void* v_bias, float qt_coef, int32_t qt_every, const float* inv_freq,
                                          int32_t rot_dims, const int32_t* positions, const int32_t* row_entry,
                                          const int32_t* page_indptr, const int32_t* page_ids, void* cache, int64_t page_stride,
                                          int64_t k_cache_off, int64_t v_cache_off, int32_t page_size, float* q_out,
                                          void* q_out_stored, int32_t n_rows, int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_qk_prep_paged_form(proj, dtype, proj_stride, q_off, k_off, v_off, heads, kv_heads, dim, vdim, q_norm, k_norm,
                                      PEGAINFER_QKNORM_HEAD_WEIGHT, eps, q_bias, k_bias, v_bias, qt_coef, qt_every, inv_freq, rot_dims,
                                      PEGAINFER_ROT_PAIRS, positions, row_entry, page_indptr, page_ids, cache, page_stride, k_cache_off,
                                      v_cache_off, page_size, q_out, q_out_stored, n_rows, dtype, stream);
}

pegainfer_status_t pegainfer_qk_prep_paged_form(const void* proj, int32_t proj_dtype, int64_t proj_stride, int64_t q_off,
                                               int64_t k_off, int64_t v_off, int32_t heads, int32_t kv_heads, int32_t dim,
                                               int32_t vdim, const void* q_norm, const void* k_norm, int32_t norm_kind, float eps,
                                               const void* q_bias, const void* k_bias, const void* v_bias, float qt_coef,
                                               int32_t qt_every, const float* inv_freq, int32_t rot_dims, int32_t rot_layout,
                                               const int32_t* positions, const int32_t* row_entry, const int32_t* page_indptr,
                                               const int32_t* page_ids, void* cache, int64_t page_stride, int64_t k_cache_off,
                                               int64_t v_cache_off, int32_t page_size, float* q_out, void* q_out_stored,
                                               int32_t n_rows, int32_t dtype, pegainfer_stream_t stream) {
  if (n_rows <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || rot_dims < 0 || rot_dims > dim || (rot_dims & 1) ||
      page_size <= 0 || (rot_dims > 0 && !inv_freq) || (!q_norm) != (!k_norm) || norm_kind < 0 || norm_kind > 2 ||
      (norm_kind == PEGAINFER_QKNORM_ALL_WEIGHT && !q_norm) || (rot_layout != PEGAINFER_ROT_PAIRS && rot_layout != PEGAINFER_ROT_HALVES))
    return PK_BAD;
  PrepForm pf;
  pf.norm_kind = norm_kind;
  pf.rot_halves = rot_layout == PEGAINFER_ROT_HALVES;
  bool ok = true;
  const bool known = by_dtype(dtype, [&](auto* t) {
    using A = std::remove_pointer_t<decltype(t)>;
    ok = by_dtype(proj_dtype, [&](auto* ti) {
      using I = std::remove_pointer_t<decltype(ti)>;
      // few rows (decoding): the heads of a row spread over several workgroups, four heads each; many rows fill the chip alone
      const int per_row = n_rows >= 512 ? 1 : std::min(16, ceil_div(heads + kv_heads, 4));
      qk_prep_paged_kernel<A, I><<<dim3(n_rows, per_row), 256, (size_t)4 * dim * sizeof(float), as_stream(stream)>>>(
          static_cast<const I*>(proj), proj_stride, q_off, k_off, v_off, heads, kv_heads, dim, vdim, static_cast<const A*>(q_norm),
          static_cast<const A*>(k_norm), eps, inv_freq, rot_dims, positions, row_entry, page_indptr, page_ids, static_cast<A*>(cache),
          page_stride, k_cache_off, v_cache_off, page_size, q_out, static_cast<A*>(q_out_stored), static_cast<const A*>(q_bias),
          static_cast<const A*>(k_bias), static_cast<const A*>(v_bias), qt_coef, qt_every, pf);
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_qk_norm_rope_paged(const void* proj, int64_t proj_stride, int64_t q_off, int64_t k_off,
                                                int64_t v_off, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim,
                                                const void* q_norm, const void* k_norm, float eps, const float* inv_freq,
                                                int32_t rot_dims, const int32_t* positions, const int32_t* row_entry,
                                                const int32_t* page_indptr, const int32_t* page_ids, void* cache,
                                                int64_t page_stride, int64_t k_cache_off, int64_t v_cache_off,
                                                int32_t page_size, float* q_out, void* q_out_stored, int32_t n_rows,
                                                int32_t dtype, pegainfer_stream_t stream) {
  if (!q_norm || !k_norm) return PK_BAD;
  return pegainfer_qk_prep_paged(proj, proj_stride, q_off, k_off, v_off, heads, kv_heads, dim, vdim, q_norm, k_norm, eps, nullptr,
                                 nullptr, nullptr, 0.f, 0, inv_freq, rot_dims, positions, row_entry, page_indptr, page_ids, cache,
                                 page_stride, k_cache_off, v_cache_off, page_size, q_out, q_out_stored, n_rows, dtype, stream);
}

pegainfer_status_t pegainfer_paged_attention_ex(const float* q, const void* cache, int64_t page_stride, int64_t k_cache_off,
                                                int64_t v_cache_off, int32_t page_size, const int32_t* positions,
                                                const int32_t* row_entry, const int32_t* page_indptr, const int32_t* page_ids,
                                                int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float scale,
                                                float factor, const int32_t* tile_row0, const int32_t* tile_ntok,
                                                const int32_t* tile_qh0, const int32_t* tile_nqh, int32_t n_tiles, void* out,
                                                int64_t out_stride, int32_t maps, float lambda, int32_t block, const void* sink,
                                                int32_t head_norm, float norm_eps, int32_t n_split, float* workspace,
                                                int32_t plain, int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_paged_attention_masked(q, cache, page_stride, k_cache_off, v_cache_off, page_size, positions, row_entry, page_indptr,
                                          page_ids, heads, kv_heads, dim, vdim, scale, factor, tile_row0, tile_ntok, tile_qh0, tile_nqh,
                                          n_tiles, out, out_stride, maps, lambda, block, sink, head_norm, norm_eps, 0.f, 0, 0, nullptr, 0,
                                          nullptr, 0, 0, n_split, workspace, plain, dtype, stream);
}

pegainfer_status_t pegainfer_paged_attention_masked(const float* q, const void* cache, int64_t page_stride, int64_t k_cache_off,
                                                    int64_t v_cache_off, int32_t page_size, const int32_t* positions,
                                                    const int32_t* row_entry, const int32_t* page_indptr, const int32_t* page_ids,
                                                    int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float scale,
                                                    float factor, const int32_t* tile_row0, const int32_t* tile_ntok,
                                                    const int32_t* tile_qh0, const int32_t* tile_nqh, int32_t n_tiles, void* out,
                                                    int64_t out_stride, int32_t maps, float lambda, int32_t block, const void* sink,
                                                    int32_t head_norm, float norm_eps, float softcap, int32_t window,
                                                    int32_t keep_first, const float* dist_bias, int32_t n_dist, const void* gate,
                                                    int64_t gate_stride, int32_t gate_kind, int32_t n_split, float* workspace,
                                                    int32_t plain, int32_t dtype, pegainfer_stream_t stream) {
  if (n_tiles <= 0) return 0;
  if (gate_kind < 0 || gate_kind > 2 || (gate_kind && !gate)) return PK_BAD;
  if (window < 0 || keep_first < 0 || (keep_first > 0 && window <= 0) || softcap < 0.f || (dist_bias && n_dist < 1)) return PK_BAD;
  if (n_split < 1) n_split = 1;
  if (n_split > 1 && (!workspace || n_split > 64)) return PK_BAD;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || (maps != 1 && maps != 2) || maps * dim > 256 || vdim <= 0 ||
      vdim > 256 || page_size <= 0 || kv_heads > 65535 || block < 0)
    return PK_BAD;
  const int qd = maps * dim;
  const size_t smem = ((size_t)kAttKeys * (qd + 1) + (size_t)kAttKeys * vdim + (size_t)kAttRows * qd + 4 * maps * 64 * kAttRpw) * sizeof(float);
  const dim3 grid(n_tiles, kv_heads, n_split);
  AttnForm form;
  form.block = block;
  form.sink = sink;
  form.lambda = lambda;
  form.head_norm = head_norm;
  form.norm_eps = norm_eps;
  form.softcap = softcap;
  form.window = window;
  form.keep_first = window > 0 ? keep_first : 0;
  form.dist_bias = dist_bias;
  form.n_dist = n_dist;
  form.gate = gate;
  form.gate_stride = gate_stride;
  form.gate_kind = gate_kind;
  bool ok = true;
  if (dtype == kDtBf16 && !plain) {   // bf16 cache: the matrix-core kernel; same tiles, same splits, same merge
    const int ncb = vdim <= 32 ? 2 : vdim <= 64 ? 4 : vdim <= 128 ? 8 : 16;
    const size_t lds = mfma_attention_lds(maps, dim, ncb);
    auto launch = [&](auto kern) {
      if (lds > 48 * 1024 &&
          hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        ok = false;
        return;
      }
      kern<<<grid, 256, lds, as_stream(stream)>>>(q, static_cast<const uint16_t*>(cache), page_stride, k_cache_off, v_cache_off, page_size,
                                                  positions, row_entry, page_indptr, page_ids, heads, kv_heads, dim, vdim, scale, factor,
                                                  tile_row0, tile_ntok, tile_qh0, tile_nqh, static_cast<uint16_t*>(out), out_stride, form,
                                                  n_split, workspace);
    };
    auto by_cols = [&](auto maps_c) {
      constexpr int M = decltype(maps_c)::value;
      if (ncb == 2) launch(paged_attention_mfma_kernel<M, 2>);
      else if (ncb == 4) launch(paged_attention_mfma_kernel<M, 4>);
      else if (ncb == 8) launch(paged_attention_mfma_kernel<M, 8>);
      else launch(paged_attention_mfma_kernel<M, 16>);
    };
    if (maps == 1) by_cols(std::integral_constant<int, 1>());
    else by_cols(std::integral_constant<int, 2>());
    if (ok && n_split > 1) {
      if (maps == 1)
        paged_attention_merge_kernel<uint16_t, 1><<<dim3(n_tiles, kv_heads), 256, 0, as_stream(stream)>>>(
            workspace, n_split, heads, kv_heads, vdim, factor, tile_row0, tile_ntok, tile_qh0, tile_nqh, static_cast<uint16_t*>(out), out_stride, form);
      else
        paged_attention_merge_kernel<uint16_t, 2><<<dim3(n_tiles, kv_heads), 256, 0, as_stream(stream)>>>(
            workspace, n_split, heads, kv_heads, vdim, factor, tile_row0, tile_ntok, tile_qh0, tile_nqh, static_cast<uint16_t*>(out), out_stride, form);
    }
    return ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
  }
  const bool known = by_dtype(dtype, [&](auto* t) {
    using A = std::remove_pointer_t<decltype(t)>;
    auto go = [&](auto kern) {
      if (smem > 48 * 1024 &&
          hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
        ok = false;
        return;
      }
      kern<<<grid, 256, smem, as_stream(stream)>>>(q, static_cast<const A*>(cache), page_stride, k_cache_off, v_cache_off,
                                                   page_size, positions, row_entry, page_indptr, page_ids, heads, kv_heads, dim,
                                                   vdim, scale, factor, tile_row0, tile_ntok, tile_qh0, tile_nqh,
                                                   static_cast<A*>(out), out_stride, form, n_split, workspace);
    };
    auto merge = [&](auto kern) {
      kern<<<dim3(n_tiles, kv_heads), 256, 0, as_stream(stream)>>>(workspace, n_split, heads, kv_heads, vdim, factor, tile_row0,
                                                                    tile_ntok, tile_qh0, tile_nqh, static_cast<A*>(out), out_stride, form);
    };
    if (maps == 1) {
      go(paged_attention_kernel<A, 1>);
      if (ok && n_split > 1) merge(paged_attention_merge_kernel<A, 1>);
    } else {
      go(paged_attention_kernel<A, 2>);
      if (ok && n_split > 1) merge(paged_attention_merge_kernel<A, 2>);
    }
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

int64_t pegainfer_paged_attention_workspace(int32_t n_tiles, int32_t kv_heads, int32_t vdim, int32_t maps, int32_t n_split) {
  return n_split > 1 ? (int64_t)n_tiles * kv_heads * n_split * kAttRows * maps * (vdim + 2) : 0;
}

pegainfer_status_t pegainfer_paged_attention(const float* q, const void* cache, int64_t page_stride, int64_t k_cache_off,
                                             int64_t v_cache_off, int32_t page_size, const int32_t* positions,
                                             const int32_t* row_entry, const int32_t* page_indptr, const int32_t* page_ids,
                                             int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float scale,
                                             float factor, const int32_t* tile_row0, const int32_t* tile_ntok,
                                             const int32_t* tile_qh0, const int32_t* tile_nqh, int32_t n_tiles, void* out,
                                             int64_t out_stride, int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_paged_attention_ex(q, cache, page_stride, k_cache_off, v_cache_off, page_size, positions, row_entry, page_indptr,
                                      page_ids, heads, kv_heads, dim, vdim, scale, factor, tile_row0, tile_ntok, tile_qh0, tile_nqh,
                                      n_tiles, out, out_stride, 1, 0.f, 0, nullptr, 0, 0.f, 1, nullptr, 1, dtype, stream);
}

pegainfer_status_t pegainfer_scale_rows(const void* in, int64_t in_stride, void* out, int64_t out_stride, int32_t cols,
                                        int32_t rows, float factor, int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0 || cols <= 0) return 0;
  const dim3 grid(rows, std::min(8, ceil_div(cols, 256)));
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        scale_rows_kernel<A><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const A*>(in), in_stride, static_cast<A*>(out),
                                                                  out_stride, cols, factor);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

}  // extern "C"

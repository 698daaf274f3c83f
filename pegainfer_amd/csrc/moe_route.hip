// Routed feed-forward: the router and the bookkeeping around the expert GEMMs (which run on the grouped form of
// pegainfer_gemm_strided).
//   route_kernel    one workgroup per token row: fp32 router logits (a wave per expert, lanes over the width), sigmoid
//                   scores, the correction added for the CHOICE only, group scores = the two largest choices of a group,
//                   the best `keep` groups stay eligible, then the `top` largest eligible choices; weights = the plain
//                   sigmoid scores of the chosen experts.  Selection runs on one wave: a lane per group for the group
//                   scores and ranks, then `top` wave-wide arg-max steps; ties go to the lower index.
//   sort_kernel     (row, choice) pairs bucketed by expert with LDS counters, an exclusive scan, and the table of <= 64-row
//                   tiles the grouped GEMM walks.  The order of pairs inside an expert comes from atomics; every pair owns
//                   its output row, so results do not depend on it.  Tiles hold <= 64 or <= 128 rows, as the GEMM form that walks them wants.
//   combine_kernel  out[row] = sum over the row's choices, in choice order, of weight * expert output (fp32 sum), plus a row
//                   every token gets (a shared expert), optionally times the sigmoid of a per-row gate logit.
// Options of the selection: a group's score = its two largest choices (default) or its largest; the chosen weights as they
// are (default) or divided by their sum.
#include <algorithm>

#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

// Selection on one wave from per-expert values in LDS (s: sigmoid scores, or logits when score is softmax; ch: s + correction):
// softmax over ALL experts if asked, group scores, kept groups, then `top` wave-wide arg-max steps.  LDS accesses of one wave
// complete in order, so no barrier is needed between its steps.
template <typename A>
__device__ __forceinline__ void route_select_wave(float* s, float* ch, float* gs, const A* __restrict__ corr,
                                                  int32_t* __restrict__ out_e, float* __restrict__ out_w, int row, int lane, int E,
                                                  int G, int keep, int top, int score, int group_kind = 0, int renorm = 0) {
  if (score == PEGAINFER_SCORE_SOFTMAX) {            // s = exp(z - max) / sum over ALL experts, then the choice scores
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, s[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) sum += expf(s[e] - mx);
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) {
      const float sc = expf(s[e] - mx) / sum;
      s[e] = sc;
      ch[e] = corr ? sc + ld(corr + e) : sc;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (G > 1) {
    const int per = E / G;
    for (int g = lane; g < G; g += 64) {             // a lane scores a group: its two largest choices
      float b0 = -INFINITY, b1 = -INFINITY;
      for (int i = 0; i < per; ++i) {
        const float v = ch[g * per + i];
        if (v > b0) { b1 = b0; b0 = v; } else if (v > b1) b1 = v;
      }
      gs[g] = per >= 2 && group_kind == PEGAINFER_GROUP_TOP2_SUM ? b0 + b1 : b0;
    }
    __builtin_amdgcn_wave_barrier();
    for (int g = lane; g < G; g += 64) {             // kept = fewer than `keep` groups rank ahead (ties: the lower index)
      const float mine = gs[g];
      int ahead = 0;
      for (int o = 0; o < G; ++o) {
        const float v = gs[o];
        ahead += (v > mine || (v == mine && o < g)) ? 1 : 0;
      }
      if (ahead >= keep)
        for (int i = 0; i < per; ++i) ch[g * per + i] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int be = 0x7FFFFFFF;
    for (int e = lane; e < E; e += 64) {             // ascending e per lane: the first maximum is the lowest index
      const float v = ch[e];
      if (v > bv) { bv = v; be = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, kWave);
      const int oe = __shfl_xor(be, off, kWave);
      if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; }
    }
    const bool found = bv != -INFINITY;
    if (lane == 0) {
      out_e[(size_t)row * top + k] = found ? be : 0;
      out_w[(size_t)row * top + k] = found ? s[be] : 0.f;
      if (found) ch[be] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (renorm && lane == 0) {   // the chosen weights divided by their sum (in choice order)
    float sum = 0.f;
    for (int k = 0; k < top; ++k) sum += out_w[(size_t)row * top + k];
    const float inv = 1.0f / (sum + 1e-20f);
    for (int k = 0; k < top; ++k) out_w[(size_t)row * top + k] *= inv;
  }
}

template <typename A>
__global__ __launch_bounds__(256) void route_kernel(const A* __restrict__ h, const A* __restrict__ wr,
                                                    const A* __restrict__ corr, int32_t* __restrict__ out_e,
                                                    float* __restrict__ out_w, int d, int E, int G, int keep, int top,
                                                    int score) {
  extern __shared__ float sm[];
  float* s = sm;            // [E] sigmoid scores
  float* ch = sm + E;       // [E] choice scores (eligible) or -inf
  float* gs = sm + 2 * E;   // [G] group scores
  const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const A* x = h + (size_t)row * d;
  const bool vec = (d & 7) == 0 && aligned16(x) && aligned16(wr);
  // a wave takes four experts at a time (four independent weight streams in flight), waves interleaved over the groups of four
  constexpr int EB = 4;
  for (int e0 = wave * EB; e0 < E; e0 += 4 * EB) {
    float a[EB] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      for (int i = lane * 8; i < d; i += 512) {
        float xv[8];
        Vec8<A>::load(x + i, xv);
#pragma unroll
        for (int q = 0; q < EB; ++q) {
          float wv[8];
          Vec8<A>::load(wr + (size_t)min(e0 + q, E - 1) * d + i, wv);
#pragma unroll
          for (int k = 0; k < 8; ++k) a[q] = fmaf(xv[k], wv[k], a[q]);
        }
      }
    } else {
      for (int i = lane; i < d; i += 64) {
        const float xv = ld(x + i);
#pragma unroll
        for (int q = 0; q < EB; ++q) a[q] = fmaf(xv, ld(wr + (size_t)min(e0 + q, E - 1) * d + i), a[q]);
      }
    }
#pragma unroll
    for (int q = 0; q < EB; ++q) {
      const float z = wave_sum(a[q]);
      const int e = e0 + q;
      if (lane == 0 && e < E) {
        const float sc = score == PEGAINFER_SCORE_SOFTMAX ? z : sigmoid_f(z);   // softmax: the logit for now
        s[e] = sc;
        ch[e] = corr ? sc + ld(corr + e) : sc;
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  route_select_wave(s, ch, gs, corr, out_e, out_w, row, lane, E, G, keep, top, score);
}

// The same selection from router logits that a GEMM has left in fp32 ([rows][E]): a wave per row, four rows per workgroup.
template <typename A>
__global__ __launch_bounds__(256) void route_from_logits_kernel(const float* __restrict__ logits, const A* __restrict__ corr,
                                                                int32_t* __restrict__ out_e, float* __restrict__ out_w, int E,
                                                                int G, int keep, int top, int rows, int score,
                                                                int64_t logits_stride, int group_kind, int renorm) {
  extern __shared__ float sm[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + wave;
  if (row >= rows) return;
  float* s = sm + wave * (2 * E + G);
  float* ch = s + E;
  float* gs = s + 2 * E;
  for (int e = lane; e < E; e += 64) {
    const float z = logits[(size_t)row * logits_stride + e];
    const float sc = score == PEGAINFER_SCORE_SOFTMAX ? z : sigmoid_f(z);
    s[e] = sc;
    ch[e] = corr ? sc + ld(corr + e) : sc;
  }
  __builtin_amdgcn_wave_barrier();
  route_select_wave(s, ch, gs, corr, out_e, out_w, row, lane, E, G, keep, top, score, group_kind, renorm);
}

__global__ __launch_bounds__(256) void route_sort_kernel(const int32_t* __restrict__ expert, int n_pairs, int top, int E,
                                                         int32_t* __restrict__ pos_pair, int32_t* __restrict__ pos_row,
                                                         int32_t* __restrict__ tile_group, int32_t* __restrict__ tile_row0,
                                                         int32_t* __restrict__ tile_rows, int32_t* __restrict__ n_tiles,
                                                         int max_tiles, int per_tile) {
  extern __shared__ int cnt[];   // [E] counts, then [E] cursors
  int* cur = cnt + E;
  for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += 256) atomicAdd(&cnt[expert[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cnt[e];
      cur[e] = off;
      for (int r0 = 0; r0 < c && nt < max_tiles; r0 += per_tile, ++nt) {
        tile_group[nt] = e;
        tile_row0[nt] = off + r0;
        tile_rows[nt] = min(per_tile, c - r0);
      }
      off += c;
    }
    *n_tiles = nt;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += 256) {
    const int at = atomicAdd(&cur[expert[p]], 1);
    pos_pair[at] = p;
    pos_row[at] = p / top;
  }
}

template <typename A>
__global__ __launch_bounds__(256) void route_combine_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                            const A* __restrict__ add, A* __restrict__ out, int d, int top,
                                                            const float* __restrict__ add_gate, int64_t add_gate_stride) {
  const int row = blockIdx.x;
  const float gate = add && add_gate ? sigmoid_f(add_gate[(size_t)row * add_gate_stride]) : 1.0f;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < d; i += gridDim.y * 256) {
    float a = add ? ld(add + (size_t)row * d + i) * gate : 0.f;
    for (int c = 0; c < top; ++c) a = fmaf(w[(size_t)row * top + c], y[((size_t)row * top + c) * d + i], a);
    st(out + (size_t)row * d + i, a);
  }
}

}  // namespace pk

extern "C" {
using namespace pk;

pegainfer_status_t pegainfer_route_topk(const void* h, const void* w_router, const void* correction, int32_t* out_expert,
                                        float* out_weight, int32_t d, int32_t experts, int32_t n_groups, int32_t keep_groups,
                                        int32_t top, int32_t rows, int32_t score_kind, int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (score_kind != PEGAINFER_SCORE_SIGMOID && score_kind != PEGAINFER_SCORE_SOFTMAX) return (pegainfer_status_t)hipErrorInvalidValue;
  if (n_groups < 1) n_groups = 1;
  if (experts <= 0 || experts % n_groups || top <= 0 || top > experts || keep_groups < 1 || keep_groups > n_groups ||
      (size_t)(2 * experts + n_groups) * 4 > 60000)
    return (pegainfer_status_t)hipErrorInvalidValue;
  const size_t smem = (size_t)(2 * experts + n_groups) * sizeof(float);
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        route_kernel<A><<<rows, 256, smem, as_stream(stream)>>>(static_cast<const A*>(h), static_cast<const A*>(w_router),
                                                                static_cast<const A*>(correction), out_expert, out_weight, d,
                                                                experts, n_groups, keep_groups, top, score_kind);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_route_from_logits_ex(const float* logits, int64_t logits_stride, const void* correction,
                                                  int32_t* out_expert, float* out_weight, int32_t experts, int32_t n_groups,
                                                  int32_t keep_groups, int32_t top, int32_t rows, int32_t score_kind,
                                                  int32_t group_kind, int32_t renorm, int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (n_groups < 1) n_groups = 1;
  if (experts <= 0 || experts % n_groups || top <= 0 || top > experts || keep_groups < 1 || keep_groups > n_groups ||
      logits_stride < experts || (size_t)(2 * experts + n_groups) * 16 > 60000 ||
      (score_kind != PEGAINFER_SCORE_SIGMOID && score_kind != PEGAINFER_SCORE_SOFTMAX) ||
      (group_kind != PEGAINFER_GROUP_TOP2_SUM && group_kind != PEGAINFER_GROUP_MAX))
    return (pegainfer_status_t)hipErrorInvalidValue;
  const size_t smem = (size_t)4 * (2 * experts + n_groups) * sizeof(float);
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        route_from_logits_kernel<A><<<ceil_div(rows, 4), 256, smem, as_stream(stream)>>>(
            logits, static_cast<const A*>(correction), out_expert, out_weight, experts, n_groups, keep_groups, top, rows, score_kind,
            logits_stride, group_kind, renorm);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_route_from_logits(const float* logits, const void* correction, int32_t* out_expert, float* out_weight,
                                               int32_t experts, int32_t n_groups, int32_t keep_groups, int32_t top, int32_t rows,
                                               int32_t score_kind, int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_route_from_logits_ex(logits, experts, correction, out_expert, out_weight, experts, n_groups, keep_groups, top, rows,
                                        score_kind, PEGAINFER_GROUP_TOP2_SUM, 0, dtype, stream);
}

pegainfer_status_t pegainfer_route_sigmoid_grouped(const void* h, const void* w_router, const void* correction,
                                                   int32_t* out_expert, float* out_weight, int32_t d, int32_t experts,
                                                   int32_t n_groups, int32_t keep_groups, int32_t top, int32_t rows,
                                                   int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_route_topk(h, w_router, correction, out_expert, out_weight, d, experts, n_groups, keep_groups, top, rows,
                              PEGAINFER_SCORE_SIGMOID, dtype, stream);
}

pegainfer_status_t pegainfer_route_sort(const int32_t* expert, int32_t n_pairs, int32_t top, int32_t experts,
                                        int32_t* pos_pair, int32_t* pos_row, int32_t* tile_group, int32_t* tile_row0,
                                        int32_t* tile_rows, int32_t* n_tiles, int32_t max_tiles, int32_t rows_per_tile,
                                        pegainfer_stream_t stream) {
  if (n_pairs <= 0) return 0;
  if ((rows_per_tile != 64 && rows_per_tile != 128) || experts <= 0 || experts > 7000 ||
      max_tiles < (n_pairs + rows_per_tile - 1) / rows_per_tile + experts)
    return (pegainfer_status_t)hipErrorInvalidValue;
  route_sort_kernel<<<1, 256, (size_t)2 * experts * sizeof(int), as_stream(stream)>>>(
      expert, n_pairs, top, experts, pos_pair, pos_row, tile_group, tile_row0, tile_rows, n_tiles, max_tiles, rows_per_tile);
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_route_combine_gated(const float* y_pairs, const float* weight, const void* add,
                                                 const float* add_gate, int64_t add_gate_stride, void* out, int32_t d,
                                                 int32_t top, int32_t rows, int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        // few rows (decoding): the row is cut over several workgroups
        const dim3 grid(rows, rows >= 256 ? 1 : std::min(16, ceil_div(d, 256)));
        route_combine_kernel<A><<<grid, 256, 0, as_stream(stream)>>>(y_pairs, weight, static_cast<const A*>(add),
                                                                     static_cast<A*>(out), d, top, add_gate, add_gate_stride);
      }))
    return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_route_combine_add(const float* y_pairs, const float* weight, const void* add, void* out, int32_t d,
                                               int32_t top, int32_t rows, int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_route_combine_gated(y_pairs, weight, add, nullptr, 0, out, d, top, rows, dtype, stream);
}

pegainfer_status_t pegainfer_route_combine(const float* y_pairs, const float* weight, void* out, int32_t d, int32_t top,
                                           int32_t rows, int32_t dtype, pegainfer_stream_t stream) {
  return pegainfer_route_combine_add(y_pairs, weight, nullptr, out, d, top, rows, dtype, stream);
}

}  // extern "C"

// Blocks around a sequence model's sublayers, each in a bf16 and an fp32 storage instance with fp32 arithmetic:
//   time_conv_kernel        causal per-channel convolution over time on a ragged batch; the inputs before an entry's first
//                           row come from the request's state (its last taps - 1 inputs)
//   time_conv_commit_kernel moves that state on by the entry's rows (one thread per (entry, channel) shifts in place,
//                           oldest first, so it never reads what it has already written)
//   group_rms_add_kernel    RMS norm in equal consecutive groups of a sublayer's OUTPUT, the residual sum, and a weighted
//                           sum over the streams of earlier layers (depth-weighted averaging) in one pass over the row
//   clamp_glu_rows_kernel   g = min(gate, L), u = clamp(up, -L, L):  g sigmoid(alpha g) (u + 1)
//   head_rms_gate_kernel    per-head RMS norm of a read-out * weight * silu / sigmoid gate * constant
//   scalar_rms_add_kernel   residual sum with a constant factor (+ bias, + extra rows, + one extra vector), then an RMS norm
//                           whose gain is a single number
//   terms_rms_add_kernel    residual sum of up to three sublayer outputs, each optionally RMS-normed with a weight first, then
//                           the RMS norm (a weight per channel) of what reads the stream next: one launch closes a layer whose
//                           sublayers all read the same normed input, and opens the next
//   glu_rows_kernel         act(gate) * up from two column ranges of a wider row (silu, relu or tanh-gelu)
//   softcap_rows_kernel     cap * tanh(x / cap) on fp32 rows
#include <algorithm>

#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

template <typename I, typename W, typename O>
__global__ __launch_bounds__(256) void time_conv_kernel(const I* __restrict__ in, int64_t in_stride, const W* __restrict__ w,
                                                        const float* __restrict__ state, int64_t slot_stride,
                                                        O* __restrict__ out, int64_t out_stride, int C, int K, int mode,
                                                        const int32_t* __restrict__ row_entry,
                                                        const int32_t* __restrict__ entry_row0,
                                                        const int32_t* __restrict__ entry_slot,
                                                        const W* __restrict__ in_bias, const W* __restrict__ out_bias) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int e = row_entry[row], r0 = entry_row0[e];
  const int local = row - r0;
  const float* tail = state + (int64_t)entry_slot[e] * slot_stride;
  const float ib = in_bias ? ld(in_bias + c) : 0.f;   // part of every real input (the carried inputs hold it already)
  float acc = 0.f;
  for (int j = 0; j < K; ++j) {
    const int src = local - (K - 1) + j;   // row of the entry this tap reads; negative = carried from earlier steps
    const float v = src >= 0 ? ld(in + (int64_t)(r0 + src) * in_stride + c) + ib : tail[(int64_t)(K - 1 + src) * C + c];
    acc = fmaf(ld(w + (int64_t)c * K + j), v, acc);
  }
  if (mode & 1) acc += ld(in + (int64_t)row * in_stride + c) + ib;
  if (out_bias) acc += ld(out_bias + c);
  if (mode & 2) acc = silu_f(acc);
  st(out + (int64_t)row * out_stride + c, acc);
}

// The same convolution for taps <= KMAX with a window in registers: a thread owns one channel and walks kConvRows rows of the
// step; while it stays inside an entry each row costs ONE load (the window slides), the taps' weights stay in registers.
// Window and weights are right-aligned (slot KMAX - 1 = the current row) and summed oldest first, the order of the plain
// kernel; slots beyond the taps hold weight 0 and input 0.
constexpr int kConvRows = 32;
template <typename I, typename W, typename O, int KMAX>
__global__ __launch_bounds__(256) void time_conv_window_kernel(const I* __restrict__ in, int64_t in_stride,
                                                               const W* __restrict__ w, const float* __restrict__ state,
                                                               int64_t slot_stride, O* __restrict__ out, int64_t out_stride,
                                                               int C, int K, int mode, int n_rows,
                                                               const int32_t* __restrict__ row_entry,
                                                               const int32_t* __restrict__ entry_row0,
                                                               const int32_t* __restrict__ entry_slot,
                                                               const W* __restrict__ in_bias, const W* __restrict__ out_bias) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const float ib = in_bias ? ld(in_bias + c) : 0.f, ob = out_bias ? ld(out_bias + c) : 0.f;
  float wr[KMAX], win[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    const int t = KMAX - 1 - j;   // rows back
    wr[j] = t < K ? ld(w + (int64_t)c * K + (K - 1 - t)) : 0.f;
    win[j] = 0.f;
  }
  const int row_begin = blockIdx.x * kConvRows, row_end = min(n_rows, row_begin + kConvRows);
  int cur_e = -1;
  for (int row = row_begin; row < row_end; ++row) {
    const int e = row_entry[row];
    if (e != cur_e) {             // first row of this walk inside the entry: fill the window's past from rows or the tail
      cur_e = e;
      const int r0 = entry_row0[e], local = row - r0;
      const float* tail = state + (int64_t)entry_slot[e] * slot_stride;
#pragma unroll
      for (int j = 0; j < KMAX - 1; ++j) {
        const int t = KMAX - 1 - j;
        const int src = local - t;
        win[j + 1] = t >= K ? 0.f : src >= 0 ? ld(in + (int64_t)(r0 + src) * in_stride + c) + ib : tail[(int64_t)(K - 1 + src) * C + c];
      }
    }
#pragma unroll
    for (int j = 0; j < KMAX - 1; ++j) win[j] = win[j + 1];
    const float cur = ld(in + (int64_t)row * in_stride + c) + ib;
    win[KMAX - 1] = cur;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < KMAX; ++j) acc = fmaf(wr[j], win[j], acc);
    if (mode & 1) acc += cur;
    acc += ob;
    if (mode & 2) acc = silu_f(acc);
    st(out + (int64_t)row * out_stride + c, acc);
  }
}

// Decoding: every entry brings ONE row.  Output and the moved-on tail in one launch: a thread owns (entry, channel), reads the
// taps - 1 carried inputs once, and writes them back shifted by one with the new input last.
template <typename I, typename W, typename O>
__global__ __launch_bounds__(256) void time_conv_step_kernel(const I* __restrict__ in, int64_t in_stride, const W* __restrict__ w,
                                                             float* __restrict__ state, int64_t slot_stride, O* __restrict__ out,
                                                             int64_t out_stride, int C, int K, int mode,
                                                             const int32_t* __restrict__ entry_slot,
                                                             const W* __restrict__ in_bias, const W* __restrict__ out_bias) {
  const int e = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  float* tail = state + (int64_t)entry_slot[e] * slot_stride;
  const float cur = ld(in + (int64_t)e * in_stride + c) + (in_bias ? ld(in_bias + c) : 0.f);
  float acc = 0.f;
  for (int j = 0; j < K - 1; ++j) {
    const float v = tail[(int64_t)j * C + c];
    acc = fmaf(ld(w + (int64_t)c * K + j), v, acc);
    if (j > 0) tail[(int64_t)(j - 1) * C + c] = v;
  }
  acc = fmaf(ld(w + (int64_t)c * K + K - 1), cur, acc);
  if (K > 1) tail[(int64_t)(K - 2) * C + c] = cur;
  if (mode & 1) acc += cur;
  if (out_bias) acc += ld(out_bias + c);
  if (mode & 2) acc = silu_f(acc);
  st(out + (int64_t)e * out_stride + c, acc);
}

template <typename I, typename W>
__global__ __launch_bounds__(256) void time_conv_commit_kernel(const I* __restrict__ in, int64_t in_stride,
                                                               float* __restrict__ state, int64_t slot_stride, int C, int K,
                                                               const int32_t* __restrict__ entry_row0,
                                                               const int32_t* __restrict__ entry_slot,
                                                               const W* __restrict__ in_bias) {
  const int e = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const float ib = in_bias ? ld(in_bias + c) : 0.f;
  const int r0 = entry_row0[e], len = entry_row0[e + 1] - r0;
  float* tail = state + (int64_t)entry_slot[e] * slot_stride;
  for (int s = 0; s < K - 1; ++s) {
    const int idx = len + s;   // position in [old state (K - 1) ; this step's inputs (len)]
    tail[(int64_t)s * C + c] = idx < K - 1 ? tail[(int64_t)idx * C + c] : ld(in + (int64_t)(r0 + idx - (K - 1)) * in_stride + c) + ib;
  }
}

// four consecutive values of a row, widened / rounded at the edges
__device__ __forceinline__ void ld4(const float* p, float* o) { const f32x4 v = *reinterpret_cast<const f32x4*>(p); o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
__device__ __forceinline__ void ld4(const uint16_t* p, float* o) {
  const u32x2 v = *reinterpret_cast<const u32x2*>(p);
  o[0] = bf_lo(v.x); o[1] = bf_hi(v.x); o[2] = bf_lo(v.y); o[3] = bf_hi(v.y);
}
__device__ __forceinline__ void st4(float* p, const float* o) { *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]}; }
__device__ __forceinline__ void st4(uint16_t* p, const float* o) { *reinterpret_cast<u32x2*>(p) = u32x2{pack_bf2(o[0], o[1]), pack_bf2(o[2], o[3])}; }

// x_in, x_out and mix_out may name the same memory (the stream is updated in place): an element is read, then written, by
// the same thread, and nothing else of those buffers is touched.  VEC: rows and groups are multiples of four values and every
// pointer is 16-byte aligned - four values per load.
template <typename Y, typename A, bool VEC>
__global__ __launch_bounds__(256) void group_rms_add_kernel(const float* x_in, const Y* __restrict__ y,
                                                            const A* __restrict__ w, int groups, float eps, float* x_out,
                                                            A* __restrict__ xb_out, int d, const float* __restrict__ stack,
                                                            int64_t stack_stride, const A* __restrict__ coef, int n_mix,
                                                            float* mix_out, A* __restrict__ mixb_out) {
  extern __shared__ float sm[];   // [groups] inverse root mean squares, then [n_mix] coefficients
  float* inv = sm;
  float* cf = sm + groups;
  const int row = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int gs = d / groups;
  const Y* yr = y + (int64_t)row * d;
  for (int j = threadIdx.x; j < n_mix; j += 256) cf[j] = ld(coef + j);
  for (int g = wave; g < groups; g += 4) {
    float ss = 0.f;
    if (VEC) {
      for (int i = lane * 4; i < gs; i += 256) {
        float v[4];
        ld4(yr + g * gs + i, v);
        ss = fmaf(v[0], v[0], ss); ss = fmaf(v[1], v[1], ss); ss = fmaf(v[2], v[2], ss); ss = fmaf(v[3], v[3], ss);
      }
    } else {
      for (int i = lane; i < gs; i += 64) {
        const float v = ld(yr + g * gs + i);
        ss = fmaf(v, v, ss);
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
  constexpr int N = VEC ? 4 : 1;
  for (int i = threadIdx.x * N; i < d; i += 256 * N) {
    const int64_t at = (int64_t)row * d + i;
    float r[N], yv[N], wv[N], xv[N], m[N];
    if (VEC) { ld4(yr + i, yv); ld4(w + i, wv); } else { yv[0] = ld(yr + i); wv[0] = ld(w + i); }
    if (x_in) { if (VEC) ld4(x_in + at, xv); else xv[0] = x_in[at]; }
    const float scale = inv[i / gs];   // VEC: a group holds whole fours
#pragma unroll
    for (int k = 0; k < N; ++k) {
      r[k] = yv[k] * scale * wv[k];
      if (x_in) r[k] += xv[k];
      m[k] = 0.f;
    }
    for (int j = 0; j < n_mix - 1; ++j) {
      float sv[N];
      if (VEC) ld4(stack + (int64_t)j * stack_stride + at, sv); else sv[0] = stack[(int64_t)j * stack_stride + at];
#pragma unroll
      for (int k = 0; k < N; ++k) m[k] = fmaf(cf[j], sv[k], m[k]);
    }
    if (n_mix > 0) {
#pragma unroll
      for (int k = 0; k < N; ++k) m[k] = fmaf(cf[n_mix - 1], r[k], m[k]);
    }
    if (VEC) {
      if (x_out) st4(x_out + at, r);
      if (xb_out) st4(xb_out + at, r);
      if (n_mix > 0 && mix_out) st4(mix_out + at, m);
      if (n_mix > 0 && mixb_out) st4(mixb_out + at, m);
    } else {
      if (x_out) x_out[at] = r[0];
      if (xb_out) st(xb_out + at, r[0]);
      if (n_mix > 0 && mix_out) mix_out[at] = m[0];
      if (n_mix > 0 && mixb_out) st(mixb_out + at, m[0]);
    }
  }
}

template <typename A>
__global__ __launch_bounds__(256) void clamp_glu_rows_kernel(const A* __restrict__ gu, A* __restrict__ out, int I, float limit,
                                                             float alpha) {
  const int row = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= I) return;
  const float g = fminf(ld(gu + (int64_t)row * 2 * I + i), limit);
  const float u = fminf(fmaxf(ld(gu + (int64_t)row * 2 * I + I + i), -limit), limit);
  st(out + (int64_t)row * I + i, g * sigmoid_f(alpha * g) * (u + 1.0f));
}

// one wave per (row, head)
template <typename A>
__global__ __launch_bounds__(256) void head_rms_gate_kernel(const float* __restrict__ o, const A* __restrict__ w, int w_per_head,
                                                            const A* __restrict__ gate, int64_t gate_stride, int gate_kind,
                                                            float factor, float eps, A* __restrict__ out, int64_t out_stride,
                                                            int heads, int vdim, int rows, int gate_first) {
  const int64_t rh = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (rh >= (int64_t)rows * heads) return;
  const int row = (int)(rh / heads), h = (int)(rh % heads);
  const float* p = o + ((int64_t)row * heads + h) * vdim;
  const A* gr = gate + (int64_t)row * gate_stride + (int64_t)h * vdim;
  auto act = [&](int i) {
    const float z = ld(gr + i);
    return gate_kind == 0 ? silu_f(z) : sigmoid_f(z);
  };
  float ss = 0.f;
  for (int i = lane; i < vdim; i += 64) {
    const float v = gate_first ? p[i] * act(i) : p[i];   // gate_first: the gated values are what is normed
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int i = lane; i < vdim; i += 64) {
    const float wv = ld(w + (w_per_head ? h * vdim : 0) + i);
    // (each order keeps its own sequence of roundings: norm, weight, gate, factor - or gate, norm, weight, factor)
    st(out + (int64_t)row * out_stride + h * vdim + i, gate_first ? p[i] * act(i) * inv * wv * factor : p[i] * inv * wv * act(i) * factor);
  }
}

// Residual sum with a constant factor, then an RMS norm whose gain is ONE number:
//   r = x_in + mult * (y + bias) + add_rows + add_vec            (every term but x_in optional)      -> x_out (fp32)
//   n = r / sqrt(mean(r^2) + eps) * gain[0]                                                          -> n_out (fp32, optional)
// x_in and x_out may name the same memory (an element is read, then written, by the same thread).  The row stays in
// registers between the sum and the norm: one pass over memory.  NPT: values a thread keeps (d <= 256 * NPT), 0 = any d
// (the row is summed a second time instead).
template <typename Y, typename A, int NPT>
__global__ __launch_bounds__(256) void scalar_rms_add_kernel(const float* x_in, const Y* __restrict__ y, const A* __restrict__ bias,
                                                             float mult, const float* __restrict__ add_rows,
                                                             const A* __restrict__ add_vec, float* x_out,
                                                             const A* __restrict__ gain, float eps, float* __restrict__ n_out,
                                                             int d) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const int64_t base = (int64_t)row * d;
  auto value = [&](int i) {
    float r = x_in[base + i];
    if (y) r = fmaf(mult, ld(y + base + i) + (bias ? ld(bias + i) : 0.f), r);
    if (add_rows) r += add_rows[base + i];
    if (add_vec) r += ld(add_vec + i);
    return r;
  };
  float ss = 0.f;
  if constexpr (NPT > 0) {
    float keep[NPT];
#pragma unroll
    for (int k = 0; k < NPT; ++k) {
      const int i = threadIdx.x + 256 * k;
      keep[k] = i < d ? value(i) : 0.f;
      ss = fmaf(keep[k], keep[k], ss);
    }
    ss = block_sum<4>(ss, red);
    const float sc = gain ? ld(gain) / sqrtf(ss / (float)d + eps) : 0.f;
#pragma unroll
    for (int k = 0; k < NPT; ++k) {
      const int i = threadIdx.x + 256 * k;
      if (i < d) {
        if (x_out) x_out[base + i] = keep[k];
        if (n_out) n_out[base + i] = keep[k] * sc;
      }
    }
  } else {
    for (int i = threadIdx.x; i < d; i += 256) {
      const float r = value(i);
      ss = fmaf(r, r, ss);
    }
    ss = block_sum<4>(ss, red);   // its barriers also order every read of x_in before the writes below
    const float sc = gain ? ld(gain) / sqrtf(ss / (float)d + eps) : 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
      const float r = value(i);
      if (x_out) x_out[base + i] = r;
      if (n_out) n_out[base + i] = r * sc;
    }
  }
}


// Up to three sublayer outputs join the stream at once; a term with a weight is RMS-normed over the row first:
//   term_t = (w_t ? (y_t + bias_t) / sqrt(mean((y_t + bias_t)^2) + eps) * w_t : y_t + bias_t) * factor_t
//   r = x_in + sum_t term_t                                  -> x_out (fp32; may alias x_in)
//   n = r / sqrt(mean(r^2) + eps) * gain                     -> n_out (N: float or the storage type; optional)
// NPT: values a thread keeps between the sum and the norm (d <= 256 * NPT), 0 = any d (the row is summed a second time).
struct SumTerm { const void* y; int64_t stride; const void* bias; const void* w; float factor; };
struct SumTerms { SumTerm t[3]; int n; };
// VEC: d, the terms' strides and every pointer allow four values per load.
template <typename A, typename N, int NPT, bool VEC>
__global__ __launch_bounds__(256) void terms_rms_add_kernel(const float* x_in, SumTerms terms, float* x_out,
                                                            const A* __restrict__ gain, float eps, N* __restrict__ n_out, int d) {
  __shared__ float red[4];
  constexpr int V = VEC ? 4 : 1;
  const int row = blockIdx.x;
  const int64_t base = (int64_t)row * d;
  auto load = [&](const auto* p, float* o) {
    if constexpr (VEC) ld4(p, o); else o[0] = ld(p);
  };
  float inv[3] = {1.f, 1.f, 1.f};
#pragma unroll
  for (int t = 0; t < 3; ++t) {
    if (t >= terms.n || !terms.t[t].w) continue;     // uniform over the workgroup
    const A* y = static_cast<const A*>(terms.t[t].y) + (int64_t)row * terms.t[t].stride;
    const A* b = static_cast<const A*>(terms.t[t].bias);
    float ss = 0.f;
    for (int i = threadIdx.x * V; i < d; i += 256 * V) {
      float v[V], bv[V];
      load(y + i, v);
      if (b) load(b + i, bv);
#pragma unroll
      for (int u = 0; u < V; ++u) {
        const float z = v[u] + (b ? bv[u] : 0.f);
        ss = fmaf(z, z, ss);
      }
    }
    inv[t] = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)d + eps);
  }
  auto value = [&](int i, float* r) {      // V values from column i on
    if (x_in) load(x_in + base + i, r);
    else {
#pragma unroll
      for (int u = 0; u < V; ++u) r[u] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < 3; ++t) {
      if (t >= terms.n) continue;
      const A* y = static_cast<const A*>(terms.t[t].y) + (int64_t)row * terms.t[t].stride;
      const A* b = static_cast<const A*>(terms.t[t].bias);
      const A* w = static_cast<const A*>(terms.t[t].w);
      float v[V], bv[V], wv[V];
      load(y + i, v);
      if (b) load(b + i, bv);
      if (w) load(w + i, wv);
#pragma unroll
      for (int u = 0; u < V; ++u) {
        float z = v[u] + (b ? bv[u] : 0.f);
        if (w) z = z * inv[t] * wv[u];
        r[u] = fmaf(terms.t[t].factor, z, r[u]);
      }
    }
  };
  auto store = [&](int i, const float* r, float sc) {
    if (x_out) {
      if constexpr (VEC) st4(x_out + base + i, r); else x_out[base + i] = r[0];
    }
    if (n_out) {
      float g[V], o[V];
      load(gain + i, g);
#pragma unroll
      for (int u = 0; u < V; ++u) o[u] = r[u] * sc * g[u];
      if constexpr (VEC) st4(n_out + base + i, o); else st(n_out + base + i, o[0]);
    }
  };
  float ss = 0.f;
  if constexpr (NPT > 0) {
    float keep[NPT];
#pragma unroll
    for (int k = 0; k < NPT; k += V) {
      const int i = (threadIdx.x + 256 * (k / V)) * V;
      if (i < d) value(i, keep + k);
      else {
#pragma unroll
        for (int u = 0; u < V; ++u) keep[k + u] = 0.f;
      }
#pragma unroll
      for (int u = 0; u < V; ++u) ss = fmaf(keep[k + u], keep[k + u], ss);
    }
    ss = block_sum<4>(ss, red);
    const float sc = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int k = 0; k < NPT; k += V) {
      const int i = (threadIdx.x + 256 * (k / V)) * V;
      if (i < d) store(i, keep + k, sc);
    }
  } else {
    for (int i = threadIdx.x * V; i < d; i += 256 * V) {
      float r[V];
      value(i, r);
#pragma unroll
      for (int u = 0; u < V; ++u) ss = fmaf(r[u], r[u], ss);
    }
    ss = block_sum<4>(ss, red);   // its barriers also order every read of x_in before the writes below
    const float sc = 1.0f / sqrtf(ss / (float)d + eps);
    for (int i = threadIdx.x * V; i < d; i += 256 * V) {
      float r[V];
      value(i, r);
      store(i, r, sc);
    }
  }
}

// out[row, i] = act(gate[row, i]) * up[row, i]; gate and up are column ranges of rows with one stride
template <typename A>
__global__ __launch_bounds__(256) void glu_rows_kernel(const A* __restrict__ gate, const A* __restrict__ up, int64_t in_stride,
                                                       A* __restrict__ out, int64_t out_stride, int I, int act) {
  const int row = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= I) return;
  const float g = ld(gate + (int64_t)row * in_stride + i), u = ld(up + (int64_t)row * in_stride + i);
  float a;
  if (act == 0) a = silu_f(g);
  else if (act == 1) a = fmaxf(g, 0.f);
  else a = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  st(out + (int64_t)row * out_stride + i, a * u);
}

__global__ __launch_bounds__(256) void softcap_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int64_t n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = cap * tanhf(in[i] / cap);
}

}  // namespace pk

extern "C" {
using namespace pk;

#define PK_BAD ((pegainfer_status_t)hipErrorInvalidValue)

pegainfer_status_t pegainfer_terms_rms_add(const float* x_in, const pegainfer_sum_term* terms, int32_t n_terms, float* x_out,
                                           const void* gain, float eps, void* n_out, int32_t n_dtype, int32_t d, int32_t rows,
                                           int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (d <= 0 || n_terms < 0 || n_terms > 3 || (n_terms > 0 && !terms) || (!x_in && n_terms == 0) || (!x_out && !n_out) ||
      (n_out && !gain))
    return PK_BAD;
  SumTerms st_{};
  st_.n = n_terms;
  for (int t = 0; t < n_terms; ++t) {
    if (!terms[t].y) return PK_BAD;
    st_.t[t] = SumTerm{terms[t].y, terms[t].y_row_stride, terms[t].bias, terms[t].norm_w, terms[t].factor};
  }
  bool ok = true;
  const bool known = by_dtype(dtype, [&](auto* ta) {
    using A = std::remove_pointer_t<decltype(ta)>;
    ok = by_dtype(n_out ? n_dtype : dtype, [&](auto* tn) {
      using N = std::remove_pointer_t<decltype(tn)>;
      bool vec = d % 4 == 0 && host_aligned16(x_in) && host_aligned16(x_out) && host_aligned16(gain) && host_aligned16(n_out);
      for (int t = 0; t < n_terms; ++t)
        vec = vec && terms[t].y_row_stride % 4 == 0 && host_aligned16(terms[t].y) && host_aligned16(terms[t].bias) && host_aligned16(terms[t].norm_w);
      auto go = [&](auto npt) {
        if (vec)
          terms_rms_add_kernel<A, N, decltype(npt)::value, true><<<rows, 256, 0, as_stream(stream)>>>(
              x_in, st_, x_out, static_cast<const A*>(gain), eps, static_cast<N*>(n_out), d);
        else
          terms_rms_add_kernel<A, N, decltype(npt)::value, false><<<rows, 256, 0, as_stream(stream)>>>(
              x_in, st_, x_out, static_cast<const A*>(gain), eps, static_cast<N*>(n_out), d);
      };
      if (d <= 1024) go(std::integral_constant<int, 4>());
      else if (d <= 4096) go(std::integral_constant<int, 16>());
      else if (d <= 8192) go(std::integral_constant<int, 32>());
      else go(std::integral_constant<int, 0>());
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_glu_rows(const void* gate, const void* up, int64_t in_row_stride, void* out, int64_t out_row_stride,
                                      int32_t I, int32_t rows, int32_t act, int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0 || I <= 0) return 0;
  if (act < 0 || act > 2) return PK_BAD;
  const dim3 grid(rows, ceil_div(I, 256));
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        glu_rows_kernel<A><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const A*>(gate), static_cast<const A*>(up), in_row_stride,
                                                                static_cast<A*>(out), out_row_stride, I, act);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_softcap_rows(const float* in, float* out, int64_t n, float cap, pegainfer_stream_t stream) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return PK_BAD;
  softcap_rows_kernel<<<ceil_div(n, 256), 256, 0, as_stream(stream)>>>(in, out, n, cap);
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_time_conv(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                       const float* state, int64_t slot_stride, void* out, int32_t out_dtype,
                                       int64_t out_row_stride, int32_t channels, int32_t taps, int32_t mode,
                                       const int32_t* row_entry, const int32_t* entry_row0, const int32_t* entry_slot,
                                       int32_t n_rows, pegainfer_stream_t stream) {
  return pegainfer_time_conv_biased(in, in_dtype, in_row_stride, w, w_dtype, nullptr, nullptr, state, slot_stride, out, out_dtype,
                                    out_row_stride, channels, taps, mode, row_entry, entry_row0, entry_slot, n_rows, stream);
}

pegainfer_status_t pegainfer_time_conv_biased(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                              const void* in_bias, const void* out_bias, const float* state, int64_t slot_stride,
                                              void* out, int32_t out_dtype, int64_t out_row_stride, int32_t channels, int32_t taps,
                                              int32_t mode, const int32_t* row_entry, const int32_t* entry_row0,
                                              const int32_t* entry_slot, int32_t n_rows, pegainfer_stream_t stream) {
  if (n_rows <= 0) return 0;
  if (channels <= 0 || taps < 1) return PK_BAD;
  const dim3 grid(n_rows, ceil_div(channels, 256));
  bool ok = true;
  const bool known = by_dtype(in_dtype, [&](auto* ti) {
    using I = std::remove_pointer_t<decltype(ti)>;
    ok = by_dtype(w_dtype, [&](auto* tw) {
           using W = std::remove_pointer_t<decltype(tw)>;
           ok = by_dtype(out_dtype, [&](auto* to) {
                  using O = std::remove_pointer_t<decltype(to)>;
                  const dim3 wgrid(ceil_div(n_rows, kConvRows), ceil_div(channels, 256));
                  if (n_rows >= 4 * kConvRows && taps <= 4)
                    time_conv_window_kernel<I, W, O, 4><<<wgrid, 256, 0, as_stream(stream)>>>(
                        static_cast<const I*>(in), in_row_stride, static_cast<const W*>(w), state, slot_stride,
                        static_cast<O*>(out), out_row_stride, channels, taps, mode, n_rows, row_entry, entry_row0, entry_slot,
                        static_cast<const W*>(in_bias), static_cast<const W*>(out_bias));
                  else if (n_rows >= 4 * kConvRows && taps <= 8)
                    time_conv_window_kernel<I, W, O, 8><<<wgrid, 256, 0, as_stream(stream)>>>(
                        static_cast<const I*>(in), in_row_stride, static_cast<const W*>(w), state, slot_stride,
                        static_cast<O*>(out), out_row_stride, channels, taps, mode, n_rows, row_entry, entry_row0, entry_slot,
                        static_cast<const W*>(in_bias), static_cast<const W*>(out_bias));
                  else
                    time_conv_kernel<I, W, O><<<grid, 256, 0, as_stream(stream)>>>(
                        static_cast<const I*>(in), in_row_stride, static_cast<const W*>(w), state, slot_stride,
                        static_cast<O*>(out), out_row_stride, channels, taps, mode, row_entry, entry_row0, entry_slot,
                        static_cast<const W*>(in_bias), static_cast<const W*>(out_bias));
                }) && ok;
         }) && ok;
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_time_conv_step(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w, int32_t w_dtype,
                                            float* state, int64_t slot_stride, void* out, int32_t out_dtype, int64_t out_row_stride,
                                            int32_t channels, int32_t taps, int32_t mode, const int32_t* entry_slot,
                                            int32_t n_entries, pegainfer_stream_t stream) {
  return pegainfer_time_conv_step_biased(in, in_dtype, in_row_stride, w, w_dtype, nullptr, nullptr, state, slot_stride, out, out_dtype,
                                         out_row_stride, channels, taps, mode, entry_slot, n_entries, stream);
}

pegainfer_status_t pegainfer_time_conv_step_biased(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* w,
                                                   int32_t w_dtype, const void* in_bias, const void* out_bias, float* state,
                                                   int64_t slot_stride, void* out, int32_t out_dtype, int64_t out_row_stride,
                                                   int32_t channels, int32_t taps, int32_t mode, const int32_t* entry_slot,
                                                   int32_t n_entries, pegainfer_stream_t stream) {
  if (n_entries <= 0) return 0;
  if (channels <= 0 || taps < 1) return PK_BAD;
  const dim3 grid(n_entries, ceil_div(channels, 256));
  bool ok = true;
  const bool known = by_dtype(in_dtype, [&](auto* ti) {
    using I = std::remove_pointer_t<decltype(ti)>;
    ok = by_dtype(w_dtype, [&](auto* tw) {
           using W = std::remove_pointer_t<decltype(tw)>;
           ok = by_dtype(out_dtype, [&](auto* to) {
                  using O = std::remove_pointer_t<decltype(to)>;
                  time_conv_step_kernel<I, W, O><<<grid, 256, 0, as_stream(stream)>>>(
                      static_cast<const I*>(in), in_row_stride, static_cast<const W*>(w), state, slot_stride,
                      static_cast<O*>(out), out_row_stride, channels, taps, mode, entry_slot, static_cast<const W*>(in_bias),
                      static_cast<const W*>(out_bias));
                }) && ok;
         }) && ok;
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_time_conv_commit(const void* in, int32_t in_dtype, int64_t in_row_stride, float* state,
                                              int64_t slot_stride, int32_t channels, int32_t taps, const int32_t* entry_row0,
                                              const int32_t* entry_slot, int32_t n_entries, pegainfer_stream_t stream) {
  return pegainfer_time_conv_commit_biased(in, in_dtype, in_row_stride, nullptr, in_dtype, state, slot_stride, channels, taps, entry_row0,
                                           entry_slot, n_entries, stream);
}

pegainfer_status_t pegainfer_time_conv_commit_biased(const void* in, int32_t in_dtype, int64_t in_row_stride, const void* in_bias,
                                                     int32_t bias_dtype, float* state, int64_t slot_stride, int32_t channels,
                                                     int32_t taps, const int32_t* entry_row0, const int32_t* entry_slot,
                                                     int32_t n_entries, pegainfer_stream_t stream) {
  if (n_entries <= 0 || taps <= 1) return 0;
  const dim3 grid(ceil_div(channels, 256), n_entries);
  bool ok = true;
  const bool known = by_dtype(in_dtype, [&](auto* ti) {
    using I = std::remove_pointer_t<decltype(ti)>;
    ok = by_dtype(bias_dtype, [&](auto* tw) {
      using W = std::remove_pointer_t<decltype(tw)>;
      time_conv_commit_kernel<I, W><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const I*>(in), in_row_stride, state, slot_stride,
                                                                         channels, taps, entry_row0, entry_slot,
                                                                         static_cast<const W*>(in_bias));
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_group_rms_add(const float* x_in, const void* y, int32_t y_dtype, const void* w, int32_t groups,
                                           float eps, float* x_out, void* xb_out, int32_t d, int32_t rows, int32_t dtype,
                                           const float* stack, int64_t stack_stride, const void* coef, int32_t n_mix,
                                           float* mix_out, void* mixb_out, pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (groups < 1 || d <= 0 || d % groups || groups > 8192 || n_mix > 4096 || (n_mix > 0 && !coef) || (n_mix > 1 && !stack)) return PK_BAD;
  bool ok = true;
  const bool known = by_dtype(y_dtype, [&](auto* ty) {
    using Y = std::remove_pointer_t<decltype(ty)>;
    ok = by_dtype(dtype, [&](auto* ta) {
      using A = std::remove_pointer_t<decltype(ta)>;
      const size_t smem = (size_t)(groups + std::max(n_mix, 0)) * sizeof(float);
      const bool vec = d % 4 == 0 && (d / groups) % 4 == 0 && stack_stride % 4 == 0 && host_aligned16(x_in) && host_aligned16(y) &&
                       host_aligned16(w) && host_aligned16(x_out) && host_aligned16(xb_out) && host_aligned16(stack) &&
                       host_aligned16(mix_out) && host_aligned16(mixb_out);
      if (vec)
        group_rms_add_kernel<Y, A, true><<<rows, 256, smem, as_stream(stream)>>>(
            x_in, static_cast<const Y*>(y), static_cast<const A*>(w), groups, eps, x_out, static_cast<A*>(xb_out), d, stack,
            stack_stride, static_cast<const A*>(coef), n_mix, mix_out, static_cast<A*>(mixb_out));
      else
        group_rms_add_kernel<Y, A, false><<<rows, 256, smem, as_stream(stream)>>>(
            x_in, static_cast<const Y*>(y), static_cast<const A*>(w), groups, eps, x_out, static_cast<A*>(xb_out), d, stack,
            stack_stride, static_cast<const A*>(coef), n_mix, mix_out, static_cast<A*>(mixb_out));
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

pegainfer_status_t pegainfer_clamp_glu_rows(const void* gate_up, void* out, int32_t I, int32_t rows, float limit, float alpha,
                                            int32_t dtype, pegainfer_stream_t stream) {
  if (rows <= 0 || I <= 0) return 0;
  const dim3 grid(rows, ceil_div(I, 256));
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        clamp_glu_rows_kernel<A><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const A*>(gate_up), static_cast<A*>(out), I,
                                                                      limit, alpha);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_head_rms_gate(const float* o, const void* w, int32_t w_per_head, const void* gate,
                                           int64_t gate_stride, int32_t gate_kind, float factor, float eps, void* out,
                                           int64_t out_stride, int32_t heads, int32_t vdim, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream) {
  return pegainfer_head_gate_rms(o, w, w_per_head, gate, gate_stride, gate_kind, 0, factor, eps, out, out_stride, heads, vdim, rows,
                                 dtype, stream);
}

pegainfer_status_t pegainfer_head_gate_rms(const float* o, const void* w, int32_t w_per_head, const void* gate, int64_t gate_stride,
                                           int32_t gate_kind, int32_t gate_first, float factor, float eps, void* out,
                                           int64_t out_stride, int32_t heads, int32_t vdim, int32_t rows, int32_t dtype,
                                           pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (heads <= 0 || vdim <= 0) return PK_BAD;
  const int blocks = ceil_div((long)rows * heads, 4);
  if (!by_dtype(dtype, [&](auto* t) {
        using A = std::remove_pointer_t<decltype(t)>;
        head_rms_gate_kernel<A><<<blocks, 256, 0, as_stream(stream)>>>(o, static_cast<const A*>(w), w_per_head,
                                                                       static_cast<const A*>(gate), gate_stride, gate_kind,
                                                                       factor, eps, static_cast<A*>(out), out_stride, heads,
                                                                       vdim, rows, gate_first);
      }))
    return PK_BAD;
  return (pegainfer_status_t)hipGetLastError();
}

pegainfer_status_t pegainfer_scalar_rms_add(const float* x_in, const void* y, int32_t y_dtype, const void* bias, float mult,
                                            const float* add_rows, const void* add_vec, float* x_out, const void* gain,
                                            float eps, float* n_out, int32_t d, int32_t rows, int32_t dtype,
                                            pegainfer_stream_t stream) {
  if (rows <= 0) return 0;
  if (d <= 0 || !x_in || (!x_out && !n_out) || (n_out && !gain)) return PK_BAD;
  bool ok = true;
  const bool known = by_dtype(y ? y_dtype : dtype, [&](auto* ty) {
    using Y = std::remove_pointer_t<decltype(ty)>;
    ok = by_dtype(dtype, [&](auto* ta) {
      using A = std::remove_pointer_t<decltype(ta)>;
      auto go = [&](auto npt) {
        scalar_rms_add_kernel<Y, A, decltype(npt)::value><<<rows, 256, 0, as_stream(stream)>>>(
            x_in, static_cast<const Y*>(y), static_cast<const A*>(bias), mult, add_rows, static_cast<const A*>(add_vec), x_out,
            static_cast<const A*>(gain), eps, n_out, d);
      };
      if (d <= 1024) go(std::integral_constant<int, 4>());
      else if (d <= 4096) go(std::integral_constant<int, 16>());
      else if (d <= 8192) go(std::integral_constant<int, 32>());
      else go(std::integral_constant<int, 0>());
    });
  });
  return known && ok ? (pegainfer_status_t)hipGetLastError() : PK_BAD;
}

}  // extern "C"

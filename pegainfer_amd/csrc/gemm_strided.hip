// Strided / batched / grouped GEMM for the shapes the weight-streaming and 128/256-tile kernels of linear.hip do not take:
// per-head products over slices of a wider row (latent-attention absorb and value up-projection), expert-grouped rows
// gathered through an index (routed feed-forward), and every product of a model served in true fp32.
//
//   y[row, g, m] = sum_k x[row, g, k] * w[g, m, k]
//
// 64 x 64 output tile per 256-thread workgroup, K in slices of 16 staged through LDS as fp32, each thread a 4 x 4 block
// of fp32 accumulators, k strictly ascending: an output's value depends on its own row and weights only (never on the
// tile it lands in, the batch or the group sizes).  Operand storage (bf16 or fp32) is a template parameter, so the bf16
// instance multiplies exact fp32 images of bf16 values and the fp32 instance is plain fp32 FMA - no reduced-precision
// matrix mode.
#include <type_traits>

#include "common.h"
#include "typed.h"
#include "pegainfer_kernels_blocks.h"

namespace pk {

constexpr int GT = 64, GM = 64, GK = 16;

template <typename TX, typename TW, typename TY, typename TG>
__global__ __launch_bounds__(256) void gemm_strided_kernel(pegainfer_gemm_desc d) {
  __shared__ float xs[GK][GT + 4];
  __shared__ float ws[GK][GM + 4];
  __shared__ int xrow[GT], yrow[GT];
  int g, row0, nrows;
  if (d.tile_group) {
    if ((int)blockIdx.x >= *d.n_tiles) return;
    g = d.tile_group[blockIdx.x];
    row0 = d.tile_row0[blockIdx.x];
    nrows = d.tile_rows[blockIdx.x];
  } else {
    g = blockIdx.z;
    row0 = blockIdx.x * GT;
    nrows = min(GT, d.rows - row0);
  }
  const int m0 = blockIdx.y * GM;
  const int tid = threadIdx.x;
  if (tid < GT) {
    const int p = row0 + tid;
    xrow[tid] = tid < nrows ? (d.x_row_index ? d.x_row_index[p] : p) : -1;
    yrow[tid] = tid < nrows ? (d.y_row_index ? d.y_row_index[p] : p) : -1;
  }
  __syncthreads();
  const TX* X = static_cast<const TX*>(d.x) + (int64_t)g * d.x_group_stride;
  const TW* W = static_cast<const TW*>(d.w) + (int64_t)g * d.w_group_stride;
  const int tr = (tid >> 4) * 4, tm = (tid & 15) * 4;   // this thread's 4 rows x 4 outputs
  float acc[4][4] = {};
  const bool w_k_fast = d.w_k_stride == 1;
  for (int k0 = 0; k0 < d.k; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      {
        const int r = idx >> 4, kk = idx & 15;
        const int src = xrow[r];
        xs[kk][r] = (src >= 0 && k0 + kk < d.k) ? ld(X + (int64_t)src * d.x_row_stride + k0 + kk) : 0.f;
      }
      {
        const int mm = w_k_fast ? idx >> 4 : idx & 63, kk = w_k_fast ? idx & 15 : idx >> 6;
        ws[kk][mm] = (m0 + mm < d.m && k0 + kk < d.k)
                         ? ld(W + (int64_t)(m0 + mm) * d.w_m_stride + (int64_t)(k0 + kk) * d.w_k_stride) : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = xs[kk][tr + i]; b[i] = ws[kk][tm + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  TY* Y = static_cast<TY*>(d.y) + (int64_t)g * d.y_group_stride;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int dst = yrow[tr + i];
    if (dst < 0) continue;
    float scale = 1.f;
    if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE)
      scale = sigmoid_f(ld(static_cast<const TG*>(d.gate) + (int64_t)xrow[tr + i] * d.gate_row_stride + g));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (m0 + tm + j >= d.m) continue;
      float v = acc[i][j];
      if (d.epilogue == PEGAINFER_EPI_RELU_SQ) { v = fmaxf(v, 0.f); v *= v; }
      else if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE) v *= scale;
      st(Y + (int64_t)dst * d.y_row_stride + m0 + tm + j, v);
    }
  }
}


// ------------------------------------------------------------------ matrix-core form (bf16 weights, k contiguous)
// The same addressing (groups, gathered rows, tile table), K in slices of 64 staged as bf16 through registers (the next slice
// is in flight while this one is multiplied), four waves in a 2 x 2 arrangement of v_mfma_f32_16x16x32_bf16 blocks.  fp32 x (the attention output in front of the value
// up-projection) is rounded to bf16 while it is staged.  Needs 16-byte chunks: K % 8 == 0, strides % 8 == 0, aligned bases.
constexpr int MK = 64, MS = MK + 8;

__device__ __forceinline__ u32x4 stage8(const uint16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ u32x4 stage8(const float* p) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
  return u32x4{pack_bf2(a.x, a.y), pack_bf2(a.z, a.w), pack_bf2(b.x, b.y), pack_bf2(b.z, b.w)};
}

// Output tile TR rows x 128 outputs (TR = 64 or 128): with 64 x 64 tiles the kernel moved 32 flop per byte staged and sat on
// the L2 -> CU bandwidth (7.5 TB/s of staging traffic at 1024 tokens x 4 experts); 128 x 128 halves the bytes per flop.
constexpr int MM = 128;

template <typename TX, typename TY, typename TG, int TR>
__global__ __launch_bounds__(256) void gemm_strided_mfma_kernel(pegainfer_gemm_desc d) {
  __shared__ __align__(16) uint16_t xs[TR * MS];
  __shared__ __align__(16) uint16_t ws[MM * MS];
  __shared__ int xrow[TR], yrow[TR];
  int g, row0, nrows;
  if (d.tile_group) {
    if ((int)blockIdx.x >= *d.n_tiles) return;
    g = d.tile_group[blockIdx.x];
    row0 = d.tile_row0[blockIdx.x];
    nrows = min(TR, d.tile_rows[blockIdx.x]);
  } else {
    g = blockIdx.z;
    row0 = blockIdx.x * TR;
    nrows = min(TR, d.rows - row0);
  }
  const int m0 = blockIdx.y * MM;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l15 = lane & 15, gq = lane >> 4;
  if (tid < TR) {
    const int p = row0 + tid;
    xrow[tid] = tid < nrows ? (d.x_row_index ? d.x_row_index[p] : p) : -1;
    yrow[tid] = tid < nrows ? (d.y_row_index ? d.y_row_index[p] : p) : -1;
  }
  __syncthreads();
  const TX* X = static_cast<const TX*>(d.x) + (int64_t)g * d.x_group_stride;
  const uint16_t* W = static_cast<const uint16_t*>(d.w) + (int64_t)g * d.w_group_stride;
  constexpr int RJ = TR / 32;                       // 16-row blocks per wave
  const int wr = (wave & 1) * (TR / 2), wm = (wave >> 1) * 64;
  f32x4 acc[4][RJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < RJ; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const u32x4 zero = {0u, 0u, 0u, 0u};
  constexpr int XC = TR * (MK / 8) / 256, WC = MM * (MK / 8) / 256;   // chunks per thread and K slice
  // this thread's rows are the same in every K slice: resolve them once
  const TX* xsrc[XC];
  const uint16_t* wsrc[WC];
#pragma unroll
  for (int i = 0; i < XC; ++i) {
    const int c = tid + i * 256, src = xrow[c >> 3];
    xsrc[i] = src >= 0 ? X + (int64_t)src * d.x_row_stride + (c & 7) * 8 : nullptr;
  }
#pragma unroll
  for (int i = 0; i < WC; ++i) {
    const int c = tid + i * 256, m = m0 + (c >> 3);
    wsrc[i] = m < d.m ? W + (int64_t)m * d.w_m_stride + (c & 7) * 8 : nullptr;
  }
  u32x4 px[XC], pw[WC];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < XC; ++i) px[i] = (xsrc[i] && k0 + ((tid + i * 256) & 7) * 8 < d.k) ? stage8(xsrc[i] + k0) : zero;
#pragma unroll
    for (int i = 0; i < WC; ++i) pw[i] = (wsrc[i] && k0 + ((tid + i * 256) & 7) * 8 < d.k) ? stage8(wsrc[i] + k0) : zero;
  };
  fetch(0);
  for (int k0 = 0; k0 < d.k; k0 += MK) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < XC; ++i) { const int c = tid + i * 256; *reinterpret_cast<u32x4*>(xs + (c >> 3) * MS + (c & 7) * 8) = px[i]; }
#pragma unroll
    for (int i = 0; i < WC; ++i) { const int c = tid + i * 256; *reinterpret_cast<u32x4*>(ws + (c >> 3) * MS + (c & 7) * 8) = pw[i]; }
    __syncthreads();
    if (k0 + MK < d.k) fetch(k0 + MK);            // the next slice's loads fly while this one is multiplied
#pragma unroll
    for (int ks = 0; ks < MK; ks += 32) {
      bf16x8_t a[4], b[RJ];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(ws + (wm + i * 16 + l15) * MS + ks + gq * 8));
#pragma unroll
      for (int j = 0; j < RJ; ++j)
        b[j] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4*>(xs + (wr + j * 16 + l15) * MS + ks + gq * 8));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < RJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }
  TY* Y = static_cast<TY*>(d.y) + (int64_t)g * d.y_group_stride;
#pragma unroll
  for (int j = 0; j < RJ; ++j) {
    const int r = wr + j * 16 + l15;
    const int dst = yrow[r];
    if (dst < 0) continue;
    float scale = 1.f;
    if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE)
      scale = sigmoid_f(ld(static_cast<const TG*>(d.gate) + (int64_t)xrow[r] * d.gate_row_stride + g));
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + wm + i * 16 + gq * 4 + e;
        if (m >= d.m) continue;
        float v = acc[i][j][e];
        if (d.epilogue == PEGAINFER_EPI_RELU_SQ) { v = fmaxf(v, 0.f); v *= v; }
        else if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE) v *= scale;
        st(Y + (int64_t)dst * d.y_row_stride + m, v);
      }
  }
}

template <typename TX, typename TY, typename TG>
static void mfma_form_launch(const pegainfer_gemm_desc& d, hipStream_t s) {
  const bool big = d.tile_group ? d.tile_rows_cap >= 128 : d.rows > 64;
  const int TR = big ? 128 : 64;
  dim3 grid(d.tile_group ? d.max_tiles : ceil_div(d.rows, TR), ceil_div(d.m, MM), d.tile_group ? 1 : d.groups);
  if (big) gemm_strided_mfma_kernel<TX, TY, TG, 128><<<grid, 256, 0, s>>>(d);
  else gemm_strided_mfma_kernel<TX, TY, TG, 64><<<grid, 256, 0, s>>>(d);
}

// ------------------------------------------------------------------ few-rows form (decode)
// At most R rows per tile (a decode step's tokens, or the pairs one expert received): the weights are streamed once with
// 16-byte loads, the rows wait in LDS as fp32 (2048 k values at a time), a wave owns one output at a time (lanes over k, butterfly sum), 32 outputs per
// workgroup - or 8 (OUT) when 32 would leave most of the chip without a workgroup (a matrix of a few thousand outputs).  fp32
// arithmetic for both storage types; the k order of an output is fixed by K alone, whatever OUT is.
constexpr int kRowsFormChunk = 2048;   // k values of the rows that wait in LDS at a time (a multiple of the 512 a wave strides by)

template <typename TX, typename TW, typename TY, typename TG, int R, int OUT = 32>
__global__ __launch_bounds__(256) void gemm_strided_rows_kernel(pegainfer_gemm_desc d) {
  extern __shared__ __attribute__((aligned(16))) float xr[];    // [R][min(K, chunk)]
  __shared__ int xrow[R], yrow[R];
  int g, row0, nrows;
  if (d.tile_group) {
    if ((int)blockIdx.x >= *d.n_tiles) return;
    g = d.tile_group[blockIdx.x];
    row0 = d.tile_row0[blockIdx.x];
    nrows = min(R, d.tile_rows[blockIdx.x]);
  } else {
    g = blockIdx.z;
    row0 = blockIdx.x * R;
    nrows = min(R, d.rows - row0);
  }
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  if (tid < R) {
    const int p = row0 + tid;
    xrow[tid] = tid < nrows ? (d.x_row_index ? d.x_row_index[p] : p) : -1;
    yrow[tid] = tid < nrows ? (d.y_row_index ? d.y_row_index[p] : p) : -1;
  }
  __syncthreads();
  const TX* X = static_cast<const TX*>(d.x) + (int64_t)g * d.x_group_stride;
  const TW* W = static_cast<const TW*>(d.w) + (int64_t)g * d.w_group_stride;
  const int K = d.k, xs = min(K, kRowsFormChunk);
  TY* Y = static_cast<TY*>(d.y) + (int64_t)g * d.y_group_stride;
  // a wave owns a quarter of the workgroup's outputs and walks them four at a time: four independent weight streams in flight.
  // The rows pass through LDS a chunk of k at a time (a long row times eight rows would leave room for one workgroup per compute
  // unit); every output's sums stay in registers across the chunks, so its k order is what it would be in one piece.
  constexpr int OW = OUT / 4, MB = OW >= 4 ? 4 : OW, NG = OW / MB;
  const int m_base = blockIdx.y * OUT + wave * OW;
  float acc[NG][MB][R];
#pragma unroll
  for (int n = 0; n < NG; ++n)
#pragma unroll
    for (int q = 0; q < MB; ++q)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[n][q][r] = 0.f;
  for (int kc0 = 0; kc0 < K; kc0 += kRowsFormChunk) {
    const int kl = min(kRowsFormChunk, K - kc0);      // a multiple of 8, as K is
    if (kc0 > 0) __syncthreads();
    for (int i = tid * 8; i < R * kl; i += 2048) {
      const int r = i / kl, k = i - r * kl;
      float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (xrow[r] >= 0) Vec8<TX>::load(X + (int64_t)xrow[r] * d.x_row_stride + kc0 + k, t);
      *reinterpret_cast<f32x4*>(xr + r * xs + k) = f32x4{t[0], t[1], t[2], t[3]};
      *reinterpret_cast<f32x4*>(xr + r * xs + k + 4) = f32x4{t[4], t[5], t[6], t[7]};
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < NG; ++n) {
      const int mw = m_base + n * MB;
      if (mw >= d.m) continue;
      for (int k = lane * 8; k < kl; k += 512) {      // (unrolling this loop by four was measured: 52 -> 66 us for a 65 536 x 2048 matrix)
        float wv[MB][8];
#pragma unroll
        for (int q = 0; q < MB; ++q) {
          const int m = min(mw + q, d.m - 1);          // a clamped row is loaded and dropped at the store
          Vec8<TW>::load(W + (int64_t)m * d.w_m_stride + kc0 + k, wv[q]);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const f32x4 xa = *reinterpret_cast<const f32x4*>(xr + r * xs + k), xb = *reinterpret_cast<const f32x4*>(xr + r * xs + k + 4);
#pragma unroll
          for (int q = 0; q < MB; ++q) {
            float a = acc[n][q][r];
            a = fmaf(wv[q][0], xa.x, a); a = fmaf(wv[q][1], xa.y, a); a = fmaf(wv[q][2], xa.z, a); a = fmaf(wv[q][3], xa.w, a);
            a = fmaf(wv[q][4], xb.x, a); a = fmaf(wv[q][5], xb.y, a); a = fmaf(wv[q][6], xb.z, a); a = fmaf(wv[q][7], xb.w, a);
            acc[n][q][r] = a;
          }
        }
      }
    }
  }
#pragma unroll
  for (int n = 0; n < NG; ++n) {
    const int mw = m_base + n * MB;
    if (mw >= d.m) continue;
#pragma unroll
    for (int q = 0; q < MB; ++q)
#pragma unroll
      for (int r = 0; r < R; ++r) acc[n][q][r] = wave_sum(acc[n][q][r]);
    if (lane == 0) {
#pragma unroll
      for (int q = 0; q < MB; ++q) {
        const int m = mw + q;
        if (m >= d.m) break;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (yrow[r] < 0) continue;
          float v = acc[n][q][r];
          if (d.epilogue == PEGAINFER_EPI_RELU_SQ) { v = fmaxf(v, 0.f); v *= v; }
          else if (d.epilogue == PEGAINFER_EPI_SIGMOID_GATE)
            v *= sigmoid_f(ld(static_cast<const TG*>(d.gate) + (int64_t)xrow[r] * d.gate_row_stride + g));
          st(Y + (int64_t)yrow[r] * d.y_row_stride + m, v);
        }
      }
    }
  }
}

template <typename TX, typename TW, typename TY, typename TG, int R>
static void rows_form_launch(const pegainfer_gemm_desc& d, hipStream_t s) {
  auto kern = &gemm_strided_rows_kernel<TX, TW, TY, TG, R, 32>;
  auto kern8 = &gemm_strided_rows_kernel<TX, TW, TY, TG, R, 8>;
  // 150 KB of rows at most (checked by the caller) next to the kernel's few static words
  static const bool once = (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024),
                            hipFuncSetAttribute(reinterpret_cast<const void*>(kern8), hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024),
                            true);
  (void)once;
  const int row_tiles = d.tile_group ? d.max_tiles : ceil_div(d.rows, R), groups = d.tile_group ? 1 : d.groups;
  // 32 outputs per workgroup unless that leaves most compute units without one
  const bool fine = (long)row_tiles * groups * ceil_div(d.m, 32) < device_cus();
  dim3 grid(row_tiles, ceil_div(d.m, fine ? 8 : 32), groups);
  const size_t lds = (size_t)R * std::min(d.k, kRowsFormChunk) * sizeof(float);
  if (fine) kern8<<<grid, 256, lds, s>>>(d);
  else kern<<<grid, 256, lds, s>>>(d);
}

static inline bool chunks_ok(const pegainfer_gemm_desc& d) {
  auto a16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return d.w_k_stride == 1 && (d.k & 7) == 0 && (d.x_row_stride & 7) == 0 && (d.x_group_stride & 7) == 0 &&
         (d.w_m_stride & 7) == 0 && (d.w_group_stride & 7) == 0 && a16(d.x) && a16(d.w);
}

template <typename TX, typename TW, typename TY>
static bool gemm_strided_launch(const pegainfer_gemm_desc& d, hipStream_t s) {
  dim3 grid(d.tile_group ? d.max_tiles : ceil_div(d.rows, GT), ceil_div(d.m, GM), d.tile_group ? 1 : d.groups);
  const bool gate32 = d.gate_dtype == kDtF32;
  if (!d.plain && chunks_ok(d)) {
    // few rows per tile: stream the weights once (both storage types, fp32 arithmetic)
    const int tr = d.tile_group ? (d.max_tile_rows > 0 ? d.max_tile_rows : (d.tile_rows_cap > 0 ? d.tile_rows_cap : GT)) : d.rows;
    const int R = tr <= 1 ? 1 : tr <= 4 ? 4 : tr <= 8 ? 8 : 0;
    if (R && (size_t)R * d.k * sizeof(float) <= 150 * 1024) {
      if (gate32) { if (R == 1) rows_form_launch<TX, TW, TY, float, 1>(d, s); else if (R == 4) rows_form_launch<TX, TW, TY, float, 4>(d, s); else rows_form_launch<TX, TW, TY, float, 8>(d, s); }
      else { if (R == 1) rows_form_launch<TX, TW, TY, uint16_t, 1>(d, s); else if (R == 4) rows_form_launch<TX, TW, TY, uint16_t, 4>(d, s); else rows_form_launch<TX, TW, TY, uint16_t, 8>(d, s); }
      return true;
    }
    if constexpr (std::is_same<TW, uint16_t>::value) {   // bf16 weights: the matrix cores
      if (gate32) mfma_form_launch<TX, TY, float>(d, s);
      else mfma_form_launch<TX, TY, uint16_t>(d, s);
      return true;
    }
  }
  if (d.tile_group && d.tile_rows_cap > GT) return false;   // a table cut for 128-row tiles cannot be walked by the 64-row form
  if (gate32) gemm_strided_kernel<TX, TW, TY, float><<<grid, 256, 0, s>>>(d);
  else gemm_strided_kernel<TX, TW, TY, uint16_t><<<grid, 256, 0, s>>>(d);
  return true;
}

}  // namespace pk

extern "C" pegainfer_status_t pegainfer_gemm_strided(const pegainfer_gemm_desc* dp, pegainfer_stream_t stream) {
  using namespace pk;
  const pegainfer_gemm_desc& d = *dp;
  if (d.m <= 0 || d.k <= 0) return 0;
  if (d.tile_group ? d.max_tiles <= 0 : (d.rows <= 0 || d.groups <= 0)) return 0;
  hipStream_t s = as_stream(stream);
  const int key = (d.x_dtype << 2) | (d.w_dtype << 1) | d.y_dtype;
  bool ok = false;
  switch (key) {
    case 0: ok = gemm_strided_launch<uint16_t, uint16_t, uint16_t>(d, s); break;
    case 1: ok = gemm_strided_launch<uint16_t, uint16_t, float>(d, s); break;
    case 4: ok = gemm_strided_launch<float, uint16_t, uint16_t>(d, s); break;
    case 5: ok = gemm_strided_launch<float, uint16_t, float>(d, s); break;
    case 7: ok = gemm_strided_launch<float, float, float>(d, s); break;
    default: break;
  }
  if (!ok) return (pegainfer_status_t)hipErrorInvalidValue;
  return (pegainfer_status_t)hipGetLastError();
}

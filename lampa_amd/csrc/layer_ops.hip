// The two HBM-bound operators either side of the gated-delta forward in a layer, on gfx950:
//   * depthwise causal short convolution (+ bias, SiLU, residual), dense or packed variable-length sequences;
//   * RMS norm with optional residual add, weight, bias and swish / sigmoid output gate.
//
// Replaces (reference chengjiang123/Lampa): causal_conv1d_fwd_kernel / causal_conv1d
// models/hattention/short_convolution.py:39-99, and layer_norm_gated_fwd_kernel / layer_norm_fwd_kernel with
// IS_RMS_NORM  models/hattention/fused_norm.py:40-111,1436-1506.
//
// Both read every input element once and write every output element once with 16-byte accesses; arithmetic is fp32,
// results are rounded to the output type (round to nearest even).
#include "gdr_common.h"

#define LO_BLOCK 256
enum { LO_ACT_NONE = 0, LO_ACT_SILU = 1, LO_ACT_SIGMOID = 2 };

__device__ __forceinline__ float lo_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T>
__device__ __forceinline__ void store8(T* p, const float* v) {
  if constexpr (sizeof(T) == 2) {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    vec8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = GdrElem<T>::from_float(v[i]);
    *reinterpret_cast<vec8*>(p) = o;
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
}

// ------------------------------------------------------------------------------------------ short convolution
// y[t, d] = act(bias[d] + sum_{j < W} weight[d, j] * x[t - (W-1) + j, d]) + residual[t, d], taps before the start of
// the token's sequence read as zero. One thread: 8 channels x CV_TOKENS consecutive tokens, the W-1 rows of history
// kept in registers, so a row of x is read 1 + (W-1)/CV_TOKENS times (the repeats hit in L2).
#define CV_TOKENS 16
#define CV_MAX_W 8

template <typename T, int W>
__global__ void __launch_bounds__(LO_BLOCK) lo_conv_kernel(const T* __restrict__ x, int64_t x_stride, int64_t n_tokens, int D,
                                                          const float* __restrict__ weight, const float* __restrict__ bias,
                                                          const T* __restrict__ residual, int64_t res_stride,
                                                          const int64_t* __restrict__ cu_seqlens, int n_seq, int64_t t_len,
                                                          int activation, T* __restrict__ y, int64_t y_stride) {
  const int groups = D / 8;                                      // channel groups of 8
  const int64_t item = (int64_t)blockIdx.x * LO_BLOCK + threadIdx.x;
  const int cg = (int)(item % groups);
  const int64_t t0 = (item / groups) * CV_TOKENS;
  if (t0 >= n_tokens) return;
  const int c0 = cg * 8;
  float w[W][8], b[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    b[c] = bias ? bias[c0 + c] : 0.0f;
#pragma unroll
    for (int j = 0; j < W; ++j) w[j][c] = weight[(int64_t)(c0 + c) * W + j];
  }
  // start of the sequence that holds token t0
  int seq = 0;
  int64_t bos, eos;
  if (cu_seqlens) {
    int lo = 0, hi = n_seq - 1;                                  // last s with cu[s] <= t0
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seqlens[mid] <= t0) lo = mid; else hi = mid - 1;
    }
    seq = lo;
    bos = cu_seqlens[seq];
    eos = cu_seqlens[seq + 1];
  } else {
    bos = t0 / t_len * t_len;
    eos = bos + t_len;
  }
  float hist[W - 1 > 0 ? W - 1 : 1][8];                          // hist[j] = x[t - (W-1) + j] for the current t
#pragma unroll
  for (int j = 0; j < W - 1; ++j) {
    const int64_t tt = t0 - (W - 1) + j;
    if (tt >= bos) load8(x + tt * x_stride + c0, hist[j]);
    else {
#pragma unroll
      for (int c = 0; c < 8; ++c) hist[j][c] = 0.0f;
    }
  }
#pragma unroll 4
  for (int i = 0; i < CV_TOKENS; ++i) {
    const int64_t t = t0 + i;
    if (t >= n_tokens) break;
    if (t >= eos) {                                              // next sequence: its history is empty
      if (cu_seqlens) {
        while (seq < n_seq - 1 && cu_seqlens[seq + 1] <= t) ++seq;  // skips empty sequences
        bos = cu_seqlens[seq];
        eos = cu_seqlens[seq + 1];
        if (t >= eos) eos = INT64_MAX;                           // tokens beyond the last boundary: one trailing run
      } else {
        bos = eos;
        eos = bos + t_len;
      }
#pragma unroll
      for (int j = 0; j < W - 1; ++j)
#pragma unroll
        for (int c = 0; c < 8; ++c) hist[j][c] = 0.0f;
    }
    float cur[8], acc[8];
    load8(x + t * x_stride + c0, cur);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      float a = 0.0f;
#pragma unroll
      for (int j = 0; j < W - 1; ++j) a = __builtin_fmaf(hist[j][c], w[j][c], a);
      a = __builtin_fmaf(cur[c], w[W - 1][c], a) + b[c];
      if (activation == LO_ACT_SILU) a = a * lo_sigmoid(a);
      acc[c] = a;
    }
    if (residual) {
      float r[8];
      load8(residual + t * res_stride + c0, r);
#pragma unroll
      for (int c = 0; c < 8; ++c) acc[c] += r[c];
    }
    store8(y + t * y_stride + c0, acc);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
#pragma unroll
      for (int j = 0; j + 1 < W - 1; ++j) hist[j][c] = hist[j + 1][c];
      if (W > 1) hist[W - 2 > 0 ? W - 2 : 0][c] = cur[c];
    }
  }
}

template <typename T>
static int lo_conv_launch(const void* x, int64_t x_stride, int64_t n_tokens, int D, int W, const float* weight,
                          const float* bias, const void* residual, int64_t res_stride, const int64_t* cu, int n_seq,
                          int64_t t_len, int activation, void* y, int64_t y_stride, hipStream_t s) {
  const int64_t items = (int64_t)(D / 8) * ((n_tokens + CV_TOKENS - 1) / CV_TOKENS);
  const dim3 grid((unsigned)((items + LO_BLOCK - 1) / LO_BLOCK)), block(LO_BLOCK);
  LAMPA_PROF(s, "start");
#define LO_CONV_CASE(WW)                                                                                              \
  case WW:                                                                                                            \
    hipLaunchKernelGGL((lo_conv_kernel<T, WW>), grid, block, 0, s, (const T*)x, x_stride, n_tokens, D, weight, bias,  \
                       (const T*)residual, res_stride, cu, n_seq, t_len, activation, (T*)y, y_stride);               \
    break;
  switch (W) {
    LO_CONV_CASE(1) LO_CONV_CASE(2) LO_CONV_CASE(3) LO_CONV_CASE(4) LO_CONV_CASE(5) LO_CONV_CASE(6) LO_CONV_CASE(7)
    LO_CONV_CASE(8)
    default: return LAMPA_ERR_UNSUPPORTED;
  }
#undef LO_CONV_CASE
  LAMPA_PROF(s, "lo_conv_kernel");
  return lampa_launch_status();
}

// x [n_tokens, D] with row stride x_stride elements (a slice of a wider projection output is fine), weight fp32 [D, W]
// (tap W-1 multiplies the current token), bias fp32 [D] or NULL, residual [n_tokens, D] (row stride res_stride) or
// NULL, y [n_tokens, D] (row stride y_stride). Sequences: cu_seqlens (device int64 [n_seq + 1]) or NULL for
// n_tokens / t_len dense sequences of t_len tokens. D % 8 == 0, strides % 8 == 0, 16-byte aligned pointers, W <= 8.
// dtype LAMPA_BF16 / LAMPA_FP16 / LAMPA_FP32 (0 / 1 / 2) of x, residual and y. activation 0 none, 1 SiLU.
extern "C" int lampa_causal_conv1d_fwd(const void* x, int64_t x_stride, int64_t n_tokens, int D, int W, const float* weight,
                                       const float* bias, const void* residual, int64_t res_stride,
                                       const int64_t* cu_seqlens, int n_seq, int64_t t_len, int activation, int dtype,
                                       void* y, int64_t y_stride, void* stream) {
  if (!x || !weight || !y || n_tokens < 0 || D < 8 || W < 1) return LAMPA_ERR_INVALID;
  if (D % 8 || x_stride % 8 || y_stride % 8 || (residual && res_stride % 8) || W > CV_MAX_W) return LAMPA_ERR_UNSUPPORTED;
  if (x_stride < D || y_stride < D || (residual && res_stride < D)) return LAMPA_ERR_INVALID;
  if (((uintptr_t)x | (uintptr_t)y | (uintptr_t)residual) % 16) return LAMPA_ERR_UNSUPPORTED;
  if (activation != LO_ACT_NONE && activation != LO_ACT_SILU) return LAMPA_ERR_INVALID;
  if (cu_seqlens ? n_seq < 1 : (t_len < 1 || n_tokens % t_len != 0)) return LAMPA_ERR_INVALID;
  if (n_tokens == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case 0: return lo_conv_launch<__bf16>(x, x_stride, n_tokens, D, W, weight, bias, residual, res_stride, cu_seqlens, n_seq, t_len, activation, y, y_stride, s);
    case 1: return lo_conv_launch<_Float16>(x, x_stride, n_tokens, D, W, weight, bias, residual, res_stride, cu_seqlens, n_seq, t_len, activation, y, y_stride, s);
    case 2: return lo_conv_launch<float>(x, x_stride, n_tokens, D, W, weight, bias, residual, res_stride, cu_seqlens, n_seq, t_len, activation, y, y_stride, s);
    default: return LAMPA_ERR_INVALID;
  }
}

// ------------------------------------------------------------------------------------------------- RMS norm
// Row r: s = x[r] (+ residual[r]); residual_out[r] = s; rstd = 1 / sqrt(mean(s^2) + eps); y = s * rstd * weight + bias;
// y *= g * sigmoid(g) (swish) or sigmoid(g). LPR lanes share a row, each owning 8 consecutive channels per step.
template <typename T, typename RT, int LPR>
__global__ void __launch_bounds__(LO_BLOCK) lo_rms_norm_kernel(const T* __restrict__ x, const T* __restrict__ g,
                                                              const float* __restrict__ weight, const float* __restrict__ bias,
                                                              const RT* __restrict__ residual, RT* __restrict__ residual_out,
                                                              T* __restrict__ y, float* __restrict__ rstd_out, int64_t rows,
                                                              int D, float eps, int activation) {
  constexpr int ROWS_PER_WAVE = 64 / LPR;
  constexpr int MAX_STEPS = 4;                                   // D <= LPR * 8 * MAX_STEPS
  const int lane = lane_id();
  const int64_t wave = ((int64_t)blockIdx.x * LO_BLOCK + threadIdx.x) >> 6;
  const int64_t row = wave * ROWS_PER_WAVE + lane / LPR;
  const int sub = lane % LPR;
  const bool live = row < rows;
  float v[MAX_STEPS][8];
  float ss = 0.0f;
#pragma unroll
  for (int st = 0; st < MAX_STEPS; ++st) {
    const int c0 = (st * LPR + sub) * 8;
    const bool on = live && c0 < D;
    if (on) {
      load8(x + row * D + c0, v[st]);
      if (residual) {
        float r[8];
        load8(residual + row * D + c0, r);
#pragma unroll
        for (int c = 0; c < 8; ++c) v[st][c] += r[c];
      }
      if (residual_out) store8(residual_out + row * D + c0, v[st]);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) v[st][c] = 0.0f;
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) ss = __builtin_fmaf(v[st][c], v[st][c], ss);
  }
#pragma unroll
  for (int off = 1; off < LPR; off <<= 1) ss += __shfl_xor(ss, off);
  const float rstd = 1.0f / sqrtf(ss / (float)D + eps);
  if (rstd_out && live && sub == 0) rstd_out[row] = rstd;
#pragma unroll
  for (int st = 0; st < MAX_STEPS; ++st) {
    const int c0 = (st * LPR + sub) * 8;
    if (!(live && c0 < D)) continue;
    float o[8], gate[8], wv[8], bv[8];
    if (g) load8(g + row * D + c0, gate);
    if (weight) load8(weight + c0, wv);
    if (bias) load8(bias + c0, bv);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      float t = v[st][c] * rstd;
      if (weight) t *= wv[c];
      if (bias) t += bv[c];
      if (g) t = activation == LO_ACT_SIGMOID ? t * lo_sigmoid(gate[c]) : t * gate[c] * lo_sigmoid(gate[c]);
      o[c] = t;
    }
    store8(y + row * D + c0, o);
  }
}

template <typename T, typename RT>
static int lo_norm_launch(const void* x, const void* g, const float* weight, const float* bias, const void* residual,
                          void* residual_out, void* y, float* rstd, int64_t rows, int D, float eps, int activation,
                          hipStream_t s) {
  int lpr = 8;
  while (lpr < 64 && lpr * 8 < D) lpr <<= 1;
  if (D > lpr * 8 * 4) return LAMPA_ERR_UNSUPPORTED;
  const int64_t waves = (rows + 64 / lpr - 1) / (64 / lpr);
  const dim3 grid((unsigned)((waves * 64 + LO_BLOCK - 1) / LO_BLOCK)), block(LO_BLOCK);
  LAMPA_PROF(s, "start");
#define LO_NORM_CASE(L)                                                                                               \
  case L:                                                                                                             \
    hipLaunchKernelGGL((lo_rms_norm_kernel<T, RT, L>), grid, block, 0, s, (const T*)x, (const T*)g, weight, bias,     \
                       (const RT*)residual, (RT*)residual_out, (T*)y, rstd, rows, D, eps, activation);               \
    break;
  switch (lpr) { LO_NORM_CASE(8) LO_NORM_CASE(16) LO_NORM_CASE(32) LO_NORM_CASE(64) }
#undef LO_NORM_CASE
  LAMPA_PROF(s, "lo_rms_norm_kernel");
  return lampa_launch_status();
}

// x, y, g [rows, D] of dtype (0 bf16, 1 fp16, 2 fp32); g NULL = no gate; weight, bias fp32 [D] or NULL;
// residual / residual_out [rows, D] of res_dtype (same codes) or NULL; rstd_out fp32 [rows] or NULL.
// activation: 1 swish / SiLU gate, 2 sigmoid gate (ignored without g). D % 8 == 0, D <= 2048.
extern "C" int lampa_rms_norm_fwd(const void* x, const void* g, const float* weight, const float* bias, const void* residual,
                                  void* residual_out, void* y, float* rstd_out, int64_t rows, int D, float eps,
                                  int activation, int dtype, int res_dtype, void* stream) {
  if (!x || !y || rows < 0 || D < 1) return LAMPA_ERR_INVALID;
  if (D % 8 || D > 2048) return LAMPA_ERR_UNSUPPORTED;
  if (g && activation != LO_ACT_SILU && activation != LO_ACT_SIGMOID) return LAMPA_ERR_INVALID;
  if (((uintptr_t)x | (uintptr_t)y | (uintptr_t)g | (uintptr_t)residual | (uintptr_t)residual_out) % 16)
    return LAMPA_ERR_UNSUPPORTED;
  if (rows == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  const bool res = residual || residual_out;
  if (!res) res_dtype = dtype;
#define LO_NORM_DISPATCH(T)                                                                                            \
  switch (res_dtype) {                                                                                                 \
    case 0: return lo_norm_launch<T, __bf16>(x, g, weight, bias, residual, residual_out, y, rstd_out, rows, D, eps, activation, s);   \
    case 1: return lo_norm_launch<T, _Float16>(x, g, weight, bias, residual, residual_out, y, rstd_out, rows, D, eps, activation, s); \
    case 2: return lo_norm_launch<T, float>(x, g, weight, bias, residual, residual_out, y, rstd_out, rows, D, eps, activation, s);    \
    default: return LAMPA_ERR_INVALID;                                                                                 \
  }
  switch (dtype) {
    case 0: LO_NORM_DISPATCH(__bf16)
    case 1: LO_NORM_DISPATCH(_Float16)
    case 2: LO_NORM_DISPATCH(float)
    default: return LAMPA_ERR_INVALID;
  }
#undef LO_NORM_DISPATCH
}

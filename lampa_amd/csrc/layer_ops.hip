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
// Hardware exp2 and reciprocal (about 1 ulp each): the element-wise kernels stay memory bound instead of spending
// their time in the correctly rounded library exp and division.
__device__ __forceinline__ float lo_sigmoid_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

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
// the token's sequence read as zero. One thread: 8 channels x CV_TOKENS consecutive tokens with their W-1 rows of
// history in registers, so a row of x is read 1 + (W-1)/CV_TOKENS times (the repeats hit in L2).
#define CV_TOKENS 16
#define CV_MAX_W 8

template <typename T>
struct LoRaw8;  // 8 consecutive elements as loaded: 16 bytes for the 2-byte types, 32 for fp32
template <>
struct LoRaw8<float> { f32x4 a, b; };
template <>
struct LoRaw8<__bf16> { typedef __bf16 vec8 __attribute__((ext_vector_type(8))); vec8 v; };
template <>
struct LoRaw8<_Float16> { typedef _Float16 vec8 __attribute__((ext_vector_type(8))); vec8 v; };

template <typename T>
__device__ __forceinline__ LoRaw8<T> lo_load_raw(const T* p) {
  LoRaw8<T> r;
  if constexpr (sizeof(T) == 2) r.v = *reinterpret_cast<const typename LoRaw8<T>::vec8*>(p);
  else { r.a = *reinterpret_cast<const f32x4*>(p); r.b = *reinterpret_cast<const f32x4*>(p + 4); }
  return r;
}
template <typename T>
__device__ __forceinline__ float lo_raw_get(const LoRaw8<T>& r, int c) {
  if constexpr (sizeof(T) == 2) return GdrElem<T>::to_float(r.v[c]);
  else return c < 4 ? r.a[c] : r.b[c - 4];
}

// All CV_TOKENS + W - 1 rows of a thread are requested before the first is used (one wait instead of one per token).
// Output column c goes to y + (c / y_split) * y_split_stride + t * y_stride + c % y_split: with y_split < D one launch
// over the q | k | v columns of a fused projection writes three separate [tokens, y_split] tensors.
template <typename T, int W>
__global__ void __launch_bounds__(LO_BLOCK) lo_conv_kernel(const T* __restrict__ x, int64_t x_stride, int64_t n_tokens, int D,
                                                          const float* __restrict__ weight, const float* __restrict__ bias,
                                                          const T* __restrict__ residual, int64_t res_stride,
                                                          const int64_t* __restrict__ cu_seqlens, int n_seq, int64_t t_len,
                                                          int activation, T* __restrict__ y, int64_t y_stride, int y_split,
                                                          int64_t y_split_stride) {
  const int groups = D / 8;                                      // channel groups of 8
  const int64_t item = (int64_t)blockIdx.x * LO_BLOCK + threadIdx.x;
  const int cg = (int)(item % groups);
  const int64_t t0 = (item / groups) * CV_TOKENS;
  if (t0 >= n_tokens) return;
  const int c0 = cg * 8;
  constexpr int ROWS = CV_TOKENS + W - 1;
  LoRaw8<T> raw[ROWS];                                           // raw[r] = x[t0 - (W-1) + r]
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    int64_t tt = t0 - (W - 1) + r;
    tt = tt < 0 ? 0 : (tt >= n_tokens ? n_tokens - 1 : tt);      // clamped: rows outside the sequence are masked below
    raw[r] = lo_load_raw(x + tt * x_stride + c0);
  }
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
  T* ybase = y + (int64_t)(c0 / y_split) * y_split_stride + (c0 % y_split);
  auto finish = [&](int64_t t, float* acc) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      acc[c] += b[c];
      if (activation == LO_ACT_SILU) acc[c] = acc[c] * lo_sigmoid_fast(acc[c]);
    }
    if (residual) {
      float r[8];
      load8(residual + t * res_stride + c0, r);
#pragma unroll
      for (int c = 0; c < 8; ++c) acc[c] += r[c];
    }
    store8(ybase + t * y_stride, acc);
  };
  if (t0 - (W - 1) >= bos && t0 + CV_TOKENS <= eos && t0 + CV_TOKENS <= n_tokens) {
    // every tap of every token lies inside one sequence: no masks
#pragma unroll
    for (int i = 0; i < CV_TOKENS; ++i) {
      float acc[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float a = 0.0f;
#pragma unroll
        for (int j = 0; j < W; ++j) a = __builtin_fmaf(lo_raw_get(raw[i + j], c), w[j][c], a);
        acc[c] = a;
      }
      finish(t0 + i, acc);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < CV_TOKENS; ++i) {
    const int64_t t = t0 + i;
    if (t < n_tokens) {
      if (t >= eos) {                                            // next sequence: its history is empty
        if (cu_seqlens) {
          while (seq < n_seq - 1 && cu_seqlens[seq + 1] <= t) ++seq;  // skips empty sequences
          bos = cu_seqlens[seq];
          eos = cu_seqlens[seq + 1];
          if (t >= eos) eos = INT64_MAX;                         // tokens beyond the last boundary: one trailing run
        } else {
          bos = eos;
          eos = bos + t_len;
        }
      }
      float acc[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float a = 0.0f;
#pragma unroll
        for (int j = 0; j < W; ++j) {
          const float xv = (t - (W - 1) + j) >= bos ? lo_raw_get(raw[i + j], c) : 0.0f;
          a = __builtin_fmaf(xv, w[j][c], a);
        }
        acc[c] = a;
      }
      finish(t, acc);
    }
  }
}

template <typename T>
static int lo_conv_launch(const void* x, int64_t x_stride, int64_t n_tokens, int D, int W, const float* weight,
                          const float* bias, const void* residual, int64_t res_stride, const int64_t* cu, int n_seq,
                          int64_t t_len, int activation, void* y, int64_t y_stride, int y_split, int64_t y_split_stride,
                          hipStream_t s) {
  const int64_t items = (int64_t)(D / 8) * ((n_tokens + CV_TOKENS - 1) / CV_TOKENS);
  const dim3 grid((unsigned)((items + LO_BLOCK - 1) / LO_BLOCK)), block(LO_BLOCK);
  LAMPA_PROF(s, "start");
#define LO_CONV_CASE(WW)                                                                                              \
  case WW:                                                                                                            \
    hipLaunchKernelGGL((lo_conv_kernel<T, WW>), grid, block, 0, s, (const T*)x, x_stride, n_tokens, D, weight, bias,  \
                       (const T*)residual, res_stride, cu, n_seq, t_len, activation, (T*)y, y_stride, y_split,      \
                       y_split_stride);                                                                              \
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
// y_split in (0, D) with D % y_split == 0 splits the output columns over D / y_split tensors of [n_tokens, y_split]
// (row stride y_stride) that lie y_split_stride elements apart; y_split <= 0 or == D: one [n_tokens, D] output.
extern "C" int lampa_causal_conv1d_fwd(const void* x, int64_t x_stride, int64_t n_tokens, int D, int W, const float* weight,
                                       const float* bias, const void* residual, int64_t res_stride,
                                       const int64_t* cu_seqlens, int n_seq, int64_t t_len, int activation, int dtype,
                                       void* y, int64_t y_stride, int y_split, int64_t y_split_stride, void* stream) {
  if (!x || !weight || !y || n_tokens < 0 || D < 8 || W < 1) return LAMPA_ERR_INVALID;
  if (y_split <= 0 || y_split == D) { y_split = D; y_split_stride = 0; }
  if (D % y_split || y_split % 8 || y_split_stride % 8 || y_stride < y_split) return LAMPA_ERR_INVALID;
  if (D % 8 || x_stride % 8 || y_stride % 8 || (residual && res_stride % 8) || W > CV_MAX_W) return LAMPA_ERR_UNSUPPORTED;
  if (x_stride < D || (residual && res_stride < D)) return LAMPA_ERR_INVALID;
  if (((uintptr_t)x | (uintptr_t)y | (uintptr_t)residual) % 16) return LAMPA_ERR_UNSUPPORTED;
  if (activation != LO_ACT_NONE && activation != LO_ACT_SILU) return LAMPA_ERR_INVALID;
  if (cu_seqlens ? n_seq < 1 : (t_len < 1 || n_tokens % t_len != 0)) return LAMPA_ERR_INVALID;
  if (n_tokens == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case 0: return lo_conv_launch<__bf16>(x, x_stride, n_tokens, D, W, weight, bias, residual, res_stride, cu_seqlens, n_seq, t_len, activation, y, y_stride, y_split, y_split_stride, s);
    case 1: return lo_conv_launch<_Float16>(x, x_stride, n_tokens, D, W, weight, bias, residual, res_stride, cu_seqlens, n_seq, t_len, activation, y, y_stride, y_split, y_split_stride, s);
    case 2: return lo_conv_launch<float>(x, x_stride, n_tokens, D, W, weight, bias, residual, res_stride, cu_seqlens, n_seq, t_len, activation, y, y_stride, y_split, y_split_stride, s);
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
                                                              int D, float eps, int activation, int g_group,
                                                              int64_t g_group_stride) {
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
    // the gate may be a slice of a wider tensor: g_group rows of D channels per token, tokens g_group_stride apart
    if (g) load8(g + (row / g_group) * g_group_stride + (row % g_group) * D + c0, gate);
    if (weight) load8(weight + c0, wv);
    if (bias) load8(bias + c0, bv);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      float t = v[st][c] * rstd;
      if (weight) t *= wv[c];
      if (bias) t += bv[c];
      if (g) t = activation == LO_ACT_SIGMOID ? t * lo_sigmoid_fast(gate[c]) : t * gate[c] * lo_sigmoid_fast(gate[c]);
      o[c] = t;
    }
    store8(y + row * D + c0, o);
  }
}

template <typename T, typename RT>
static int lo_norm_launch(const void* x, const void* g, const float* weight, const float* bias, const void* residual,
                          void* residual_out, void* y, float* rstd, int64_t rows, int D, float eps, int activation,
                          int g_group, int64_t g_group_stride, hipStream_t s) {
  int lpr = 8;
  while (lpr < 64 && lpr * 8 < D) lpr <<= 1;
  if (D > lpr * 8 * 4) return LAMPA_ERR_UNSUPPORTED;
  const int64_t waves = (rows + 64 / lpr - 1) / (64 / lpr);
  const dim3 grid((unsigned)((waves * 64 + LO_BLOCK - 1) / LO_BLOCK)), block(LO_BLOCK);
  LAMPA_PROF(s, "start");
#define LO_NORM_CASE(L)                                                                                               \
  case L:                                                                                                             \
    hipLaunchKernelGGL((lo_rms_norm_kernel<T, RT, L>), grid, block, 0, s, (const T*)x, (const T*)g, weight, bias,     \
                       (const RT*)residual, (RT*)residual_out, (T*)y, rstd, rows, D, eps, activation, g_group,       \
                       g_group_stride);                                                                              \
    break;
  switch (lpr) { LO_NORM_CASE(8) LO_NORM_CASE(16) LO_NORM_CASE(32) LO_NORM_CASE(64) }
#undef LO_NORM_CASE
  LAMPA_PROF(s, "lo_rms_norm_kernel");
  return lampa_launch_status();
}

// x, y, g [rows, D] of dtype (0 bf16, 1 fp16, 2 fp32); g NULL = no gate; weight, bias fp32 [D] or NULL;
// residual / residual_out [rows, D] of res_dtype (same codes) or NULL; rstd_out fp32 [rows] or NULL.
// activation: 1 swish / SiLU gate, 2 sigmoid gate (ignored without g). D % 8 == 0, D <= 2048.
// g_group > 0: the gate is a slice of a wider tensor, g_group rows of D channels per token and g_group_stride elements
// from one token to the next (a multiple of 8); g_group <= 0: g is [rows, D] contiguous.
extern "C" int lampa_rms_norm_fwd(const void* x, const void* g, const float* weight, const float* bias, const void* residual,
                                  void* residual_out, void* y, float* rstd_out, int64_t rows, int D, float eps,
                                  int activation, int dtype, int res_dtype, int g_group, int64_t g_group_stride,
                                  void* stream) {
  if (!x || !y || rows < 0 || D < 1) return LAMPA_ERR_INVALID;
  if (g_group <= 0) { g_group = 1; g_group_stride = D; }
  if (g && (g_group_stride % 8 || g_group_stride < (int64_t)g_group * D)) return LAMPA_ERR_INVALID;
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
    case 0: return lo_norm_launch<T, __bf16>(x, g, weight, bias, residual, residual_out, y, rstd_out, rows, D, eps, activation, g_group, g_group_stride, s);   \
    case 1: return lo_norm_launch<T, _Float16>(x, g, weight, bias, residual, residual_out, y, rstd_out, rows, D, eps, activation, g_group, g_group_stride, s); \
    case 2: return lo_norm_launch<T, float>(x, g, weight, bias, residual, residual_out, y, rstd_out, rows, D, eps, activation, g_group, g_group_stride, s);    \
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

// --------------------------------------------------------------------------------------- decay and write gates
// g[t, h] = -exp(A_log[h]) * softplus(a[t, h] + dt_bias[h]),  beta[t, h] = sigmoid(b[t, h]) * beta_scale, in fp32.
// softplus(x) = x for x > 20, else log1p(exp(x)) (the threshold of torch.nn.functional.softplus).
template <typename T>
__global__ void __launch_bounds__(LO_BLOCK) lo_gates_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ b,
                                                           int64_t b_stride, const float* __restrict__ A_log,
                                                           const float* __restrict__ dt_bias, int64_t n_tokens, int H,
                                                           float beta_scale, float* __restrict__ g, float* __restrict__ beta) {
  const int64_t i = (int64_t)blockIdx.x * LO_BLOCK + threadIdx.x;
  if (i >= n_tokens * H) return;
  const int64_t t = i / H;
  const int h = (int)(i - t * H);
  const float x = GdrElem<T>::to_float(a[t * a_stride + h]) + dt_bias[h];
  const float sp = x > 20.0f ? x : log1pf(expf(x));
  g[i] = -expf(A_log[h]) * sp;
  beta[i] = lo_sigmoid(GdrElem<T>::to_float(b[t * b_stride + h])) * beta_scale;
}

// a, b [n_tokens, H] of dtype with row strides in elements (slices of a wider projection output are fine);
// A_log, dt_bias fp32 [H]; g, beta fp32 [n_tokens, H] contiguous.
extern "C" int lampa_gdr_gates_fwd(const void* a, int64_t a_stride, const void* b, int64_t b_stride, const float* A_log,
                                   const float* dt_bias, int64_t n_tokens, int H, float beta_scale, int dtype, float* g,
                                   float* beta, void* stream) {
  if (!a || !b || !A_log || !dt_bias || !g || !beta || n_tokens < 0 || H < 1 || a_stride < H || b_stride < H)
    return LAMPA_ERR_INVALID;
  if (n_tokens == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((n_tokens * H + LO_BLOCK - 1) / LO_BLOCK)), block(LO_BLOCK);
  LAMPA_PROF(s, "start");
  switch (dtype) {
    case 0: hipLaunchKernelGGL(lo_gates_kernel<__bf16>, grid, block, 0, s, (const __bf16*)a, a_stride, (const __bf16*)b, b_stride, A_log, dt_bias, n_tokens, H, beta_scale, g, beta); break;
    case 1: hipLaunchKernelGGL(lo_gates_kernel<_Float16>, grid, block, 0, s, (const _Float16*)a, a_stride, (const _Float16*)b, b_stride, A_log, dt_bias, n_tokens, H, beta_scale, g, beta); break;
    case 2: hipLaunchKernelGGL(lo_gates_kernel<float>, grid, block, 0, s, (const float*)a, a_stride, (const float*)b, b_stride, A_log, dt_bias, n_tokens, H, beta_scale, g, beta); break;
    default: return LAMPA_ERR_INVALID;
  }
  LAMPA_PROF(s, "lo_gates_kernel");
  return lampa_launch_status();
}

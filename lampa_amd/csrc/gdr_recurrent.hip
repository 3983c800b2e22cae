// Token-serial gated-delta-rule forward with an fp32 state held in registers (gfx950).
//
// One wave owns up to 64 value columns of one (sequence, value head): lane = value column, and every lane keeps
// the K state rows of its column in registers, so the three contractions of a step (S^T k, the rank-one update
// and S^T q) are per-lane loops with no cross-lane traffic; k_t and q_t are loaded one element per lane,
// normalised with a wave reduction and broadcast with v_readlane.
//
// Replaces fused_recurrent_gated_delta_rule_fwd_kernel, models/hattention/gated_delta_rule_ori.py:372-464
// (same order of operations; state layout [N, HV, K, V] fp32; grouped value heads HV >= H).  It is also the
// fp32 mode of the chunk operator and the on-GPU cross-check of the chunk kernels.
#include "gdr_common.h"

// value of lane `src` (a compile-time constant) in every lane: one v_readlane into a scalar register
__device__ __forceinline__ float bcast(float x, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), src));
}

template <typename T, int KT>
__global__ void __launch_bounds__(64) gdr_recurrent_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                          const T* __restrict__ v, const float* __restrict__ g,
                                                          const float* __restrict__ beta, T* __restrict__ o,
                                                          const float* __restrict__ h0, float* __restrict__ ht,
                                                          const int64_t* __restrict__ cu_seqlens, int64_t t_len,
                                                          int H, int HV, int K, int V, float scale, int l2norm) {
  constexpr int KR = KT / 64 > 0 ? KT / 64 : 1;  // k/q elements held per lane
  const int lane = threadIdx.x;
  const int col = blockIdx.x * 64 + lane;
  const bool active = col < V;
  const int seq = blockIdx.y / HV, hv = blockIdx.y % HV;
  const int h = hv / (HV / H);
  const int64_t bos = cu_seqlens ? cu_seqlens[seq] : seq * t_len;
  const int64_t eos = cu_seqlens ? cu_seqlens[seq + 1] : bos + t_len;

  float S[KT];
#pragma unroll
  for (int i = 0; i < KT; ++i)
    S[i] = (h0 && active && i < K) ? h0[(((int64_t)seq * HV + hv) * K + i) * V + col] : 0.0f;

  // The inputs of the coming tokens are loaded PF tokens ahead into a ring of registers (a step depends on the
  // previous one through the state only, so without this every token pays a full memory latency). Loads past the end
  // of the sequence re-read its last token and are dropped.
  constexpr int PF = 8;
  struct Tok {
    float kv[KR], qv[KR], g, b, v;
  };
  Tok ring[PF];
  auto issue = [&](int64_t t, Tok& x) __attribute__((always_inline)) {
    t = t < eos ? t : eos - 1;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = r * 64 + lane;
      x.kv[r] = i < K ? GdrElem<T>::to_float(k[(t * H + h) * K + i]) : 0.0f;
      x.qv[r] = i < K ? GdrElem<T>::to_float(q[(t * H + h) * K + i]) : 0.0f;
    }
    x.g = g[t * HV + hv];
    x.b = beta[t * HV + hv];
    x.v = active ? GdrElem<T>::to_float(v[(t * HV + hv) * V + col]) : 0.0f;
  };
  auto step = [&](int64_t t, const Tok& x) __attribute__((always_inline)) {
    float kv[KR], qv[KR];
    float kss = 0.0f, qss = 0.0f;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      kv[r] = x.kv[r];
      qv[r] = x.qv[r];
      kss += kv[r] * kv[r];
      qss += qv[r] * qv[r];
    }
    float kinv = 1.0f, qinv = 1.0f;
    if (l2norm != GDR_L2_NONE) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        kss += __shfl_xor(kss, off);
        qss += __shfl_xor(qss, off);
      }
      if (l2norm == GDR_L2_CHUNK) {
        kinv = 1.0f / __fsqrt_rn(kss + 1e-6f);
        qinv = 1.0f / __fsqrt_rn(qss + 1e-6f);
      } else {
        kinv = 1.0f / (__fsqrt_rn(kss) + 1e-6f);
        qinv = 1.0f / (__fsqrt_rn(qss) + 1e-6f);
      }
    }
#pragma unroll
    for (int r = 0; r < KR; ++r) { kv[r] *= kinv; qv[r] *= qinv * scale; }
    const float decay = expf(x.g);
    const float b = x.b;
    const float vt = x.v;

    float dot4[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // four interleaved partial sums: a single chain of KT dependent FMAs
#pragma unroll                                  // would be the step's critical path
    for (int i = 0; i < KT; ++i) {
      const float ki = bcast(kv[i / 64], i % 64);
      S[i] *= decay;
      dot4[i & 3] = __builtin_fmaf(S[i], ki, dot4[i & 3]);
    }
    const float d = b * (vt - ((dot4[0] + dot4[1]) + (dot4[2] + dot4[3])));
    float out4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < KT; ++i) {
      const float ki = bcast(kv[i / 64], i % 64);
      const float qi = bcast(qv[i / 64], i % 64);
      S[i] = __builtin_fmaf(ki, d, S[i]);
      out4[i & 3] = __builtin_fmaf(S[i], qi, out4[i & 3]);
    }
    const float out = (out4[0] + out4[1]) + (out4[2] + out4[3]);
    if (active) o[(t * HV + hv) * V + col] = GdrElem<T>::from_float(out);
  };
  if (bos < eos) {
#pragma unroll
    for (int p = 0; p < PF; ++p) issue(bos + p, ring[p]);
    for (int64_t t0 = bos; t0 < eos; t0 += PF) {
#pragma unroll
      for (int p = 0; p < PF; ++p) {
        const Tok cur = ring[p];
        issue(t0 + p + PF, ring[p]);
        if (t0 + p < eos) step(t0 + p, cur);
      }
    }
  }
  if (ht && active) {
#pragma unroll
    for (int i = 0; i < KT; ++i)
      if (i < K) ht[(((int64_t)seq * HV + hv) * K + i) * V + col] = S[i];
  }
}

template <typename T>
static int gdr_recurrent_launch(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                void* o, const float* h0, float* ht, const int64_t* cu, int n_seq, int64_t t_len,
                                int H, int HV, int K, int V, float scale, int l2norm, hipStream_t s) {
  const dim3 grid((V + 63) / 64, n_seq * HV), block(64);
  LAMPA_PROF(s, "start");
#define GDR_REC_CASE(KT)                                                                                         \
  hipLaunchKernelGGL((gdr_recurrent_kernel<T, KT>), grid, block, 0, s, (const T*)q, (const T*)k, (const T*)v, g, \
                     beta, (T*)o, h0, ht, cu, t_len, H, HV, K, V, scale, l2norm)
  if (K <= 32) GDR_REC_CASE(32);
  else if (K <= 64) GDR_REC_CASE(64);
  else GDR_REC_CASE(128);
#undef GDR_REC_CASE
  LAMPA_PROF(s, "gdr_recurrent_kernel");
  return lampa_launch_status();
}

// q, k [total_tokens, H, K]; v, o [total_tokens, HV, V]; g, beta fp32 [total_tokens, HV]; h0, ht fp32
// [n_seq, HV, K, V] (nullable). Sequences are [cu_seqlens[i], cu_seqlens[i+1]) (device int64, n_seq + 1 entries) or,
// when cu_seqlens is NULL, n_seq blocks of t_len tokens. dtype: 0 bf16, 1 fp16, 2 fp32 (q, k, v and o).
// l2norm: 0 none, 1 x / sqrt(sum x^2 + 1e-6), 2 x / (sqrt(sum x^2) + 1e-6).
extern "C" int lampa_gdr_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                       void* o, const float* h0, float* ht, const int64_t* cu_seqlens, int n_seq,
                                       int64_t t_len, int H, int HV, int K, int V, int dtype, float scale, int l2norm,
                                       void* stream) {
  if (!q || !k || !v || !g || !beta || !o) return LAMPA_ERR_INVALID;
  if (n_seq < 0 || H < 1 || HV < H || HV % H != 0 || K < 1 || V < 1 || t_len < 0) return LAMPA_ERR_INVALID;
  if (K > 128) return LAMPA_ERR_UNSUPPORTED;
  if (l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (n_seq == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case GDR_BF16:
      return gdr_recurrent_launch<__bf16>(q, k, v, g, beta, o, h0, ht, cu_seqlens, n_seq, t_len, H, HV, K, V, scale,
                                          l2norm, s);
    case GDR_FP16:
      return gdr_recurrent_launch<_Float16>(q, k, v, g, beta, o, h0, ht, cu_seqlens, n_seq, t_len, H, HV, K, V,
                                            scale, l2norm, s);
    case GDR_FP32:
      return gdr_recurrent_launch<float>(q, k, v, g, beta, o, h0, ht, cu_seqlens, n_seq, t_len, H, HV, K, V, scale,
                                         l2norm, s);
    default:
      return LAMPA_ERR_INVALID;
  }
}

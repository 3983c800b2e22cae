// Token-serial gated-delta-rule forward with an fp32 state held in registers (gfx950). Two kernels:
//
// gdr_recurrent_kernel: one wave owns up to 64 value columns of one (sequence, value head): lane = value column, and
// every lane keeps the K state rows of its column in registers, so the three contractions of a step (S^T k, the
// rank-one update and S^T q) are per-lane loops with no cross-lane traffic; k_t and q_t are loaded one element per
// lane, normalised with a wave reduction and broadcast with v_readlane.
// gdr_recurrent_split_kernel (further down): 32 columns per wave, the state rows of a column split over the two halves
// of the wave -- fewer instructions per token and wave, for launches of few waves.
//
// Replaces fused_recurrent_gated_delta_rule_fwd_kernel, models/hattention/gated_delta_rule_ori.py:372-464
// (state layout [N, HV, K, V] fp32; grouped value heads HV >= H).  It is also the fp32 mode of the chunk operator and
// the on-GPU cross-check of the chunk kernels.
#include "gdr_common.h"

// value of lane `src` (a compile-time constant) in every lane: one v_readlane into a scalar register
__device__ __forceinline__ float bcast(float x, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), src));
}

// BETA_V: beta holds one value per value column, [tokens, HV, V] (IS_BETA_HEADWISE of the reference kernel,
// gated_delta_rule_ori.py:415-418,444-448), instead of one per (token, value head).
template <typename T, int KT, bool BETA_V = false>
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
    if constexpr (BETA_V) x.b = active ? beta[(t * HV + hv) * V + col] : 0.0f;
    else x.b = beta[t * HV + hv];
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

// ---- the same recurrence with the state rows of a column split over the two halves of the wave ----------------------
// One wave owns 32 value columns of one (sequence, value head): lane = (half, column), and a lane keeps KT / 2 state
// rows of its column, so a step is half as many instructions per wave as above and V <= 32 fills the wave; the two
// partial sums of S^T k and of S^T q meet through one cross-half exchange each. The wave is bound by instruction issue
// (one wave per SIMD: four cycles per instruction), so everything that is not the recurrence leaves the step: k and q
// of a group of tokens are loaded 4 elements at a time one group ahead, widened and parked in LDS (a lane reads its
// KT / 2 values of a token with 16-byte broadcast reads instead of one cross-lane read per element), and the per-token
// scalars (1 / |k|, scale / |q|, e^g, beta) are computed for the whole group at once, lane = token. The l2 norms are
// applied as factors on the sums, not on the vectors. K a multiple of 4, q and k 16-byte aligned.
// x of the lower half of the wave plus x of the upper half, in every lane (one cross-half swap, no LDS)
__device__ __forceinline__ float rec_half_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // r[0] = lower half's, r[1] = upper half's
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <bool B>
struct RecLazy {
  static constexpr bool value = B;
};

template <typename T>
__device__ __forceinline__ float4 rec_load4(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *reinterpret_cast<const float4*>(p);
  } else {
    typedef T vec4 __attribute__((ext_vector_type(4)));
    const vec4 x = *reinterpret_cast<const vec4*>(p);
    return make_float4(GdrElem<T>::to_float(x[0]), GdrElem<T>::to_float(x[1]), GdrElem<T>::to_float(x[2]),
                       GdrElem<T>::to_float(x[3]));
  }
}

// COMPOSITE: the affine map of the sequence instead of its outputs. The state of a gated delta sequence is affine in
// the state it starts from, S_end = M S_0 + N: the wave's columns are columns of [M | N] (V = K + the value width),
// started from [I | 0], the M columns see v = 0; nothing is written but ht (fp32 [n_seq, HV, K, V]). ht_map (nullable)
// gives the row of ht that a sequence's final state goes to (negative: not stored).
template <typename T, int KT, bool COMPOSITE, bool SHORT_GROUPS = false>
__global__ void __launch_bounds__(64)
    gdr_recurrent_split_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                               const float* __restrict__ g, const float* __restrict__ beta, T* __restrict__ o,
                               const float* __restrict__ h0, float* __restrict__ ht,
                               const int64_t* __restrict__ cu_seqlens, int64_t t_len, int H, int HV, int K, int V,
                               float scale, int l2norm, const int32_t* __restrict__ ht_map) {
  constexpr int RP = KT / 2;                          // state rows per lane
  // tokens per group: 24 KB of LDS per wave at K >= 64 (six waves per CU); SHORT_GROUPS halves that for launches of
  // more waves than that holds at once (built for KT = 64, where eight then fit and a launch of 2016 waves needs one
  // round instead of two: 1.11 -> 0.73 ms; with fewer waves the longer groups are faster, 207 against 230 us)
  constexpr int G = (SHORT_GROUPS ? 512 : 1024) / KT < 64 ? (SHORT_GROUPS ? 512 : 1024) / KT : 64;
  constexpr int ROW4 = (2 * KT + 4) / 4;              // 16-byte pieces per token in LDS: k | q, padded against conflicts
  constexpr int PPT = 2 * KT / 4;                     // 4-element pieces of k | q per token
  constexpr int PIECES = G * PPT / 64;                // pieces per lane and group
  constexpr int VALS = G * 32 / 64;                   // v elements per lane and group
  static_assert((G * PPT) % 64 == 0, "group shape");
  // two buffers of a group each; two more tokens' room behind each group, so that the reads ahead need no bound
  // (what they return for tokens after the group is never used)
  __shared__ float4 s_kq[2][(G + 2) * ROW4];
  __shared__ float4 s_sc[2][G + 2];
  __shared__ float s_v[2][(G + 2) * 32];
  __shared__ float s_fold[2];  // per group: the decay over the whole group if it runs in the lazy form, else 0
  const int lane = threadIdx.x, half = lane >> 5, cl = lane & 31;
  const int col = blockIdx.x * 32 + cl;
  const bool active = col < V;
  const int seq = blockIdx.y / HV, hv = blockIdx.y % HV;
  const int h = hv / (HV / H);
  const int64_t bos = cu_seqlens ? cu_seqlens[seq] : seq * t_len;
  const int64_t eos = cu_seqlens ? cu_seqlens[seq + 1] : bos + t_len;

  const int v_dim = COMPOSITE ? V - K : V;   // width of a row of v
  const int v_col = COMPOSITE ? col - K : col;  // this lane's column of v (negative: an M column, v = 0)
  float S[RP];  // rows half * RP + r
#pragma unroll
  for (int r = 0; r < RP; ++r) {
    const int i = half * RP + r;
    if constexpr (COMPOSITE) S[r] = (i == col && col < K) ? 1.0f : 0.0f;
    else S[r] = (h0 && active && i < K) ? h0[(((int64_t)seq * HV + hv) * K + i) * V + col] : 0.0f;
  }
  if (bos < eos) {
    float4 piece[PIECES];
    float vals[VALS];
    float g_tok = 0.0f, b_tok = 0.0f;
    // loads of the group that starts at token t0: every address is inside the tensors (tokens past the end re-read the
    // last one, elements past K or V the last element) and what is out of range is replaced when it is parked
    auto fetch = [&](int64_t t0) __attribute__((always_inline)) {
#pragma unroll
      for (int n = 0; n < PIECES; ++n) {
        const int pi = lane + 64 * n, j = pi / PPT, c = 4 * (pi % PPT);
        const int64_t t = t0 + j < eos ? t0 + j : eos - 1;
        const int e = c < KT ? c : c - KT;
        if (COMPOSITE && c >= KT) piece[n] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);  // (q is not used)
        else piece[n] = rec_load4<T>((c < KT ? k : q) + (t * H + h) * K + (e < K ? e : K - 4));
      }
#pragma unroll
      for (int n = 0; n < VALS; ++n) {
        const int vi = lane + 64 * n, j = vi / 32;
        const int cc = (int)blockIdx.x * 32 + vi % 32 - (COMPOSITE ? K : 0);
        const int64_t t = t0 + j < eos ? t0 + j : eos - 1;
        vals[n] = GdrElem<T>::to_float(v[(t * HV + hv) * v_dim + max(0, min(cc, v_dim - 1))]);
      }
      const int64_t t = t0 + lane < eos ? t0 + lane : eos - 1;
      g_tok = g[t * HV + hv];
      b_tok = beta[t * HV + hv];
    };
    // the fetched group into LDS buffer `buf`, then its per-token scalars (lane = token)
    auto commit = [&](int buf, bool live) __attribute__((always_inline)) {
#pragma unroll
      for (int n = 0; n < PIECES; ++n) {
        const int pi = lane + 64 * n, j = pi / PPT, c4 = pi % PPT;
        const int c = 4 * c4, e = c < KT ? c : c - KT;
        s_kq[buf][j * ROW4 + c4] = e < K ? piece[n] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
#pragma unroll
      for (int n = 0; n < VALS; ++n) {
        const int cc = (int)blockIdx.x * 32 + (lane + 64 * n) % 32 - (COMPOSITE ? K : 0);
        s_v[buf][lane + 64 * n] = (COMPOSITE && cc < 0) ? 0.0f : vals[n];
      }
      // The decay is not applied to the state token by token: within a group the registers hold S / c_j, c_j = the
      // decay from the group's start up to token j, and c_j goes into the token's scalars instead (a multiply per
      // state element and token less); the state is brought back to scale once per group. With more than e^60 of
      // decay (or growth) inside one group 1 / c_j would leave the fp32 range: such a group runs in the direct form.
      const float g_use = (lane < G && live) ? g_tok : 0.0f;
      const float cum = wave_inclusive_scan(g_use);
      const float span = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_inclusive_scan(fabsf(g_use))), 63));
      const bool lazy = span <= 60.0f;  // (false for a NaN as well)
      if (lane == G - 1) s_fold[buf] = lazy ? expf(cum) : 0.0f;
      if (lane < G) {
        float kss = 0.0f, qss = 0.0f;
#pragma unroll
        for (int c4 = 0; c4 < KT / 4; ++c4) {
          const float4 a = s_kq[buf][lane * ROW4 + c4], b = s_kq[buf][lane * ROW4 + KT / 4 + c4];
          kss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
          qss += b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
        }
        float kinv = 1.0f, qinv = 1.0f;
        if (l2norm == GDR_L2_CHUNK) {
          kinv = 1.0f / __fsqrt_rn(kss + 1e-6f);
          qinv = 1.0f / __fsqrt_rn(qss + 1e-6f);
        } else if (l2norm == GDR_L2_RECURRENT) {
          kinv = 1.0f / (__fsqrt_rn(kss) + 1e-6f);
          qinv = 1.0f / (__fsqrt_rn(qss) + 1e-6f);
        }
        // a token past the end is a step that changes nothing (d = 0, decay 1), so the steps need no branch
        // direct: 1 / |k|, scale / |q|, e^g, beta; lazy: c / |k|, c scale / |q|, 1 / (c |k|), beta
        float4 sc = live ? make_float4(kinv, qinv * scale, expf(g_tok), b_tok) : make_float4(0.0f, 0.0f, 1.0f, 0.0f);
        if (lazy) {
          const float c = expf(cum), rc = expf(-cum);
          sc = live ? make_float4(kinv * c, qinv * scale * c, kinv * rc, b_tok) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        s_sc[buf][lane] = sc;
      }
    };
    // a token's operands: its scalars, this lane's RP elements of k and of q, its v
    struct Operands {
      float4 sc, kk[RP / 4], qq[RP / 4];
      float v;
    };
    auto read_token = [&](int buf, int j, Operands& x) __attribute__((always_inline)) {
      x.sc = s_sc[buf][j];  // the token's four scalars (direct or lazy form, see commit)
      const float4* kr = &s_kq[buf][j * ROW4 + half * (RP / 4)];
#pragma unroll
      for (int r4 = 0; r4 < RP / 4; ++r4) {
        x.kk[r4] = kr[r4];
        x.qq[r4] = kr[KT / 4 + r4];
      }
      x.v = s_v[buf][j * 32 + cl];
    };
    fetch(bos);
    commit(0, bos + lane < eos);
    int buf = 0;
    for (int64_t t0 = bos; t0 < eos; t0 += G, buf ^= 1) {
      const bool more = t0 + G < eos;
      if (more) fetch(t0 + G);
      const int n_tok = eos - t0 < G ? (int)(eos - t0) : G;
      // two tokens per round on two operand sets: a token's operands are requested before the arithmetic of the token
      // before it starts, so their LDS latency hides behind it. The token after the last of an odd count is a step
      // that changes nothing.
      auto run_group = [&](auto lazy_tag) __attribute__((always_inline)) {
        constexpr bool LAZY = decltype(lazy_tag)::value;
        auto step = [&](const Operands& x, int64_t t) __attribute__((always_inline)) {
          float kk[RP], qq[RP];
#pragma unroll
          for (int r4 = 0; r4 < RP / 4; ++r4) {
            kk[4 * r4] = x.kk[r4].x; kk[4 * r4 + 1] = x.kk[r4].y; kk[4 * r4 + 2] = x.kk[r4].z; kk[4 * r4 + 3] = x.kk[r4].w;
            qq[4 * r4] = x.qq[r4].x; qq[4 * r4 + 1] = x.qq[r4].y; qq[4 * r4 + 2] = x.qq[r4].z; qq[4 * r4 + 3] = x.qq[r4].w;
          }
          float dot4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int r = 0; r < RP; ++r) dot4[r & 3] = __builtin_fmaf(S[r], kk[r], dot4[r & 3]);
          const float dot = rec_half_sum((dot4[0] + dot4[1]) + (dot4[2] + dot4[3]));
          // S <- e^g S, then d = beta (v - S^T k), S <- S + k d^T, o = S^T q, with k = k_raw / |k|; in the lazy form on
          // S / c_j, where the decay is part of the scalars
          const float4 sc = x.sc;
          const float d = LAZY ? sc.w * (x.v - sc.x * dot) : sc.w * (x.v - sc.z * sc.x * dot);
          const float dk = LAZY ? d * sc.z : d * sc.x;
          if constexpr (COMPOSITE) {
#pragma unroll
            for (int r = 0; r < RP; ++r) S[r] = __builtin_fmaf(kk[r], dk, LAZY ? S[r] : sc.z * S[r]);
          } else {
            float out4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int r = 0; r < RP; ++r) {
              S[r] = __builtin_fmaf(kk[r], dk, LAZY ? S[r] : sc.z * S[r]);
              out4[r & 3] = __builtin_fmaf(S[r], qq[r], out4[r & 3]);
            }
            const float out = rec_half_sum((out4[0] + out4[1]) + (out4[2] + out4[3]));
            if (active && half == 0 && t < eos) o[(t * HV + hv) * V + col] = GdrElem<T>::from_float(out * sc.y);
          }
        };
        Operands xa, xb;
        read_token(buf, 0, xa);
        for (int j = 0; j < n_tok; j += 2) {
          read_token(buf, j + 1, xb);
          __builtin_amdgcn_sched_barrier(0);
          step(xa, t0 + j);
          read_token(buf, j + 2, xa);
          __builtin_amdgcn_sched_barrier(0);
          step(xb, t0 + j + 1);
        }
      };
      const float fold = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(s_fold[buf])));
      if (fold != 0.0f) {
        run_group(RecLazy<true>{});
#pragma unroll
        for (int r = 0; r < RP; ++r) S[r] *= fold;  // back to scale: S = c_last (S / c_last)
      } else {
        run_group(RecLazy<false>{});
      }
      if (more) commit(buf ^ 1, t0 + G + lane < eos);
    }
  }
  const int out_row = ht_map ? ht_map[seq] : seq;
  if (ht && active && out_row >= 0) {
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      const int i = half * RP + r;
      if (i < K) ht[(((int64_t)out_row * HV + hv) * K + i) * V + col] = S[r];
    }
  }
}

// more waves than six per CU of the 256 (what the long groups' LDS holds at once)
static inline bool gdr_rec_short_groups(const dim3& grid) { return (int64_t)grid.x * grid.y > 6 * 256; }

template <typename T>
static int gdr_recurrent_launch(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                void* o, const float* h0, float* ht, const int64_t* cu, int n_seq, int64_t t_len,
                                int H, int HV, int K, int V, float scale, int l2norm, hipStream_t s,
                                const int32_t* ht_map = nullptr) {
  LAMPA_PROF(s, "start");
  // the split form while its waves (twice as many) still find a SIMD each or nearly so
  const int64_t split_waves = (int64_t)((V + 31) / 32) * n_seq * HV;
  if (K % 4 == 0 && ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 15) == 0 &&
      split_waves <= 2048) {
    const dim3 grid2((V + 31) / 32, n_seq * HV);
#define GDR_REC_SPLIT(KT)                                                                                          \
  hipLaunchKernelGGL((gdr_recurrent_split_kernel<T, KT, false>), grid2, dim3(64), 0, s, (const T*)q, (const T*)k,  \
                     (const T*)v, g, beta, (T*)o, h0, ht, cu, t_len, H, HV, K, V, scale, l2norm, ht_map)
    if (K <= 16) GDR_REC_SPLIT(16);
    else if (K <= 32) GDR_REC_SPLIT(32);
    else if (K <= 64) {
      if (gdr_rec_short_groups(grid2))
        hipLaunchKernelGGL((gdr_recurrent_split_kernel<T, 64, false, true>), grid2, dim3(64), 0, s, (const T*)q,
                           (const T*)k, (const T*)v, g, beta, (T*)o, h0, ht, cu, t_len, H, HV, K, V, scale, l2norm,
                           ht_map);
      else GDR_REC_SPLIT(64);
    } else GDR_REC_SPLIT(128);
#undef GDR_REC_SPLIT
    LAMPA_PROF(s, "gdr_recurrent_split_kernel");
    return lampa_launch_status();
  }
  const dim3 grid((V + 63) / 64, n_seq * HV), block(64);
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

// ---- long sequences in parallel ---------------------------------------------------------------------------------
// A token-serial kernel gives a (sequence, head) to one or two waves, so a few long sequences leave the chip idle. The
// state a run of tokens ends with is affine in the state it starts from, so the sequences are cut into segments:
//   A  every segment's map [M | N] from [I | 0]            (gdr_recurrent_split_kernel<COMPOSITE>, K + V columns)
//   S  S_{p+1} = M_p S_p + N_p over a sequence's segments  (gdr_segment_scan_kernel, serial, small)
//   B  every segment again from the state it really starts with, writing o (the plain kernel, segments as sequences)
// all in fp32: the same function as the token loop up to fp32 rounding.

// 32 columns of the state per workgroup; mn [n_seg, HV, K, K + V], sinit [n_seg, HV, K, V]. A step is short, so what
// counts is that nothing serial is left in it but the product itself:
//  - M_p is loaded with 16-byte accesses into registers DEPTH segments ahead (its 1 - 2 us of memory latency would
//    otherwise be paid once per segment) and parked in LDS; the register sets are fixed per step of an unrolled group
//    (moving a set would wait for its load), and every memory operation of a step is unconditional (under a condition
//    it becomes a branch, after which the compiler no longer counts the operations in flight and drains them);
//  - M_p S runs on the fp32 MFMA (v_mfma_f32_32x32x2f32: 4 bytes per lane and operand from LDS). As multiply-adds with
//    M read as broadcasts it was bound by LDS bandwidth (512 KB per step at K = 64: 4.8 us). The four waves split the
//    product into row tiles of 32 and, where there are fewer than four of those, into parts of the contraction whose
//    partial tiles are added afterwards;
//  - LDS-only barriers.
// LDS: M [max(KT, 32)][KT + 4] | S [KT][33] | partial tiles [KS][max(KT, 32)][33], floats.
typedef float rs_f32x16 __attribute__((ext_vector_type(16)));
template <int KT>
struct RsScanShape {
  static constexpr int RT = KT >= 32 ? KT / 32 : 1;  // row tiles of 32
  static constexpr int KS = 4 / RT;                  // parts of the contraction (one wave each)
  static constexpr int ROWS = RT * 32;
  static constexpr int MS = KT + 4;                  // row stride of M in LDS (floats)
  static constexpr size_t LDS_BYTES = ((size_t)ROWS * MS + (size_t)KT * 33 + (size_t)KS * ROWS * 33) * sizeof(float);
};

// What a workgroup's range of maps is (blockIdx.y) and what it writes:
//   RS_PLAIN    a sequence's segments; the state each segment starts from (the last map is not applied)
//   RS_COMPOSE  group `grp` (gs consecutive segments) of sequence `seq`, blockIdx.y = seq * maxg + grp, on the K + V
//               columns of [I | 0]: every map of the group is applied and only the result, the group's own map
//               [M | N], is stored (template COMPOSE; V counts all K + V columns there)
//   RS_GROUPS   a sequence's groups, the maps being the groups' maps: the state each group starts from
//   RS_WITHIN   a group's segments from the state the group starts with (h0 row = blockIdx.y)
// A long sequence is scanned as RS_COMPOSE -> RS_GROUPS -> RS_WITHIN: three launches of about sqrt(n) dependent steps
// each instead of one of n.
enum { RS_PLAIN = 0, RS_COMPOSE = 1, RS_GROUPS = 2, RS_WITHIN = 3 };

template <int KT, int DEPTH, bool COMPOSE = false>
__global__ void __launch_bounds__(256) gdr_segment_scan_kernel(const float* __restrict__ mn, const float* __restrict__ h0,
                                                              const int32_t* __restrict__ seq_seg0, int HV, int K, int V,
                                                              float* __restrict__ sinit, int mode, int gs, int maxg,
                                                              int W) {
  using SH = RsScanShape<KT>;
  constexpr int MS = SH::MS, RT = SH::RT, KS = SH::KS, ROWS = SH::ROWS;
  constexpr int K4 = KT / 4;                          // 16-byte pieces per row of M
  constexpr int RPB = 256 / K4 < ROWS ? 256 / K4 : ROWS;  // rows of M that the workgroup stores to LDS at once
  constexpr int MREGS = (ROWS + RPB - 1) / RPB;       // such batches = pieces per thread
  constexpr int NR = KT / 8;                          // rows of the new column per thread in the combine step
  constexpr int KL = KT / KS;                         // contraction length of a wave
  static_assert(KT % 8 == 0 && KL % 2 == 0, "shape");
  extern __shared__ float4 s_scan4[];
  float* s_M = reinterpret_cast<float*>(s_scan4);
  float* s_S = s_M + ROWS * MS;
  float* s_P = s_S + KT * 33;
  const int tid = threadIdx.x, c = tid & 31, rg = tid >> 5;
  const int wave = tid >> 6, ln = tid & 31, hh = (tid >> 5) & 1;
  const int rt = wave % RT, ks = wave / RT;
  const int hv = blockIdx.z;
  const int col = blockIdx.x * 32 + c;
  const int colc = col < V ? col : V - 1;  // (lanes past V shadow the last column: same loads, same stores)
  // the range of maps [p0, p1) and the row of h0
  int p0, p1, row0 = blockIdx.y;
  if (mode == RS_PLAIN) {
    p0 = seq_seg0[blockIdx.y];
    p1 = seq_seg0[blockIdx.y + 1];
  } else if (mode == RS_GROUPS) {
    const int n = seq_seg0[blockIdx.y + 1] - seq_seg0[blockIdx.y];
    p0 = blockIdx.y * maxg;
    p1 = p0 + (n + gs - 1) / gs;
  } else {  // a group of a sequence
    const int seq = blockIdx.y / maxg, grp = blockIdx.y - seq * maxg;
    const int s1 = seq_seg0[seq + 1];
    p0 = seq_seg0[seq] + grp * gs;
    p1 = min(p0 + gs, s1);
  }
  if (p0 >= p1) return;
  const int p_last = p1 - 1;      // the last map that exists in the range
  if (COMPOSE) p1 += 1;           // one more (virtual) segment, so that the loop below applies all of them
#pragma unroll
  for (int n = 0; n < NR; ++n) {
    const int i = rg + 8 * n;
    if (COMPOSE) s_S[i * 33 + c] = (i == col && col < K) ? 1.0f : 0.0f;
    else s_S[i * 33 + c] = (h0 && i < K) ? h0[(((int64_t)row0 * HV + hv) * K + i) * V + colc] : 0.0f;
  }
  // the column of the maps' N part that goes with this column of the state (COMPOSE: none for the first K columns)
  const int ncol = COMPOSE ? min(max(col - K, 0), W - K - 1) : colc;
  const bool has_n = !COMPOSE || col >= K;
  const int my_row = tid / K4, my_c4 = tid % K4;
  const bool loader = my_row < RPB;
  float4 mreg[DEPTH][MREGS];
  float nreg[DEPTH][NR];
  // M_p and this thread's entries of N_p into register set `slot`: unconditional loads from clamped addresses (a
  // segment index past the end, a row or column past K); what lies past K is replaced by zero when it is used
  auto fetch = [&](int p, int slot) __attribute__((always_inline)) {
    p = min(p, p_last);
    const float* M = mn + ((int64_t)p * HV + hv) * K * W;
#pragma unroll
    for (int u = 0; u < MREGS; ++u)
      mreg[slot][u] = *reinterpret_cast<const float4*>(M + (int64_t)min(u * RPB + my_row, K - 1) * W + min(4 * my_c4, K - 4));
#pragma unroll
    for (int n = 0; n < NR; ++n) nreg[slot][n] = M[(int64_t)min(rg + 8 * n, K - 1) * W + K + ncol];
  };
  // the state segment p starts from (every lane stores every time: rows past K repeat the last row's store)
  auto store_start = [&](int p) __attribute__((always_inline)) {
    if (COMPOSE) return;
    float* out = sinit + ((int64_t)p * HV + hv) * K * V;
#pragma unroll
    for (int n = 0; n < NR; ++n) {
      const int i = min(rg + 8 * n, K - 1);
      out[(int64_t)i * V + colc] = s_S[i * 33 + c];
    }
  };
  // one step: the state segment p starts from is stored, then S <- M_p S + N_p from register set `slot`, which is then
  // loaded again for segment p + DEPTH
  auto advance = [&](int p, int slot) __attribute__((always_inline)) {
    store_start(p);
#pragma unroll
    for (int u = 0; u < MREGS; ++u) {
      const int i = u * RPB + my_row;
      const bool inside = i < K && 4 * my_c4 < K;
      if (loader && i < ROWS)
        *reinterpret_cast<float4*>(s_M + i * MS + 4 * my_c4) = inside ? mreg[slot][u] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    float acc[NR];
#pragma unroll
    for (int n = 0; n < NR; ++n) acc[n] = (has_n && rg + 8 * n < K) ? nreg[slot][n] : 0.0f;
    lds_barrier();  // M_p is in LDS (an LDS-only barrier: the loads issued ahead stay in flight)
    fetch(p + DEPTH, slot);
    {
      // this wave's tile: rows 32 rt .., contraction indices ks KL .. ; step s takes the indices s (lanes 0-31) and
      // KL / 2 + s (lanes 32-63) of that range, so that a lane walks consecutive addresses
      const float* ap = s_M + (32 * rt + ln) * MS + ks * KL + hh * (KL / 2);
      const float* bp = s_S + (ks * KL + hh * (KL / 2)) * 33 + ln;
      rs_f32x16 t;
#pragma unroll
      for (int r = 0; r < 16; ++r) t[r] = 0.0f;
#pragma unroll
      for (int s0 = 0; s0 < KL / 2; s0 += 8) {  // operands of eight steps, then their MFMAs
        float av[8], bv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < KL / 2) {
            av[u] = ap[s0 + u];
            bv[u] = bp[(s0 + u) * 33];
          }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < KL / 2) t = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u], bv[u], t, 0, 0, 0);
      }
      float* pp = s_P + (ks * ROWS + 32 * rt + 4 * hh) * 33 + ln;  // accumulator register r: row 8 (r / 4) + 4 hh + r % 4
#pragma unroll
      for (int r = 0; r < 16; ++r) pp[(8 * (r / 4) + (r % 4)) * 33] = t[r];
    }
    lds_barrier();  // the partial tiles are in LDS; every wave has read the old S and M_p
#pragma unroll
    for (int n = 0; n < NR; ++n) {
      const int i = rg + 8 * n;
#pragma unroll
      for (int part = 0; part < KS; ++part) acc[n] += s_P[(part * ROWS + i) * 33 + c];
      s_S[i * 33 + c] = acc[n];
    }
    lds_barrier();
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) fetch(p0 + d, d);
  __syncthreads();
  int p = p0;
  for (; p + DEPTH < p1; p += DEPTH) {  // DEPTH steps on fixed register sets
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) advance(p + d, d);
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (p + d + 1 < p1) advance(p + d, d);
  store_start(p1 - 1);
  if (COMPOSE) {  // the group's map, in the layout of the segments' maps
    float* out = sinit + ((int64_t)blockIdx.y * HV + hv) * K * W;
#pragma unroll
    for (int n = 0; n < NR; ++n) {
      const int i = min(rg + 8 * n, K - 1);
      out[(int64_t)i * W + colc] = s_S[i * 33 + c];
    }
  }
}

template <typename T>
static int gdr_recurrent_segmented(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                   void* o, const float* h0, float* ht, const int64_t* cu_seg,
                                   const int32_t* seq_seg0, const int32_t* seg_out, int n_seq, int n_seg, int H, int HV,
                                   int K, int V, float scale, int l2norm, float* mn, float* sinit, float* groups,
                                   hipStream_t s) {
  LAMPA_PROF(s, "start");
  const dim3 grid_a((K + V + 31) / 32, n_seg * HV), grid_b((V + 31) / 32, n_seg * HV);
#define GDR_REC_SEG(KT) GDR_REC_SEG2(KT, false, false)
#define GDR_REC_SEG2(KT, SHORT_A, SHORT_B)                                                                           \
  do {                                                                                                               \
    hipLaunchKernelGGL((gdr_recurrent_split_kernel<T, KT, true, SHORT_A>), grid_a, dim3(64), 0, s, (const T*)k, (const T*)k,  \
                       (const T*)v, g, beta, (T*)nullptr, (const float*)nullptr, mn, cu_seg, (int64_t)0, H, HV, K,   \
                       K + V, scale, l2norm, (const int32_t*)nullptr);                                               \
    LAMPA_PROF(s, "gdr_recurrent_split_kernel<composite>");                                                          \
    if (gdr_segment_scan(mn, h0, seq_seg0, n_seq, n_seg, HV, K, V, sinit, groups, s) != LAMPA_OK)                    \
      return LAMPA_ERR_LAUNCH;                                                                                       \
    LAMPA_PROF(s, "start");                                                                                          \
    hipLaunchKernelGGL((gdr_recurrent_split_kernel<T, KT, false, SHORT_B>), grid_b, dim3(64), 0, s, (const T*)q, (const T*)k, \
                       (const T*)v, g, beta, (T*)o, sinit, ht, cu_seg, (int64_t)0, H, HV, K, V, scale, l2norm,       \
                       seg_out);                                                                                     \
    LAMPA_PROF(s, "gdr_recurrent_split_kernel");                                                                     \
  } while (0)
  const bool short_a = gdr_rec_short_groups(grid_a), short_b = gdr_rec_short_groups(grid_b);
  if (K <= 16) GDR_REC_SEG(16);
  else if (K <= 32) GDR_REC_SEG(32);
  else if (K <= 64) {
    if (short_a && short_b) GDR_REC_SEG2(64, true, true);
    else if (short_a) GDR_REC_SEG2(64, true, false);
    else if (short_b) GDR_REC_SEG2(64, false, true);
    else GDR_REC_SEG(64);
  } else GDR_REC_SEG(128);
#undef GDR_REC_SEG
#undef GDR_REC_SEG2
  return lampa_launch_status();
}

// The first two launches above on their own, for the backward pass (gdr_backward.hip), which needs the maps and the
// states the segments start from but not the outputs; the scan is also run a second time there, over the transposed
// maps in reverse segment order.
static int gdr_scan_attr() {
  static bool attr_set[64] = {};  // per device: the widest scans' dynamic LDS limit (a repeated set is harmless)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LAMPA_ERR_LAUNCH;
  if (!attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)gdr_segment_scan_kernel<128, 1, false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)RsScanShape<128>::LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute((const void*)gdr_segment_scan_kernel<128, 1, true>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)RsScanShape<128>::LDS_BYTES) != hipSuccess)
      return LAMPA_ERR_LAUNCH;
    attr_set[dev] = true;
  }
  return LAMPA_OK;
}

template <typename T>
static void gdr_segment_maps_typed(const void* k, const void* v, const float* g, const float* beta,
                                   const int64_t* cu_seg, int n_seg, int H, int HV, int K, int V, int l2norm, float* mn,
                                   hipStream_t s) {
  const dim3 grid_a((K + V + 31) / 32, n_seg * HV);
#define GDR_REC_MAPS(KT)                                                                                            \
  hipLaunchKernelGGL((gdr_recurrent_split_kernel<T, KT, true>), grid_a, dim3(64), 0, s, (const T*)k, (const T*)k,   \
                     (const T*)v, g, beta, (T*)nullptr, (const float*)nullptr, mn, cu_seg, (int64_t)0, H, HV, K,    \
                     K + V, 1.0f, l2norm, (const int32_t*)nullptr)
  if (K <= 16) GDR_REC_MAPS(16);
  else if (K <= 32) GDR_REC_MAPS(32);
  else if (K <= 64) {
    if (gdr_rec_short_groups(grid_a))
      hipLaunchKernelGGL((gdr_recurrent_split_kernel<T, 64, true, true>), grid_a, dim3(64), 0, s, (const T*)k,
                         (const T*)k, (const T*)v, g, beta, (T*)nullptr, (const float*)nullptr, mn, cu_seg, (int64_t)0,
                         H, HV, K, K + V, 1.0f, l2norm, (const int32_t*)nullptr);
    else GDR_REC_MAPS(64);
  } else GDR_REC_MAPS(128);
#undef GDR_REC_MAPS
}

int gdr_segment_maps(const void* k, const void* v, const float* g, const float* beta, const int64_t* cu_seg, int n_seg,
                     int H, int HV, int K, int V, int dtype, int l2norm, float* mn, hipStream_t s) {
  LAMPA_PROF(s, "start");
  switch (dtype) {
    case GDR_BF16: gdr_segment_maps_typed<__bf16>(k, v, g, beta, cu_seg, n_seg, H, HV, K, V, l2norm, mn, s); break;
    case GDR_FP16: gdr_segment_maps_typed<_Float16>(k, v, g, beta, cu_seg, n_seg, H, HV, K, V, l2norm, mn, s); break;
    case GDR_FP32: gdr_segment_maps_typed<float>(k, v, g, beta, cu_seg, n_seg, H, HV, K, V, l2norm, mn, s); break;
    default: return LAMPA_ERR_INVALID;
  }
  LAMPA_PROF(s, "gdr_recurrent_split_kernel<composite>");
  return lampa_launch_status();
}

// Group slots of the three-launch scan: at most GDR_SCAN_GROUP_SEQS sequences of together at most
// GDR_SCAN_GROUP_SEGS segments take it; groups of gs = ceil(sqrt(n_seg / n_seq)) segments, at most
// maxg = ceil(n_seg / gs) of them in a sequence however the segments are spread, so n_seq * maxg <=
// n_seq^1.5 sqrt(n_seg) + n_seq slots of a map [K, K + V] and a state [K, V] each.
#define GDR_SCAN_GROUP_SEQS 4
#define GDR_SCAN_GROUP_SEGS 4096
int64_t gdr_scan_group_floats(int n_seg, int HV, int K, int V) {
  if (n_seg > GDR_SCAN_GROUP_SEGS) return 0;
  int64_t root = 1;
  while (root * root < n_seg) ++root;
  return (8 * root + GDR_SCAN_GROUP_SEQS) * HV * K * (int64_t)(K + 2 * V);
}

int gdr_segment_scan(const float* mn, const float* h0, const int32_t* seq_seg0, int n_seq, int n_seg, int HV, int K,
                     int V, float* sinit, float* groups, hipStream_t s) {
  const int rc = gdr_scan_attr();
  if (rc != LAMPA_OK) return rc;
  const int W = K + V;
#define GDR_REC_SCAN(KT, COMPOSE, GRID, MAPS, H0, COLS, OUT, MODE, GS, MAXG)                                      \
  hipLaunchKernelGGL((gdr_segment_scan_kernel<KT, (KT <= 32 ? 4 : KT == 64 ? 2 : 1), COMPOSE>), GRID, dim3(256),   \
                     RsScanShape<KT>::LDS_BYTES, s, MAPS, H0, seq_seg0, HV, K, COLS, OUT, MODE, GS, MAXG, W)
#define GDR_REC_SCAN_ANY(...)                        \
  do {                                               \
    if (K <= 16) GDR_REC_SCAN(16, __VA_ARGS__);      \
    else if (K <= 32) GDR_REC_SCAN(32, __VA_ARGS__); \
    else if (K <= 64) GDR_REC_SCAN(64, __VA_ARGS__); \
    else GDR_REC_SCAN(128, __VA_ARGS__);             \
  } while (0)
  // a few long sequences: groups of about sqrt(segments per sequence) segments, three launches of that many steps
  if (groups && n_seq <= GDR_SCAN_GROUP_SEQS && n_seg <= GDR_SCAN_GROUP_SEGS && n_seg >= 24 * n_seq) {
    int gs = 1;
    while (gs * gs * n_seq < n_seg) ++gs;
    const int maxg = (n_seg + gs - 1) / gs;
    float* gmaps = groups;                                                  // [n_seq * maxg, HV, K, K + V]
    float* gstart = groups + (int64_t)n_seq * maxg * HV * K * W;            // [n_seq * maxg, HV, K, V]
    LAMPA_PROF(s, "start");
    const dim3 grid_a((W + 31) / 32, n_seq * maxg, HV), grid_b((V + 31) / 32, n_seq, HV),
        grid_c((V + 31) / 32, n_seq * maxg, HV);
    GDR_REC_SCAN_ANY(true, grid_a, mn, (const float*)nullptr, W, gmaps, RS_COMPOSE, gs, maxg);
    LAMPA_PROF(s, "gdr_segment_scan_kernel<compose>");
    GDR_REC_SCAN_ANY(false, grid_b, (const float*)gmaps, h0, V, gstart, RS_GROUPS, gs, maxg);
    LAMPA_PROF(s, "gdr_segment_scan_kernel<groups>");
    GDR_REC_SCAN_ANY(false, grid_c, mn, (const float*)gstart, V, sinit, RS_WITHIN, gs, maxg);
    LAMPA_PROF(s, "gdr_segment_scan_kernel<within>");
    return lampa_launch_status();
  }
  LAMPA_PROF(s, "start");
  const dim3 grid((V + 31) / 32, n_seq, HV);
  GDR_REC_SCAN_ANY(false, grid, mn, h0, V, sinit, RS_PLAIN, 0, 1);
#undef GDR_REC_SCAN_ANY
#undef GDR_REC_SCAN
  LAMPA_PROF(s, "gdr_segment_scan_kernel");
  return lampa_launch_status();
}

// Workspace of lampa_gdr_recurrent_segmented_fwd: the segments' maps [n_seg, HV, K, K + V] and the states they start
// from [n_seg, HV, K, V], fp32.
extern "C" int64_t lampa_gdr_recurrent_segmented_workspace_bytes(int n_seg, int HV, int K, int V) {
  if (n_seg < 0 || HV < 1 || K < 1 || V < 1) return LAMPA_ERR_INVALID;
  return lampa_align_up((int64_t)n_seg * HV * K * (K + V) * 4, 256) + lampa_align_up((int64_t)n_seg * HV * K * V * 4, 256) +
         lampa_align_up(gdr_scan_group_floats(n_seg, HV, K, V) * 4, 256);
}

// lampa_gdr_recurrent_fwd for a few long sequences: the caller cuts every sequence into segments (cu_seg: device int64,
// n_seg + 1 token offsets, every sequence boundary among them; seq_seg0: device int32, n_seq + 1, first segment of
// every sequence; seg_out: device int32, n_seg, the sequence whose last segment this is, else -1) and the segments run
// in parallel. Same arguments and results otherwise; K and V multiples of 4, q and k 16-byte aligned, K <= 128.
extern "C" int lampa_gdr_recurrent_segmented_fwd(const void* q, const void* k, const void* v, const float* g,
                                                 const float* beta, void* o, const float* h0, float* ht,
                                                 const int64_t* cu_seg, const int32_t* seq_seg0, const int32_t* seg_out,
                                                 int n_seq, int n_seg, int H, int HV, int K, int V, int dtype,
                                                 float scale, int l2norm, void* workspace, int64_t workspace_bytes,
                                                 void* stream) {
  if (!q || !k || !v || !g || !beta || !o || !cu_seg || !seq_seg0 || !seg_out) return LAMPA_ERR_INVALID;
  if (n_seq < 0 || n_seg < n_seq || H < 1 || HV < H || HV % H != 0 || K < 1 || V < 1) return LAMPA_ERR_INVALID;
  if (l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (K > 128 || K % 4 != 0 || V % 4 != 0 ||
      ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 15) != 0)
    return LAMPA_ERR_UNSUPPORTED;
  if (n_seq == 0 || n_seg == 0) return LAMPA_OK;
  if (!workspace || workspace_bytes < lampa_gdr_recurrent_segmented_workspace_bytes(n_seg, HV, K, V))
    return LAMPA_ERR_WORKSPACE;
  float* mn = (float*)workspace;
  float* sinit = (float*)((char*)workspace + lampa_align_up((int64_t)n_seg * HV * K * (K + V) * 4, 256));
  float* groups = (float*)((char*)sinit + lampa_align_up((int64_t)n_seg * HV * K * V * 4, 256));
  if (gdr_scan_group_floats(n_seg, HV, K, V) == 0) groups = nullptr;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case GDR_BF16:
      return gdr_recurrent_segmented<__bf16>(q, k, v, g, beta, o, h0, ht, cu_seg, seq_seg0, seg_out, n_seq, n_seg, H,
                                             HV, K, V, scale, l2norm, mn, sinit, groups, s);
    case GDR_FP16:
      return gdr_recurrent_segmented<_Float16>(q, k, v, g, beta, o, h0, ht, cu_seg, seq_seg0, seg_out, n_seq, n_seg, H,
                                               HV, K, V, scale, l2norm, mn, sinit, groups, s);
    case GDR_FP32:
      return gdr_recurrent_segmented<float>(q, k, v, g, beta, o, h0, ht, cu_seg, seq_seg0, seg_out, n_seq, n_seg, H, HV,
                                            K, V, scale, l2norm, mn, sinit, groups, s);
    default:
      return LAMPA_ERR_INVALID;
  }
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

// The same operator with one beta per value column: beta fp32 [total_tokens, HV, V] (the reference kernel's
// IS_BETA_HEADWISE, gated_delta_rule_ori.py:415-418,444-448). Always the lane-per-column kernel: a lane owns one
// value column, so its beta is one more load per token.
template <typename T>
static int gdr_recurrent_headwise_launch(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                         void* o, const float* h0, float* ht, const int64_t* cu, int n_seq,
                                         int64_t t_len, int H, int HV, int K, int V, float scale, int l2norm,
                                         hipStream_t s) {
  LAMPA_PROF(s, "start");
  const dim3 grid((V + 63) / 64, n_seq * HV), block(64);
#define GDR_REC_CASE(KT)                                                                                              \
  hipLaunchKernelGGL((gdr_recurrent_kernel<T, KT, true>), grid, block, 0, s, (const T*)q, (const T*)k, (const T*)v, g, \
                     beta, (T*)o, h0, ht, cu, t_len, H, HV, K, V, scale, l2norm)
  if (K <= 32) GDR_REC_CASE(32);
  else if (K <= 64) GDR_REC_CASE(64);
  else GDR_REC_CASE(128);
#undef GDR_REC_CASE
  LAMPA_PROF(s, "gdr_recurrent_kernel<headwise beta>");
  return lampa_launch_status();
}

extern "C" int lampa_gdr_recurrent_headwise_fwd(const void* q, const void* k, const void* v, const float* g,
                                                const float* beta, void* o, const float* h0, float* ht,
                                                const int64_t* cu_seqlens, int n_seq, int64_t t_len, int H, int HV,
                                                int K, int V, int dtype, float scale, int l2norm, void* stream) {
  if (!q || !k || !v || !g || !beta || !o) return LAMPA_ERR_INVALID;
  if (n_seq < 0 || H < 1 || HV < H || HV % H != 0 || K < 1 || V < 1 || t_len < 0) return LAMPA_ERR_INVALID;
  if (K > 128) return LAMPA_ERR_UNSUPPORTED;
  if (l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (n_seq == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case GDR_BF16:
      return gdr_recurrent_headwise_launch<__bf16>(q, k, v, g, beta, o, h0, ht, cu_seqlens, n_seq, t_len, H, HV, K, V,
                                                   scale, l2norm, s);
    case GDR_FP16:
      return gdr_recurrent_headwise_launch<_Float16>(q, k, v, g, beta, o, h0, ht, cu_seqlens, n_seq, t_len, H, HV, K,
                                                     V, scale, l2norm, s);
    case GDR_FP32:
      return gdr_recurrent_headwise_launch<float>(q, k, v, g, beta, o, h0, ht, cu_seqlens, n_seq, t_len, H, HV, K, V,
                                                  scale, l2norm, s);
    default:
      return LAMPA_ERR_INVALID;
  }
}

// Backward pass of the gated delta rule (gfx950), fp32 throughout: the gradients of
//   S_t = a_t S_{t-1} + k_t u_t^T,  u_t = b_t (v_t - (a_t S_{t-1})^T k_t),  o_t = scale S_t^T q_t,  a_t = exp(g_t)
// with respect to q, k, v, g, beta and the initial state, given d o and d (final state).
// Replaces chunk_gated_delta_rule_bwd, models/hattention/gated_delta_rule_ori.py:83-160 (and the l2norm_bwd calls of
// ChunkGatedDeltaRuleFunction.backward, gated_delta_rule_ori.py:205-233).
//
// With G_t = dL/dS_t (everything that reaches S_t) and Sd_t = a_t S_{t-1}:
//   G_t   = H_{t+1} + scale q_t do_t^T                  H_{T+1} = d (final state)
//   du_t  = G_t^T k_t        dv_t = b_t du_t            db_t = du_t . (v_t - w_t),  w_t = Sd_t^T k_t
//   dk_t  = G_t u_t - b_t Sd_t du_t                     dq_t = scale S_t do_t = scale (Sd_t do_t + k_t (u_t . do_t))
//   dg_t  = <G_t, Sd_t> - b_t du_t . w_t                H_t  = a_t (G_t - b_t k_t du_t^T)      d (initial state) = H_1
// H runs backwards in time and needs no state; the other gradients need Sd_t at the same time as G_t. Both recurrences
// are affine in the state they start from, so the sequences are cut into segments as in the segmented forward:
//   1  forward maps [M | N] of the segments and the states they start from      (gdr_recurrent.hip, two launches)
//   2  every segment's H from zero backwards: N'; the linear part is M^T        (gdr_bwd_segment_kernel<COMPOSITE>)
//   3  H_end over the segments of a sequence, last to first                     (the forward scan kernel on [M^T | N'])
//   4  every segment: forward once, leaving S at every 8th token in memory; then block by block from the end: the
//      block's 8 decayed states rebuilt (every second one into a spill area of the workgroup -- all eight are 32 KB at
//      K = 64, which as LDS would leave three waves per CU --, the others from those by one more step on the way
//      back), then its tokens backwards                                         (gdr_bwd_segment_kernel)
//   5  partial sums over the column slabs and grouped value heads, the chain rule of the q/k normalisation, output
//      types                                                                    (gdr_bwd_finish_kernel)
// A wave owns 16 value columns of one (segment, value head): lane = (row group, column), a lane keeps K / 4 rows of
// its column of S and of H in registers. Sums over the rows of a column cross the four row groups (two register
// swaps); sums over the columns (dk, dq) go through LDS; db and dg are reduced once per block. A token's step is a
// chain of dependent LDS round trips, so the kernel lives on waves per SIMD: at most GB_MAX_GRID workgroups of one wave
// walk through the (segment, head, slab) units.
#include "gdr_common.h"
#include <mutex>

#define GB_BT 8     // tokens per block: decayed states rebuilt at a time, distance of the states kept in memory
#define GB_COLS 16  // value columns per wave
#define GB_FIN_TOKENS 4  // tokens per wave of the finish kernel
// what the segment kernel writes once and reads once or never (the states every GB_BT tokens, the partial dq / dk)
// goes around the caches' replacement order, which leaves the L2 to the spill areas (segment kernel 2.45 -> 2.32 ms)
#define GB_STREAM_STORE(v, p) __builtin_nontemporal_store((v), (p))
#define GB_STREAM_LOAD(p) __builtin_nontemporal_load(p)
#define GB_MAX_GRID 4096  // workgroups of the segment kernel (each owns a spill area for a block's states)

template <typename T>
__device__ __forceinline__ float4 gb_load4(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *reinterpret_cast<const float4*>(p);
  } else {
    typedef T vec4 __attribute__((ext_vector_type(4)));
    const vec4 x = *reinterpret_cast<const vec4*>(p);
    return make_float4(GdrElem<T>::to_float(x[0]), GdrElem<T>::to_float(x[1]), GdrElem<T>::to_float(x[2]),
                       GdrElem<T>::to_float(x[3]));
  }
}

template <int KT>
struct GbShape {
  static constexpr int KR = KT / 4;                    // state rows per lane
  static constexpr int Q4 = KR / 4;                    // 16-byte pieces of those
  static constexpr int LPT = KT / 8;                   // lanes that load one token's k (8 elements each)
  static constexpr int PASSES = (GB_BT * LPT + 63) / 64;
  static constexpr int C_GROUP = KR * GB_COLS + 16;    // floats per row group in the column-sum buffer (+16: banks)
  // LDS (floats): k [GB_BT][KT] | q | v [GB_BT][16] | do | w | (a, b) [GB_BT][4] | column sums [2][4][C_GROUP] |
  // db / dg partials [GB_BT][2][64]
  static constexpr int OFF_K = 0;
  static constexpr int OFF_Q = OFF_K + GB_BT * KT;
  static constexpr int OFF_V = OFF_Q + GB_BT * KT;
  static constexpr int OFF_DO = OFF_V + GB_BT * GB_COLS;
  static constexpr int OFF_W = OFF_DO + GB_BT * GB_COLS;
  static constexpr int OFF_SC = OFF_W + GB_BT * GB_COLS;
  static constexpr int OFF_C = OFF_SC + GB_BT * 4;
  static constexpr int OFF_RED = OFF_C + 2 * 4 * C_GROUP;
  static constexpr int FLOATS = OFF_RED + GB_BT * 2 * 64;
  static constexpr size_t LDS_BYTES = (size_t)FLOATS * sizeof(float);
  static constexpr int CKPT = KT * GB_COLS;            // floats of one stored state slab
  static constexpr int HIST = GB_BT / 2 * CKPT;        // every second decayed state of a block (per workgroup, in memory)
};

template <typename T>
struct GbArgs {
  const T *q, *k, *v, *dout;
  const float *g, *beta;
  const float* sinit;       // [n_seg, HV, K, V]: the state each segment starts from
  const float* hend;        // rows [HV, K, V]: row seg_rev[seg] is the state gradient the segment ends with
  const int32_t* seg_rev;   // [n_seg]: the segment's row in hend (and in mn_rev)
  const int64_t* cu_seg;    // [n_seg + 1]
  const float* mn;          // forward maps [n_seg, HV, K, K + V]
  float* mn_rev;            // COMPOSITE: rows [HV, K, K + V] = [M^T | N']
  float* ckpt;              // states at every GB_BT-th token of every (segment, head, slab)
  float* hist;              // per workgroup: decayed states of the block it works on, [GB_BT / 2][Q4][64][4]
  int64_t units;            // n_seg * HV * slabs (segment, head, slab) units, dealt to the workgroups round robin
  T* dv;
  float *dq_part, *dk_part; // [slabs, total, HV, K]
  float *db_part, *dg_part; // [slabs, total, HV]
  int64_t total;
  int H, HV, K, V, slabs;
  float scale;
  int l2norm;
};

// x summed over the four row groups of a column (lanes 16 apart), in every lane: two register swaps, no LDS
// (permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second, so the two
// results are (x of row 0 | 0 | 2 | 2) and (1 | 1 | 3 | 3); permlane32_swap does the same with the halves of the wave)
__device__ __forceinline__ float gb_rows_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned w = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// A workgroup is one wave, and a wave's LDS instructions execute in the order they were issued: what one lane wrote is
// there for another lane's later read without a barrier or a wait. Only the compiler has to keep that order.
__device__ __forceinline__ void gb_wave_fence() { asm volatile("" ::: "memory"); }

template <typename T, int KT, bool COMPOSITE>
__device__ __forceinline__ void gb_unit(const GbArgs<T>& A, int64_t unit, float* lds) {
  using SH = GbShape<KT>;
  constexpr int KR = SH::KR, Q4 = SH::Q4, LPT = SH::LPT, PASSES = SH::PASSES, CG = SH::C_GROUP;
  float* s_k = lds + SH::OFF_K;
  float* s_q = lds + SH::OFF_Q;
  float* s_v = lds + SH::OFF_V;
  float* s_do = lds + SH::OFF_DO;
  float* s_w = lds + SH::OFF_W;
  float* s_sc = lds + SH::OFF_SC;
  float* s_c = lds + SH::OFF_C;
  float* s_red = lds + SH::OFF_RED;

  const int lane = threadIdx.x, rg = lane >> 4, j = lane & 15;
  // the block's decayed states: every lane reads back exactly the 16-byte pieces it wrote (a spill area of its own,
  // rewritten block after block, so it stays in the caches)
  float* hist = A.hist + (int64_t)blockIdx.x * SH::HIST + lane * 4;
  int64_t bid = unit;
  const int slab = (int)(bid % A.slabs);
  bid /= A.slabs;
  const int hv = (int)(bid % A.HV);
  const int seg = (int)(bid / A.HV);
  const int H = A.H, HV = A.HV, K = A.K, V = A.V;
  const int h = hv / (HV / H);
  const int col = slab * GB_COLS + j;
  const bool active = col < V;
  const int64_t t0 = A.cu_seg[seg], t1 = A.cu_seg[seg + 1];
  const int n_blk = (int)((t1 - t0 + GB_BT - 1) / GB_BT);
  const int64_t total = A.total;

  // ---- a block's inputs: loaded into registers one block ahead, then normalised and parked in LDS ------------------
  float4 kreg[PASSES][2], qreg[PASSES][2];
  float vreg[2], dreg[2], greg = 0.0f, breg = 0.0f;
  auto fetch = [&](int b) __attribute__((always_inline)) {  // every load from a clamped address, dropped at commit
    const int64_t tb = t0 + (int64_t)b * GB_BT;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int idx = lane + 64 * p, tok = idx / LPT, part = idx % LPT;
      const int64_t t = min(max(tb + tok, t0), t1 - 1);
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const int e = min(part * 8 + 4 * hf, K - 4);
        kreg[p][hf] = gb_load4<T>(A.k + (t * H + h) * K + e);
        qreg[p][hf] = gb_load4<T>(A.q + (t * H + h) * K + e);
      }
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int idx = lane + 64 * p, tok = idx >> 4, cc = min(slab * GB_COLS + (idx & 15), V - 1);
      const int64_t t = min(max(tb + tok, t0), t1 - 1);
      vreg[p] = GdrElem<T>::to_float(A.v[(t * HV + hv) * V + cc]);
      dreg[p] = GdrElem<T>::to_float(A.dout[(t * HV + hv) * V + cc]);
    }
    const int64_t t = min(max(tb + (lane & (GB_BT - 1)), t0), t1 - 1);
    greg = A.g[t * HV + hv];
    breg = A.beta[t * HV + hv];
  };
  auto commit = [&](int b) __attribute__((always_inline)) {
    const int64_t tb = t0 + (int64_t)b * GB_BT;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int idx = lane + 64 * p, tok = idx / LPT, part = idx % LPT;
      const bool live = tb + tok >= t0 && tb + tok < t1;
      float kv[8], qv[8];
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const bool in = part * 8 + 4 * hf < K;
        const float4 a = kreg[p][hf], c = qreg[p][hf];
        kv[4 * hf] = in ? a.x : 0.0f; kv[4 * hf + 1] = in ? a.y : 0.0f;
        kv[4 * hf + 2] = in ? a.z : 0.0f; kv[4 * hf + 3] = in ? a.w : 0.0f;
        qv[4 * hf] = in ? c.x : 0.0f; qv[4 * hf + 1] = in ? c.y : 0.0f;
        qv[4 * hf + 2] = in ? c.z : 0.0f; qv[4 * hf + 3] = in ? c.w : 0.0f;
      }
      float kinv = 1.0f, qinv = 1.0f;
      if (A.l2norm != GDR_L2_NONE) {
        float kss = 0.0f, qss = 0.0f;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          kss = __builtin_fmaf(kv[x], kv[x], kss);
          qss = __builtin_fmaf(qv[x], qv[x], qss);
        }
#pragma unroll
        for (int off = 1; off < LPT; off <<= 1) {
          kss += __shfl_xor(kss, off);
          qss += __shfl_xor(qss, off);
        }
        if (A.l2norm == GDR_L2_CHUNK) {
          kinv = 1.0f / __fsqrt_rn(kss + 1e-6f);
          qinv = 1.0f / __fsqrt_rn(qss + 1e-6f);
        } else {
          kinv = 1.0f / (__fsqrt_rn(kss) + 1e-6f);
          qinv = 1.0f / (__fsqrt_rn(qss) + 1e-6f);
        }
      }
      if (!live) kinv = qinv = 0.0f;  // a token outside the segment: k = q = 0, a = 1, b = 0 leaves both states alone
      if (tok < GB_BT) {
        float4* kd = reinterpret_cast<float4*>(s_k + tok * KT + part * 8);
        float4* qd = reinterpret_cast<float4*>(s_q + tok * KT + part * 8);
        kd[0] = make_float4(kv[0] * kinv, kv[1] * kinv, kv[2] * kinv, kv[3] * kinv);
        kd[1] = make_float4(kv[4] * kinv, kv[5] * kinv, kv[6] * kinv, kv[7] * kinv);
        qd[0] = make_float4(qv[0] * qinv, qv[1] * qinv, qv[2] * qinv, qv[3] * qinv);
        qd[1] = make_float4(qv[4] * qinv, qv[5] * qinv, qv[6] * qinv, qv[7] * qinv);
      }
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int idx = lane + 64 * p, tok = idx >> 4;
      const bool live = tb + tok >= t0 && tb + tok < t1 && slab * GB_COLS + (idx & 15) < V;
      s_v[idx] = live ? vreg[p] : 0.0f;
      s_do[idx] = live ? dreg[p] * A.scale : 0.0f;
    }
    if (lane < GB_BT) {
      const bool live = tb + lane >= t0 && tb + lane < t1;
      s_sc[lane * 4] = live ? expf(greg) : 1.0f;
      s_sc[lane * 4 + 1] = live ? breg : 0.0f;
    }
    gb_wave_fence();
  };
  auto read_rows = [&](const float* base, float (&x)[KR]) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < Q4; ++m) {
      const float4 a = *reinterpret_cast<const float4*>(base + rg * KR + 4 * m);
      x[4 * m] = a.x; x[4 * m + 1] = a.y; x[4 * m + 2] = a.z; x[4 * m + 3] = a.w;
    }
  };

  // one token forwards: S <- a S (kept for the way back when `keep`), then the delta update
  auto fwd_step = [&](int tok, float (&S)[KR], bool keep) __attribute__((always_inline)) {
    const float a = s_sc[tok * 4], bt = s_sc[tok * 4 + 1];
    float kr[KR];
    read_rows(s_k + tok * KT, kr);
    float wp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      S[r] *= a;
      wp[r & 3] = __builtin_fmaf(S[r], kr[r], wp[r & 3]);
    }
    if (keep && (tok & 1) == 0) {  // every second decayed state is kept; the way back rebuilds the one after it
#pragma unroll
      for (int m = 0; m < Q4; ++m)
        *reinterpret_cast<float4*>(hist + ((tok >> 1) * Q4 + m) * 256) =
            make_float4(S[4 * m], S[4 * m + 1], S[4 * m + 2], S[4 * m + 3]);
    }
    const float w = gb_rows_sum((wp[0] + wp[1]) + (wp[2] + wp[3]));
    if (keep && rg == 0) s_w[tok * GB_COLS + j] = w;
    const float u = bt * (s_v[tok * GB_COLS + j] - w);
#pragma unroll
    for (int r = 0; r < KR; ++r) S[r] = __builtin_fmaf(kr[r], u, S[r]);
    __builtin_amdgcn_sched_barrier(0);  // (the next token's operands are not hoisted above this one)
  };

  float Hs[KR];
  const float* hsrc = nullptr;
  if (!COMPOSITE && A.hend) hsrc = A.hend + ((int64_t)A.seg_rev[seg] * HV + hv) * K * V;
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int i = rg * KR + r;
    Hs[r] = (hsrc && active && i < K) ? hsrc[(int64_t)i * V + col] : 0.0f;
  }

  if constexpr (COMPOSITE) {
    // ---- H from zero, backwards over the segment ----------------------------------------------------------------
    if (n_blk > 0) fetch(n_blk - 1);
    for (int b = n_blk - 1; b >= 0; --b) {
      commit(b);
      fetch(b - 1);
#pragma unroll
      for (int tok = GB_BT - 1; tok >= 0; --tok) {
        const float a = s_sc[tok * 4], bt = s_sc[tok * 4 + 1], dj = s_do[tok * GB_COLS + j];
        float kr[KR], qr[KR];
        read_rows(s_k + tok * KT, kr);
        read_rows(s_q + tok * KT, qr);
        float dup[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int r = 0; r < KR; ++r) {
          Hs[r] = __builtin_fmaf(qr[r], dj, Hs[r]);
          dup[r & 3] = __builtin_fmaf(Hs[r], kr[r], dup[r & 3]);
        }
        const float bdu = bt * gb_rows_sum((dup[0] + dup[1]) + (dup[2] + dup[3]));
#pragma unroll
        for (int r = 0; r < KR; ++r) Hs[r] = a * __builtin_fmaf(-bdu, kr[r], Hs[r]);
        __builtin_amdgcn_sched_barrier(0);  // (the next token's operands are not hoisted above this one)
      }
      gb_wave_fence();
    }
    const int W = K + V;
    float* out = A.mn_rev + ((int64_t)A.seg_rev[seg] * HV + hv) * K * W;
#pragma unroll
    for (int r = 0; r < KR; ++r) {
      const int i = rg * KR + r;
      if (active && i < K) out[(int64_t)i * W + K + col] = Hs[r];
    }
    const float* M = A.mn + ((int64_t)seg * HV + hv) * K * W;
    for (int l = slab; l < K; l += A.slabs)  // this wave's share of the transpose of M
      for (int i = lane; i < K; i += 64) out[(int64_t)i * W + l] = M[(int64_t)l * W + i];
  } else {
    // ---- the segment forwards: the state at every block start goes to memory ----------------------------------------
    float S[KR];
    {
      const float* src = A.sinit + ((int64_t)seg * HV + hv) * K * V;
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        const int i = rg * KR + r;
        S[r] = (active && i < K) ? src[(int64_t)i * V + col] : 0.0f;
      }
    }
    float* ck = A.ckpt + (((t0 / GB_BT + seg) * HV + hv) * A.slabs + slab) * (int64_t)SH::CKPT + lane;
    const int64_t ck_stride = (int64_t)HV * A.slabs * SH::CKPT;  // from one block to the next
    if (n_blk > 0) fetch(0);
    for (int b = 0; b < n_blk; ++b) {
      commit(b);
      fetch(b + 1);
#pragma unroll
      for (int r = 0; r < KR; ++r) GB_STREAM_STORE(S[r], &ck[b * ck_stride + r * 64]);
#pragma unroll
      for (int tok = 0; tok < GB_BT; ++tok) fwd_step(tok, S, false);
      gb_wave_fence();
    }
    // ---- block by block from the end ---------------------------------------------------------------------------------
    float Sn[KR];
    if (n_blk > 0) {
      fetch(n_blk - 1);
#pragma unroll
      for (int r = 0; r < KR; ++r) Sn[r] = GB_STREAM_LOAD(&ck[(n_blk - 1) * ck_stride + r * 64]);
    }
    for (int b = n_blk - 1; b >= 0; --b) {
      const int64_t tb = t0 + (int64_t)b * GB_BT;
      commit(b);
      fetch(b - 1);
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        S[r] = Sn[r];
        Sn[r] = GB_STREAM_LOAD(&ck[max(b - 1, 0) * ck_stride + r * 64]);
      }
#pragma unroll
      for (int tok = 0; tok < GB_BT; ++tok) fwd_step(tok, S, true);
      gb_wave_fence();
      float4 sdn[Q4];
#pragma unroll
      for (int m = 0; m < Q4; ++m)
        sdn[m] = *reinterpret_cast<const float4*>(hist + (((GB_BT - 2) >> 1) * Q4 + m) * 256);
#pragma unroll
      for (int tok = GB_BT - 1; tok >= 0; --tok) {
        const int64_t t = tb + tok;
        const bool live = t < t1;
        const float a = s_sc[tok * 4], bt = s_sc[tok * 4 + 1];
        const float vj = s_v[tok * GB_COLS + j], dj = s_do[tok * GB_COLS + j], wj = s_w[tok * GB_COLS + j];
        float kr[KR], qr[KR], Sd[KR];
        read_rows(s_k + tok * KT, kr);
        read_rows(s_q + tok * KT, qr);
        if (tok & 1) {
          // an odd token's decayed state from the kept one of the token before: one forward step, the same operations
          // in the same order as on the way forth
          float kp[KR];
          read_rows(s_k + (tok - 1) * KT, kp);
          const float up = s_sc[(tok - 1) * 4 + 1] * (s_v[(tok - 1) * GB_COLS + j] - s_w[(tok - 1) * GB_COLS + j]);
#pragma unroll
          for (int m = 0; m < Q4; ++m) {
            const float4 x = sdn[m];
            Sd[4 * m] = a * __builtin_fmaf(kp[4 * m], up, x.x);
            Sd[4 * m + 1] = a * __builtin_fmaf(kp[4 * m + 1], up, x.y);
            Sd[4 * m + 2] = a * __builtin_fmaf(kp[4 * m + 2], up, x.z);
            Sd[4 * m + 3] = a * __builtin_fmaf(kp[4 * m + 3], up, x.w);
          }
        } else {
#pragma unroll
          for (int m = 0; m < Q4; ++m) {  // a kept state; the one two tokens back is asked for now
            const float4 x = sdn[m];
            Sd[4 * m] = x.x; Sd[4 * m + 1] = x.y; Sd[4 * m + 2] = x.z; Sd[4 * m + 3] = x.w;
            if (tok >= 2) sdn[m] = *reinterpret_cast<const float4*>(hist + (((tok - 2) >> 1) * Q4 + m) * 256);
          }
        }
        float dup[4] = {0.0f, 0.0f, 0.0f, 0.0f}, pgp[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int r = 0; r < KR; ++r) {
          Hs[r] = __builtin_fmaf(qr[r], dj, Hs[r]);  // G
          dup[r & 3] = __builtin_fmaf(Hs[r], kr[r], dup[r & 3]);
          pgp[r & 3] = __builtin_fmaf(Hs[r], Sd[r], pgp[r & 3]);
        }
        const float du = gb_rows_sum((dup[0] + dup[1]) + (dup[2] + dup[3]));
        const float e = vj - wj, u = bt * e, bdu = bt * du, udj = u * dj;
        if (rg == 0 && active && live) A.dv[(t * HV + hv) * V + col] = GdrElem<T>::from_float(bdu);
        s_red[(tok * 2) * 64 + lane] = rg == 0 ? du * e : 0.0f;
        s_red[(tok * 2 + 1) * 64 + lane] = ((pgp[0] + pgp[1]) + (pgp[2] + pgp[3])) - (rg == 0 ? bdu * wj : 0.0f);
#pragma unroll
        for (int r = 0; r < KR; ++r) {
          s_c[rg * CG + r * GB_COLS + j] = __builtin_fmaf(Sd[r], dj, kr[r] * udj);              // dq (scaled)
          s_c[(4 + rg) * CG + r * GB_COLS + j] = __builtin_fmaf(Hs[r], u, -bdu * Sd[r]);        // dk
          Hs[r] = a * __builtin_fmaf(-bdu, kr[r], Hs[r]);
        }
        gb_wave_fence();
#pragma unroll
        for (int o = lane; o < 2 * KT; o += 64) {  // the sums over this wave's 16 columns, one (gradient, row) per lane
          const int which = o / KT, i = o % KT;
          const float4* p = reinterpret_cast<const float4*>(s_c + (which * 4 + i / KR) * CG + (i % KR) * GB_COLS);
          const float4 x0 = p[0], x1 = p[1], x2 = p[2], x3 = p[3];
          const float sum = (((x0.x + x0.y) + (x0.z + x0.w)) + ((x1.x + x1.y) + (x1.z + x1.w))) +
                            (((x2.x + x2.y) + (x2.z + x2.w)) + ((x3.x + x3.y) + (x3.z + x3.w)));
          if (i < K && live)
            GB_STREAM_STORE(sum, &(which ? A.dk_part : A.dq_part)[(((int64_t)slab * total + t) * HV + hv) * K + i]);
        }
        gb_wave_fence();
      }
      {  // db and dg of the block's tokens: 8 lanes per token
        const int tok = lane >> 3, sub = lane & 7;
        const float4* pb = reinterpret_cast<const float4*>(s_red + (tok * 2) * 64 + sub * 8);
        const float4* pg = reinterpret_cast<const float4*>(s_red + (tok * 2 + 1) * 64 + sub * 8);
        float sb = ((pb[0].x + pb[0].y) + (pb[0].z + pb[0].w)) + ((pb[1].x + pb[1].y) + (pb[1].z + pb[1].w));
        float sg = ((pg[0].x + pg[0].y) + (pg[0].z + pg[0].w)) + ((pg[1].x + pg[1].y) + (pg[1].z + pg[1].w));
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) {
          sb += __shfl_xor(sb, off);
          sg += __shfl_xor(sg, off);
        }
        if (sub == 0 && tb + tok < t1) {
          A.db_part[((int64_t)slab * total + tb + tok) * HV + hv] = sb;
          A.dg_part[((int64_t)slab * total + tb + tok) * HV + hv] = sg;
        }
      }
      gb_wave_fence();
    }
  }
}

template <typename T, int KT, bool COMPOSITE>
__global__ void __launch_bounds__(64, (KT <= 64 ? 2 : 1)) gdr_bwd_segment_kernel(const GbArgs<T> A) {
  extern __shared__ float4 s_gb4[];
  for (int64_t unit = blockIdx.x; unit < A.units; unit += gridDim.x) {
    gb_unit<T, KT, COMPOSITE>(A, unit, reinterpret_cast<float*>(s_gb4));
    gb_wave_fence();
  }
}

// One wave per (token, q/k head): dq and dk summed over the column slabs and the value heads of the group, taken
// through the normalisation of q and k (y = x inv: dx = inv (dy - y (y . dy)) for inv = 1 / sqrt(|x|^2 + eps), and
// dx = inv dy - y (y . dy) / |x| for inv = 1 / (|x| + eps)), written in the input type; lanes below the group size
// also sum db and dg of their value head.
template <typename T>
__global__ void __launch_bounds__(256) gdr_bwd_finish_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                            const float* __restrict__ dq_part,
                                                            const float* __restrict__ dk_part,
                                                            const float* __restrict__ db_part,
                                                            const float* __restrict__ dg_part, T* __restrict__ dq,
                                                            T* __restrict__ dk, float* __restrict__ dbeta,
                                                            float* __restrict__ dg, int64_t total, int H, int HV, int K,
                                                            int slabs, int l2norm) {
  const int64_t wave = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  const int lane = threadIdx.x & 63;
  const int h = (int)(wave % H), G = HV / H;
  // GB_FIN_TOKENS consecutive tokens per wave (a wave per token is over before its loads are back)
  for (int64_t t = wave / H * GB_FIN_TOKENS; t < min(total, (wave / H + 1) * GB_FIN_TOKENS); ++t) {
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    const T* x_in = which ? k : q;
    const float* part = which ? dk_part : dq_part;
    T* out = which ? dk : dq;
    float x[2], dy[2];
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int i = lane + 64 * n;
      x[n] = 0.0f;
      dy[n] = 0.0f;
      if (i < K) {
        x[n] = GdrElem<T>::to_float(x_in[(t * H + h) * K + i]);
        // the partial sums of this entry: (slab, value head of the group), four loads in flight at a time
        const int n_part = slabs * G;
        for (int c0 = 0; c0 < n_part; c0 += 4) {
          float p4[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int c = min(c0 + u, n_part - 1), sl = c / G, gq = c - sl * G;
            p4[u] = part[(((int64_t)sl * total + t) * HV + h * G + gq) * K + i];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) dy[n] += c0 + u < n_part ? p4[u] : 0.0f;
        }
      }
    }
    if (l2norm != GDR_L2_NONE) {
      float ss = x[0] * x[0] + x[1] * x[1];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
      const float nrm = __fsqrt_rn(ss);
      const float inv = l2norm == GDR_L2_CHUNK ? 1.0f / __fsqrt_rn(ss + 1e-6f) : 1.0f / (nrm + 1e-6f);
      float dot = x[0] * inv * dy[0] + x[1] * inv * dy[1];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
#pragma unroll
      for (int n = 0; n < 2; ++n) {
        const float y = x[n] * inv;
        if (l2norm == GDR_L2_CHUNK) dy[n] = inv * (dy[n] - y * dot);
        else dy[n] = inv * dy[n] - (nrm > 0.0f ? y * dot / nrm : 0.0f);
      }
    }
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int i = lane + 64 * n;
      if (i < K) out[(t * H + h) * K + i] = GdrElem<T>::from_float(dy[n]);
    }
  }
  if (lane < G) {
    const int hv = h * G + lane;
    float sb = 0.0f, sg = 0.0f;
    for (int s = 0; s < slabs; ++s) {
      sb += db_part[((int64_t)s * total + t) * HV + hv];
      sg += dg_part[((int64_t)s * total + t) * HV + hv];
    }
    dbeta[t * HV + hv] = sb;
    dg[t * HV + hv] = sg;
  }
  }
}

// d (initial state) of every sequence: the row the reversed scan ends with
__global__ void __launch_bounds__(256) gdr_bwd_dh0_kernel(const float* __restrict__ hends,
                                                         const int32_t* __restrict__ seq_seg0_rev, int64_t row,
                                                         float* __restrict__ dh0) {
  const int seq = blockIdx.y;
  const float* src = hends + (int64_t)(seq_seg0_rev[seq + 1] - 1) * row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < row; i += (int64_t)gridDim.x * 256)
    dh0[(int64_t)seq * row + i] = src[i];
}

static int gb_padded_k(int K) { return K <= 16 ? 16 : K <= 32 ? 32 : K <= 64 ? 64 : 128; }

struct GbWorkspace {
  int64_t mn, sinit, mn_rev, hends, groups, ckpt, hist, dq_part, dk_part, db_part, dg_part, bytes;
};
static GbWorkspace gb_workspace(int64_t total, int n_seq, int n_seg, int HV, int K, int V) {
  const int slabs = (V + GB_COLS - 1) / GB_COLS;
  GbWorkspace w;
  int64_t at = 0;
  auto take = [&](int64_t floats) {
    const int64_t here = at;
    at += lampa_align_up(floats * 4, 256);
    return here;
  };
  w.mn = take((int64_t)n_seg * HV * K * (K + V));
  w.sinit = take((int64_t)n_seg * HV * K * V);
  w.mn_rev = take((int64_t)(n_seg + n_seq) * HV * K * (K + V));
  w.hends = take((int64_t)(n_seg + n_seq) * HV * K * V);
  w.groups = take(gdr_scan_group_floats(n_seg + n_seq, HV, K, V));
  w.ckpt = take((total / GB_BT + n_seg + 1) * HV * slabs * (int64_t)gb_padded_k(K) * GB_COLS);
  w.hist = take((int64_t)GB_MAX_GRID * (GB_BT / 2) * gb_padded_k(K) * GB_COLS);
  w.dq_part = take((int64_t)slabs * total * HV * K);
  w.dk_part = take((int64_t)slabs * total * HV * K);
  w.db_part = take((int64_t)slabs * total * HV);
  w.dg_part = take((int64_t)slabs * total * HV);
  w.bytes = at;
  return w;
}

// d(initial state) of sequences without tokens: a copy of d(final state), or zero
__global__ void gdr_bwd_dh0_empty_kernel(const float* __restrict__ dht, float* __restrict__ dh0, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dh0[i] = dht ? dht[i] : 0.0f;
}

extern "C" int64_t lampa_gdr_bwd_workspace_bytes(int64_t total_tokens, int n_seq, int n_seg, int HV, int K, int V) {
  if (total_tokens < 0 || n_seq < 0 || n_seg < 0 || HV < 1 || K < 1 || V < 1 || K > 128) return LAMPA_ERR_INVALID;
  return gb_workspace(total_tokens, n_seq, n_seg, HV, K, V).bytes;
}

template <typename T>
static int gb_run(const void* q, const void* k, const void* v, const float* g, const float* beta, const float* h0,
                  const void* dout, const float* dht, void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
                  const int64_t* cu_seg, const int32_t* seq_seg0, const int32_t* seq_seg0_rev, const int32_t* seg_rev,
                  int64_t total, int n_seq, int n_seg, int H, int HV, int K, int V, int dtype, float scale, int l2norm,
                  char* ws, const GbWorkspace& w, hipStream_t s) {
  static bool attr_set[64] = {};  // per device: the widest kernels' dynamic LDS limit
  static std::mutex attr_lock;    // (several host threads may call at once)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LAMPA_ERR_LAUNCH;
  std::unique_lock<std::mutex> hold(attr_lock);
  if (!attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)gdr_bwd_segment_kernel<T, 128, false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)GbShape<128>::LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute((const void*)gdr_bwd_segment_kernel<T, 128, true>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)GbShape<128>::LDS_BYTES) != hipSuccess)
      return LAMPA_ERR_LAUNCH;
    attr_set[dev] = true;
  }
  hold.unlock();
  float* mn = (float*)(ws + w.mn);
  float* sinit = (float*)(ws + w.sinit);
  float* mn_rev = (float*)(ws + w.mn_rev);
  float* hends = (float*)(ws + w.hends);
  int rc = gdr_segment_maps(k, v, g, beta, cu_seg, n_seg, H, HV, K, V, dtype, l2norm, mn, s);
  if (rc != LAMPA_OK) return rc;
  float* groups = gdr_scan_group_floats(n_seg + n_seq, HV, K, V) ? (float*)(ws + w.groups) : nullptr;
  rc = gdr_segment_scan(mn, h0, seq_seg0, n_seq, n_seg, HV, K, V, sinit, groups, s);
  if (rc != LAMPA_OK) return rc;

  GbArgs<T> a;
  a.q = (const T*)q; a.k = (const T*)k; a.v = (const T*)v; a.dout = (const T*)dout;
  a.g = g; a.beta = beta;
  a.sinit = sinit; a.hend = hends; a.seg_rev = seg_rev; a.cu_seg = cu_seg;
  a.mn = mn; a.mn_rev = mn_rev; a.ckpt = (float*)(ws + w.ckpt); a.hist = (float*)(ws + w.hist);
  a.dv = (T*)dv;
  a.dq_part = (float*)(ws + w.dq_part); a.dk_part = (float*)(ws + w.dk_part);
  a.db_part = (float*)(ws + w.db_part); a.dg_part = (float*)(ws + w.dg_part);
  a.total = total;
  a.H = H; a.HV = HV; a.K = K; a.V = V; a.slabs = (V + GB_COLS - 1) / GB_COLS;
  a.scale = scale; a.l2norm = l2norm;
  a.units = (int64_t)n_seg * HV * a.slabs;
  const dim3 grid((unsigned)(a.units < GB_MAX_GRID ? a.units : GB_MAX_GRID));
#define GB_SEG(KT, COMP) \
  hipLaunchKernelGGL((gdr_bwd_segment_kernel<T, KT, COMP>), grid, dim3(64), GbShape<KT>::LDS_BYTES, s, a)
#define GB_SEG_ANY(COMP)                \
  do {                                  \
    if (K <= 16) GB_SEG(16, COMP);      \
    else if (K <= 32) GB_SEG(32, COMP); \
    else if (K <= 64) GB_SEG(64, COMP); \
    else GB_SEG(128, COMP);             \
  } while (0)
  LAMPA_PROF(s, "start");
  GB_SEG_ANY(true);
  LAMPA_PROF(s, "gdr_bwd_segment_kernel<composite>");
  rc = lampa_launch_status();
  if (rc != LAMPA_OK) return rc;
  rc = gdr_segment_scan(mn_rev, dht, seq_seg0_rev, n_seq, n_seg + n_seq, HV, K, V, hends, groups, s);
  if (rc != LAMPA_OK) return rc;
  LAMPA_PROF(s, "start");
  GB_SEG_ANY(false);
  LAMPA_PROF(s, "gdr_bwd_segment_kernel");
#undef GB_SEG_ANY
#undef GB_SEG
  const int64_t waves = (total + GB_FIN_TOKENS - 1) / GB_FIN_TOKENS * H;
  hipLaunchKernelGGL((gdr_bwd_finish_kernel<T>), dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, (const T*)q,
                     (const T*)k, a.dq_part, a.dk_part, a.db_part, a.dg_part, (T*)dq, (T*)dk, dbeta, dg, total, H, HV, K,
                     a.slabs, l2norm);
  LAMPA_PROF(s, "gdr_bwd_finish_kernel");
  if (dh0) {
    const int64_t row = (int64_t)HV * K * V;
    hipLaunchKernelGGL(gdr_bwd_dh0_kernel, dim3((unsigned)((row + 255) / 256 < 64 ? (row + 255) / 256 : 64), n_seq), dim3(256), 0, s,
                       hends, seq_seg0_rev, row, dh0);
    LAMPA_PROF(s, "gdr_bwd_dh0_kernel");
  }
  return lampa_launch_status();
}

// Gradients of the gated-delta forward (lampa_gdr_chunk_fwd / lampa_gdr_recurrent_fwd compute the same function).
// q, k [total, H, K]; v, dout, dv [total, HV, V]; g, beta, dg, dbeta fp32 [total, HV]; dq, dk like q; h0, dht, dh0 fp32
// [n_seq, HV, K, V] (each nullable: zero initial state, no gradient into the final state, d h0 not wanted).
// The caller cuts every sequence into segments, as for lampa_gdr_recurrent_segmented_fwd: cu_seg (device int64,
// n_seg + 1 token offsets, every sequence boundary among them), seq_seg0 (device int32, n_seq + 1: first segment of
// every sequence) and, for the pass that runs backwards, seq_seg0_rev (device int32, n_seq + 1: seq_seg0[s] + s, one
// extra row per sequence) and seg_rev (device int32, n_seg: seq_seg0_rev[s] + (last segment of s) - p for segment p of
// sequence s). K <= 128, K and V multiples of 4; q, k 16-byte aligned; at most 64 value heads per q/k head.
extern "C" int lampa_gdr_bwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                             const float* h0, const void* dout, const float* dht, void* dq, void* dk, void* dv,
                             float* dg, float* dbeta, float* dh0, const int64_t* cu_seg, const int32_t* seq_seg0,
                             const int32_t* seq_seg0_rev, const int32_t* seg_rev, int64_t total_tokens, int n_seq,
                             int n_seg, int H, int HV, int K, int V, int dtype, float scale, int l2norm, void* workspace,
                             int64_t workspace_bytes, void* stream) {
  if (!q || !k || !v || !g || !beta || !dout || !dq || !dk || !dv || !dg || !dbeta) return LAMPA_ERR_INVALID;
  if (!cu_seg || !seq_seg0 || !seq_seg0_rev || !seg_rev) return LAMPA_ERR_INVALID;
  if (total_tokens < 0 || n_seq < 0 || n_seg < n_seq || H < 1 || HV < H || HV % H != 0 || K < 1 || V < 1)
    return LAMPA_ERR_INVALID;
  if (l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (K > 128 || K % 4 != 0 || V % 4 != 0 || HV / H > 64 || n_seq > 65535 ||
      ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 15) != 0)
    return LAMPA_ERR_UNSUPPORTED;
  if (n_seq == 0) return LAMPA_OK;
  if (n_seg == 0 || total_tokens == 0) {
    // no tokens: the final state is the initial state, so d(initial state) = d(final state) (zero when none is given)
    if (dh0) {
      const int64_t n = (int64_t)n_seq * HV * K * V;
      hipLaunchKernelGGL(gdr_bwd_dh0_empty_kernel, dim3((unsigned)((n + 255) / 256 < 1024 ? (n + 255) / 256 : 1024)),
                         dim3(256), 0, (hipStream_t)stream, dht, dh0, n);
      return lampa_launch_status();
    }
    return LAMPA_OK;
  }
  const GbWorkspace w = gb_workspace(total_tokens, n_seq, n_seg, HV, K, V);
  if (!workspace || workspace_bytes < w.bytes) return LAMPA_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char* ws = (char*)workspace;
#define GB_RUN(TT)                                                                                                     \
  gb_run<TT>(q, k, v, g, beta, h0, dout, dht, dq, dk, dv, dg, dbeta, dh0, cu_seg, seq_seg0, seq_seg0_rev, seg_rev,     \
             total_tokens, n_seq, n_seg, H, HV, K, V, dtype, scale, l2norm, ws, w, s)
  switch (dtype) {
    case GDR_BF16: return GB_RUN(__bf16);
    case GDR_FP16: return GB_RUN(_Float16);
    case GDR_FP32: return GB_RUN(float);
    default: return LAMPA_ERR_INVALID;
  }
#undef GB_RUN
}

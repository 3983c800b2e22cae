// Chunkwise gated-delta-rule forward on gfx950 (bf16 MFMA 32x32x16, fp32 accumulate, fp32 state).
//
// Replaces the forward pipeline of chunk_gated_delta_rule (reference chengjiang123/Lampa,
// models/hattention/gated_delta_rule_ori.py:29-80): chunk_local_cumsum (cumsum.py:27-62), l2norm_fwd
// (l2norm.py:87-103), chunk_scaled_dot_kkt_fwd (chunk_scaled_dot_kkt.py:27-71), solve_tril (solve_tril.py),
// recompute_w_u_fwd (wy_fast.py:140-189), chunk_gated_delta_rule_fwd_h (chunk_delta_h.py:34-189) and
// chunk_fwd_o (chunk_o.py:33-111).
//
// Per chunk of C = 64 tokens of one head, with gamma the in-chunk cumulative log-decay, rk / rq the l2-norm
// factors of the raw k / q rows and S the K x V state entering the chunk:
//   A     = strict_lower( beta_i rk_i rk_j (k_i . k_j) e^{gamma_i - gamma_j} ),   T = (I + A)^-1
//   R     = beta_i ( v_i - e^{gamma_i} rk_i (K S)_i )                v_new = T R
//   o_i   = scale e^{gamma_i} rq_i (Q S)_i + (P v_new)_i,    P_ij = scale rq_i rk_j (q_i . k_j) e^{gamma_i - gamma_j}, j <= i
//   S'    = e^{gamma_last} S + K^T ( e^{gamma_last - gamma_j} rk_j v_new_j )
// All per-token factors are applied to accumulator rows in fp32, so the MFMA operands are the RAW bf16 k, q, v
// tiles and the only intermediate that goes through HBM is T (6 KiB per chunk and head).
//
// Kernels:
//   tinv     wave per (chunk, head): K K^T on MFMA with operand fragments loaded straight from HBM, gating, blocked
//            inverse (two 32x32 forward substitutions in fp32 + an MFMA merge with bf16 high/remainder splits);
//            T goes to HBM as three 32x32 bf16 blocks.
//   segment  workgroup per (segment of chunks, head), one "chain" wave per 32 columns plus two "stager" waves. Each
//            chunk's k, v, q, T tiles are staged once in LDS (row-major only), the coming chunks' global loads are
//            in flight meanwhile, and every chain wave runs the recurrence on its columns with the state in
//            accumulator registers. PASS_A: columns of [M | N] of the segment's affine map S -> M S + N (start
//            identity / zero). PASS_B: value columns, from the segment's true initial state, writing o (and the
//            final state).
//   scan     S_{p+1} = M_p S_p + N_p over the segments of a sequence, storing each segment's initial state.
// The state tile is fed back as the next MFMA's B operand straight from the accumulator registers: register r of
// lane l is row 8*(r/4) + 4*(l/32) + r%4, and since a contraction may visit its index in any order as long as
// both operands agree, every A operand is read from LDS in that slot order (ld_kappa).
#pragma once
#include "gdr_common.h"
#include "gdr_ops.h"
#include "gdr_plan.h"

// Device pointers to the tables of the plan (resolved on the host, so that a kernel reaches an entry with one
// load instead of a dependent pair).
struct GdrPlanView {
  const int32_t *chunk_tok0, *chunk_len, *seg_chunk0, *seg_nchunks, *seg_seq, *seg_flags, *seq_seg0, *seq_nseg, *seg_order;
};
static GdrPlanView gdr_plan_view(const int32_t* plan_host, const int32_t* plan_dev) {
  GdrPlanView pv;
  pv.chunk_tok0 = plan_dev + plan_host[PLAN_OFF_CHUNK_TOK0];
  pv.chunk_len = plan_dev + plan_host[PLAN_OFF_CHUNK_LEN];
  pv.seg_chunk0 = plan_dev + plan_host[PLAN_OFF_SEG_CHUNK0];
  pv.seg_nchunks = plan_dev + plan_host[PLAN_OFF_SEG_NCHUNKS];
  pv.seg_seq = plan_dev + plan_host[PLAN_OFF_SEG_SEQ];
  pv.seg_flags = plan_dev + plan_host[PLAN_OFF_SEG_FLAGS];
  pv.seq_seg0 = plan_dev + plan_host[PLAN_OFF_SEQ_SEG0];
  pv.seq_nseg = plan_dev + plan_host[PLAN_OFF_SEQ_NSEG];
  pv.seg_order = plan_dev + plan_host[PLAN_OFF_SEG_ORDER];
  return pv;
}

// T of one chunk and head in HBM, 16-bit elements: the lower-triangular blocks T11 and T22 packed by rows in 16-byte
// pieces of 8 columns -- row r keeps its pieces 0 .. r / 8 (rows 0-7 one piece, 8-15 two, 16-23 three, 24-31 four: 80
// of the 128 pieces of a 32x32 block; what lies above the diagonal inside a kept piece is stored as the zero it is)
// -- after the full block T21, 32x32 row-major: T21 | T11 packed | T22 packed (so that the 128 threads that stage a
// record read pieces t, 128 + t and 256 + t % 32 of it: two of the three loads share their address).
#define T_DIAG_PIECES 80
#define T_OFF_21 0
#define T_OFF_11 (32 * 32 * 2)
#define T_OFF_22 (T_OFF_11 + T_DIAG_PIECES * 16)
#define T_BYTES (T_OFF_22 + T_DIAG_PIECES * 16)
// (row, 8-column piece) of piece p of a packed block
__device__ __forceinline__ void tri_piece(int p, int& row, int& part) {
  const int x2 = p - 8, x3 = p - 24, x4 = p - 48;
  const int q3 = (x3 * 11) >> 5;  // x3 / 3 for 0 <= x3 < 24
  row = p < 8 ? p : p < 24 ? 8 + (x2 >> 1) : p < 48 ? 16 + q3 : 24 + (x4 >> 2);
  part = p < 8 ? 0 : p < 24 ? (x2 & 1) : p < 48 ? x3 - 3 * q3 : (x4 & 3);
}
// (row, piece) of the u-th of the 48 pieces of a 32x32 block that lie entirely above the diagonal
__device__ __forceinline__ void tri_upper_piece(int u, int& row, int& part) {
  const int q3 = (u * 11) >> 5, x2 = u - 24;
  row = u < 24 ? q3 : u < 40 ? 8 + (x2 >> 1) : 16 + (u - 40);
  part = u < 24 ? 1 + (u - 3 * q3) : u < 40 ? 2 + (x2 & 1) : 3;
}
// Record of one chunk and head: T, then the chunk's cumulative log-decay (units of log 2) and beta per token, fp32
// [64] each. The segment kernels take the two factor rows from here: in g and beta themselves a head's 64 values sit
// 4 bytes apart in rows that interleave all heads, so every workgroup would fetch the sectors of all of them.
#define REC_BYTES (T_BYTES + 3 * 64 * 4)  // (third row: the l2-norm factors of the k rows, written by gdr_local_kernel)
#define GDR_SCAN_GROUP 8  // segments per group of the two-level scan; a multiple of its ring depth

__device__ __forceinline__ bf16x8 frag_load(const unsigned char* base, int frag, int lane) {
  return *reinterpret_cast<const bf16x8*>(base + (size_t)frag * 1024 + lane * 16);
}
__device__ __forceinline__ void frag_store(unsigned char* base, int frag, int lane, bf16x8 v) {
  *reinterpret_cast<bf16x8*>(base + (size_t)frag * 1024 + lane * 16) = v;
}

// A-operand fragment (rows row0..row0+31 of a row-major bf16 array with `stride` elements per row, contraction
// step starting at column col0) in accumulator slot order: slots 0-3 = columns col0 + 4hh + 0..3,
// slots 4-7 = columns col0 + 8 + 4hh + 0..3.
__device__ __forceinline__ bf16x8 ld_kappa(const __bf16* arr, int stride, int row, int col0, int hh) {
  const bf16x4 lo = *reinterpret_cast<const bf16x4*>(arr + row * stride + col0 + 4 * hh);
  const bf16x4 hi = *reinterpret_cast<const bf16x4*>(arr + row * stride + col0 + 8 + 4 * hh);
  bf16x8 out;
#pragma unroll
  for (int s = 0; s < 4; ++s) { out[s] = lo[s]; out[4 + s] = hi[s]; }
  return out;
}

__device__ __forceinline__ f32x16 zero16() {
  f32x16 z;
#pragma unroll
  for (int r = 0; r < 16; ++r) z[r] = 0.0f;
  return z;
}

// Tells the compiler that x is the same in every lane, so that a table lookup with it becomes a scalar load: a
// vector load would join the queue of the prefetches and its wait would drain all of them.
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

__device__ __forceinline__ int acc_row(int r, int hh) { return 8 * (r / 4) + 4 * hh + (r % 4); }

// 2^x for x <= 0, otherwise 0 (also for NaN): the reference's safe_exp (models/hattention/fla_op.py:27-29), which it
// applies to every DIFFERENCE of cumulative log-decays (chunk_scaled_dot_kkt.py:67, chunk_o.py:98, chunk_delta_h.py:152).
// With g <= 0 those differences are never positive and this is a plain exp2.
__device__ __forceinline__ float safe_exp2(float x) { return __builtin_amdgcn_exp2f(x <= 0.0f ? x : -1e30f); }

__device__ __forceinline__ float l2_factor(float ss, int l2norm) {
  if (l2norm == GDR_L2_CHUNK) return 1.0f / __fsqrt_rn(ss + 1e-6f);
  if (l2norm == GDR_L2_RECURRENT) return 1.0f / (__fsqrt_rn(ss) + 1e-6f);
  return 1.0f;
}

// 16-byte vector of the input element type
template <typename T>
struct Raw8 {
  typedef T type __attribute__((ext_vector_type(8)));
};

// Raw input piece -> bf16 operand piece (+ its sum of squares when the rows get l2-normalised). bf16 inputs are
// passed through bit for bit; fp16 inputs are rounded to bf16 here.
template <typename T>
__device__ __forceinline__ bf16x8 raw_to_bf16(typename Raw8<T>::type v, float& ss, bool want_ss) {
  bf16x8 out;
  if constexpr (sizeof(T) == 2 && !__is_same(T, _Float16)) {
    out = __builtin_bit_cast(bf16x8, v);
    if (want_ss) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (float)out[e];
        ss = __builtin_fmaf(f, f, ss);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (float)v[e];
      if (want_ss) ss = __builtin_fmaf(f, f, ss);
      out[e] = (__bf16)f;
    }
  }
  return out;
}

// Raw input piece (type T) -> operand piece (type OT) (+ its sum of squares when the rows get l2-normalised): a bit
// copy when the operands keep the input type, a conversion otherwise.
template <typename T, typename OT>
__device__ __forceinline__ typename OpVec<OT>::x8 raw_to_op(typename Raw8<T>::type v, float& ss, bool want_ss) {
  typename OpVec<OT>::x8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float f = (float)v[e];
    if (want_ss) ss = __builtin_fmaf(f, f, ss);
    if constexpr (!__is_same(T, OT)) out[e] = (OT)f;
  }
  if constexpr (__is_same(T, OT)) out = __builtin_bit_cast(typename OpVec<OT>::x8, v);
  return out;
}

// ---- T = (I + A)^-1 ------------------------------------------------------------------------------------------
// c ? a : b on two accumulator registers. Written plainly, "c ? acc[i] : acc[j]" is folded into acc[c ? i : j], a
// register-indexed access that costs a 16-way compare-and-select chain; hiding one operand keeps it one v_cndmask.
__device__ __forceinline__ float gdr_pick(bool c, float a, float b) {
  asm volatile("" : "+v"(a));
  return c ? a : b;
}

// n consecutive floats (n = 1..4) from LDS into the first n components of a vector: exactly the bytes needed, so that
// partially used vectors of neighbouring loads never share (and wait for) a register
template <int N>
__device__ __forceinline__ f32x4 lds_ld_n(const float* p) {
  f32x4 out;
  if constexpr (N >= 4) {
    out = *reinterpret_cast<const f32x4*>(p);
  } else if constexpr (N == 3) {
    typedef float f32x3 __attribute__((ext_vector_type(3)));
    const f32x3 t3 = *reinterpret_cast<const f32x3*>(p);
    out[0] = t3[0]; out[1] = t3[1]; out[2] = t3[2]; out[3] = 0.0f;
  } else if constexpr (N == 2) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 t2 = *reinterpret_cast<const f32x2*>(p);
    out[0] = t2[0]; out[1] = t2[1]; out[2] = 0.0f; out[3] = 0.0f;
  } else {
    out[0] = *p; out[1] = 0.0f; out[2] = 0.0f; out[3] = 0.0f;
  }
  return out;
}

// One wave per (chunk, head), many per CU (every step is a short dependent chain on one wave, so it needs other waves
// to fill the gaps): K K^T on MFMA with operand fragments loaded straight from HBM (the k tile never touches LDS),
// gating, T by forward substitution on the four 16x16 diagonal blocks at once (lane = block and column: 15 dependent
// steps) and two levels of MFMA merges T21 = -T22 (A21 T11), each product a single fp16 instruction (T is rounded to
// the operand type OT afterwards, the coarser or an equal rounding). LDS holds the two diagonal 32x32 blocks in fp32
// and the per-token factor rows, all wave-private. Output: the record of the chunk and head.
// Built for four waves per SIMD (128 registers; its 10.5 KB of LDS then allow 15 of these one-wave workgroups per CU).
static inline int gdr_local_grid(int n_chunks, int HV) { return 8 * ((n_chunks + 7) / 8) * HV; }

template <typename T, typename OT, int KT>
__global__ void __launch_bounds__(64, 4) gdr_local_kernel(const T* __restrict__ k, const float* __restrict__ g,
                                                          const float* __restrict__ beta,
                                                          const int32_t* __restrict__ chunk_tok0,
                                                          const int32_t* __restrict__ chunk_len,
                                                          unsigned char* __restrict__ rec, int n_chunks, int H, int HV,
                                                          int l2norm) {
  using X8 = typename OpVec<T>::x8;    // input fragments (the K K^T products run in the input type)
  using O8 = typename OpVec<OT>::x8;   // record elements
  using O2 = typename OpVec<OT>::x2;
  constexpr int SB = 36, NKS = KT / 16;
  __shared__ __align__(16) float s_Ad[2 * 32 * SB];  // the two diagonal 32x32 blocks of A, later of T
  __shared__ __align__(16) float s_gamma[64], s_beta[64], s_rk[64], s_ra[64], s_ca[64];
  float* s_A11 = s_Ad;
  float* s_A22 = s_Ad + 32 * SB;
  // 1-D grid of gdr_local_grid(n_chunks, HV) workgroups. Workgroups go to the 8 XCDs round robin by their id and
  // every XCD has its own L2: the HV heads of a chunk are given to consecutive workgroups of ONE XCD, because g and
  // beta are [T, H] rows of which a head uses 4 bytes per 32-byte sector, and the sector should be fetched once.
  const int chunk = ((int)blockIdx.x / 8 / HV) * 8 + (int)blockIdx.x % 8, hv = ((int)blockIdx.x / 8) % HV;
  if (chunk >= n_chunks) return;
  const int h = hv / (HV / H);
  const int tok0 = chunk_tok0[chunk], len = chunk_len[chunk];
  const int lane = threadIdx.x, hh = lane >> 5, ln = lane & 31;
  const bool want_ss = l2norm != GDR_L2_NONE;

  // operand fragments of the k tile: fk[tm][ks] = k[32 tm + ln][16 ks + 8 hh .. + 7]; rows past the end of a partial
  // chunk behave as k = 0, g = 0, beta = 0
  X8 fk[2][NKS];
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    const size_t row = (size_t)(tok0 + min(32 * tm + ln, len - 1)) * H + h;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) fk[tm][ks] = *reinterpret_cast<const X8*>(k + row * KT + 16 * ks + 8 * hh);
  }
  const size_t gi = (size_t)(tok0 + min(lane, len - 1)) * HV + hv;
  const float rg = g[gi], rb = beta[gi];
  if (len < 64) {
    X8 zero;
#pragma unroll
    for (int x = 0; x < 8; ++x) zero[x] = (T)0.0f;
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) fk[tm][ks] = 32 * tm + ln < len ? fk[tm][ks] : zero;
  }
  float rk2[2] = {1.0f, 1.0f};
  if (want_ss) {
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      float ss = 0.0f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) ss = op_sumsq<T>(fk[tm][ks], ss);
      ss += __shfl_xor(ss, 32);
      rk2[tm] = l2_factor(ss, l2norm);
    }
  }
  f32x16 accA[3];
#pragma unroll
  for (int tt = 0; tt < 3; ++tt) {
    const int tr = tt == 2 ? 1 : 0, tc = tt == 0 ? 0 : 1;  // tiles (0,0), (0,1) = A21^T, (1,1)
    accA[tt] = zero16();
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) accA[tt] = mfma32(fk[tr][ks], fk[tc][ks], accA[tt]);
  }
  // per-token factors, lane = token (gamma in units of log 2)
  float gcum = 1.44269504f * wave_cumulative_decay(lane < len ? rg : 0.0f);
  // The product must be ROUNDED before it enters any difference of two gammas: contracted into it as an fma, the
  // difference of equal gammas comes out as a rounding residual of either sign, and a positive exponent is masked to
  // zero. The empty asm hides the product from the compiler.
  asm volatile("" : "+v"(gcum));
  const float bz = lane < len ? rb : 0.0f;
  const float g_last = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gcum), 63));
  const float rk_tok = hh ? rk2[1] : rk2[0];
  {
    float* fact = reinterpret_cast<float*>(rec + ((size_t)chunk * HV + hv) * REC_BYTES + T_BYTES);
    fact[lane] = gcum;
    fact[64 + lane] = bz;
    fact[128 + lane] = rk_tok;
  }
  // Fast gating: e^{gamma_i - gamma_j} = E_i / E_j with E = e^{gamma - gamma_ref}, gamma_ref = gamma_last / 2, as long as
  // no exponent can leave the fp32 range (total decay of the chunk above 2^-120) and no g is positive (then every ratio
  // has to go through safe_exp one by one).
  const bool fast = !__ballot(rg > 0.0f && lane < len) && g_last > -120.0f;
  const float E = __builtin_amdgcn_exp2f(gcum - 0.5f * g_last), iE = __builtin_amdgcn_exp2f(0.5f * g_last - gcum);
  s_gamma[lane] = gcum;
  s_beta[lane] = bz;
  s_rk[lane] = rk_tok;
  s_ra[lane] = bz * rk_tok * E;
  s_ca[lane] = rk_tok * iE;
  lds_fence();
  f32x16 a21t;
  if (fast) {
#pragma unroll
    for (int tt = 0; tt < 3; ++tt) {
      const int tr = tt == 2 ? 1 : 0, tc = tt == 0 ? 0 : 1;
      f32x4 rowa[4], rowc[4];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        rowa[b4] = *reinterpret_cast<const f32x4*>(&s_ra[32 * tr + 8 * b4 + 4 * hh]);
        rowc[b4] = *reinterpret_cast<const f32x4*>(&s_ca[32 * tr + 8 * b4 + 4 * hh]);
      }
      const int cidx = 32 * tc + ln;
      const float cola = s_ca[cidx], cola_t = s_ra[cidx];
      lds_fence();
      if (tt == 1) {  // A21^T: rows j (tile 0), columns i (tile 1): A_ij = ra_i ca_j (k_i.k_j)
#pragma unroll
        for (int r = 0; r < 16; ++r) a21t[r] = accA[1][r] * cola_t * rowc[r / 4][r % 4];
      } else {        // diagonal blocks: rows i, columns j, strictly lower
        float* blk = tt == 0 ? s_A11 : s_A22;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int il = acc_row(r, hh);
          blk[il * SB + ln] = il > ln ? accA[tt][r] * cola * rowa[r / 4][r % 4] : 0.0f;
        }
      }
    }
  } else {
#pragma unroll
    for (int tt = 0; tt < 3; ++tt) {
      const int tr = tt == 2 ? 1 : 0, tc = tt == 0 ? 0 : 1;
      f32x4 gr4[4], rr4[4], br4[4];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        gr4[b4] = *reinterpret_cast<const f32x4*>(&s_gamma[32 * tr + 8 * b4 + 4 * hh]);
        rr4[b4] = *reinterpret_cast<const f32x4*>(&s_rk[32 * tr + 8 * b4 + 4 * hh]);
        br4[b4] = *reinterpret_cast<const f32x4*>(&s_beta[32 * tr + 8 * b4 + 4 * hh]);
      }
      const int cidx = 32 * tc + ln;
      const float gc = s_gamma[cidx], rc = s_rk[cidx], bc = s_beta[cidx];
      lds_fence();
      if (tt == 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          a21t[r] = accA[1][r] * (bc * rc) * rr4[r / 4][r % 4] * safe_exp2(gc - gr4[r / 4][r % 4]);
      } else {
        float* blk = tt == 0 ? s_A11 : s_A22;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int il = acc_row(r, hh);
          blk[il * SB + ln] = accA[tt][r] * (br4[r / 4][r % 4] * rr4[r / 4][r % 4] * rc) *
                              safe_exp2(il > ln ? gr4[r / 4][r % 4] - gc : 1.0f);
        }
      }
    }
  }
  lds_fence();
  // ---- the four 16x16 diagonal blocks by forward substitution: lane 16 b + c owns column c of block b (block b = rows
  //      and columns 16 (b % 2) .. + 15 of the 32x32 diagonal block b / 2), fp32 throughout
  {
    const int b4 = lane >> 4, c = lane & 15;
    float* Ab = s_Ad + (b4 >> 1) * (32 * SB) + (16 * (b4 & 1)) * SB + 16 * (b4 & 1);
    float x[16];
    // every row this lane needs, requested at once (row i: columns 0 .. i-1, exactly those)
    f32x4 rows[16][4];
#define GDR_ROW(i)                                                                                    \
  {                                                                                                   \
    constexpr int full = (i) / 4, rem = (i) % 4;                                                      \
    _Pragma("unroll") for (int qq = 0; qq < full; ++qq) rows[i][qq] = lds_ld_n<4>(Ab + (i) * SB + 4 * qq); \
    if constexpr (rem > 0) rows[i][full] = lds_ld_n<rem>(Ab + (i) * SB + 4 * full);                   \
  }
    GDR_ROW(1) GDR_ROW(2) GDR_ROW(3) GDR_ROW(4) GDR_ROW(5) GDR_ROW(6) GDR_ROW(7) GDR_ROW(8)
    GDR_ROW(9) GDR_ROW(10) GDR_ROW(11) GDR_ROW(12) GDR_ROW(13) GDR_ROW(14) GDR_ROW(15)
#undef GDR_ROW
    x[0] = (c == 0) ? 1.0f : 0.0f;
#pragma unroll
    for (int i = 1; i < 16; ++i) {
      // the terms with x[0 .. i-2] first, the one that waits for x[i-1] last
      float acc0 = (i == c) ? 1.0f : 0.0f, acc1 = 0.0f;
#pragma unroll
      for (int j = 0; j + 1 < i; ++j) {
        if (j & 1) acc1 = __builtin_fmaf(-rows[i][j / 4][j % 4], x[j], acc1);
        else acc0 = __builtin_fmaf(-rows[i][j / 4][j % 4], x[j], acc0);
      }
      x[i] = __builtin_fmaf(-rows[i][(i - 1) / 4][(i - 1) % 4], x[i - 1], acc0 + acc1);
    }
    lds_fence();
#pragma unroll
    for (int i = 0; i < 16; ++i) Ab[i * SB + c] = x[i];  // T in place of A
  }
  lds_fence();
  // ---- first merge, both 32x32 diagonal blocks in ONE 32x32x16 product per stage: operand row / column ln = 16 B + i
  //      belongs to diagonal block B; the quadrants (B, B) of the result are the two products wanted. fp16 operands: T is
  //      rounded to the input type afterwards, which is the coarser rounding for bf16 inputs and the same for fp16.
  {
    const int B = ln >> 4, i = ln & 15;
    float* blk = s_Ad + B * (32 * SB);
    f16x8 a1, b1, a2, b2;
    const f32x4 p0 = *reinterpret_cast<const f32x4*>(blk + (16 + i) * SB + 4 * hh);       // A21'[i][slots]
    const f32x4 p1 = *reinterpret_cast<const f32x4*>(blk + (16 + i) * SB + 8 + 4 * hh);
    const f32x4 q0 = *reinterpret_cast<const f32x4*>(blk + (16 + i) * SB + 16 + 4 * hh);  // T22'[i][slots]
    const f32x4 q1 = *reinterpret_cast<const f32x4*>(blk + (16 + i) * SB + 24 + 4 * hh);
    float colv[8];
#pragma unroll
    for (int qq = 0; qq < 8; ++qq) colv[qq] = blk[kappa(hh, qq) * SB + i];                  // T11'[slots][i]
    lds_fence();
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) {
      a1[qq] = (_Float16)p0[qq]; a1[4 + qq] = (_Float16)p1[qq];
      a2[qq] = (_Float16)q0[qq]; a2[4 + qq] = (_Float16)q1[qq];
    }
#pragma unroll
    for (int qq = 0; qq < 8; ++qq) b1[qq] = (_Float16)colv[qq];
    const f32x16 y = mfma32(a1, b1, zero16());  // quadrant (B, B): A21' T11'
#pragma unroll
    for (int qq = 0; qq < 8; ++qq) b2[qq] = (_Float16)gdr_pick(B != 0, y[8 + qq], y[qq]);
    const f32x16 z = mfma32(a2, b2, zero16());  // quadrant (B, B): T22' (A21' T11')
#pragma unroll
    for (int qq = 0; qq < 8; ++qq)              // T21'[row][i] = -z: rows 16 B + kappa(hh, qq) of the product
      blk[(16 + kappa(hh, qq)) * SB + i] = -gdr_pick(B != 0, z[8 + qq], z[qq]);
  }
  lds_fence();
  // ---- second merge: T21 = -T22 (A21 T11), A21 from the transposed accumulator
  f32x16 y = zero16(), t21 = zero16();
  {
    float colv[16];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int qq = 0; qq < 8; ++qq) colv[8 * ks + qq] = s_A11[(16 * ks + kappa(hh, qq)) * SB + ln];
    f32x4 rowv[4];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      rowv[2 * ks + 0] = *reinterpret_cast<const f32x4*>(&s_A22[ln * SB + 16 * ks + 4 * hh]);
      rowv[2 * ks + 1] = *reinterpret_cast<const f32x4*>(&s_A22[ln * SB + 16 * ks + 8 + 4 * hh]);
    }
    lds_fence();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      f16x8 bb;
#pragma unroll
      for (int qq = 0; qq < 8; ++qq) bb[qq] = (_Float16)colv[8 * ks + qq];
      y = mfma32(acc_to_op<_Float16>(a21t, 8 * ks), bb, y);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      f16x8 aa;
#pragma unroll
      for (int qq = 0; qq < 4; ++qq) { aa[qq] = (_Float16)rowv[2 * ks][qq]; aa[4 + qq] = (_Float16)rowv[2 * ks + 1][qq]; }
      t21 = mfma32(aa, acc_to_op<_Float16>(y, 8 * ks), t21);
    }
  }
  // ---- T -> HBM: the diagonal blocks from LDS in 16-byte pieces; T21 from the accumulator, two columns per store
  //      (lanes 2j and 2j+1 swap one value of every adjacent row pair)
  OT* out = reinterpret_cast<OT*>(rec + ((size_t)chunk * HV + hv) * REC_BYTES);
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    const float* src = blk == 0 ? s_A11 : s_A22;
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int piece = lane + 64 * jj;  // of the packed block
      if (piece < T_DIAG_PIECES) {
        int row, part;
        tri_piece(piece, row, part);
        const f32x4 lo = *reinterpret_cast<const f32x4*>(&src[row * SB + 8 * part]);
        const f32x4 hi = *reinterpret_cast<const f32x4*>(&src[row * SB + 8 * part + 4]);
        O8 pk;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) { pk[e4] = (OT)lo[e4]; pk[4 + e4] = (OT)hi[e4]; }
        *reinterpret_cast<O8*>(out + (blk == 0 ? T_OFF_11 : T_OFF_22) / 2 + 8 * piece) = pk;
      }
    }
  }
  {
    const bool odd = ln & 1;
#pragma unroll
    for (int pr = 0; pr < 8; ++pr) {
      const int r0 = 2 * pr, r1 = r0 + 1;
      const float x0 = -t21[r0], x1 = -t21[r1];
      const float keep = gdr_pick(odd, x1, x0);
      const float got = dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, gdr_pick(odd, x0, x1));
      O2 pk;
      pk[0] = (OT)(odd ? got : keep);
      pk[1] = (OT)(odd ? keep : got);
      const int row = acc_row(r0, hh) + (odd ? 1 : 0);
      *reinterpret_cast<O2*>(out + T_OFF_21 / 2 + row * 32 + (ln & ~1)) = pk;
    }
  }
}

// ---- segment kernel --------------------------------------------------------------------------------------------
// Workgroup per (segment, head). Waves 0 .. SLABS-1 ("chain" waves) each own 32 columns of the state and run the
// recurrence; the last two waves ("stagers") load the coming chunks' tiles from HBM, stage them ROW-MAJOR in LDS
// (16-byte writes only), derive the per-token factors and (PASS_B) build the P fragments. Operands that contract
// over the tokens (K^T, and v in accumulator layout) are read from the row-major tiles with the transposing LDS
// load (ds_read_b64_tr_b16), so no transposed copy is ever written.
//
// The k, v, T tiles and the per-token factors are DOUBLE-buffered in LDS, so the stagers fill the tiles of chunk c+1
// while the chain waves work on chunk c; q, P and the o tile exist once. LDS-only barriers per chunk (every barrier is
// a rendezvous of all waves, so the stagers' work is spread such that they are never the slower side):
//   B(c)  the chain waves hold every k / v / T operand of chunk c in registers, and tiles (c+1) [PASS_A: also its
//         factors], q(c) and P(c) are complete             -> buffer c%2 is free for chunk c+2
//         (a stager stages the q rows of ONE 32-row tile and builds exactly the P tiles of those rows -- stager 0
//         the tile (0,0), stager 1 the tiles (1,0) and (1,1) -- so no barrier separates staging q from building P)
//   C(c)  (PASS_B) the chain waves hold the q and P operands of chunk c, factors (c+1) are complete
//                                                          -> the stagers may write q(c+1)
// Global loads are issued about one chunk period before their data is staged.
// Output pass of the heads up to 64 x 64: the chain waves only write their slab of the o tile; the stagers carry the
// tile of chunk c - 1 to HBM after B(c) (whole rows), and one more barrier after the last chunk lets them write the last.
// Narrow form of the output pass (CW = 16, GdrSegShape): chain waves of 16 columns on the 16x16x32 MFMA, two PAIRS of
// stager waves (k / v / T / factors and q / P), the same barriers; for heads wider than 64 x 64 q and P exist twice.
// NQ: copies of the q tile, the P fragments and the q factor rows (2: by chunk parity, like the tile sets)
template <int KT, int VT, bool PASS_B, bool SCALED = !PASS_B, int NQ = 1>
struct GdrSegSmem {
  static constexpr int SK = KT + 8;  // row stride of the k / q tiles (bf16 elements)
  static constexpr int SV = VT + 8;  // row stride of the v and o tiles
  static constexpr int ST = 40;      // row stride of a 32x32 block of T (blocks T11, T21, T22)
  // one set of tiles (two of them)
  static constexpr int T_OFF_K = 0;
  static constexpr int T_OFF_V = T_OFF_K + 64 * SK * 2;
  static constexpr int T_OFF_T = T_OFF_V + 64 * SV * 2;
  static constexpr int T_OFF_F = T_OFF_T + 3 * 32 * ST * 2;
  static constexpr int N_FACT = 6;  // beta, ek, dk, gamma, rk, misc
  static constexpr int T_OFF_KD = T_OFF_F + N_FACT * 64 * 4;  // PASS_A: second scaled copy of the k tile
  static constexpr int TILE_BYTES = T_OFF_KD + (SCALED ? 64 * SK * 2 : 0);
  static constexpr int Q_BYTES = 64 * SK * 2, P_BYTES = 6 * 1024, QF_BYTES = 2 * 64 * 4;
  static constexpr int OFF_Q = 2 * TILE_BYTES;
  static constexpr int OFF_P = OFF_Q + (PASS_B ? NQ * Q_BYTES : 0);
  static constexpr int OFF_O = OFF_P + (PASS_B ? NQ * P_BYTES : 0);
  static constexpr int OFF_QF = OFF_O + (PASS_B ? 64 * SV * 2 : 0);  // qs, rq
  static constexpr int BYTES = OFF_QF + (PASS_B ? NQ * QF_BYTES : 0);
};

// pointers into one of the two tile sets
template <typename OT>
struct GdrTilesT {
  // k = the raw k tile; or (composite pass with SCALED tiles) k = diag(ek) K and kd = diag(dk) K, rounded to bf16
  // once: the stagers fold the per-token gate and norm factors into the tiles, so the chain waves neither read nor
  // apply them. That takes a third of the chain waves' LDS traffic away and pays when many short segments share the
  // CUs; with few long segments (one workgroup per CU) the stagers' extra work is the longer pole, so the
  // hierarchical forward instantiates the composite pass with SCALED = false.
  OT *k, *kd, *v, *t;
  float *beta, *ek, *dk, *gamma, *rk, *misc;  // ek = e^{gamma_i} rk_i, dk = e^{gamma_last - gamma_i} rk_i, misc[0] = e^{gamma_last}
};

// CW: columns of the state per chain wave. 32: products on the 32x32x16 MFMA. 16 (output pass, K >= 64): "narrow" chain
// waves on the 16x16x32 MFMA -- twice as many waves, each with half the dependent MFMA -> convert -> MFMA chain of a chunk
// and half the state registers (K / 4 per lane).
template <int KT, int VT, bool PASS_B, int CW = 32>
struct GdrSegShape {
  static_assert(CW == 32 || (CW == 16 && PASS_B && KT >= 64), "narrow chain waves: output pass, K >= 64");
  static constexpr int SLABS = PASS_B ? VT / CW : (KT + VT) / 32;  // chain waves
  // + the stager waves: two (each stages half the rows of every tile and builds part of P), or, beside narrow chain
  // waves, two pairs -- one for k, v, T and the per-token factors, one for q and P -- so that neither role needs more
  // registers than four waves per SIMD leave
  static constexpr int STAGERS = CW == 16 ? 4 : 2;
  static constexpr bool DOUBLE_Q = CW == 16 && KT + VT > 128;  // q tile and P fragments double-buffered (LDS allows it)
  static constexpr int WAVES = SLABS + STAGERS;
  // The k and q tiles are stored swizzled (op_swizzle16 in gdr_ops.h: one conflict-free 16-byte LDS read per operand
  // fragment instead of two 8-byte reads). It pays in the output pass of the 128-wide heads (-10 %); at K = V = 64
  // the output pass times the same and the composite pass loses: the wider reads cost it 24 registers, and two of
  // its six-wave workgroups only share a CU below 128 (the hardware deals a workgroup's waves out to the SIMDs in a
  // fixed rotation and starts the next workgroup one step further on, so one SIMD carries four of the twelve waves).
  // (the composite pass of the 128-wide heads, whose LDS is 90 % busy with half of it bank conflicts, gets slower with
  // swizzled scaled tiles: 814 -> 909 us at config 4 -- the swizzled 16-byte reads cost it registers it does not have)
  static constexpr bool SWIZZLED = CW == 32 && PASS_B && (KT > 64 || VT > 64);
  // Waves per SIMD the register allocation has to leave room for (the second argument of the launch bounds). The
  // composite pass at K = V = 64 runs two six-wave workgroups per CU, and the hardware's rotation puts four of those
  // twelve waves on one SIMD: 128 registers each.
  // Narrow output pass: K = V = 64 runs two eight-wave workgroups per CU (four waves per SIMD), the wider heads one
  // workgroup of up to twelve waves (three per SIMD).
  static constexpr int WAVES_PER_SIMD = CW == 16 ? (KT + VT <= 128 ? 4 : 3) : (!PASS_B && KT + VT <= 128) ? 4 : 2;
};

typedef short s16x4 __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: lane i of every block of 16 lanes receives element (i % 4) of the four 8-byte rows that
// lanes i/4, i/4 + 4, i/4 + 8 and i/4 + 12 of its block point at.
__device__ __forceinline__ bf16x4 lds_read_tr4(const __bf16* p) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p));
}

// Four consecutive rows row0 + 4hh .. +3 of column col0 + (lane % 32) of a row-major bf16 tile: lane L of a block
// points at row L / 4, column group L % 4 of the block's 16 columns.
__device__ __forceinline__ bf16x4 ld_col4(const __bf16* arr, int stride, int col0, int row0, int lane) {
  const int L = lane & 15, blk = (lane >> 4) & 1, hh = lane >> 5;
  return lds_read_tr4(arr + (row0 + 4 * hh + (L >> 2)) * stride + col0 + 16 * blk + 4 * (L & 3));
}

// A-operand fragment of the TRANSPOSE of a row-major tile: operand row = tile column col0 + (lane % 32),
// contraction over the tile rows row0 .. row0 + 15 in accumulator slot order.
__device__ __forceinline__ bf16x8 ld_kappa_tr(const __bf16* arr, int stride, int col0, int row0, int lane) {
  const bf16x4 lo = ld_col4(arr, stride, col0, row0, lane), hi = ld_col4(arr, stride, col0, row0 + 8, lane);
  bf16x8 out;
#pragma unroll
  for (int s = 0; s < 4; ++s) { out[s] = lo[s]; out[4 + s] = hi[s]; }
  return out;
}

template <typename T, int KT, int VT, bool PASS_B, bool SCALED_K = !PASS_B, typename OT = T, int CW = 32>
__global__ void __launch_bounds__((64 * GdrSegShape<KT, VT, PASS_B, CW>::WAVES),
                                  ((SCALED_K || CW == 16) ? GdrSegShape<KT, VT, PASS_B, CW>::WAVES_PER_SIMD : 2))
    gdr_segment_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                       const float* __restrict__ g, const float* __restrict__ beta, const GdrPlanView pv,
                       const int32_t* __restrict__ chunk_tok0, const int32_t* __restrict__ chunk_len,
                       const unsigned char* __restrict__ tmat,
                       const float* __restrict__ Sinit, unsigned char* __restrict__ Mcomp,
                       unsigned char* __restrict__ Ncomp, float* __restrict__ Dcomp, T* __restrict__ o,
                       float* __restrict__ ht, int H, int HV, float scale, int l2norm,
                       const unsigned char* __restrict__ Mgrp, const unsigned char* __restrict__ Ngrp,
                       const float* __restrict__ Dgrp, const float* __restrict__ h0, int gmax) {
  // OT: the 16-bit type of every MFMA operand (tiles in LDS, T, R, v_new, P, the state as operand, M' of the
  // composites): the input type, so that fp16 inputs run on the fp16 MFMA without losing mantissa bits
  using X8 = typename OpVec<OT>::x8;
  using X4 = typename OpVec<OT>::x4;
  constexpr bool SCALED = !PASS_B && SCALED_K;
  constexpr bool SWZ = GdrSegShape<KT, VT, PASS_B, CW>::SWIZZLED;
  // narrow chain waves: the k, q and T tiles keep every 32 columns in the order of op_perm32 (gdr_ops.h)
  constexpr bool P16 = CW == 16;
  // The narrow form keeps the k, q and T tiles in op_perm32 order (one 16-byte read per operand fragment). With the
  // tiles in plain order and two 8-byte reads per fragment the output pass is slower: 71.0 against 68.2 us at
  // K = V = 64, 1 463 against 1 290 us at K = V = 128 (config 4).
  constexpr bool PERM = P16;
  // 32-column output pass: the o tile of a chunk is written to HBM by the STAGER waves (after the next chunk's barrier
  // B, whole rows), so the read-back and the stores are off the recurrence waves' chain.
  constexpr bool STAGER_FLUSH = PASS_B && CW == 32 && KT + VT <= 128;  // (the wider heads have no registers for it)
  // Output pass at K <= 64: a stager builds the P tiles of the q rows it staged itself (stager 0 the tile (0,0),
  // stager 1 the tiles (1,0) and (1,1)), so no barrier separates staging q from building P. At K = 128 a P tile is
  // twice the work, the two stagers share the middle tile, and the barrier Qb(c) (q(c) is staged) comes back.
  constexpr bool OWN_Q = KT <= 64 || CW == 16;  // (the narrow form's q / P stagers have registers of their own to spare)
  // Narrow form of the heads wider than 64 x 64 (one workgroup per CU, LDS to spare): q, P and the q factor rows exist
  // twice, so the q / P stagers stage q(c + 1) while the chain waves still read q(c) and P(c).
  constexpr bool DBQ = GdrSegShape<KT, VT, PASS_B, CW>::DOUBLE_Q;
  using SM = GdrSegSmem<KT, VT, PASS_B, SCALED, DBQ ? 2 : 1>;
  constexpr int NSLAB = GdrSegShape<KT, VT, PASS_B, CW>::SLABS;
  constexpr int SK = SM::SK, SV = SM::SV, ST = SM::ST;
  extern __shared__ __align__(16) unsigned char smem[];
  auto tiles = [&](int par) {
    unsigned char* base = smem + par * SM::TILE_BYTES;
    GdrTilesT<OT> t;
    t.k = reinterpret_cast<OT*>(base + SM::T_OFF_K);
    t.kd = reinterpret_cast<OT*>(base + (SCALED ? SM::T_OFF_KD : SM::T_OFF_K));
    t.v = reinterpret_cast<OT*>(base + SM::T_OFF_V);
    t.t = reinterpret_cast<OT*>(base + SM::T_OFF_T);
    t.beta = reinterpret_cast<float*>(base + SM::T_OFF_F);
    t.ek = t.beta + 64;
    t.dk = t.beta + 128;
    t.gamma = t.beta + 192;
    t.rk = t.beta + 256;
    t.misc = t.beta + 320;
    return t;
  };
  OT* const s_q0 = reinterpret_cast<OT*>(smem + SM::OFF_Q);
  unsigned char* const s_P0 = smem + SM::OFF_P;
  T* s_o = reinterpret_cast<T*>(smem + SM::OFF_O);
  float* const s_qs0 = reinterpret_cast<float*>(smem + SM::OFF_QF);  // scale e^{gamma_i} rq_i, then rq_i
  // the copy of the q tile / the P fragments / the factor rows that belongs to a chunk of parity par
#define GDR_Q_BUFFERS(par)                                                          \
  OT* const s_q = s_q0 + (DBQ ? (par) : 0) * (SM::Q_BYTES / 2);                     \
  unsigned char* const s_P = s_P0 + (DBQ ? (par) : 0) * SM::P_BYTES;                \
  float* const s_qs = s_qs0 + (DBQ ? (par) : 0) * (SM::QF_BYTES / 4);               \
  float* const s_rq = s_qs + 64;                                                    \
  (void)s_q; (void)s_P; (void)s_qs; (void)s_rq

  // long segments first (see the plan). Grid (segments, heads), or one row of segments x heads workgroups in which the
  // heads of a segment are neighbours, so that the order holds over all heads
  const int seg = pv.seg_order[gridDim.y > 1 ? blockIdx.x : blockIdx.x / HV];
  const int hv = gridDim.y > 1 ? blockIdx.y : blockIdx.x % HV;
  const int h = hv / (HV / H);
  const int flags = pv.seg_flags[seg];
  if (!PASS_B && (flags & SEG_LAST)) return;  // nothing follows the last segment of a sequence
  const int c0 = pv.seg_chunk0[seg], nc = pv.seg_nchunks[seg];
  const int c1 = c0 + nc;
  // (the per-chunk tables are separate restrict parameters: read through the view they could alias the kernel's
  // stores, would be fetched with vector loads and would sit in the same queue as the stagers' prefetches)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;

  if (wave >= NSLAB) {
    // ================================================ stager ================================================
    // Narrow output pass: with eight or more chain waves beside them the four stagers are the longer pole, so they get
    // the SIMDs' issue slots first (config 4: output pass 1 168 -> 993 - 1 012 us). In the other forms the chain is
    // the longer pole and a raised priority on either side changes nothing or costs a little.
    if constexpr (PASS_B && CW == 16) __builtin_amdgcn_s_setprio(3);
    constexpr int KU = KT / 16, VU = VT / 16;  // 16-byte pieces per thread: half a row of k / q, of v
    // (narrow form: pair 0 = waves NSLAB, NSLAB + 1 stages k, v, T and the factors, pair 1 = the next two q and P; a
    // pair is the 128 threads the staging code is written for)
    const int spair = P16 ? (wave - NSLAB) >> 1 : 0;
    const int stid = tid - 64 * (NSLAB + 2 * spair), sw = (wave - NSLAB) & 1;
    const int srow = stid >> 1, spart = stid & 1;
    // PASS_A keeps the raw k rows of two chunks (sets by chunk parity): the scaled tiles are written from the
    // registers after the row norms are known, and the next k loads must already be on their way by then
    typename Raw8<T>::type rk0_[KU], rk1_[SCALED ? KU : 1], rv_[VU];
    typename Raw8<T>::type rq0_[PASS_B ? KU : 1], rq1_[PASS_B ? KU : 1];  // q of even / odd chunks of the segment
    X8 rt_[3];
    float rg = 0.0f, rb = 0.0f;
    float grow = 0.0f;  // gamma of row srow of the chunk whose tiles were staged last
    float ghalf = 0.0f;  // half the total log-decay of that chunk
    bool pfast = false;  // that chunk's P takes the factored gating (stage_factors)
    // where this thread's pieces of the packed diagonal blocks of T go in the LDS tile; the pieces above the diagonal
    // are never staged and are zeroed once, in both tile sets
    int ta_off, tb_off;  // element offsets into the T area of a tile set of this thread's two packed pieces
    {
      int row, part;
      const int da = stid, db = 128 + (stid & 31);  // indices among the 160 packed pieces (T11: 0 .. 79, T22: 80 .. 159)
      tri_piece(da < T_DIAG_PIECES ? da : da - T_DIAG_PIECES, row, part);
      ta_off = ((da < T_DIAG_PIECES ? 0 : 2) * 32 + row) * ST + (PERM ? op_perm32_piece(part) : 8 * part);
      tri_piece(db - T_DIAG_PIECES, row, part);
      tb_off = (2 * 32 + row) * ST + (PERM ? op_perm32_piece(part) : 8 * part);
    }
    const int t21_off = (1 * 32 + (stid >> 2)) * ST + (PERM ? op_perm32_piece(stid & 3) : 8 * (stid & 3));
    // a 16-byte piece of T into a tile: as it is, or (P16) its two halves 8 elements apart
    auto put_t = [&](OT* at, X8 v) __attribute__((always_inline)) {
      if constexpr (PERM) {
        X4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) { lo[e] = v[e]; hi[e] = v[4 + e]; }
        *reinterpret_cast<X4*>(at) = lo;
        *reinterpret_cast<X4*>(at + 8) = hi;
      } else {
        *reinterpret_cast<X8*>(at) = v;
      }
    };
    if (stid < 128 - T_DIAG_PIECES) {
      int ur, up;
      tri_upper_piece(stid, ur, up);
      X8 z8;
#pragma unroll
      for (int e = 0; e < 8; ++e) z8[e] = (OT)0.0f;
#pragma unroll
      for (int par = 0; par < 2; ++par) {
        OT* tt = tiles(par).t;
        put_t(&tt[(0 * 32 + ur) * ST + (PERM ? op_perm32_piece(up) : 8 * up)], z8);
        put_t(&tt[(2 * 32 + ur) * ST + (PERM ? op_perm32_piece(up) : 8 * up)], z8);
      }
    }
    // Loads are unconditional (rows past the end of a partial chunk read its last row and are zeroed when staged):
    // a select on a freshly loaded value would make the wave wait for the load at once.
    // (tok0, len: the chunk's entries of the tables, which the caller holds in scalar registers: fetched here they
    // would put a dependent scalar-memory round trip in front of every use)
    auto issue_tiles = [&](int c, int tok0, int len, typename Raw8<T>::type* rk_) {  // k, v, T
      c = uniform(c);
      const T* kb = k + ((size_t)tok0 * H + h) * KT;
      const T* vb = v + ((size_t)tok0 * HV + hv) * VT;
      const int r = min(srow, len - 1);
      const int koff = r * H * KT + spart * (KT / 2), voff = r * HV * VT + spart * (VT / 2);
#pragma unroll
      for (int u = 0; u < KU; ++u) rk_[u] = *reinterpret_cast<const typename Raw8<T>::type*>(kb + koff + 8 * u);
#pragma unroll
      for (int u = 0; u < VU; ++u) rv_[u] = *reinterpret_cast<const typename Raw8<T>::type*>(vb + voff + 8 * u);
      // three pieces per thread, unconditional loads (the last 32 pieces are loaded by four threads each, which then
      // store the same values to the same place)
      const X8* tp = reinterpret_cast<const X8*>(tmat + ((size_t)c * HV + hv) * REC_BYTES);
      rt_[0] = tp[stid];                    // T21
      rt_[1] = tp[128 + stid];              // packed diagonal pieces 0 .. 127 (T11, then the first 48 of T22)
      rt_[2] = tp[256 + (stid & 31)];       // packed diagonal pieces 128 .. 159 (the rest of T22), four times over
    };
    auto issue_gb = [&](int c) {  // cumulative log-decay and beta of the chunk's tokens (lane = token)
      c = uniform(c);
      const float* fact = reinterpret_cast<const float*>(tmat + ((size_t)c * HV + hv) * REC_BYTES + T_BYTES);
      rg = fact[lane];
      rb = fact[64 + lane];
    };
    auto issue_q = [&](int tok0, int len, typename Raw8<T>::type* rq_) {
      const T* qb = q + ((size_t)tok0 * H + h) * KT;
      const int koff = min(srow, len - 1) * H * KT + spart * (KT / 2);
#pragma unroll
      for (int u = 0; u < KU; ++u) rq_[u] = *reinterpret_cast<const typename Raw8<T>::type*>(qb + koff + 8 * u);
    };
    typename Raw8<T>::type zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = (T)0.0f;
    const bool want_ss = l2norm != GDR_L2_NONE;

    float kss = 0.0f;  // sum of squares of this thread's half of k row srow (stage_data -> stage_factors)
    // k, v and T of chunk c from the registers to tile set par
    // rows past the end of a partial chunk become zero (a uniform branch: whole chunks pay nothing for it)
    auto zero_dead_rows = [&](int len, typename Raw8<T>::type* regs, int n) __attribute__((always_inline)) {
      if (len < 64) {
        const bool live = srow < len;
#pragma unroll
        for (int u = 0; u < n; ++u) regs[u] = live ? regs[u] : zero;
      }
    };
    auto stage_data = [&](int len, int par, typename Raw8<T>::type* rk_) {
      const GdrTilesT<OT> tl = tiles(par);
      zero_dead_rows(len, rk_, KU);
      zero_dead_rows(len, rv_, VU);
      put_t(&tl.t[t21_off], rt_[0]);
      put_t(&tl.t[ta_off], rt_[1]);
      put_t(&tl.t[tb_off], rt_[2]);
      kss = 0.0f;
      if constexpr (PERM) {
#pragma unroll
        for (int u = 0; u < KU; u += 4) {  // (a thread's half row is one or two groups of 32 columns)
          X8 p0 = raw_to_op<T, OT>(rk_[u], kss, want_ss), p1 = raw_to_op<T, OT>(rk_[u + 1], kss, want_ss);
          X8 p2 = raw_to_op<T, OT>(rk_[u + 2], kss, want_ss), p3 = raw_to_op<T, OT>(rk_[u + 3], kss, want_ss);
          op_perm32<OT>(p0, p1, p2, p3);
          OT* at = &tl.k[srow * SK + spart * (KT / 2) + 8 * u];
          *reinterpret_cast<X8*>(at) = p0;
          *reinterpret_cast<X8*>(at + 8) = p1;
          *reinterpret_cast<X8*>(at + 16) = p2;
          *reinterpret_cast<X8*>(at + 24) = p3;
        }
      }
#pragma unroll
      for (int u = 0; u < (PERM ? 0 : KU); u += 2) {
        X8 pa = raw_to_op<T, OT>(rk_[u], kss, want_ss), pb = raw_to_op<T, OT>(rk_[u + 1], kss, want_ss);
        if constexpr (!SCALED) {
          if constexpr (SWZ) op_swizzle16<OT>(pa, pb);
          *reinterpret_cast<X8*>(&tl.k[srow * SK + spart * (KT / 2) + 8 * u]) = pa;
          *reinterpret_cast<X8*>(&tl.k[srow * SK + spart * (KT / 2) + 8 * u + 8]) = pb;
        }
      }
#pragma unroll
      for (int u = 0; u < VU; ++u) {
        float unused = 0.0f;
        *reinterpret_cast<X8*>(&tl.v[srow * SV + spart * (VT / 2) + 8 * u]) =
            raw_to_op<T, OT>(rv_[u], unused, false);
      }
    };
    // per-token factors of chunk c (gate, beta, norms) into tile set par
    auto stage_factors = [&](int c, int par, const typename Raw8<T>::type* rk_) {
      const GdrTilesT<OT> tl = tiles(par);
      // in-chunk cumulative log-decay in units of log 2 (exp2 is a single instruction) and beta, lane = token; both
      // come ready from the chunk's record (zero decay increment and zero beta past the end of a partial chunk)
      const float bv = rb, gv = rg;
      const float g_last = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gv), 63));
      const float kss2 = kss + dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, kss);
      // the thread that owns row srow derives that token's factors (gamma / beta of the row sit in lane srow)
      grow = __shfl(gv, srow);
      const float brow = __shfl(bv, srow);
      const float rk = l2_factor(kss2, l2norm);
      const float ekr = __builtin_amdgcn_exp2f(grow) * rk, dkr = safe_exp2(g_last - grow) * rk;
      if constexpr (PASS_B && OWN_Q) {  // (the 128-wide heads have no registers to spare for a second form)
        // Gating of P in factored form, e^{gamma_i - gamma_j} = E_i / E_j with E = 2^(gamma - gamma_last / 2): one exp2
        // per token instead of one per element. Allowed while no exponent can leave the fp32 range (the chunk's total
        // decay above 2^-120) and no log-decay of the chunk is positive (the cumulative sums never rise); otherwise
        // every ratio goes through safe_exp2 one by one. Lanes past the end of a partial chunk repeat the last sum.
        const float gprev = __shfl_up(gv, 1);
        pfast = !__ballot(lane > 0 && gv > gprev) && !__ballot(gv > 0.0f) && g_last > -120.0f;
        ghalf = 0.5f * g_last;
      }
      if (spart == 0) {
        tl.beta[srow] = brow;
        tl.ek[srow] = ekr;
        tl.dk[srow] = dkr;
        tl.gamma[srow] = grow;
        tl.rk[srow] = (PASS_B && pfast) ? rk * __builtin_amdgcn_exp2f(ghalf - grow) : rk;  // column factor of P
        if (srow == 0) {
          tl.misc[0] = __builtin_amdgcn_exp2f(g_last);
          tl.misc[1] = (PASS_B && pfast) ? 1.0f : 0.0f;
          tl.misc[2] = ghalf;
        }
      }
      if constexpr (SCALED) {  // the two scaled k tiles, from the raw row that is still in registers
#pragma unroll
        for (int u = 0; u < KU; u += 2) {
          X8 pe[2], pd[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const typename Raw8<T>::type piece = rk_[u + h];  // (dead rows were zeroed by stage_data)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float f = (float)piece[e];
              pe[h][e] = (OT)(f * ekr);
              pd[h][e] = (OT)(f * dkr);
            }
          }
          if constexpr (SWZ) { op_swizzle16<OT>(pe[0], pe[1]); op_swizzle16<OT>(pd[0], pd[1]); }
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            *reinterpret_cast<X8*>(&tl.k[srow * SK + spart * (KT / 2) + 8 * (u + h)]) = pe[h];
            *reinterpret_cast<X8*>(&tl.kd[srow * SK + spart * (KT / 2) + 8 * (u + h)]) = pd[h];
          }
        }
      }
    };
    auto stage_q = [&](int len, typename Raw8<T>::type* rq_, int par = 0) {
      GDR_Q_BUFFERS(par);
      if constexpr (P16) {  // the factors of this chunk were derived by the other pair of stagers
        const GdrTilesT<OT> tl = tiles(par);
        grow = tl.gamma[srow];
        pfast = tl.misc[1] != 0.0f;
        ghalf = tl.misc[2];
      }
      zero_dead_rows(len, rq_, KU);
      float qss = 0.0f;
      if constexpr (PERM) {
#pragma unroll
        for (int u = 0; u < KU; u += 4) {
          X8 p0 = raw_to_op<T, OT>(rq_[u], qss, want_ss), p1 = raw_to_op<T, OT>(rq_[u + 1], qss, want_ss);
          X8 p2 = raw_to_op<T, OT>(rq_[u + 2], qss, want_ss), p3 = raw_to_op<T, OT>(rq_[u + 3], qss, want_ss);
          op_perm32<OT>(p0, p1, p2, p3);
          OT* at = &s_q[srow * SK + spart * (KT / 2) + 8 * u];
          *reinterpret_cast<X8*>(at) = p0;
          *reinterpret_cast<X8*>(at + 8) = p1;
          *reinterpret_cast<X8*>(at + 16) = p2;
          *reinterpret_cast<X8*>(at + 24) = p3;
        }
      }
#pragma unroll
      for (int u = 0; u < (PERM ? 0 : KU); u += 2) {
        X8 pa = raw_to_op<T, OT>(rq_[u], qss, want_ss), pb = raw_to_op<T, OT>(rq_[u + 1], qss, want_ss);
        if constexpr (SWZ) op_swizzle16<OT>(pa, pb);
        *reinterpret_cast<X8*>(&s_q[srow * SK + spart * (KT / 2) + 8 * u]) = pa;
        *reinterpret_cast<X8*>(&s_q[srow * SK + spart * (KT / 2) + 8 * u + 8]) = pb;
      }
      qss += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, qss);
      if (spart == 0) {
        const float rq = l2_factor(qss, l2norm);
        s_qs[srow] = scale * __builtin_amdgcn_exp2f(grow) * rq;
        s_rq[srow] = pfast ? rq * __builtin_amdgcn_exp2f(grow - ghalf) : rq;  // row factor of P (without scale)
      }
    };

    auto build_p = [&](int par) {
      if constexpr (PASS_B) {
        GDR_Q_BUFFERS(par);
        const GdrTilesT<OT> tl = tiles(par);
        // P^T tiles (0,0), (0,1), (1,1) -> P fragments; tile (1,0) is zero. Stager 0 takes tile 0, stager 1 tile 2,
        // and they share tile 1: both run its four MFMAs, each finishes and stores one of its two fragments.
        const bool fast = OWN_Q && uniform(__float_as_int(tl.misc[1])) != 0;
        auto p_tile = [&](int t, int half) {  // half: -1 = whole tile, 0 / 1 = accumulator registers 0-7 / 8-15
          const int jm = t == 2 ? 1 : 0, tn = t == 0 ? 0 : 1;
          X8 fa[KT / 16], fb[KT / 16];
#pragma unroll
          for (int ks = 0; ks < KT / 16; ++ks) {
            fa[ks] = *reinterpret_cast<const X8*>(&tl.k[(32 * jm + ln) * SK + 16 * ks + 8 * hh]);
            fb[ks] = *reinterpret_cast<const X8*>(&s_q[(32 * tn + ln) * SK + 16 * ks + 8 * hh]);
          }
          f32x4 gj[4], rj[4];  // gamma_j (slow path only) and the column factor of this lane's 16 accumulator rows
#pragma unroll
          for (int b4 = 0; b4 < 4; ++b4) {
            if (!fast) gj[b4] = *reinterpret_cast<const f32x4*>(&tl.gamma[32 * jm + 8 * b4 + 4 * hh]);
            rj[b4] = *reinterpret_cast<const f32x4*>(&tl.rk[32 * jm + 8 * b4 + 4 * hh]);
          }
          const int i = 32 * tn + ln;
          const float gi = fast ? 0.0f : tl.gamma[i], fi = scale * s_rq[i];
          lds_fence();
          f32x16 acc = zero16();
#pragma unroll
          for (int ks = 0; ks < KT / 16; ++ks) acc = mfma32(fa[ks], fb[ks], acc);
          if constexpr (P16) {
            // Narrow chain waves read P as the B operand of the 16x16x32 shape: lane 16 g + i' of fragment (tt, ts)
            // holds P[token 16 tt + i'][32 ts + 4 g .. + 3 and 32 ts + 16 + 4 g .. + 3]. Of this tile (columns = tokens
            // 32 tn + ln, rows j = 32 jm + 8 b + 4 hh + e in register 4 b + e) a lane therefore holds two pieces:
            // registers {0-3, 8-11} for g = hh and {4-7, 12-15} for g = hh + 2, both of fragment (2 tn + ln / 16, jm).
            const int tt = 2 * tn + (ln >> 4), f16 = tt < 2 ? tt : 2 + 2 * (tt - 2) + jm;
#pragma unroll
            for (int pc = 0; pc < 2; ++pc) {
              if (half >= 0 && half != pc) continue;
              X8 piece;
              if (fast) {  // (one branch per piece, not per element)
#pragma unroll
                for (int x = 0; x < 8; ++x) {
                  const int r = (x < 4 ? 0 : 8) + 4 * pc + (x & 3);
                  const float t = acc[r] * (fi * rj[r / 4][r % 4]);
                  piece[x] = (OT)((jm != tn || ln >= acc_row(r, hh)) ? t : 0.0f);
                }
              } else {
#pragma unroll
                for (int x = 0; x < 8; ++x) {
                  const int r = (x < 4 ? 0 : 8) + 4 * pc + (x & 3);
                  const int j = 32 * jm + acc_row(r, hh);
                  piece[x] = (OT)(acc[r] * (fi * rj[r / 4][r % 4] * safe_exp2(i >= j ? gi - gj[r / 4][r % 4] : 1.0f)));
                }
              }
              op_frag_store<OT>(s_P, f16, 16 * (hh + 2 * pc) + (ln & 15), piece);
            }
            return;
          }
          const int f0 = tn == 0 ? 0 : 2 + 2 * jm;  // fragments: tm=0 -> 0,1 ; tm=1 -> 2..5
#pragma unroll
          for (int part = 0; part < 2; ++part) {
            if (half >= 0 && half != part) continue;
            if (fast) {
#pragma unroll
              for (int r = 8 * part; r < 8 * part + 8; ++r) {
                const float val = acc[r] * (fi * rj[r / 4][r % 4]);
                acc[r] = (jm != tn || ln >= acc_row(r, hh)) ? val : 0.0f;  // (the tile below the diagonal is full)
              }
            } else {
#pragma unroll
              for (int r = 8 * part; r < 8 * part + 8; ++r) {  // the mask goes on the exponent: branch-free
                const int j = 32 * jm + acc_row(r, hh);
                acc[r] *= fi * rj[r / 4][r % 4] * safe_exp2(i >= j ? gi - gj[r / 4][r % 4] : 1.0f);
              }
            }
            op_frag_store<OT>(s_P, f0 + part, lane, acc_to_op<OT>(acc, 8 * part));
          }
        };
        if constexpr (P16 && KT <= 64) {
          // Narrow form (the P builders are on the critical path there): one batch of operand reads for all tiles of the
          // wave -- stager 1's two tiles share their q rows --, the tiles' MFMA chains interleaved, the column factors
          // requested behind the MFMAs. Fragment layout as in p_tile.
          const int tn = sw;
          const int i = 32 * tn + ln;
          X8 fb[KT / 16], fa0[KT / 16], fa1[KT / 16];
#pragma unroll
          for (int ks = 0; ks < KT / 16; ++ks) {
            fb[ks] = *reinterpret_cast<const X8*>(&s_q[(32 * tn + ln) * SK + 16 * ks + 8 * hh]);
            fa0[ks] = *reinterpret_cast<const X8*>(&tl.k[ln * SK + 16 * ks + 8 * hh]);
            if (sw == 1) fa1[ks] = *reinterpret_cast<const X8*>(&tl.k[(32 + ln) * SK + 16 * ks + 8 * hh]);
          }
          const float gi = fast ? 0.0f : tl.gamma[i], fi = scale * s_rq[i];
          lds_fence();
          f32x16 acc0 = zero16(), acc1 = zero16();
#pragma unroll
          for (int ks = 0; ks < KT / 16; ++ks) {
            acc0 = mfma32(fa0[ks], fb[ks], acc0);
            if (sw == 1) acc1 = mfma32(fa1[ks], fb[ks], acc1);
          }
          asm volatile("" ::: "memory");
          auto finish = [&](const f32x16& acc, int jm) __attribute__((always_inline)) {
            f32x4 gj[4], rj[4];
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
              if (!fast) gj[b4] = *reinterpret_cast<const f32x4*>(&tl.gamma[32 * jm + 8 * b4 + 4 * hh]);
              rj[b4] = *reinterpret_cast<const f32x4*>(&tl.rk[32 * jm + 8 * b4 + 4 * hh]);
            }
            const int tt = 2 * tn + (ln >> 4), f16 = tt < 2 ? tt : 2 + 2 * (tt - 2) + jm;
            f32x16 val;
            if (fast) {  // (one branch for the tile: inside the element loop it becomes a branch per element)
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const float t = acc[r] * (fi * rj[r / 4][r % 4]);
                val[r] = (jm != tn || ln >= acc_row(r, hh)) ? t : 0.0f;
              }
            } else {
#pragma unroll
              for (int r = 0; r < 16; ++r) {
                const int j = 32 * jm + acc_row(r, hh);
                val[r] = acc[r] * (fi * rj[r / 4][r % 4] * safe_exp2(i >= j ? gi - gj[r / 4][r % 4] : 1.0f));
              }
            }
#pragma unroll
            for (int pc = 0; pc < 2; ++pc) {
              X8 piece;
#pragma unroll
              for (int x = 0; x < 8; ++x) piece[x] = (OT)val[(x < 4 ? 0 : 8) + 4 * pc + (x & 3)];
              op_frag_store<OT>(s_P, f16, 16 * (hh + 2 * pc) + (ln & 15), piece);
            }
          };
          finish(acc0, 0);
          if (sw == 1) finish(acc1, 1);
          return;
        }
        // P^T tiles (0,0), (0,1), (1,1) -> P fragments; tile (1,0) is zero.
        if constexpr (OWN_Q) {  // a stager builds the tiles whose q rows it staged itself
          if (sw == 0) p_tile(0, -1);
          else { p_tile(1, -1); p_tile(2, -1); }
        } else {                // stager 0 takes tile 0, stager 1 tile 2, and they share tile 1: both run its MFMAs,
          p_tile(sw == 0 ? 0 : 2, -1);  // each finishes and stores one of its two fragments
          p_tile(1, sw);
        }
      }
    };
    // Chunk indices past the end of the segment are clamped (the last chunk is fetched again for nothing), so that
    // every iteration issues the same loads: with conditional issues the compiler could not count the loads in
    // flight any more and would drain the queue at every wait. q(c) / q(c+2) share a register set.
    const int cl = c1 - 1;
    if constexpr (P16) {
      if (nc > 0) {
        const int ca = uniform(c0), cb = uniform(min(c0 + 1, cl)), cc = uniform(min(c0 + 2, cl));
        const int tk0 = chunk_tok0[ca], ln0 = chunk_len[ca], tk1 = chunk_tok0[cb], ln1 = chunk_len[cb];
        int ln_c = ln0, ln_c1 = ln1, tk_c1 = tk1, tk_c2 = chunk_tok0[cc], ln_c2 = chunk_len[cc];
        if (spair == 0) {
          // ---- k, v, T and the factors: tiles and factors (c + 1) are staged and the loads (c + 2) issued before B(c)
          issue_tiles(c0, tk0, ln0, rk0_);
          issue_gb(c0);
          stage_data(ln0, 0, rk0_);
          stage_factors(c0, 0, rk0_);
          issue_tiles(min(c0 + 1, cl), tk1, ln1, rk0_);
          issue_gb(min(c0 + 1, cl));
          lds_barrier();  // tiles (c0) are ready
          for (int c = c0; c < c1; ++c) {
            const int par = (c - c0) & 1;
            const int cn = uniform(min(c + 3, cl));
            const int tk_n = chunk_tok0[cn], ln_n = chunk_len[cn];
            if constexpr (!OWN_Q) lds_barrier();  // Qb(c) (this pair only takes part)
            if (c + 1 < c1) {
              stage_data(ln_c1, par ^ 1, rk0_);
              stage_factors(c + 1, par ^ 1, rk0_);  // (that set's factor rows are free since B(c - 1))
            }
            issue_tiles(min(c + 2, cl), tk_c2, ln_c2, rk0_);
            issue_gb(min(c + 2, cl));
            lds_barrier();  // B(c)
            lds_barrier();  // C(c)
            ln_c = ln_c1; ln_c1 = ln_c2; tk_c2 = tk_n; ln_c2 = ln_n;
          }
        } else {
          // ---- q and P: q(c) staged and P(c) built before B(c) (from the k tile and the factors of chunk c, complete
          //      since C(c - 1)); the loads of q(c + 1) follow the staging of q(c) into the same registers
          issue_q(tk0, ln0, rq0_);
          lds_barrier();  // tiles (c0) are ready
          if constexpr (DBQ) {
            // q and P exist twice: q(c + 1) is staged between B(c) and C(c) (its factors are complete at B(c), its buffer
            // free since C(c - 1)), P(c + 1) is built after C(c) -- so only the P products sit between C(c) and B(c + 1)
            stage_q(ln_c, rq0_, 0);
            issue_q(tk_c1, ln_c1, rq0_);
            lds_fence();
            build_p(0);
            for (int c = c0; c < c1; ++c) {
              const int par = (c - c0) & 1;
              const int cn = uniform(min(c + 3, cl));
              const int tk_n = chunk_tok0[cn], ln_n = chunk_len[cn];
              lds_barrier();  // B(c)
              if (c + 1 < c1) {
                stage_q(ln_c1, rq0_, par ^ 1);
                issue_q(tk_c2, ln_c2, rq0_);
              }
              lds_barrier();  // C(c)
              if (c + 1 < c1) build_p(par ^ 1);
              ln_c = ln_c1; tk_c1 = tk_c2; ln_c1 = ln_c2; tk_c2 = tk_n; ln_c2 = ln_n;
            }
          } else
          for (int c = c0; c < c1; ++c) {
            const int par = (c - c0) & 1;
            const int cn = uniform(min(c + 3, cl));
            const int tk_n = chunk_tok0[cn], ln_n = chunk_len[cn];
            stage_q(ln_c, rq0_, par);
            issue_q(tk_c1, ln_c1, rq0_);
            if constexpr (OWN_Q) lds_fence();  // this wave's own q rows are in LDS (it builds P from no others)
            else lds_barrier();                // Qb(c)
            build_p(par);
            lds_barrier();  // B(c)
            lds_barrier();  // C(c)
            ln_c = ln_c1; tk_c1 = tk_c2; ln_c1 = ln_c2; tk_c2 = tk_n; ln_c2 = ln_n;
          }
        }
        lds_barrier();  // the o tile of the last chunk is complete (the chain waves' last flush)
      }
      return;
    }
    if (nc > 0) {
      typename Raw8<T>::type* const rkA = rk0_;
      typename Raw8<T>::type* const rkB = SCALED ? rk1_ : rk0_;
      // the chunks' table entries live in scalar registers and are fetched a chunk period before their first use
      const int ca = uniform(c0), cb = uniform(min(c0 + 1, cl)), cc = uniform(min(c0 + 2, cl));
      const int tk0 = chunk_tok0[ca], ln0 = chunk_len[ca], tk1 = chunk_tok0[cb], ln1 = chunk_len[cb];
      int ln_c = ln0, ln_c1 = ln1, tk_c2 = chunk_tok0[cc], ln_c2 = chunk_len[cc];  // of chunks c, c + 1, c + 2 (clamped)
      int tk_c = tk0, tk_c1 = tk1, tk_p = 0, ln_p = 0;                              // (tk_p, ln_p: of chunk c - 1)
      // the o tile (rows of chunk `tok0`) -> HBM, 16-byte pieces, whole rows (non-temporal: o is not read again here)
      auto stager_flush = [&](int tok0, int len) __attribute__((always_inline)) {
        constexpr int PPR = VT / 8, NP = 64 * PPR / 128;
        T* ob = o + ((size_t)tok0 * HV + hv) * VT;
        uint4 val[NP];
#pragma unroll
        for (int j = 0; j < NP; ++j) {
          const int x = stid + 128 * j;
          val[j] = *reinterpret_cast<const uint4*>(&s_o[(x / PPR) * SV + 8 * (x % PPR)]);
        }
#pragma unroll
        for (int j = 0; j < NP; ++j) {
          const int x = stid + 128 * j, row = x / PPR, part = x % PPR;
          typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4)));
          nt_u32x4 nv;
          nv[0] = val[j].x; nv[1] = val[j].y; nv[2] = val[j].z; nv[3] = val[j].w;
          if (row < len)
            __builtin_nontemporal_store(nv, reinterpret_cast<nt_u32x4*>(ob + (unsigned)(row * (HV * VT) + 8 * part)));
        }
      };
      issue_tiles(c0, tk0, ln0, rkA);
      issue_gb(c0);
      if constexpr (PASS_B) { issue_q(tk0, ln0, rq0_); issue_q(tk1, ln1, rq1_); }
      stage_data(ln0, 0, rkA);
      stage_factors(c0, 0, rkA);
      issue_tiles(min(c0 + 1, cl), tk1, ln1, rkB);
      issue_gb(min(c0 + 1, cl));
      lds_barrier();  // tiles (c0) are ready
      // rk_next holds the raw k rows of chunk c + 1, rk_free is loaded with those of chunk c + 2
      auto one_chunk = [&](int c, int par, typename Raw8<T>::type* rq_, typename Raw8<T>::type* rk_next,
                           typename Raw8<T>::type* rk_free) {
        const int cn = uniform(min(c + 3, cl));
        const int tk_n = chunk_tok0[cn], ln_n = chunk_len[cn];  // used from the next chunk on
        if (c + 1 < c1) stage_data(ln_c1, par ^ 1, rk_next);
        issue_tiles(min(c + 2, cl), tk_c2, ln_c2, rk_free);
        if constexpr (PASS_B) {
          stage_q(ln_c, rq_);
          issue_q(tk_c2, ln_c2, rq_);
          if constexpr (OWN_Q) lds_fence();  // this wave's own q rows are in LDS (it builds P from no others)
          else lds_barrier();                // Qb(c)
          build_p(par);
          lds_barrier();  // B(c)
          if constexpr (STAGER_FLUSH) {
            if (c > c0) stager_flush(tk_p, ln_p);  // o(c - 1): written after C(c - 1), next written after C(c)
          }
          if (c + 1 < c1) stage_factors(c + 1, par ^ 1, rk_next);
          issue_gb(min(c + 2, cl));
          lds_barrier();  // C(c)
        } else {
          if (c + 1 < c1) stage_factors(c + 1, par ^ 1, rk_next);
          issue_gb(min(c + 2, cl));
          lds_barrier();  // B(c)
        }
        tk_p = tk_c; ln_p = ln_c; tk_c = tk_c1; tk_c1 = tk_c2;
        ln_c = ln_c1; ln_c1 = ln_c2; tk_c2 = tk_n; ln_c2 = ln_n;
      };
      for (int c = c0; c < c1; c += 2) {
        one_chunk(c, 0, rq0_, rkB, rkA);
        if (c + 1 < c1) one_chunk(c + 1, 1, rq1_, rkA, rkB);
      }
      if constexpr (STAGER_FLUSH) {
        lds_barrier();  // the o tile of the last chunk is complete
        stager_flush(tk_p, ln_p);
      }
    }
    return;
  }

  if constexpr (CW == 16) {
    // ============================================ narrow chain wave ============================================
    // Wave w owns the 16 value columns 16 w .. + 15 and all K rows of them: S as K / 16 accumulator tiles of the
    // 16x16x32 shape (lane 16 g + i: rows 16 km + 4 g + r, column i). Same stages and barriers as the 32-column chain
    // wave below; every operand fragment from memory is one 16-byte LDS read (tiles in op_perm32 order).
    constexpr int NKM = KT / 16, NKS = KT / 32, NF = 4 * NKS;  // state tiles, contraction steps over K, k / q fragments
    const int g4 = lane >> 4, li = lane & 15;
    const int col = 16 * wave + li;
    f32x4 S[NKM];
    // where this lane's part of a state tile sits in the 32-column accumulator order the scan kernels use: tile
    // (column slab wave / 2, row block km / 2), plane 2 (km % 2) + g / 2, lane 32 (g % 2) + 16 (wave % 2) + i
    const int lane32 = 32 * (g4 & 1) + 16 * (wave & 1) + li;
    auto slab_piece = [&](int km) { return ((km >> 1) * 4 + 2 * (km & 1) + (g4 >> 1)) * 64 + lane32; };
    bool walked = false;
    if constexpr (KT == 64) if (gmax > 0) {
      walked = true;
      // second level of the two-level scan (see the 32-column chain wave): the composites of the groups before this
      // segment's group, then of the segments before it inside its group
      constexpr int M_BYTES = KT * KT * 2, N_BYTES = KT * 32 * 4;
      const int seq = pv.seg_seq[seg], local = seg - pv.seq_seg0[seq];
      const int lead = local / GDR_SCAN_GROUP, nst = lead + local % GDR_SCAN_GROUP;
      const int item0 = seg - local % GDR_SCAN_GROUP;
#pragma unroll
      for (int km = 0; km < NKM; ++km)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          S[km][r] = h0 ? h0[(((size_t)seq * HV + hv) * KT + 16 * km + 4 * g4 + r) * VT + col] : 0.0f;
      X8 rm[2][NKM * NKS];
      f32x4 rn[2][NKM];
      float rd[2];
      // M' is stored as A-operand fragments of the 32x32x16 shape: element (row, c) in fragment (row / 32, c / 16), lane
      // 32 ((c % 16 / 4) & 1) + row % 32, slot 4 (c % 16 / 8) + c % 4. This lane's share of the step ks (columns
      // 32 ks + 4 g .. and 32 ks + 16 + 4 g ..) of rows 16 km + i: the 8-byte half g / 2 of lane 32 (g % 2) + (16 km + i) % 32
      // in the fragments (km / 2, 2 ks) and (km / 2, 2 ks + 1).
      auto issue = [&](int p, X8* m, f32x4* n, float& d) __attribute__((always_inline)) {
        p = uniform(max(0, min(p, nst - 1)));
        const bool top = p < lead;
        const size_t sh = (size_t)(top ? seq * gmax + p : item0 + (p - lead)) * HV + hv;
        const unsigned char* M = (top ? Mgrp : Mcomp) + sh * M_BYTES;
        const f32x4* N = reinterpret_cast<const f32x4*>((top ? Ngrp : Ncomp) + (sh * (VT / 32) + (wave >> 1)) * N_BYTES);
#pragma unroll
        for (int km = 0; km < NKM; ++km)
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const int l32 = 32 * (g4 & 1) + 16 * (km & 1) + li;
            const unsigned char* f = M + ((size_t)((km >> 1) * (KT / 16) + 2 * ks) * 64 + l32) * 16 + 8 * (g4 >> 1);
            const X4 lo = *reinterpret_cast<const X4*>(f), hi = *reinterpret_cast<const X4*>(f + 1024);
            X8 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
            m[km * NKS + ks] = v;
          }
#pragma unroll
        for (int km = 0; km < NKM; ++km) n[km] = N[slab_piece(km)];
        d = (top ? Dgrp : Dcomp)[sh];
      };
      auto step = [&](const X8* m, const f32x4* n, float d) __attribute__((always_inline)) {
        X8 Sb[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) Sb[ks] = acc2_to_op<OT>(S[2 * ks], S[2 * ks + 1]);
#pragma unroll
        for (int km = 0; km < NKM; ++km) {
          f32x4 acc;
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] = __builtin_fmaf(d, S[km][e], n[km][e]);
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) acc = mfma16(m[km * NKS + ks], Sb[ks], acc);
          S[km] = acc;
        }
      };
      if (nst > 0) {
        issue(0, rm[0], rn[0], rd[0]);
        issue(1, rm[1], rn[1], rd[1]);
        for (int p = 0; p < nst; p += 2) {
          step(rm[0], rn[0], rd[0]);
          issue(p + 2, rm[0], rn[0], rd[0]);
          if (p + 1 < nst) step(rm[1], rn[1], rd[1]);
          issue(p + 3, rm[1], rn[1], rd[1]);
        }
      }
    }
    if (!walked) {  // the scan leaves every segment's initial state as 32-column slabs in accumulator order
      const f32x4* si = reinterpret_cast<const f32x4*>(Sinit + (((size_t)seg * HV + hv) * (VT / 32) + (wave >> 1)) * (KT * 32));
#pragma unroll
      for (int km = 0; km < NKM; ++km) S[km] = si[slab_piece(km)];
    }

    // this wave's rows of the o tile -> HBM: 64 / NSLAB whole rows of V values, two 16-byte pieces per lane (piece
    // lane + 64 j of the wave's rows: the same part of a row 64 / PPR rows further down)
    constexpr int RW = 64 / NSLAB, PPR = VT / 8;
    const int fo_row = wave * RW + lane / PPR;
    const T* fo_lds = s_o + fo_row * SV + 8 * (lane % PPR);
    const unsigned fo_off = (unsigned)(fo_row * (HV * VT) + 8 * (lane % PPR));  // elements, from the chunk's first o row
    auto flush_o = [&](int tok0, int len) __attribute__((always_inline)) {
      T* ob = o + ((size_t)tok0 * HV + hv) * VT;  // uniform base; per-lane 32-bit offsets
      const uint4 v0 = *reinterpret_cast<const uint4*>(fo_lds);
      const uint4 v1 = *reinterpret_cast<const uint4*>(fo_lds + (64 / PPR) * SV);
      // (o is written once and not read again by this pipeline: non-temporal, see the 32-column chain wave)
      typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4)));
      nt_u32x4 n0, n1;
      n0[0] = v0.x; n0[1] = v0.y; n0[2] = v0.z; n0[3] = v0.w;
      n1[0] = v1.x; n1[1] = v1.y; n1[2] = v1.z; n1[3] = v1.w;
      if (fo_row < len) __builtin_nontemporal_store(n0, reinterpret_cast<nt_u32x4*>(ob + fo_off));
      if (fo_row + 64 / PPR < len)
        __builtin_nontemporal_store(n1, reinterpret_cast<nt_u32x4*>(ob + fo_off + (unsigned)((64 / PPR) * (HV * VT))));
    };
    // A-operand fragment of a row-major tile: row `row`, the 32-wide contraction step that starts at column c32, in
    // the slot order of the narrow shape (columns 4 g .. + 3 and 16 + 4 g .. + 3): one 16-byte piece of a tile in
    // op_perm32 order, two 8-byte pieces otherwise
    auto row_frag = [&](const OT* arr, int stride, int row, int c32) __attribute__((always_inline)) {
      if constexpr (PERM) {
        return *reinterpret_cast<const X8*>(&arr[row * stride + c32 + 8 * g4]);
      } else {
        const X4 lo = *reinterpret_cast<const X4*>(&arr[row * stride + c32 + 4 * g4]);
        const X4 hi = *reinterpret_cast<const X4*>(&arr[row * stride + c32 + 16 + 4 * g4]);
        X8 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) { out[e] = lo[e]; out[4 + e] = hi[e]; }
        return out;
      }
    };
    // T fragment (tm, ts): rows 16 tm + i of the block T11 (tm < 2) or of T21 / T22 (tm >= 2, ts = 0 / 1)
    auto t_frag = [&](const OT* tt, int tm, int ts) {
      const int blk = tm < 2 ? 0 : 1 + ts;
      return row_frag(tt, ST, blk * 32 + 16 * (tm & 1) + li, 0);
    };

    int o_tok0 = 0, o_len = 0, p_tok0 = 0, p_len = 0;  // table entries of this chunk and of the one before it
    if (nc > 0) { o_tok0 = chunk_tok0[uniform(c0)]; o_len = chunk_len[uniform(c0)]; }
    if (nc > 0) lds_barrier();  // tiles (c0) are ready
    for (int c = c0; c < c1; ++c) {
      const GdrTilesT<OT> tl = tiles((c - c0) & 1);
      GDR_Q_BUFFERS((c - c0) & 1);
      if constexpr (!OWN_Q) lds_barrier();  // Qb(c) (the chain waves only take part)
      const int c_nx = uniform(min(c + 1, c1 - 1));
      const int n_tok0 = chunk_tok0[c_nx], n_len = chunk_len[c_nx];
      // Registers: four waves share a SIMD at K = V = 64 (128 registers each), so every batch of LDS reads is requested
      // behind the MFMAs whose operands it replaces (an MFMA has read its operands once it is issued), not a stage ahead;
      // the MFMAs in flight and the epilogue arithmetic cover the reads. (The empty asm statements keep the compiler from
      // hoisting the reads back up.)
      X8 fk[NF];  // K rows (stage 1), K^T rows (stage 3), Q rows (output)
      X8 ft[6];   // T (stage 2), P (output)
#pragma unroll
      for (int tm = 0; tm < 4; ++tm)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
          fk[tm * NKS + ks] = row_frag(tl.k, SK, 16 * tm + li, 32 * ks);
      X8 Sb[NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) Sb[ks] = acc2_to_op<OT>(S[2 * ks], S[2 * ks + 1]);
      lds_fence();
      f32x4 R[4];
#pragma unroll
      for (int tm = 0; tm < 4; ++tm) {  // K S
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) acc = mfma16(fk[tm * NKS + ks], Sb[ks], acc);
        R[tm] = acc;
      }
      asm volatile("" ::: "memory");
      // the per-token factors and the v tile (in accumulator layout) of stage 1's epilogue, then the T fragments
      f32x4 be[4], ek[4];
      X4 vv[4];
#pragma unroll
      for (int tm = 0; tm < 4; ++tm) {
        be[tm] = *reinterpret_cast<const f32x4*>(&tl.beta[16 * tm + 4 * g4]);
        ek[tm] = *reinterpret_cast<const f32x4*>(&tl.ek[16 * tm + 4 * g4]);
        vv[tm] = op_lds_read_tr4<OT>(tl.v + (16 * tm + 4 * g4 + (li >> 2)) * SV + 16 * wave + 4 * (li & 3));
      }
      ft[0] = t_frag(tl.t, 0, 0); ft[1] = t_frag(tl.t, 1, 0); ft[2] = t_frag(tl.t, 2, 0);
      ft[3] = t_frag(tl.t, 2, 1); ft[4] = t_frag(tl.t, 3, 0); ft[5] = t_frag(tl.t, 3, 1);
#pragma unroll
      for (int tm = 0; tm < 4; ++tm)  // R = beta (v - ek (K S))
#pragma unroll
        for (int e = 0; e < 4; ++e) R[tm][e] = be[tm][e] * ((float)vv[tm][e] - ek[tm][e] * R[tm][e]);
      X8 Rb[2];
      Rb[0] = acc2_to_op<OT>(R[0], R[1]);
      Rb[1] = acc2_to_op<OT>(R[2], R[3]);
      f32x4 Vn[4];
#pragma unroll
      for (int tm = 0; tm < 4; ++tm) {  // v_new = T R (T is lower triangular: rows 32 .. 63 need both steps)
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        acc = mfma16(ft[tm < 2 ? tm : 2 * tm - 2], Rb[0], acc);
        if (tm >= 2) acc = mfma16(ft[2 * tm - 1], Rb[1], acc);
        Vn[tm] = acc;
      }
      asm volatile("" ::: "memory");
      // K^T fragments (transposing reads of the row-major k tile) and the decay factors of the state update
#pragma unroll
      for (int km = 0; km < NKM; ++km)
#pragma unroll
        for (int ts = 0; ts < 2; ++ts) fk[km * 2 + ts] = op_ld_tr16<OT, PERM>(tl.k, SK, 16 * km, 32 * ts, lane);
      f32x4 dk[4];
#pragma unroll
      for (int tm = 0; tm < 4; ++tm) dk[tm] = *reinterpret_cast<const f32x4*>(&tl.dk[16 * tm + 4 * g4]);
      const float dec = tl.misc[0];
      X8 Vb[2], Vsb[2];
#pragma unroll
      for (int ts = 0; ts < 2; ++ts) {
        Vb[ts] = acc2_to_op<OT>(Vn[2 * ts], Vn[2 * ts + 1]);
        f32x4 a = Vn[2 * ts], b = Vn[2 * ts + 1];
#pragma unroll
        for (int e = 0; e < 4; ++e) { a[e] *= dk[2 * ts][e]; b[e] *= dk[2 * ts + 1][e]; }
        Vsb[ts] = acc2_to_op<OT>(a, b);
      }
      lds_fence();
      lds_barrier();  // B(c): every operand that comes from the k, v and T tiles of chunk c is in registers; the o
                      // tile of chunk c - 1 is complete
#pragma unroll
      for (int km = 0; km < NKM; ++km) {  // S <- dec S + K^T (dk v_new)
#pragma unroll
        for (int e = 0; e < 4; ++e) S[km][e] *= dec;
#pragma unroll
        for (int ts = 0; ts < 2; ++ts) S[km] = mfma16(fk[km * 2 + ts], Vsb[ts], S[km]);
      }
      asm volatile("" ::: "memory");
      if (c > c0) flush_o(p_tok0, p_len);  // (behind the MFMAs of the state update, where few registers are live)
      asm volatile("" ::: "memory");
      // Q rows, P fragments, output factors
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
          fk[tt * NKS + ks] = row_frag(s_q, SK, 16 * tt + li, 32 * ks);
#pragma unroll
      for (int f = 0; f < 6; ++f) ft[f] = op_frag_load<OT>(s_P, f, lane);
      float qsv[4];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) qsv[tt] = s_qs[16 * tt + li];  // scale e^{gamma} rq of this lane's token per row tile
      lds_fence();
      lds_barrier();  // C(c): the q and P operands of chunk c are in registers, the o tile of chunk c - 1 has been read
      // o^T = S_old^T (qs Q)^T + v_new^T P^T (computed transposed: the lane holds a token and four value columns, see
      // the 32-column chain wave): tile tt = tokens 16 tt .. + 15, rows of the result = this wave's 16 value columns
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        f32x4 a1 = {0.0f, 0.0f, 0.0f, 0.0f}, a2 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) a1 = mfma16(Sb[ks], fk[tt * NKS + ks], a1);
        a2 = mfma16(Vb[0], ft[tt < 2 ? tt : 2 * tt - 2], a2);
        if (tt >= 2) a2 = mfma16(Vb[1], ft[2 * tt - 1], a2);
        typedef T T4 __attribute__((ext_vector_type(4)));
        T4 pk;
#pragma unroll
        for (int e = 0; e < 4; ++e) pk[e] = GdrElem<T>::from_float(__builtin_fmaf(qsv[tt], a1[e], a2[e]));
        *reinterpret_cast<T4*>(&s_o[(16 * tt + li) * SV + 16 * wave + 4 * g4]) = pk;
      }
      p_tok0 = o_tok0; p_len = o_len;
      o_tok0 = n_tok0; o_len = n_len;
    }
    if (nc > 0) {
      lds_barrier();  // the o tile of the last chunk is complete
      flush_o(p_tok0, p_len);
    }
    int late = 0;  // (keeps the compiler from computing these addresses before the loop)
    asm volatile("" : "+v"(late));
    if (ht && (flags & SEG_LAST)) {
      const int seq = pv.seg_seq[seg];
      float* out = ht + ((size_t)seq * HV + hv) * KT * VT + late;
#pragma unroll
      for (int km = 0; km < NKM; ++km)
#pragma unroll
        for (int r = 0; r < 4; ++r) out[(16 * km + 4 * g4 + r) * VT + col] = S[km][r];
    }
    return;
  } else {

  // ================================================== chain ==================================================
  // this wave's 32 columns: PASS_B value columns; PASS_A columns of [M | N]
  const bool is_m = !PASS_B && wave < KT / 32;
  const int vslab = PASS_B ? wave : (is_m ? 0 : wave - KT / 32);
  const int col = 32 * vslab + ln;  // value column (unused for M slabs)
  const float vmask = is_m ? 0.0f : 1.0f;

  f32x16 S[KT / 32];
  bool walked = false;
  if constexpr (PASS_B && KT == 64) if (gmax > 0) {
    walked = true;
    // Two-level scan, second level done here: the state this segment starts from = the sequence's initial state
    // pushed through the composites of the groups before this segment's group (Mgrp / Ngrp / Dgrp, written by the
    // group pass) and then through the composites of the segments before it inside its group (at most
    // 2 (GDR_SCAN_GROUP - 1) steps S <- d S + N + M' S). This wave owns all rows of its 32 columns, so the state
    // feeds the next step's B operand straight from the accumulators.
    constexpr int NKS = KT / 16, NKM = KT / 32;
    constexpr int M_BYTES = KT * KT * 2, N_BYTES = KT * 32 * 4;
    const int seq = pv.seg_seq[seg], local = seg - pv.seq_seg0[seq];
    const int lead = local / GDR_SCAN_GROUP, nst = lead + local % GDR_SCAN_GROUP;
    const int item0 = seg - local % GDR_SCAN_GROUP;
#pragma unroll
    for (int km = 0; km < NKM; ++km)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        S[km][r] = h0 ? h0[(((size_t)seq * HV + hv) * KT + 32 * km + acc_row(r, hh)) * VT + col] : 0.0f;
    X8 rm[2][NKM * NKS];
    f32x4 rn[2][NKM * 4];
    float rd[2];
    auto issue = [&](int p, X8* m, f32x4* n, float& d) __attribute__((always_inline)) {
      p = uniform(max(0, min(p, nst - 1)));
      const bool top = p < lead;
      const size_t sh = (size_t)(top ? seq * gmax + p : item0 + (p - lead)) * HV + hv;
      const X8* M = reinterpret_cast<const X8*>((top ? Mgrp : Mcomp) + sh * M_BYTES);
      const f32x4* N = reinterpret_cast<const f32x4*>((top ? Ngrp : Ncomp) + (sh * (VT / 32) + vslab) * N_BYTES);
#pragma unroll
      for (int f = 0; f < NKM * NKS; ++f) m[f] = M[f * 64 + lane];
#pragma unroll
      for (int f = 0; f < NKM * 4; ++f) n[f] = N[f * 64 + lane];
      d = (top ? Dgrp : Dcomp)[sh];
    };
    auto step = [&](const X8* m, const f32x4* n, float d) __attribute__((always_inline)) {
      X8 Sb[NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) Sb[ks] = acc_to_op<OT>(S[ks / 2], 8 * (ks % 2));
#pragma unroll
      for (int km = 0; km < NKM; ++km) {
        f32x16 acc;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[4 * q4 + e] = __builtin_fmaf(d, S[km][4 * q4 + e], n[km * 4 + q4][e]);
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) acc = mfma32(m[km * NKS + ks], Sb[ks], acc);
        S[km] = acc;
      }
    };
    if (nst > 0) {
      issue(0, rm[0], rn[0], rd[0]);
      issue(1, rm[1], rn[1], rd[1]);
      for (int p = 0; p < nst; p += 2) {
        step(rm[0], rn[0], rd[0]);
        issue(p + 2, rm[0], rn[0], rd[0]);
        if (p + 1 < nst) step(rm[1], rn[1], rd[1]);
        issue(p + 3, rm[1], rn[1], rd[1]);
      }
    }
  }
  if (walked) {
  } else if (PASS_B) {  // the scan leaves every segment's initial state as 32-column slabs in accumulator order
    const f32x4* si = reinterpret_cast<const f32x4*>(Sinit + (((size_t)seg * HV + hv) * (VT / 32) + vslab) * (KT * 32));
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 t = si[(km * 4 + q4) * 64 + lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) S[km][4 * q4 + e] = t[e];
      }
  } else {
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int r = 0; r < 16; ++r) S[km][r] = (is_m && 32 * km + acc_row(r, hh) == 32 * wave + ln) ? 1.0f : 0.0f;
  }

  GDR_Q_BUFFERS(0);
  float dtot = 1.0f;  // product of the chunks' decays over the segment (PASS_A)
  // The LDS operand reads of a stage are issued as one batch one stage ahead of the MFMAs that use them
  // (lds_fence() pins that order); left alone the compiler fetches each fragment right before its MFMA and
  // pays the LDS latency once per MFMA.
  // The q rows and the P fragments of the output are requested right after B(c), before the state update's MFMAs,
  // where the registers allow a second set of fragments (K = 64 and below).
  constexpr bool EARLY_Q = PASS_B && KT <= 64;
  int o_tok0 = 0, o_len = 0;  // table entries of the chunk whose o rows are stored, fetched a chunk ahead
  if (PASS_B && nc > 0) { o_tok0 = chunk_tok0[uniform(c0)]; o_len = chunk_len[uniform(c0)]; }
  // Output pass at K <= 64: the K rows of chunk c + 1 are requested behind the barrier C(c), in front of the output's
  // MFMAs (the fragment registers are free from the state update on, and the tiles of chunk c + 1 are complete since
  // B(c)), so the next chunk does not start with an LDS round trip.
  constexpr bool EARLY_K = EARLY_Q && KT == 64;  // (the 32 x 32 form has no registers for it)
  X8 fk[2 * (KT / 16)];  // K rows (stage 1), K^T rows (stage 3), Q rows (output)
  auto load_k_rows = [&](const GdrTilesT<OT>& tx) __attribute__((always_inline)) {
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int ks = 0; ks < KT / 16; ++ks) fk[tm * (KT / 16) + ks] = SWZ ? op_ld_kappa_swz<OT>(tx.k, SK, 32 * tm + ln, 16 * ks, hh)
                                        : op_ld_kappa<OT>(tx.k, SK, 32 * tm + ln, 16 * ks, hh);
  };
  if (nc > 0) lds_barrier();  // tiles (c0) are ready
  if constexpr (EARLY_K) load_k_rows(tiles(0));
  for (int c = c0; c < c1; ++c) {
    const GdrTilesT<OT> tl = tiles((c - c0) & 1);
    if constexpr (PASS_B && !OWN_Q) lds_barrier();  // Qb(c) (the chain waves only take part)
    const int c_nx = uniform(min(c + 1, c1 - 1));
    const int n_tok0 = PASS_B ? chunk_tok0[c_nx] : 0, n_len = PASS_B ? chunk_len[c_nx] : 0;
    X8 fq[EARLY_Q ? 2 * (KT / 16) : 1];
    X8 ft[6];              // T (stage 2), P (output)
    if constexpr (!EARLY_K) load_k_rows(tl);
    X8 Sb[KT / 16];
#pragma unroll
    for (int ks = 0; ks < KT / 16; ++ks) Sb[ks] = acc_to_op<OT>(S[ks / 2], 8 * (ks % 2));
    lds_fence();
    // batch for stage 2: T fragments and the per-token factors / v tile of stage 1's epilogue
#pragma unroll
    for (int tm = 0; tm < 2; ++tm)
#pragma unroll
      for (int ks = 0; ks < 2 * (tm + 1); ++ks)  // blocks T11 | T21, T22
        ft[2 * tm + ks] = op_ld_kappa<OT>(tl.t + (tm == 0 ? 0 : (ks < 2 ? 1 : 2)) * 32 * ST, ST, ln, 16 * (ks & 1), hh);
    f32x4 be[8], ek[8];
    X4 vv[8];
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
      const int i0 = 8 * t8 + 4 * hh;
      be[t8] = *reinterpret_cast<const f32x4*>(&tl.beta[i0]);
      if constexpr (!SCALED) ek[t8] = *reinterpret_cast<const f32x4*>(&tl.ek[i0]);
      // v[8 t8 + 4 hh + e][col]. The M slabs (v = 0) issue the same transposing loads and drop the result with
      // vmask: the load must run with every lane enabled, so it is kept out of any per-wave branch.
      vv[t8] = op_ld_col4<OT>(tl.v, SV, 32 * vslab, 8 * t8, lane);
    }
    X8 Rb[4];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {  // R = beta (v - ek (K S))
      f32x16 acc = zero16();
#pragma unroll
      for (int ks = 0; ks < KT / 16; ++ks) acc = mfma32(fk[tm * (KT / 16) + ks], Sb[ks], acc);
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float ks_ = SCALED ? acc[4 * b4 + e] : ek[4 * tm + b4][e] * acc[4 * b4 + e];
          acc[4 * b4 + e] = be[4 * tm + b4][e] * (vmask * (float)vv[4 * tm + b4][e] - ks_);
        }
      Rb[2 * tm + 0] = acc_to_op<OT>(acc, 0);
      Rb[2 * tm + 1] = acc_to_op<OT>(acc, 8);
    }
    lds_fence();
    // batch for stage 3: K^T fragments (transposing reads of the row-major k tile) and the decay factors
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) fk[km * 4 + ks] = op_ld_kappa_tr<OT, SWZ>(tl.kd, SK, 32 * km, 16 * ks, lane);
    f32x4 dk[8];
    if constexpr (!SCALED) {
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) dk[t8] = *reinterpret_cast<const f32x4*>(&tl.dk[8 * t8 + 4 * hh]);
    }
    const float dec = tl.misc[0];
    X8 Vb[4], Vsb[4];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {  // v_new = T R (T is lower triangular: tile tm needs 2 (tm + 1) steps)
      f32x16 acc = zero16();
#pragma unroll
      for (int ks = 0; ks < 2 * (tm + 1); ++ks) acc = mfma32(ft[2 * tm + ks], Rb[ks], acc);
      Vb[2 * tm + 0] = acc_to_op<OT>(acc, 0);
      Vb[2 * tm + 1] = acc_to_op<OT>(acc, 8);
      if constexpr (!SCALED) {
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[4 * b4 + e] *= dk[4 * tm + b4][e];
        Vsb[2 * tm + 0] = acc_to_op<OT>(acc, 0);
        Vsb[2 * tm + 1] = acc_to_op<OT>(acc, 8);
      } else {  // (the decay factors are in the kd tile)
        Vsb[2 * tm + 0] = Vb[2 * tm + 0];
        Vsb[2 * tm + 1] = Vb[2 * tm + 1];
      }
    }
    lds_fence();
    lds_barrier();  // B(c): every operand that comes from the k, v and T tiles of chunk c is in registers
    dtot *= dec;
    float qs0 = 0.0f, qs1 = 0.0f;
    if constexpr (EARLY_Q) {  // batch: Q rows, P fragments, output factors (in flight during the state update)
#pragma unroll
      for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int ks = 0; ks < KT / 16; ++ks) fq[tm * (KT / 16) + ks] = SWZ ? op_ld_kappa_swz<OT>(s_q, SK, 32 * tm + ln, 16 * ks, hh)
                                        : op_ld_kappa<OT>(s_q, SK, 32 * tm + ln, 16 * ks, hh);
#pragma unroll
      for (int f = 0; f < 6; ++f) ft[f] = op_frag_load<OT>(s_P, f, lane);
      qs0 = s_qs[ln];
      qs1 = s_qs[32 + ln];
    }
#pragma unroll
    for (int km = 0; km < KT / 32; ++km) {  // S <- dec S + K^T (dk v_new)
#pragma unroll
      for (int r = 0; r < 16; ++r) S[km][r] *= dec;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) S[km] = mfma32(fk[km * 4 + ks], Vsb[ks], S[km]);
    }
    if constexpr (PASS_B) {
      if constexpr (!EARLY_Q) {  // batch: Q rows, P fragments, output factors
#pragma unroll
        for (int tm = 0; tm < 2; ++tm)
#pragma unroll
          for (int ks = 0; ks < KT / 16; ++ks) fk[tm * (KT / 16) + ks] = SWZ ? op_ld_kappa_swz<OT>(s_q, SK, 32 * tm + ln, 16 * ks, hh)
                                          : op_ld_kappa<OT>(s_q, SK, 32 * tm + ln, 16 * ks, hh);
#pragma unroll
        for (int f = 0; f < 6; ++f) ft[f] = op_frag_load<OT>(s_P, f, lane);
        qs0 = s_qs[ln];  // scale e^{gamma_i} rq_i of this lane's token in either row tile
        qs1 = s_qs[32 + ln];
      }
      lds_fence();
      lds_barrier();  // C(c): the q and P operands of chunk c are in registers
      if constexpr (EARLY_K) load_k_rows(tiles((c + 1 - c0) & 1));  // (after the last chunk: read and dropped)
      // o^T = S_old^T (qs Q)^T + v_new^T P^T: the state and v_new, which this wave holds in accumulator layout (lane =
      // value column), are read as the A operands (operand row = value column), the Q and P fragments as the B
      // operands (operand column = token). The result tile has the TOKEN in the lane and 16 value columns (four runs
      // of four) in the registers, so the token's factor is one scalar per lane and a run packs into one 8-byte piece
      // of the token's row without any exchange between lanes. The slab goes to this wave's own part of the o tile
      // and from there to HBM in 16-byte pieces.
#pragma unroll
      for (int tm = 0; tm < 2; ++tm) {
        f32x16 a1 = zero16(), a2 = zero16();
#pragma unroll
        for (int ks = 0; ks < KT / 16; ++ks) a1 = mfma32(Sb[ks], (EARLY_Q ? fq : fk)[tm * (KT / 16) + ks], a1);
#pragma unroll
        for (int ks = 0; ks < 2 * (tm + 1); ++ks) a2 = mfma32(Vb[ks], ft[2 * tm + ks], a2);
        const float qsv = tm ? qs1 : qs0;
        typedef T T4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          T4 pk;
#pragma unroll
          for (int e = 0; e < 4; ++e) pk[e] = GdrElem<T>::from_float(__builtin_fmaf(qsv, a1[4 * b4 + e], a2[4 * b4 + e]));
          *reinterpret_cast<T4*>(&s_o[(32 * tm + ln) * SV + 32 * vslab + 8 * b4 + 4 * hh]) = pk;
        }
      }
      if constexpr (!STAGER_FLUSH) {
        lds_fence();
        const int tok0 = o_tok0, len = o_len;
        T* ob = o + ((size_t)tok0 * HV + hv) * VT;  // uniform base; per-lane 32-bit offsets below
        const int rs = HV * VT;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int piece = lane + 64 * j, row = piece >> 2, part = piece & 3;
          const uint4 val = *reinterpret_cast<const uint4*>(&s_o[row * SV + 32 * vslab + 8 * part]);
          // o is written once and not read again by this pipeline: a non-temporal store keeps it from pushing the
          // tiles and composites out of the L2 (layer 136.6 -> 132.9 us; the same hint on the loads of q, k, v costs
          // 10 - 30 us, on the records' stores it changes nothing)
          typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4)));
          nt_u32x4 nv;
          nv[0] = val.x; nv[1] = val.y; nv[2] = val.z; nv[3] = val.w;
          if (row < len) __builtin_nontemporal_store(nv, reinterpret_cast<nt_u32x4*>(ob + row * rs + 32 * vslab + 8 * part));
        }
      }
      o_tok0 = n_tok0;
      o_len = n_len;
    }
  }

  if constexpr (STAGER_FLUSH) {
    if (nc > 0) lds_barrier();  // the o tile of the last chunk is complete (the stagers write it out)
  }
  // epilogue; the opaque zero keeps the compiler from computing all these addresses before the loop
  int late = 0;
  asm volatile("" : "+v"(late));
  if constexpr (PASS_B) {
    if (ht && (flags & SEG_LAST)) {
      const int seq = pv.seg_seq[seg];
      float* out = ht + ((size_t)seq * HV + hv) * KT * VT + late;
#pragma unroll
      for (int km = 0; km < KT / 32; ++km)
#pragma unroll
        for (int r = 0; r < 16; ++r) out[(32 * km + acc_row(r, hh)) * VT + col] = S[km][r];
    }
  } else if (is_m) {
    // M = dtot I + M': M' as bf16 A-operand fragments (rows = state rows, contraction over the columns in
    // accumulator slot order), element (row, col) -> fragment (row/32, col/16), lane 32*hh' + row%32, slot s
    unsigned char* out = Mcomp + ((size_t)seg * HV + hv) * (KT * KT * 2) + late;
    const int mcol = 32 * wave + ln, ks = mcol >> 4, c16 = mcol & 15;
    const int hs = (c16 >> 2) & 1, slot = 4 * (c16 >> 3) + (c16 & 3);
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * km + acc_row(r, hh);
        const float val = S[km][r] - (row == mcol ? dtot : 0.0f);
        *reinterpret_cast<OT*>(out + ((size_t)((km * (KT / 16) + ks) * 64 + 32 * hs + (row & 31))) * 16 + 2 * slot) =
            (OT)val;
      }
    if (wave == 0 && lane == 0) Dcomp[(size_t)seg * HV + hv] = dtot;
  } else {
    // N slab in accumulator order: tile (vslab, km), plane q (registers 4q..4q+3), lane -> 16 bytes
    unsigned char* out = Ncomp + (((size_t)seg * HV + hv) * (VT / 32) + vslab) * (KT * 32 * 4) + late;
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 t;
#pragma unroll
        for (int e = 0; e < 4; ++e) t[e] = S[km][4 * q4 + e];
        reinterpret_cast<f32x4*>(out)[(km * 4 + q4) * 64 + lane] = t;
      }
  }
  }  // (the 32-column chain wave)
#undef GDR_Q_BUFFERS
}

// ---- scan ---------------------------------------------------------------------------------------------------------
// grid (n_seq, HV, VT/32), KT/32 waves. S_{p+1} = M_p S_p + N_p over the segments of one sequence for a 32-column
// slab of the state; Sinit receives the state every segment starts from, as 32-column slabs in accumulator order
// (the layout the output pass loads with 16-byte reads).
// The composite pass stores M_p as d_p I + M'_p (d_p = the segment's total decay, exact in fp32) with M' in bf16
// MFMA A-operand fragment order and N_p in accumulator order, so a step is
//   S <- d S + N + M' S      (one MFMA per fragment; the state feeds the B operand straight from the accumulator).
// The chain is serial in p, so nothing else may sit on it. Wave w owns rows 32w .. 32w+31 of the slab: it loads
// only its own row tile of M' and N (DEPTH steps ahead, straight into registers in operand order: no staging) and
// needs the other waves' rows of the state only as B operand: every wave publishes its two operand fragments in
// LDS (double-buffered by step parity, one LDS-only barrier per step) and starts the step's MFMAs with its own
// fragments while the others' are on their way.
template <typename OT, int KT, int VT, int DEPTH>
__global__ void __launch_bounds__(64 * (KT / 32)) gdr_scan_kernel(const GdrPlanView pv,
                                                                 const unsigned char* __restrict__ Mcomp,
                                                                 const unsigned char* __restrict__ Ncomp,
                                                                 const float* __restrict__ Dcomp,
                                                                 const float* __restrict__ h0,
                                                                 float* __restrict__ Sinit, int HV, int n_segments) {
  using X8 = typename OpVec<OT>::x8;
  constexpr int NKS = KT / 16;
  constexpr int M_BYTES = KT * KT * 2, N_BYTES = KT * 32 * 4;
  __shared__ __align__(16) unsigned char s_x[2][NKS * 1024];
  // grid (n_seq, HV, VT / 32): workgroups go to the 8 XCDs round robin by their linear id, so with the column slab as the
  // SLOWEST index the slabs of one (sequence, head) -- which all read the same M' -- sit n_seq * HV ids apart, on one XCD
  // whenever that is a multiple of 8, and its L2 serves M' to all but the first of them
  const int seq = blockIdx.x, hv = blockIdx.y, vn = blockIdx.z;
  const int seg0 = pv.seq_seg0[seq], nseg = pv.seq_nseg[seq];
  const int nsteps = nseg - 1;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  const int col = 32 * vn + ln;

  f32x16 S = zero16();
  if (h0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = h0[(((size_t)seq * HV + hv) * KT + 32 * wave + acc_row(r, hh)) * VT + col];
  }

  X8 rm[DEPTH][NKS];
  f32x4 rn[DEPTH][4];
  float rd[DEPTH];
  auto issue = [&](int p, X8* m, f32x4* n, float& d) {
    const size_t sh = (size_t)(seg0 + p) * HV + hv;
    const X8* M = reinterpret_cast<const X8*>(Mcomp + sh * M_BYTES);
    const f32x4* N = reinterpret_cast<const f32x4*>(Ncomp + (sh * (VT / 32) + vn) * N_BYTES);
#pragma unroll
    for (int j = 0; j < NKS; ++j) m[j] = M[(wave * NKS + (2 * wave + j) % NKS) * 64 + lane];  // own fragments first
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) n[q4] = N[(wave * 4 + q4) * 64 + lane];
    d = Dcomp[sh];
  };
  // (every step issues the same loads, clamped at the end, so that the waits can leave younger loads in flight)
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue(max(0, min(d, nsteps - 1)), rm[d], rn[d], rd[d]);

  auto step = [&](int p, X8* m, f32x4* n, float& dd) {
    {  // the state segment seg0 + p starts from; steps past the end write to the spare slot behind the last segment
      const size_t slot = p <= nsteps ? (size_t)(seg0 + p) : (size_t)n_segments;
      f32x4* si = reinterpret_cast<f32x4*>(Sinit + ((slot * HV + hv) * (VT / 32) + vn) * (KT * 32));
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 t;
#pragma unroll
        for (int e = 0; e < 4; ++e) t[e] = S[4 * q4 + e];
        si[(wave * 4 + q4) * 64 + lane] = t;
      }
    }
    const float dec = dd;
    unsigned char* xbuf = s_x[p & 1];
    const X8 own0 = acc_to_op<OT>(S, 0), own1 = acc_to_op<OT>(S, 8);
    op_frag_store<OT>(xbuf, 2 * wave + 0, lane, own0);
    op_frag_store<OT>(xbuf, 2 * wave + 1, lane, own1);
    f32x16 acc;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[4 * q4 + e] = __builtin_fmaf(dec, S[4 * q4 + e], n[q4][e]);
    acc = mfma32(m[0], own0, acc);
    acc = mfma32(m[1], own1, acc);
    lds_barrier();
#pragma unroll
    for (int j = 2; j < NKS; ++j) acc = mfma32(m[j], op_frag_load<OT>(xbuf, (2 * wave + j) % NKS, lane), acc);
    S = acc;
    issue(max(0, min(p + DEPTH, nsteps - 1)), m, n, dd);
  };
  // The step loops have NO early exit: they run in whole groups, and the steps past the last segment work on clamped
  // operands and store to the spare slot. With a branch around a step the compiler can no longer count the loads in
  // flight and waits for all of them at every step; and since it drains the queue at every loop header anyway (the
  // ring registers are loaded in one iteration and used in the next), the main loop covers LONG groups of steps.
  constexpr int LONG = 4 * DEPTH;
  int p0 = 0;
  for (; p0 + LONG <= nsteps + 1; p0 += LONG) {
#pragma unroll
    for (int u = 0; u < LONG; ++u) step(p0 + u, rm[u % DEPTH], rn[u % DEPTH], rd[u % DEPTH]);
  }
  for (; p0 <= nsteps; p0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) step(p0 + d, rm[d], rn[d], rd[d]);
  }
}

// ---- two-level scan ------------------------------------------------------------------------------------------------
// A long sequence has many segments and the scan above walks them one after the other (0.45 us per step, a chain of
// dependent MFMA / LDS-exchange stages with 16 workgroups on the whole chip). With groups of G segments the serial
// depth drops from n to about n / G + 2 G:
//   GROUP  every group but the last of a sequence, in parallel: the composite of its G segments, i.e. the scan step
//          applied to the KT + VT columns [P_M | P_N] starting from [I | 0]; written as a segment composite is
//          (D = product of the decays, M' = P_M - D I as bf16 A-operand fragments, N = P_N in accumulator order);
//   LEAF   every group in parallel: the workgroup of group j first walks the composites of groups 0 .. j-1 from the
//          sequence's initial state (at most gmax - 1 redundant steps; a separate serial pass over the groups would
//          cost a launch more), then its own segments, writing the state every segment starts from (what the
//          single-level scan writes).
// Same step code in both modes; loops are branch free with clamped operands and a spare store slot as above.
enum { SCAN_GROUP = 1, SCAN_LEAF = 2 };

template <typename OT, int KT, int VT, int DEPTH, int MODE>
__global__ void __launch_bounds__(64 * (KT / 32)) gdr_scan2_kernel(const GdrPlanView pv,
                                                                  const unsigned char* __restrict__ Msrc,
                                                                  const unsigned char* __restrict__ Nsrc,
                                                                  const float* __restrict__ Dsrc,
                                                                  const float* __restrict__ h0,
                                                                  float* __restrict__ dst, unsigned char* __restrict__ Mout,
                                                                  unsigned char* __restrict__ Nout, float* __restrict__ Dout,
                                                                  int HV, int spare_slot, int gmax) {
  using X8 = typename OpVec<OT>::x8;
  constexpr int G = GDR_SCAN_GROUP;
  static_assert(G % DEPTH == 0, "a group must be a whole number of ring rounds");
  constexpr int NKS = KT / 16;
  constexpr int M_BYTES = KT * KT * 2, N_BYTES = KT * 32 * 4;
  constexpr int NCB = MODE == SCAN_GROUP ? (KT + VT) / 32 : VT / 32;  // 32-column blocks per item of the grid
  __shared__ __align__(16) unsigned char s_x[2][NKS * 1024];
  const int vn = blockIdx.x % NCB, j = blockIdx.x / NCB, seq = blockIdx.y, hv = blockIdx.z;
  const int seg0 = pv.seq_seg0[seq], nseg = pv.seq_nseg[seq];
  const int ngroups = (nseg + G - 1) / G;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  // items = the maps this workgroup applies, slots = where it stores the running state before each of them
  int item0, nsteps, slot0, lead = 0;  // lead: group-level maps walked before the workgroup's own items (LEAF)
  if (MODE == SCAN_GROUP) {
    if (j >= ngroups - 1) return;  // the composite of a sequence's last group is never needed
    item0 = seg0 + j * G; nsteps = G - 1; slot0 = 0;
  } else {
    if (j >= ngroups) return;
    item0 = seg0 + j * G; lead = j; nsteps = lead + min(G, nseg - j * G) - 1; slot0 = item0;
  }
  const int last = MODE == SCAN_GROUP ? nsteps : nsteps - 1;   // last map that is really applied (prefetches are clamped to it)
  const bool is_pm = MODE == SCAN_GROUP && vn < KT / 32;       // a block of P_M: no additive term, starts from I
  const int nblk = MODE == SCAN_GROUP ? max(vn - KT / 32, 0) : vn;  // 32-column block of N / of the state

  f32x16 S = zero16();
  if (MODE == SCAN_GROUP) {
    if (is_pm) {
#pragma unroll
      for (int r = 0; r < 16; ++r) S[r] = (32 * wave + acc_row(r, hh) == 32 * vn + ln) ? 1.0f : 0.0f;
    }
  } else if (h0) {
#pragma unroll
    for (int r = 0; r < 16; ++r)
      S[r] = h0[(((size_t)seq * HV + hv) * KT + 32 * wave + acc_row(r, hh)) * VT + 32 * vn + ln];
  }

  X8 rm[DEPTH][NKS];
  f32x4 rn[DEPTH][4];
  float rd[DEPTH];
  auto issue = [&](int p, X8* m, f32x4* n, float& d) {
    const bool top = MODE == SCAN_LEAF && p < lead;  // a group composite (read through the *out pointers)
    const size_t sh = (size_t)(top ? seq * gmax + p : item0 + (p - lead)) * HV + hv;
    const X8* M = reinterpret_cast<const X8*>((top ? Mout : Msrc) + sh * M_BYTES);
    const f32x4* N = reinterpret_cast<const f32x4*>((top ? Nout : Nsrc) + (sh * (VT / 32) + nblk) * N_BYTES);
#pragma unroll
    for (int f = 0; f < NKS; ++f) m[f] = M[(wave * NKS + (2 * wave + f) % NKS) * 64 + lane];  // own fragments first
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) n[q4] = N[(wave * 4 + q4) * 64 + lane];
    d = (top ? Dout : Dsrc)[sh];
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue(max(0, min(d, last)), rm[d], rn[d], rd[d]);

  float dprod = 1.0f;
  auto step = [&](int p, X8* m, f32x4* n, float& dd) {
    if (MODE != SCAN_GROUP) {
      const size_t slot = (p >= lead && p <= nsteps) ? (size_t)(slot0 + (p - lead)) : (size_t)spare_slot;
      f32x4* si = reinterpret_cast<f32x4*>(dst + ((slot * HV + hv) * (VT / 32) + vn) * (KT * 32));
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 t;
#pragma unroll
        for (int e = 0; e < 4; ++e) t[e] = S[4 * q4 + e];
        si[(wave * 4 + q4) * 64 + lane] = t;
      }
    }
    const float dec = dd;
    dprod *= dec;
    unsigned char* xbuf = s_x[p & 1];
    const X8 own0 = acc_to_op<OT>(S, 0), own1 = acc_to_op<OT>(S, 8);
    op_frag_store<OT>(xbuf, 2 * wave + 0, lane, own0);
    op_frag_store<OT>(xbuf, 2 * wave + 1, lane, own1);
    f32x16 acc;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[4 * q4 + e] = __builtin_fmaf(dec, S[4 * q4 + e], is_pm ? 0.0f : n[q4][e]);
    acc = mfma32(m[0], own0, acc);
    acc = mfma32(m[1], own1, acc);
    lds_barrier();
#pragma unroll
    for (int f = 2; f < NKS; ++f) acc = mfma32(m[f], op_frag_load<OT>(xbuf, (2 * wave + f) % NKS, lane), acc);
    S = acc;
    issue(max(0, min(p + DEPTH, last)), m, n, dd);
  };
  constexpr int LONG = 4 * DEPTH;
  int p0 = 0;
  if (MODE != SCAN_GROUP) {
    for (; p0 + LONG <= nsteps + 1; p0 += LONG) {
#pragma unroll
      for (int u = 0; u < LONG; ++u) step(p0 + u, rm[u % DEPTH], rn[u % DEPTH], rd[u % DEPTH]);
    }
  }
  for (; p0 <= nsteps; p0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) step(p0 + d, rm[d], rn[d], rd[d]);
  }

  if (MODE == SCAN_GROUP) {  // exactly G maps were applied (G is a multiple of DEPTH): store the composite
    const size_t gh = (size_t)(seq * gmax + j) * HV + hv;
    if (is_pm) {
      unsigned char* out = Mout + gh * M_BYTES;
      const int mcol = 32 * vn + ln, ks = mcol >> 4, c16 = mcol & 15;
      const int hs = (c16 >> 2) & 1, slot = 4 * (c16 >> 3) + (c16 & 3);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * wave + acc_row(r, hh);
        const float val = S[r] - (row == mcol ? dprod : 0.0f);
        *reinterpret_cast<OT*>(out + ((size_t)((wave * NKS + ks) * 64 + 32 * hs + (row & 31))) * 16 + 2 * slot) = (OT)val;
      }
      if (vn == 0 && tid == 0) Dout[gh] = dprod;
    } else {
      f32x4* out = reinterpret_cast<f32x4*>(Nout + (gh * (VT / 32) + nblk) * N_BYTES);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 t;
#pragma unroll
        for (int e = 0; e < 4; ++e) t[e] = S[4 * q4 + e];
        out[(wave * 4 + q4) * 64 + lane] = t;
      }
    }
  }
}

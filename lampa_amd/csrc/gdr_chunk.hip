// Chunkwise gated-delta-rule forward on gfx950 (bf16 MFMA 32x32x16, fp32 accumulate, fp32 state).
//
// Replaces the forward pipeline of chunk_gated_delta_rule (reference chengjiang123/Lampa,
// models/hattention/gated_delta_rule_ori.py:29-80): chunk_local_cumsum (cumsum.py:27-62), l2norm_fwd
// (l2norm.py:87-103), chunk_scaled_dot_kkt_fwd (chunk_scaled_dot_kkt.py:27-71), solve_tril (solve_tril.py),
// recompute_w_u_fwd (wy_fast.py:140-189), chunk_gated_delta_rule_fwd_h (chunk_delta_h.py:34-189) and
// chunk_fwd_o (chunk_o.py:33-111).
//
// Four kernels:
//   prep       one workgroup per (chunk, head): l2norm, cumulative log-decay, KK^T and QK^T on MFMA, the
//              unit-lower-triangular inverse by forward substitution in LDS, then W, U.  Everything the
//              sequential part needs is written as ready-made MFMA operand fragments ("record" of the chunk).
//   composite  the state map of a chunk is affine, S' = M S + N.  The sequence is cut into segments of a few
//              chunks; one wave per (segment, head, 32 columns of [M | N]) runs the recurrence on the identity
//              and on zero to obtain the segment's composite (M, N).
//   scan       one wave per (sequence, head, 32 value columns) walks the segments: S_{p+1} = M_p S_p + N_p
//              (hi/lo split bf16 MFMA, fp32 state) and stores every segment's initial state.
//   output     one wave per (segment, head, 32 value columns) replays its segment from the right initial state:
//              v_new = U - W S,  o = Q~ S + P v_new,  S <- e^{g_last} S + K~^T v_new.
// The sequential kernels keep the state in accumulator registers and feed it straight back as the next MFMA's
// B operand (accumulator rows 8*(r/4) + 4*hh + r%4 become contraction slots), so the state never touches LDS.
#include "gdr_common.h"

#define GDR_C 64  // chunk length

// ---- plan (host-built tables, int32) -------------------------------------------------------------------------
enum {
  PLAN_N_SEQ = 0,
  PLAN_TOTAL_CHUNKS = 1,
  PLAN_N_SEGMENTS = 2,
  PLAN_CHUNKS_PER_SEGMENT = 3,
  PLAN_OFF_CHUNK_TOK0 = 4,
  PLAN_OFF_CHUNK_LEN = 5,
  PLAN_OFF_SEG_CHUNK0 = 6,
  PLAN_OFF_SEG_NCHUNKS = 7,
  PLAN_OFF_SEG_SEQ = 8,
  PLAN_OFF_SEG_FLAGS = 9,
  PLAN_OFF_SEQ_SEG0 = 10,
  PLAN_OFF_SEQ_NSEG = 11,
  PLAN_TOTAL_TOKENS = 12,
  PLAN_HEADER = 16
};
#define SEG_FIRST 1
#define SEG_LAST 2

static int64_t plan_counts(const int64_t* cu, int n_seq, int cps, int64_t* n_chunks, int64_t* n_segments) {
  int64_t chunks = 0, segs = 0;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t len = cu[s + 1] - cu[s];
    if (len < 0) return -1;
    const int64_t nc = (len + GDR_C - 1) / GDR_C;
    chunks += nc;
    segs += nc == 0 ? 1 : (nc + cps - 1) / cps;  // an empty sequence still owns one (empty) segment
  }
  *n_chunks = chunks;
  *n_segments = segs;
  return 0;
}

// Number of int32 entries of the plan for these sequences (negative on error).
extern "C" int64_t lampa_gdr_plan_size(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment) {
  if (!cu_seqlens_host || n_seq < 1 || chunks_per_segment < 1) return LAMPA_ERR_INVALID;
  int64_t chunks, segs;
  if (plan_counts(cu_seqlens_host, n_seq, chunks_per_segment, &chunks, &segs) != 0) return LAMPA_ERR_INVALID;
  if (cu_seqlens_host[n_seq] > INT32_MAX) return LAMPA_ERR_UNSUPPORTED;
  return PLAN_HEADER + 2 * chunks + 4 * segs + 2 * (int64_t)n_seq;
}

// Fills plan_host (lampa_gdr_plan_size entries). The caller copies it to the device and passes that pointer on.
extern "C" int lampa_gdr_plan_fill(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment,
                                   int32_t* plan_host) {
  if (!plan_host) return LAMPA_ERR_INVALID;
  const int64_t size = lampa_gdr_plan_size(cu_seqlens_host, n_seq, chunks_per_segment);
  if (size < 0) return (int)size;
  int64_t chunks, segs;
  plan_counts(cu_seqlens_host, n_seq, chunks_per_segment, &chunks, &segs);
  int32_t* p = plan_host;
  for (int i = 0; i < PLAN_HEADER; ++i) p[i] = 0;
  p[PLAN_N_SEQ] = n_seq;
  p[PLAN_TOTAL_CHUNKS] = (int32_t)chunks;
  p[PLAN_N_SEGMENTS] = (int32_t)segs;
  p[PLAN_CHUNKS_PER_SEGMENT] = chunks_per_segment;
  p[PLAN_TOTAL_TOKENS] = (int32_t)cu_seqlens_host[n_seq];
  int64_t off = PLAN_HEADER;
  p[PLAN_OFF_CHUNK_TOK0] = (int32_t)off; off += chunks;
  p[PLAN_OFF_CHUNK_LEN] = (int32_t)off; off += chunks;
  p[PLAN_OFF_SEG_CHUNK0] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEG_NCHUNKS] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEG_SEQ] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEG_FLAGS] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEQ_SEG0] = (int32_t)off; off += n_seq;
  p[PLAN_OFF_SEQ_NSEG] = (int32_t)off; off += n_seq;
  int64_t c = 0, g = 0;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t bos = cu_seqlens_host[s], len = cu_seqlens_host[s + 1] - bos;
    const int64_t nc = (len + GDR_C - 1) / GDR_C;
    const int64_t ns = nc == 0 ? 1 : (nc + chunks_per_segment - 1) / chunks_per_segment;
    p[p[PLAN_OFF_SEQ_SEG0] + s] = (int32_t)g;
    p[p[PLAN_OFF_SEQ_NSEG] + s] = (int32_t)ns;
    for (int64_t i = 0; i < ns; ++i) {
      const int64_t c0 = i * chunks_per_segment;
      const int64_t cn = nc - c0 < chunks_per_segment ? nc - c0 : chunks_per_segment;
      p[p[PLAN_OFF_SEG_CHUNK0] + g] = (int32_t)(c + c0);
      p[p[PLAN_OFF_SEG_NCHUNKS] + g] = (int32_t)(cn < 0 ? 0 : cn);
      p[p[PLAN_OFF_SEG_SEQ] + g] = s;
      p[p[PLAN_OFF_SEG_FLAGS] + g] = (i == 0 ? SEG_FIRST : 0) | (i == ns - 1 ? SEG_LAST : 0);
      ++g;
    }
    for (int64_t i = 0; i < nc; ++i) {
      p[p[PLAN_OFF_CHUNK_TOK0] + c] = (int32_t)(bos + i * GDR_C);
      p[p[PLAN_OFF_CHUNK_LEN] + c] = (int32_t)(len - i * GDR_C < GDR_C ? len - i * GDR_C : GDR_C);
      ++c;
    }
  }
  return LAMPA_OK;
}

// ---- record layout ----------------------------------------------------------------------------------------------
// A fragment is 64 lanes x 8 bf16 (1 KiB): lane l's 16 bytes are its share of one MFMA 32x32x16 A operand.
//   Wf[tm][ks]   -W rows 32tm..+31 (tokens), contraction step ks over the key dimension     2*(K/16) fragments
//   Kf[km][ks]   K~^T rows 32km..+31 (key dims), contraction step ks over the tokens         (K/32)*4
//   Qf[tm][ks]   Q~ rows (tokens), contraction over the key dimension                        2*(K/16)
//   Pf[tm][ks]   P rows (tokens i), contraction over the tokens j (tm = 0 only needs ks < 2) 2*4
//   Uf[tm][vn]   U tile in accumulator layout, 16 bf16 per lane (2 KiB)                      2*(V/32)
template <int KT, int VT>
struct GdrRecord {
  static constexpr int W_FRAGS = 2 * (KT / 16);
  static constexpr int K_FRAGS = (KT / 32) * 4;
  static constexpr int Q_FRAGS = 2 * (KT / 16);
  static constexpr int P_FRAGS = 8;
  static constexpr int U_TILES = 2 * (VT / 32);
  static constexpr int W_OFF = 0;
  static constexpr int K_OFF = W_OFF + W_FRAGS;
  static constexpr int Q_OFF = K_OFF + K_FRAGS;
  static constexpr int P_OFF = Q_OFF + Q_FRAGS;
  static constexpr int U_OFF = P_OFF + P_FRAGS;            // in units of 1 KiB
  static constexpr int BYTES = (U_OFF + 2 * U_TILES) * 1024;
};

static int64_t gdr_record_bytes(int K, int V) {
  return (int64_t)(2 * (K / 16) * 2 + (K / 32) * 4 + 8 + 2 * 2 * (V / 32)) * 1024;
}

__device__ __forceinline__ bf16x8 frag_load(const unsigned char* rec, int frag, int lane) {
  return *reinterpret_cast<const bf16x8*>(rec + (size_t)frag * 1024 + lane * 16);
}
__device__ __forceinline__ void frag_store(unsigned char* rec, int frag, int lane, bf16x8 v) {
#ifndef GDR_DBG_SKIP_STORE
  *reinterpret_cast<bf16x8*>(rec + (size_t)frag * 1024 + lane * 16) = v;
#else
  if (v[0] == (__bf16)123.456f) *reinterpret_cast<bf16x8*>(rec + (size_t)frag * 1024 + lane * 16) = v;
#endif
}

// ---- prep kernel ----------------------------------------------------------------------------------------------
template <int KT, int VT>
struct GdrPrepSmem {
  static constexpr int SK = KT + 8;  // row stride of the row-major k / q tiles (bf16)
  static constexpr int SX = 72;      // row stride of the [dim][token] tiles and of the [token][token] tiles (bf16)
  static constexpr int SA = 68;      // row stride of the fp32 A tile
  static constexpr int OFF_K = 0;
  static constexpr int OFF_Q = OFF_K + 64 * SK * 2;
  static constexpr int OFF_KT = OFF_Q + 64 * SK * 2;
  static constexpr int OFF_VT = OFF_KT + KT * SX * 2;
  static constexpr int OFF_A = OFF_VT + VT * SX * 2;
  static constexpr int OFF_TW = OFF_A + 64 * SA * 4;
  static constexpr int OFF_TU = OFF_TW + 64 * SX * 2;
  static constexpr int OFF_GAMMA = OFF_TU + 64 * SX * 2;
  static constexpr int OFF_BETA = OFF_GAMMA + 64 * 4;
  static constexpr int BYTES = OFF_BETA + 64 * 4;
};

template <typename T, int KT, int VT>
__global__ void __launch_bounds__(256) gdr_prep_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                      const T* __restrict__ v, const float* __restrict__ g,
                                                      const float* __restrict__ beta,
                                                      const int32_t* __restrict__ plan,
                                                      unsigned char* __restrict__ records,
                                                      float* __restrict__ decs, int H, int HV, float scale,
                                                      int l2norm) {
  using SM = GdrPrepSmem<KT, VT>;
  using REC = GdrRecord<KT, VT>;
  extern __shared__ __align__(16) unsigned char smem[];
  __bf16* s_k = reinterpret_cast<__bf16*>(smem + SM::OFF_K);
  __bf16* s_q = reinterpret_cast<__bf16*>(smem + SM::OFF_Q);
  __bf16* s_kT = reinterpret_cast<__bf16*>(smem + SM::OFF_KT);
  __bf16* s_vT = reinterpret_cast<__bf16*>(smem + SM::OFF_VT);
  float* s_A = reinterpret_cast<float*>(smem + SM::OFF_A);
  __bf16* s_TW = reinterpret_cast<__bf16*>(smem + SM::OFF_TW);
  __bf16* s_TU = reinterpret_cast<__bf16*>(smem + SM::OFF_TU);
  float* s_gamma = reinterpret_cast<float*>(smem + SM::OFF_GAMMA);
  float* s_beta = reinterpret_cast<float*>(smem + SM::OFF_BETA);
  constexpr int SK = SM::SK, SX = SM::SX, SA = SM::SA;

  const int chunk = blockIdx.x, hv = blockIdx.y;
  const int h = hv / (HV / H);
  const int tok0 = plan[plan[PLAN_OFF_CHUNK_TOK0] + chunk];
  const int len = plan[plan[PLAN_OFF_CHUNK_LEN] + chunk];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  unsigned char* rec = records + ((size_t)chunk * HV + hv) * REC::BYTES;

  // (1) cumulative log-decay and beta of the chunk; rows past the end behave as g = 0, beta = 0, k = v = q = 0
  if (wave == 0) {
    float gv = lane < len ? g[(size_t)(tok0 + lane) * HV + hv] : 0.0f;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float up = __shfl_up(gv, off);
      if (lane >= off) gv += up;
    }
    s_gamma[lane] = gv;
    s_beta[lane] = lane < len ? beta[(size_t)(tok0 + lane) * HV + hv] : 0.0f;
  }

  // (2) load, l2-normalise, stage in LDS: k row-major and transposed, q row-major, v transposed
  {
    const int row = tid >> 2, q4 = tid & 3;
    const bool valid = row < len;
    constexpr int EPT = KT / 4;
    float kf[EPT], qf[EPT];
    float kss = 0.0f, qss = 0.0f;
    const T* kp = k + ((size_t)(tok0 + row) * H + h) * KT + q4 * EPT;
    const T* qp = q + ((size_t)(tok0 + row) * H + h) * KT + q4 * EPT;
#pragma unroll
    for (int c = 0; c < EPT / 8; ++c) {
      if (valid) {
        load8<T>(kp + 8 * c, kf + 8 * c);
        load8<T>(qp + 8 * c, qf + 8 * c);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) { kf[8 * c + e] = 0.0f; qf[8 * c + e] = 0.0f; }
      }
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e) { kss += kf[e] * kf[e]; qss += qf[e] * qf[e]; }
    float kinv = 1.0f, qinv = 1.0f;
    if (l2norm != GDR_L2_NONE) {
      kss += __shfl_xor(kss, 1); kss += __shfl_xor(kss, 2);
      qss += __shfl_xor(qss, 1); qss += __shfl_xor(qss, 2);
      if (l2norm == GDR_L2_CHUNK) {
        kinv = 1.0f / __fsqrt_rn(kss + 1e-6f);
        qinv = 1.0f / __fsqrt_rn(qss + 1e-6f);
      } else {
        kinv = 1.0f / (__fsqrt_rn(kss) + 1e-6f);
        qinv = 1.0f / (__fsqrt_rn(qss) + 1e-6f);
      }
    }
#pragma unroll
    for (int c = 0; c < EPT / 8; ++c) {
      bf16x8 kb, qb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        kb[e] = (__bf16)(kf[8 * c + e] * kinv);
        qb[e] = (__bf16)(qf[8 * c + e] * qinv);
#ifndef GDR_DBG_SKIP_TR
        s_kT[(q4 * EPT + 8 * c + e) * SX + row] = kb[e];
#endif
      }
      *reinterpret_cast<bf16x8*>(&s_k[row * SK + q4 * EPT + 8 * c]) = kb;
      *reinterpret_cast<bf16x8*>(&s_q[row * SK + q4 * EPT + 8 * c]) = qb;
    }
    constexpr int VPT = VT / 4;
    const T* vp = v + ((size_t)(tok0 + row) * HV + hv) * VT + q4 * VPT;
#pragma unroll
    for (int c = 0; c < VPT / 8; ++c) {
      float vf[8];
      if (valid) {
        load8<T>(vp + 8 * c, vf);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) vf[e] = 0.0f;
      }
#pragma unroll
#ifndef GDR_DBG_SKIP_TR
      for (int e = 0; e < 8; ++e) s_vT[(q4 * VPT + 8 * c + e) * SX + row] = (__bf16)vf[e];
#endif
    }
  }
  __syncthreads();

  // (3) A = strict_lower(beta_i (k_i . k_j) e^{gamma_i - gamma_j}) -> LDS fp32; one 32x32 tile per wave
  {
    const int tm = wave >> 1, tn = wave & 1;
    if (!(tm == 0 && tn == 1)) {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KT / 16; ++ks) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&s_k[(32 * tm + ln) * SK + 16 * ks + 8 * hh]);
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(&s_k[(32 * tn + ln) * SK + 16 * ks + 8 * hh]);
        acc = mfma32(a, b, acc);
      }
      const int j = 32 * tn + ln;
      const float gj = s_gamma[j];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 32 * tm + 8 * (r / 4) + 4 * hh + (r % 4);
        const float val = i > j ? acc[r] * s_beta[i] * __expf(s_gamma[i] - gj) : 0.0f;
        s_A[i * SA + j] = val;
      }
    }
  }
  __syncthreads();

  if (wave == 0) {
    // (4a) T = (I + A)^-1, A strictly lower triangular, as a 2x2 block matrix of 32x32 blocks:
    //      T11 = (I + A11)^-1, T22 = (I + A22)^-1 by forward substitution -- lane 32b + c owns column c of block b,
    //      every lane of a half-wave reads the same A element (LDS broadcast), fp32 throughout;
    //      T21 = -T22 (A21 T11) with two MFMA products whose operands are split into bf16 high and remainder parts.
    const int b = hh, c = ln;
    const float* Ab = s_A + (32 * b) * SA + 32 * b;
    float x[32];
    f32x4 rowbuf[2][8];  // rows i and i+1 of the block, so that the next row loads while this one is reduced
    rowbuf[1][0] = *reinterpret_cast<const f32x4*>(Ab + 1 * SA);
    x[0] = (c == 0) ? 1.0f : 0.0f;
#pragma unroll
    for (int i = 1; i < 32; ++i) {
      if (i + 1 < 32) {
#pragma unroll
        for (int q = 0; q < (i + 1 + 3) / 4; ++q)
          rowbuf[(i + 1) & 1][q] = *reinterpret_cast<const f32x4*>(Ab + (i + 1) * SA + 4 * q);
      }
      float acc0 = (i == c) ? 1.0f : 0.0f, acc1 = 0.0f;
#pragma unroll
      for (int j = 0; j < i; ++j) {
        if (j & 1) acc1 = __builtin_fmaf(-rowbuf[i & 1][j / 4][j % 4], x[j], acc1);
        else acc0 = __builtin_fmaf(-rowbuf[i & 1][j / 4][j % 4], x[j], acc0);
      }
      x[i] = acc0 + acc1;
      // pins the order "loads of row i+1, arithmetic of row i" so the compiler neither serialises every load
      // behind a wait nor hoists all 124 loads to the top (which spills)
      asm volatile("" : "+v"(x[i]) : : "memory");
    }
    __builtin_amdgcn_wave_barrier();
    // diagonal blocks: fp32 copy in place of A11 / A22 (operands of the merge) and the scaled bf16 outputs;
    // the upper-right block of T is zero
    const float bc = s_beta[lane];
    const float wc = bc * __expf(s_gamma[lane]);
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      s_A[(32 * b + i) * SA + lane] = x[i];
      s_TW[(32 * b + i) * SX + lane] = (__bf16)(x[i] * wc);
      s_TU[(32 * b + i) * SX + lane] = (__bf16)(x[i] * bc);
      if (b == 1) {
        s_TW[i * SX + lane] = (__bf16)0.0f;
        s_TU[i * SX + lane] = (__bf16)0.0f;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x16 y0, y1, y2;
#pragma unroll
    for (int r = 0; r < 16; ++r) { y0[r] = 0.0f; y1[r] = 0.0f; y2[r] = 0.0f; }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {  // Y = A21 T11
      bf16x8 ahi, alo, bhi, blo;
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(&s_A[(32 + ln) * SA + 16 * ks + 8 * hh]);
      const f32x4 a1 = *reinterpret_cast<const f32x4*>(&s_A[(32 + ln) * SA + 16 * ks + 8 * hh + 4]);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float av = q < 4 ? a0[q % 4] : a1[q % 4];
        const float bv = s_A[(16 * ks + 8 * hh + q) * SA + ln];
        const __bf16 ah = (__bf16)av, bh = (__bf16)bv;
        ahi[q] = ah; alo[q] = (__bf16)(av - (float)ah);
        bhi[q] = bh; blo[q] = (__bf16)(bv - (float)bh);
      }
      y0 = mfma32(ahi, bhi, y0);
      y1 = mfma32(alo, bhi, y1);
      y2 = mfma32(ahi, blo, y2);
    }
    f32x16 t0, t1, t2;
#pragma unroll
    for (int r = 0; r < 16; ++r) { y0[r] += y1[r] + y2[r]; t0[r] = 0.0f; t1[r] = 0.0f; t2[r] = 0.0f; }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {  // T22 Y, Y taken straight from the accumulator as the B operand
      bf16x8 ahi, alo, bhi, blo;
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(&s_A[(32 + ln) * SA + 32 + 16 * ks + 4 * hh]);
      const f32x4 a1 = *reinterpret_cast<const f32x4*>(&s_A[(32 + ln) * SA + 32 + 16 * ks + 8 + 4 * hh]);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float av = q < 4 ? a0[q % 4] : a1[q % 4];
        const float bv = y0[8 * ks + q];
        const __bf16 ah = (__bf16)av, bh = (__bf16)bv;
        ahi[q] = ah; alo[q] = (__bf16)(av - (float)ah);
        bhi[q] = bh; blo[q] = (__bf16)(bv - (float)bh);
      }
      t0 = mfma32(ahi, bhi, t0);
      t1 = mfma32(alo, bhi, t1);
      t2 = mfma32(ahi, blo, t2);
    }
    const float bl = s_beta[ln];
    const float wl = bl * __expf(s_gamma[ln]);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 32 + 8 * (r / 4) + 4 * hh + (r % 4);
      const float t21 = -(t0[r] + (t1[r] + t2[r]));
      s_TW[row * SX + ln] = (__bf16)(t21 * wl);
      s_TU[row * SX + ln] = (__bf16)(t21 * bl);
    }
    if (lane == 0) decs[(size_t)chunk * HV + hv] = __expf(s_gamma[63]);
  } else {
    // (4b) meanwhile: P^T tiles, K~^T fragments, Q~ fragments
    constexpr int N_TASKS = 3 + REC::K_FRAGS + REC::Q_FRAGS;
    const float g_last = s_gamma[63];
    for (int task = wave - 1; task < N_TASKS; task += 3) {
      if (task < 3) {
        const int jm = task == 2 ? 1 : 0, tn = task == 0 ? 0 : 1;  // tiles (0,0), (0,1), (1,1); (1,0) is all zero
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KT / 16; ++ks) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(&s_k[(32 * jm + ln) * SK + 16 * ks + 8 * hh]);
          const bf16x8 b = *reinterpret_cast<const bf16x8*>(&s_q[(32 * tn + ln) * SK + 16 * ks + 8 * hh]);
          acc = mfma32(a, b, acc);
        }
        const int i = 32 * tn + ln;
        const float gi = s_gamma[i];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = 32 * jm + 8 * (r / 4) + 4 * hh + (r % 4);
          acc[r] = i >= j ? acc[r] * scale * __expf(gi - s_gamma[j]) : 0.0f;
        }
        frag_store(rec, REC::P_OFF + tn * 4 + 2 * jm + 0, lane, acc_to_operand(acc, 0));
        frag_store(rec, REC::P_OFF + tn * 4 + 2 * jm + 1, lane, acc_to_operand(acc, 8));
      } else if (task < 3 + REC::K_FRAGS) {
        const int f = task - 3, km = f / 4, ks = f % 4;
        const int kd = 32 * km + ln;
        const bf16x4 lo = *reinterpret_cast<const bf16x4*>(&s_kT[kd * SX + 16 * ks + 4 * hh]);
        const bf16x4 hi = *reinterpret_cast<const bf16x4*>(&s_kT[kd * SX + 16 * ks + 8 + 4 * hh]);
        bf16x8 out;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          const int tok = 16 * ks + kappa(hh, s);
          const float kv = (float)(s < 4 ? lo[s % 4] : hi[s % 4]);
          out[s] = (__bf16)(kv * __expf(g_last - s_gamma[tok]));
        }
        frag_store(rec, REC::K_OFF + f, lane, out);
      } else {
        const int f = task - 3 - REC::K_FRAGS, tm = f / (KT / 16), ks = f % (KT / 16);
        const int tok = 32 * tm + ln;
        const bf16x4 lo = *reinterpret_cast<const bf16x4*>(&s_q[tok * SK + 16 * ks + 4 * hh]);
        const bf16x4 hi = *reinterpret_cast<const bf16x4*>(&s_q[tok * SK + 16 * ks + 8 + 4 * hh]);
        const float sc = scale * __expf(s_gamma[tok]);
        bf16x8 out;
#pragma unroll
        for (int s = 0; s < 8; ++s) out[s] = (__bf16)((float)(s < 4 ? lo[s % 4] : hi[s % 4]) * sc);
        frag_store(rec, REC::Q_OFF + f, lane, out);
      }
    }
  }
  __syncthreads();

  // (5) -W^T = -(k^T TW^T) -> A fragments of W S;  U = TU v -> accumulator-layout tiles
  {
    constexpr int W_TILES = (KT / 32) * 2, U_TILES = 2 * (VT / 32);
    for (int task = wave; task < W_TILES + U_TILES; task += 4) {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
      if (task < W_TILES) {
        const int km = task >> 1, tn = task & 1;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(&s_kT[(32 * km + ln) * SX + 16 * ks + 8 * hh]);
          const bf16x8 b = *reinterpret_cast<const bf16x8*>(&s_TW[(32 * tn + ln) * SX + 16 * ks + 8 * hh]);
          acc = mfma32(a, b, acc);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = -acc[r];
        frag_store(rec, REC::W_OFF + tn * (KT / 16) + 2 * km + 0, lane, acc_to_operand(acc, 0));
        frag_store(rec, REC::W_OFF + tn * (KT / 16) + 2 * km + 1, lane, acc_to_operand(acc, 8));
      } else {
        const int t = task - W_TILES, tm = t / (VT / 32), vn = t % (VT / 32);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(&s_TU[(32 * tm + ln) * SX + 16 * ks + 8 * hh]);
          const bf16x8 b = *reinterpret_cast<const bf16x8*>(&s_vT[(32 * vn + ln) * SX + 16 * ks + 8 * hh]);
          acc = mfma32(a, b, acc);
        }
        unsigned char* up = rec + (size_t)REC::U_OFF * 1024 + (size_t)t * 2048 + lane * 32;
        *reinterpret_cast<bf16x8*>(up) = acc_to_operand(acc, 0);
        *reinterpret_cast<bf16x8*>(up + 16) = acc_to_operand(acc, 8);
      }
    }
  }
}

// ---- sequential kernels -----------------------------------------------------------------------------------------
// State tile km of a wave: rows 32km..+31 (key dims), 32 columns; register r of lane l = (row 8*(r/4)+4*hh+r%4, col ln).
template <int KT>
__device__ __forceinline__ void state_operands(const f32x16* S, bf16x8* Sb) {
#pragma unroll
  for (int ks = 0; ks < KT / 16; ++ks) Sb[ks] = acc_to_operand(S[ks / 2], 8 * (ks % 2));
}

// Operand fragments of one chunk for one wave of the sequential kernels, held in registers so that the next
// chunk's loads are in flight while the current chunk computes.
template <int KT, int VT, bool WITH_OUTPUT>
struct GdrChunkOps {
  bf16x8 W[2 * (KT / 16)];
  bf16x8 Kf[(KT / 32) * 4];
  bf16x8 Q[WITH_OUTPUT ? 2 * (KT / 16) : 1];
  bf16x8 P[WITH_OUTPUT ? 6 : 1];
  bf16x8 U[4];  // U tiles tm = 0, 1 of this wave's 32 columns, two halves each
  float dec;
};

template <int KT, int VT, bool WITH_OUTPUT>
__device__ __forceinline__ void chunk_ops_load(GdrChunkOps<KT, VT, WITH_OUTPUT>& ops,
                                               const unsigned char* __restrict__ rec, const float* __restrict__ decp,
                                               int lane, int vn, bool with_u) {
  using REC = GdrRecord<KT, VT>;
#pragma unroll
  for (int f = 0; f < 2 * (KT / 16); ++f) ops.W[f] = frag_load(rec, REC::W_OFF + f, lane);
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    const unsigned char* up = rec + (size_t)REC::U_OFF * 1024 + (size_t)(tm * (VT / 32) + vn) * 2048 + lane * 32;
    if (with_u) {
      ops.U[2 * tm + 0] = *reinterpret_cast<const bf16x8*>(up);
      ops.U[2 * tm + 1] = *reinterpret_cast<const bf16x8*>(up + 16);
    } else {
#pragma unroll
      for (int q = 0; q < 8; ++q) { ops.U[2 * tm][q] = (__bf16)0.0f; ops.U[2 * tm + 1][q] = (__bf16)0.0f; }
    }
  }
  if constexpr (WITH_OUTPUT) {
#pragma unroll
    for (int f = 0; f < 2 * (KT / 16); ++f) ops.Q[f] = frag_load(rec, REC::Q_OFF + f, lane);
#pragma unroll
    for (int f = 0; f < 2; ++f) ops.P[f] = frag_load(rec, REC::P_OFF + f, lane);
#pragma unroll
    for (int f = 0; f < 4; ++f) ops.P[2 + f] = frag_load(rec, REC::P_OFF + 4 + f, lane);
  }
#pragma unroll
  for (int f = 0; f < (KT / 32) * 4; ++f) ops.Kf[f] = frag_load(rec, REC::K_OFF + f, lane);
  ops.dec = *decp;
}

__device__ __forceinline__ f32x16 utile_widen(bf16x8 a, bf16x8 b) {
  f32x16 out;
#pragma unroll
  for (int s = 0; s < 8; ++s) { out[s] = (float)a[s]; out[8 + s] = (float)b[s]; }
  return out;
}

// One chunk of the recurrence on a 32-column slab: v_new = U - W S (Vb = its B-operand fragments),
// S <- dec S + K~^T v_new. With output: o tile tm = Q~ S + P v_new is handed to `emit(tm, acc)`.
template <int KT, int VT, bool WITH_OUTPUT, typename Emit>
__device__ __forceinline__ void chunk_step(const GdrChunkOps<KT, VT, WITH_OUTPUT>& ops, f32x16* S, Emit emit) {
  bf16x8 Sb[KT / 16];
  state_operands<KT>(S, Sb);
  bf16x8 Vb[4];
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    f32x16 acc = utile_widen(ops.U[2 * tm], ops.U[2 * tm + 1]);
#pragma unroll
    for (int ks = 0; ks < KT / 16; ++ks) acc = mfma32(ops.W[tm * (KT / 16) + ks], Sb[ks], acc);
    Vb[2 * tm + 0] = acc_to_operand(acc, 0);
    Vb[2 * tm + 1] = acc_to_operand(acc, 8);
  }
  if constexpr (WITH_OUTPUT) {
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KT / 16; ++ks) acc = mfma32(ops.Q[tm * (KT / 16) + ks], Sb[ks], acc);
#pragma unroll
      for (int ks = 0; ks < 2 * (tm + 1); ++ks) acc = mfma32(ops.P[2 * tm + ks], Vb[ks], acc);
      emit(tm, acc);
    }
  }
#pragma unroll
  for (int km = 0; km < KT / 32; ++km) {
#pragma unroll
    for (int r = 0; r < 16; ++r) S[km][r] *= ops.dec;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) S[km] = mfma32(ops.Kf[km * 4 + ks], Vb[ks], S[km]);
  }
}

// composite: grid (n_segments, HV), one wave per 32-column slab of [M | N] ((KT+VT)/32 waves per workgroup, so the
// waves that read the same W and K~ fragments share one CU's L1 and one XCD's L2). Slabs < KT/32 carry columns of
// M (start: identity, no U term), the others columns of N (start: zero).
// Mcomp [seg, HV, KT, KT], Ncomp [seg, HV, KT, VT] fp32 row-major.
template <int KT, int VT>
__global__ void __launch_bounds__(2 * (KT + VT)) gdr_composite_kernel(const int32_t* __restrict__ plan,
                                                          const unsigned char* __restrict__ records,
                                                          const float* __restrict__ decs,
                                                          float* __restrict__ Mcomp, float* __restrict__ Ncomp,
                                                          int HV) {
  using REC = GdrRecord<KT, VT>;
  using OPS = GdrChunkOps<KT, VT, false>;
  const int slab = threadIdx.x >> 6, seg = blockIdx.x, hv = blockIdx.y;
  const int flags = plan[plan[PLAN_OFF_SEG_FLAGS] + seg];
  if (flags & SEG_LAST) return;  // nothing follows the last segment of a sequence
  const int c0 = plan[plan[PLAN_OFF_SEG_CHUNK0] + seg], nc = plan[plan[PLAN_OFF_SEG_NCHUNKS] + seg];
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  const bool is_m = slab < KT / 32;
  const int vn = is_m ? 0 : slab - KT / 32;

  f32x16 S[KT / 32];
#pragma unroll
  for (int km = 0; km < KT / 32; ++km)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      S[km][r] = (is_m && (32 * km + 8 * (r / 4) + 4 * hh + (r % 4)) == 32 * slab + ln) ? 1.0f : 0.0f;

  auto rec_of = [&](int c) { return records + ((size_t)c * HV + hv) * REC::BYTES; };
  auto dec_of = [&](int c) { return decs + (size_t)c * HV + hv; };
  auto no_emit = [](int, const f32x16&) {};
  const int c1 = c0 + nc;
  OPS a, b;
  if (nc > 0) chunk_ops_load<KT, VT, false>(a, rec_of(c0), dec_of(c0), lane, vn, !is_m);
  for (int c = c0; c < c1; c += 2) {
    if (c + 1 < c1) chunk_ops_load<KT, VT, false>(b, rec_of(c + 1), dec_of(c + 1), lane, vn, !is_m);
    chunk_step<KT, VT, false>(a, S, no_emit);
    if (c + 1 < c1) {
      if (c + 2 < c1) chunk_ops_load<KT, VT, false>(a, rec_of(c + 2), dec_of(c + 2), lane, vn, !is_m);
      chunk_step<KT, VT, false>(b, S, no_emit);
    }
  }
  float* out = is_m ? Mcomp + ((size_t)seg * HV + hv) * KT * KT : Ncomp + ((size_t)seg * HV + hv) * KT * VT;
  const int ncols = is_m ? KT : VT, col = (is_m ? 32 * slab : 32 * vn) + ln;
#pragma unroll
  for (int km = 0; km < KT / 32; ++km)
#pragma unroll
    for (int r = 0; r < 16; ++r) out[(size_t)(32 * km + 8 * (r / 4) + 4 * hh + (r % 4)) * ncols + col] = S[km][r];
}

// scan: grid (VT/32, n_seq, HV), KT/32 waves per workgroup. Wave w owns state rows 32w..32w+31 of a 32-column slab.
// Per segment: store the state as the segment's initial state, then S <- M S + N with M and S split into bf16
// high and remainder parts (three MFMA products, close to fp32 accuracy). The waves exchange their share of S as
// B-operand fragments through a double-buffered LDS array (one barrier per step); the M rows and N tile of the
// next step are loaded while the current one computes.
// Sinit [seg, HV, KT, VT] fp32 row-major receives the state every segment starts from.
template <int KT>
struct GdrScanRegs {
  f32x4 m[KT / 16][2];
  float n[16];
};

template <int KT, int VT>
__device__ __forceinline__ void scan_load(GdrScanRegs<KT>& r, const float* __restrict__ M,
                                          const float* __restrict__ N, int wave, int hh, int ln, int col) {
#pragma unroll
  for (int ks = 0; ks < KT / 16; ++ks) {
    const float* mrow = M + (size_t)(32 * wave + ln) * KT + 16 * ks;
    r.m[ks][0] = *reinterpret_cast<const f32x4*>(mrow + 4 * hh);
    r.m[ks][1] = *reinterpret_cast<const f32x4*>(mrow + 8 + 4 * hh);
  }
#pragma unroll
  for (int q = 0; q < 16; ++q) r.n[q] = N[(size_t)(32 * wave + 8 * (q / 4) + 4 * hh + (q % 4)) * VT + col];
}

template <int KT, int VT>
__global__ void __launch_bounds__(KT * 2) gdr_scan_kernel(const int32_t* __restrict__ plan,
                                                         const float* __restrict__ Mcomp,
                                                         const float* __restrict__ Ncomp,
                                                         const float* __restrict__ h0, float* __restrict__ Sinit,
                                                         int HV) {
  __shared__ __align__(16) bf16x8 s_frag[2][2][KT / 16][64];  // [buffer][hi/lo][contraction step][lane]
  const int vn = blockIdx.x, seq = blockIdx.y, hv = blockIdx.z;
  const int seg0 = plan[plan[PLAN_OFF_SEQ_SEG0] + seq], nseg = plan[plan[PLAN_OFF_SEQ_NSEG] + seq];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  const int col = 32 * vn + ln;
  f32x16 S;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = 32 * wave + 8 * (r / 4) + 4 * hh + (r % 4);
    S[r] = h0 ? h0[(((size_t)seq * HV + hv) * KT + row) * VT + col] : 0.0f;
  }
  GdrScanRegs<KT> nxt;
  if (nseg > 1)
    scan_load<KT, VT>(nxt, Mcomp + ((size_t)seg0 * HV + hv) * KT * KT, Ncomp + ((size_t)seg0 * HV + hv) * KT * VT, wave,
                      hh, ln, col);
  for (int p = 0; p < nseg; ++p) {
    const int seg = seg0 + p;
    float* si = Sinit + ((size_t)seg * HV + hv) * KT * VT;
#pragma unroll
    for (int r = 0; r < 16; ++r) si[(size_t)(32 * wave + 8 * (r / 4) + 4 * hh + (r % 4)) * VT + col] = S[r];
    if (p == nseg - 1) break;
    // this step's M rows (hi / lo operand fragments) and N tile arrived in nxt; start fetching the next step's
    bf16x8 Mhi[KT / 16], Mlo[KT / 16];
    f32x16 acc0, acc1, acc2;
#pragma unroll
    for (int ks = 0; ks < KT / 16; ++ks)
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float x = nxt.m[ks][q / 4][q % 4];
        const __bf16 hi = (__bf16)x;
        Mhi[ks][q] = hi;
        Mlo[ks][q] = (__bf16)(x - (float)hi);
      }
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = nxt.n[r]; acc1[r] = 0.0f; acc2[r] = 0.0f; }
    if (p + 2 < nseg)
      scan_load<KT, VT>(nxt, Mcomp + ((size_t)(seg + 1) * HV + hv) * KT * KT,
                        Ncomp + ((size_t)(seg + 1) * HV + hv) * KT * VT, wave, hh, ln, col);
    // publish this wave's rows of S as B-operand fragments (contraction steps 2*wave and 2*wave+1)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      bf16x8 hi, lo;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const float x = S[8 * half + q];
        const __bf16 h = (__bf16)x;
        hi[q] = h;
        lo[q] = (__bf16)(x - (float)h);
      }
      s_frag[p & 1][0][2 * wave + half][lane] = hi;
      s_frag[p & 1][1][2 * wave + half][lane] = lo;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < KT / 16; ++ks) {
      const bf16x8 Shi = s_frag[p & 1][0][ks][lane];
      const bf16x8 Slo = s_frag[p & 1][1][ks][lane];
      acc0 = mfma32(Mhi[ks], Shi, acc0);
      acc1 = mfma32(Mlo[ks], Shi, acc1);
      acc2 = mfma32(Mhi[ks], Slo, acc2);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = acc0[r] + (acc1[r] + acc2[r]);
  }
}

// output: grid (n_segments, HV), one wave per 32 value columns (VT/32 waves per workgroup).
template <typename T, int KT, int VT>
__global__ void __launch_bounds__(2 * VT) gdr_output_kernel(const int32_t* __restrict__ plan,
                                                       const unsigned char* __restrict__ records,
                                                       const float* __restrict__ decs,
                                                       const float* __restrict__ Sinit, T* __restrict__ o,
                                                       float* __restrict__ ht, int HV) {
  using REC = GdrRecord<KT, VT>;
  using OPS = GdrChunkOps<KT, VT, true>;
  const int vn = threadIdx.x >> 6, seg = blockIdx.x, hv = blockIdx.y;
  const int c0 = plan[plan[PLAN_OFF_SEG_CHUNK0] + seg], nc = plan[plan[PLAN_OFF_SEG_NCHUNKS] + seg];
  const int flags = plan[plan[PLAN_OFF_SEG_FLAGS] + seg], seq = plan[plan[PLAN_OFF_SEG_SEQ] + seg];
  const int* chunk_tok0 = plan + plan[PLAN_OFF_CHUNK_TOK0];
  const int* chunk_len = plan + plan[PLAN_OFF_CHUNK_LEN];
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  const int col = 32 * vn + ln;
  f32x16 S[KT / 32];
  {
    const float* si = Sinit + ((size_t)seg * HV + hv) * KT * VT;
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int r = 0; r < 16; ++r) S[km][r] = si[(size_t)(32 * km + 8 * (r / 4) + 4 * hh + (r % 4)) * VT + col];
  }
  auto rec_of = [&](int c) { return records + ((size_t)c * HV + hv) * REC::BYTES; };
  auto dec_of = [&](int c) { return decs + (size_t)c * HV + hv; };
  auto run = [&](const OPS& ops, int c) {
    const int tok0 = chunk_tok0[c], len = chunk_len[c];
    chunk_step<KT, VT, true>(ops, S, [&](int tm, const f32x16& acc) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int tok = 32 * tm + 8 * (r / 4) + 4 * hh + (r % 4);
        if (tok < len) o[((size_t)(tok0 + tok) * HV + hv) * VT + col] = GdrElem<T>::from_float(acc[r]);
      }
    });
  };
  const int c1 = c0 + nc;
  if constexpr (KT <= 64) {
    OPS a, b;  // two register sets: the next chunk's fragments load while the current chunk computes
    if (nc > 0) chunk_ops_load<KT, VT, true>(a, rec_of(c0), dec_of(c0), lane, vn, true);
    for (int c = c0; c < c1; c += 2) {
      if (c + 1 < c1) chunk_ops_load<KT, VT, true>(b, rec_of(c + 1), dec_of(c + 1), lane, vn, true);
      run(a, c);
      if (c + 1 < c1) {
        if (c + 2 < c1) chunk_ops_load<KT, VT, true>(a, rec_of(c + 2), dec_of(c + 2), lane, vn, true);
        run(b, c + 1);
      }
    }
  } else {
    for (int c = c0; c < c1; ++c) {
      OPS a;
      chunk_ops_load<KT, VT, true>(a, rec_of(c), dec_of(c), lane, vn, true);
      run(a, c);
    }
  }
  if (ht && (flags & SEG_LAST)) {
    float* out = ht + ((size_t)seq * HV + hv) * KT * VT;
#pragma unroll
    for (int km = 0; km < KT / 32; ++km)
#pragma unroll
      for (int r = 0; r < 16; ++r) out[(size_t)(32 * km + 8 * (r / 4) + 4 * hh + (r % 4)) * VT + col] = S[km][r];
  }
}

// ---- host side ------------------------------------------------------------------------------------------------
struct GdrWorkspace {
  int64_t off_records, off_decs, off_m, off_n, off_sinit, bytes;
};

static GdrWorkspace gdr_workspace(int64_t chunks, int64_t segs, int HV, int K, int V) {
  GdrWorkspace w;
  int64_t off = 0;
  w.off_records = off; off += lampa_align_up(chunks * HV * gdr_record_bytes(K, V), 256);
  w.off_decs = off;    off += lampa_align_up(chunks * HV * 4, 256);
  w.off_m = off;       off += lampa_align_up(segs * HV * (int64_t)K * K * 4, 256);
  w.off_n = off;       off += lampa_align_up(segs * HV * (int64_t)K * V * 4, 256);
  w.off_sinit = off;   off += lampa_align_up(segs * HV * (int64_t)K * V * 4, 256);
  w.bytes = off > 0 ? off : 256;
  return w;
}

static bool gdr_chunk_supported(int K, int V) { return (K == 64 || K == 128) && (V == 64 || V == 128); }

extern "C" int64_t lampa_gdr_chunk_workspace_bytes(int64_t total_chunks, int64_t n_segments, int HV, int K, int V) {
  if (total_chunks < 0 || n_segments < 0 || HV < 1) return LAMPA_ERR_INVALID;
  if (!gdr_chunk_supported(K, V)) return LAMPA_ERR_UNSUPPORTED;
  return gdr_workspace(total_chunks, n_segments, HV, K, V).bytes;
}

template <typename T, int KT, int VT>
static int gdr_chunk_launch(const void* q, const void* k, const void* v, const float* g, const float* beta, void* o,
                            const float* h0, float* ht, const int32_t* plan_dev, int n_seq, int chunks, int segs, int H,
                            int HV, float scale, int l2norm, unsigned char* ws, hipStream_t s) {
  const GdrWorkspace w = gdr_workspace(chunks, segs, HV, KT, VT);
  unsigned char* records = ws + w.off_records;
  float* decs = (float*)(ws + w.off_decs);
  float* Mc = (float*)(ws + w.off_m);
  float* Nc = (float*)(ws + w.off_n);
  float* Si = (float*)(ws + w.off_sinit);
  constexpr int smem = GdrPrepSmem<KT, VT>::BYTES;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)gdr_prep_kernel<T, KT, VT>, hipFuncAttributeMaxDynamicSharedMemorySize, smem) !=
        hipSuccess)
      return LAMPA_ERR_LAUNCH;
    attr_set = true;
  }
  LAMPA_PROF(s, "start");
  if (chunks > 0) {
    hipLaunchKernelGGL((gdr_prep_kernel<T, KT, VT>), dim3(chunks, HV), dim3(256), smem, s, (const T*)q, (const T*)k,
                       (const T*)v, g, beta, plan_dev, records, decs, H, HV, scale, l2norm);
    LAMPA_PROF(s, "gdr_prep_kernel");
    if (segs > n_seq) {
      hipLaunchKernelGGL((gdr_composite_kernel<KT, VT>), dim3(segs, HV), dim3(2 * (KT + VT)), 0, s, plan_dev, records,
                         decs, Mc, Nc, HV);
      LAMPA_PROF(s, "gdr_composite_kernel");
    }
  }
  hipLaunchKernelGGL((gdr_scan_kernel<KT, VT>), dim3(VT / 32, n_seq, HV), dim3(KT * 2), 0, s, plan_dev, Mc, Nc, h0, Si,
                     HV);
  LAMPA_PROF(s, "gdr_scan_kernel");
  hipLaunchKernelGGL((gdr_output_kernel<T, KT, VT>), dim3(segs, HV), dim3(2 * VT), 0, s, plan_dev, records, decs, Si,
                     (T*)o, ht, HV);
  LAMPA_PROF(s, "gdr_output_kernel");
  return lampa_launch_status();
}

// Chunkwise forward. q, k [total_tokens, H, K]; v, o [total_tokens, HV, V] (dtype 0 bf16 / 1 fp16); g, beta fp32
// [total_tokens, HV]; h0, ht fp32 [n_seq, HV, K, V] (nullable). plan_host / plan_dev: the same plan
// (lampa_gdr_plan_fill) in host and in device memory. workspace: lampa_gdr_chunk_workspace_bytes bytes.
extern "C" int lampa_gdr_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                   void* o, const float* h0, float* ht, const int32_t* plan_host,
                                   const int32_t* plan_dev, int H, int HV, int K, int V, int dtype, float scale,
                                   int l2norm, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!q || !k || !v || !g || !beta || !o || !plan_host || !plan_dev) return LAMPA_ERR_INVALID;
  if (H < 1 || HV < H || HV % H != 0 || l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (!gdr_chunk_supported(K, V) || (dtype != GDR_BF16 && dtype != GDR_FP16)) return LAMPA_ERR_UNSUPPORTED;
  const int n_seq = plan_host[PLAN_N_SEQ], chunks = plan_host[PLAN_TOTAL_CHUNKS], segs = plan_host[PLAN_N_SEGMENTS];
  if (n_seq < 1 || segs < n_seq) return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < gdr_workspace(chunks, segs, HV, K, V).bytes) return LAMPA_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  unsigned char* ws = (unsigned char*)workspace;
#define GDR_CASE(TT, KK, VV)                                                                                       \
  return gdr_chunk_launch<TT, KK, VV>(q, k, v, g, beta, o, h0, ht, plan_dev, n_seq, chunks, segs, H, HV, scale, \
                                      l2norm, ws, s)
  if (dtype == GDR_BF16) {
    if (K == 64 && V == 64) GDR_CASE(__bf16, 64, 64);
    if (K == 64 && V == 128) GDR_CASE(__bf16, 64, 128);
    if (K == 128 && V == 64) GDR_CASE(__bf16, 128, 64);
    if (K == 128 && V == 128) GDR_CASE(__bf16, 128, 128);
  } else {
    if (K == 64 && V == 64) GDR_CASE(_Float16, 64, 64);
    if (K == 64 && V == 128) GDR_CASE(_Float16, 64, 128);
    if (K == 128 && V == 64) GDR_CASE(_Float16, 128, 64);
    if (K == 128 && V == 128) GDR_CASE(_Float16, 128, 128);
  }
#undef GDR_CASE
  return LAMPA_ERR_UNSUPPORTED;
}

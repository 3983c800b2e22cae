// Backward pass of the gated-delta forward in the chunked (WY) form on the MFMA (gfx950), K = V = 64, bf16 / fp16.
//
// Replaces chunk_gated_delta_rule_bwd (reference chengjiang123/Lampa, models/hattention/gated_delta_rule_ori.py:83-160:
// chunk_bwd_dv_local chunk_o.py:372, chunk_gated_delta_rule_bwd_dhu chunk_delta_h.py:209, chunk_bwd_dqkwg chunk_o.py:128,
// prepare_wy_repr_bwd wy_fast.py:27) and the l2norm_bwd calls of ChunkGatedDeltaRuleFunction.backward
// (gated_delta_rule_ori.py:205-233).
//
// Per chunk of 64 tokens of one head (Kh, Qh the l2-normalised rows, gamma the in-chunk cumulative log-decay, S the
// state entering the chunk, G' the gradient of the loss with respect to the state leaving it):
//   forward   A = strict_lower(beta_i (kh_i . kh_j) e^{gamma_i - gamma_j}),  T = (I + A)^-1,  E = diag(e^gamma),
//             D = diag(e^{gamma_L - gamma}),  W = T B E Kh,  U = T B V,  Vn = U - W S,  S' = e^{gamma_L} S + (D Kh)^T Vn,
//             O = scale (E Qh S + P Vn),  P_ij = (qh_i . kh_j) e^{gamma_i - gamma_j}  (i >= j)
//   backward  dVn = scale P^T dO + D Kh G',   dS = e^{gamma_L} G' + scale (E Qh)^T dO - W^T dVn,
//             X = T^T dVn (dV = B X),  dW = -dVn S^T,  Xw = T^T dW,  grad A = -X Vn^T, grad P = scale dO Vn^T, ...
// Both state sequences are affine recurrences over the chunks (S' = M S + N forwards, dS = M^T G' + N' backwards, with the
// same M = e^{gamma_L} I - (D Kh)^T W), so nothing here is serial in the tokens and only a short scan is serial in the
// chunks:
//   maps   one workgroup per (chunk, head): the chunk's map (M - dI as 16-bit MFMA A-operand fragments, N in the 16-bit
//          operand type, the decay d in fp32), once for the forward direction and once for the reverse one;
//   scan   the states entering every chunk (forwards) and the gradients leaving every chunk (backwards) by a scan
//          over the maps in three levels of groups of 8 (the step of the forward pass's scan kernels; the maps of the
//          groups keep N and the states in fp32, the states in front of the chunks are stored in the operand type);
//   grads  one workgroup per (chunk, head): every gradient of the chunk from its tiles, S and G'.
#include "gdr_chunk_kernels.h"
#include <mutex>

#define GB_LS 68                    // row stride (16-bit elements) of the 64 x 64 tiles in LDS: 8-byte aligned rows
#define GB_TILE (64 * GB_LS)        // elements of one tile
#define GB_THREADS 256
#define GB_G GDR_SCAN_GROUP         // items per group of the scan levels

// ---- plan (host) -------------------------------------------------------------------------------------------------
// int32 tables, the same in host and device memory. An "item" is a chunk's map; every sequence owns one more item
// than it has chunks (the scan stores the state in front of every item and never applies a sequence's last one, so
// the slot of the extra item receives the state behind the last chunk). Forward items of a sequence are its chunks in
// order, reverse items its chunks from the last to the first.
enum {
  BP_N_SEQ = 0, BP_CHUNKS, BP_ITEMS, BP_GMAX1, BP_GMAX2,
  BP_OFF_TOK0, BP_OFF_LEN, BP_OFF_ITEM_F, BP_OFF_ITEM_R, BP_OFF_EXTRA_R,
  BP_OFF_L1G, BP_OFF_L2G, BP_OFF_TOP, BP_OFF_LEAF2, BP_OFF_LEAF1,  // each: seg0[n] then nseg[n]
  BP_HEADER = 16
};

static int64_t bp_counts(const int64_t* cu, int n_seq, int64_t* chunks, int* gmax1, int* gmax2) {
  int64_t c = 0;
  int g1 = 1, g2 = 1;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t len = cu[s + 1] - cu[s];
    if (len < 0) return -1;
    const int64_t nc = (len + GDR_C - 1) / GDR_C, items = nc + 1;
    const int n1 = (int)((items + GB_G - 1) / GB_G), n2 = (n1 + GB_G - 1) / GB_G;
    c += nc;
    g1 = n1 > g1 ? n1 : g1;
    g2 = n2 > g2 ? n2 : g2;
  }
  *chunks = c;
  *gmax1 = g1;
  *gmax2 = g2;
  return 0;
}

extern "C" int64_t lampa_gdr_bwd_chunk_plan_size(const int64_t* cu_seqlens_host, int n_seq) {
  if (!cu_seqlens_host || n_seq < 1) return LAMPA_ERR_INVALID;
  int64_t chunks;
  int g1, g2;
  if (bp_counts(cu_seqlens_host, n_seq, &chunks, &g1, &g2) != 0) return LAMPA_ERR_INVALID;
  if (cu_seqlens_host[n_seq] > INT32_MAX) return LAMPA_ERR_UNSUPPORTED;
  return BP_HEADER + 4 * chunks + n_seq + 2 * (3 * (int64_t)n_seq + (int64_t)n_seq * g2 + (int64_t)n_seq * g1);
}

extern "C" int lampa_gdr_bwd_chunk_plan_fill(const int64_t* cu_seqlens_host, int n_seq, int32_t* plan) {
  if (!plan) return LAMPA_ERR_INVALID;
  const int64_t size = lampa_gdr_bwd_chunk_plan_size(cu_seqlens_host, n_seq);
  if (size < 0) return (int)size;
  int64_t chunks;
  int g1, g2;
  bp_counts(cu_seqlens_host, n_seq, &chunks, &g1, &g2);
  int32_t* p = plan;
  for (int i = 0; i < BP_HEADER; ++i) p[i] = 0;
  p[BP_N_SEQ] = n_seq; p[BP_CHUNKS] = (int32_t)chunks; p[BP_ITEMS] = (int32_t)(chunks + n_seq);
  p[BP_GMAX1] = g1; p[BP_GMAX2] = g2;
  int64_t off = BP_HEADER;
  p[BP_OFF_TOK0] = (int32_t)off; off += chunks;
  p[BP_OFF_LEN] = (int32_t)off; off += chunks;
  p[BP_OFF_ITEM_F] = (int32_t)off; off += chunks;
  p[BP_OFF_ITEM_R] = (int32_t)off; off += chunks;
  p[BP_OFF_EXTRA_R] = (int32_t)off; off += n_seq;
  p[BP_OFF_L1G] = (int32_t)off; off += 2 * n_seq;
  p[BP_OFF_L2G] = (int32_t)off; off += 2 * n_seq;
  p[BP_OFF_TOP] = (int32_t)off; off += 2 * n_seq;
  p[BP_OFF_LEAF2] = (int32_t)off; off += 2 * (int64_t)n_seq * g2;
  p[BP_OFF_LEAF1] = (int32_t)off; off += 2 * (int64_t)n_seq * g1;
  int64_t c = 0, item = 0;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t bos = cu_seqlens_host[s], len = cu_seqlens_host[s + 1] - bos;
    const int nc = (int)((len + GDR_C - 1) / GDR_C), items = nc + 1;
    const int n1 = (items + GB_G - 1) / GB_G, n2 = (n1 + GB_G - 1) / GB_G;
    for (int i = 0; i < nc; ++i) {
      p[p[BP_OFF_TOK0] + c + i] = (int32_t)(bos + (int64_t)i * GDR_C);
      p[p[BP_OFF_LEN] + c + i] = (int32_t)(len - (int64_t)i * GDR_C < GDR_C ? len - (int64_t)i * GDR_C : GDR_C);
      p[p[BP_OFF_ITEM_F] + c + i] = (int32_t)(item + i);
      p[p[BP_OFF_ITEM_R] + c + i] = (int32_t)(item + (nc - 1 - i));
    }
    p[p[BP_OFF_EXTRA_R] + s] = (int32_t)(item + nc);
    p[p[BP_OFF_L1G] + s] = (int32_t)item;        p[p[BP_OFF_L1G] + n_seq + s] = items;
    p[p[BP_OFF_L2G] + s] = s * g1;               p[p[BP_OFF_L2G] + n_seq + s] = n1;
    p[p[BP_OFF_TOP] + s] = s * g2;               p[p[BP_OFF_TOP] + n_seq + s] = n2;
    for (int j = 0; j < g2; ++j) {  // supergroup j of the sequence: its groups (level-1 composites)
      const int cnt = n1 - j * GB_G;
      p[p[BP_OFF_LEAF2] + s * g2 + j] = s * g1 + j * GB_G;
      p[p[BP_OFF_LEAF2] + n_seq * g2 + s * g2 + j] = j < n2 ? (cnt < GB_G ? cnt : GB_G) : 0;
    }
    for (int j = 0; j < g1; ++j) {  // group j of the sequence: its items
      const int cnt = items - j * GB_G;
      p[p[BP_OFF_LEAF1] + s * g1 + j] = (int32_t)(item + (j < n1 ? j * GB_G : 0));
      p[p[BP_OFF_LEAF1] + n_seq * g1 + s * g1 + j] = j < n1 ? (cnt < GB_G ? cnt : GB_G) : 0;
    }
    c += nc;
    item += items;
  }
  return LAMPA_OK;
}

// ---- device helpers ------------------------------------------------------------------------------------------------
template <typename OT>
__device__ __forceinline__ typename OpVec<OT>::x8 gb_row(const OT* buf, int row, int k0, int hh) {
  return op_ld_kappa<OT>(buf, GB_LS, row, k0, hh);
}
template <typename OT>
__device__ __forceinline__ typename OpVec<OT>::x8 gb_tr(const OT* buf, int col0, int k0, int lane) {
  return op_ld_kappa_tr<OT, false>(buf, GB_LS, col0, k0, lane);
}

// 32 x 32 tile of a product, contraction index k0 .. k1 in steps of 16. A operand: rows a0 .. a0 + 31 of the product;
// ATR false: buffer A[row][k], true: buffer A[k][row]. B operand: columns b0 .. b0 + 31 of the product; BTR false:
// buffer B[col][k], true: buffer B[k][col].
template <typename OT, bool ATR, bool BTR>
__device__ __forceinline__ f32x16 gb_mm(const OT* A, int a0, const OT* B, int b0, int k0, int k1, f32x16 acc, int lane) {
  const int hh = lane >> 5, ln = lane & 31;
  for (int ks = k0; ks < k1; ks += 16) {
    const typename OpVec<OT>::x8 fa = ATR ? gb_tr<OT>(A, a0, ks, lane) : gb_row<OT>(A, a0 + ln, ks, hh);
    const typename OpVec<OT>::x8 fb = BTR ? gb_tr<OT>(B, b0, ks, lane) : gb_row<OT>(B, b0 + ln, ks, hh);
    acc = mfma32(fa, fb, acc);
  }
  return acc;
}

// accumulator tile -> rows r0 .., columns c0 .. of a 16-bit LDS tile
template <typename OT>
__device__ __forceinline__ void gb_store(OT* buf, int r0, int c0, const f32x16& acc, int lane) {
  const int hh = lane >> 5, ln = lane & 31;
#pragma unroll
  for (int r = 0; r < 16; ++r) buf[(r0 + acc_row(r, hh)) * GB_LS + c0 + ln] = (OT)acc[r];
}

// this lane's 16 accumulator rows' worth of a per-row factor (rows r0 + 8 b + 4 hh + e)
__device__ __forceinline__ void gb_row_factors(const float* f, int r0, int hh, float* out) {
#pragma unroll
  for (int b4 = 0; b4 < 4; ++b4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(&f[r0 + 8 * b4 + 4 * hh]);
#pragma unroll
    for (int e = 0; e < 4; ++e) out[4 * b4 + e] = t[e];
  }
}

// the elements of a 16-bit LDS tile that sit where this lane's accumulator registers sit: rows r0 + ..., column c0 + ln
template <typename OT>
__device__ __forceinline__ void gb_acc_view(const OT* buf, int r0, int c0, int lane, float* out) {
#pragma unroll
  for (int b4 = 0; b4 < 4; ++b4) {
    const typename OpVec<OT>::x4 t = op_ld_col4<OT>(buf, GB_LS, c0, r0 + 8 * b4, lane);
#pragma unroll
    for (int e = 0; e < 4; ++e) out[4 * b4 + e] = (float)t[e];
  }
}

// sum over the 32 lanes of this lane's half of the wave (every lane of the half receives it)
__device__ __forceinline__ float gb_half_sum(float x) {
  x += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, x);
  x += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, x);
  x += dpp_f32<0x141, 0xF>(0.0f, x);  // row_half_mirror
  x += dpp_f32<0x140, 0xF>(0.0f, x);  // row_mirror
  x += __shfl_xor(x, 16);
  return x;
}
// sum over the 8 consecutive lanes that share lane / 8
__device__ __forceinline__ float gb_sum8(float x) {
  x += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, x);
  x += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, x);
  x += dpp_f32<0x141, 0xF>(0.0f, x);
  return x;
}

// 64 rows x 64 columns of 16-bit elements from global memory (row stride `ld` elements) into an LDS tile; rows from
// `len` on become zero; with `norm` every row is scaled by its l2 factor (stored to rfac when given) and rounded once.
template <typename T, typename OT>
__device__ __forceinline__ void gb_stage_rows(const T* src, int64_t ld, int len, OT* dst, int l2norm, bool norm,
                                              float* rfac, const float* rfac_in) {
  using X4 = typename OpVec<OT>::x4;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int p = threadIdx.x + GB_THREADS * u, row = p >> 3, part = p & 7;
    typename Raw8<T>::type raw;
#pragma unroll
    for (int e = 0; e < 8; ++e) raw[e] = (T)0.0f;
    if (row < len) raw = *reinterpret_cast<const typename Raw8<T>::type*>(src + (int64_t)row * ld + 8 * part);
    float f[8], ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { f[e] = (float)raw[e]; ss = __builtin_fmaf(f[e], f[e], ss); }
    float c = 1.0f;
    if (norm) {
      if (rfac_in) c = rfac_in[row];
      else c = l2_factor(gb_sum8(ss), l2norm);
      if (rfac && part == 0) rfac[row] = c;
    }
    X4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) { lo[e] = (OT)(f[e] * c); hi[e] = (OT)(f[4 + e] * c); }
    *reinterpret_cast<X4*>(&dst[row * GB_LS + 8 * part]) = lo;
    *reinterpret_cast<X4*>(&dst[row * GB_LS + 8 * part + 4]) = hi;
  }
}

// T of a record (block T21 full, the diagonal blocks packed by rows) as a full 64 x 64 tile, zeros above the diagonal
template <typename OT>
__device__ __forceinline__ void gb_stage_T(const unsigned char* rec, OT* dst) {
  using X8 = typename OpVec<OT>::x8;
  using X4 = typename OpVec<OT>::x4;
  X4 z;
#pragma unroll
  for (int e = 0; e < 4; ++e) z[e] = (OT)0.0f;
  auto put = [&](int row, int col, X8 v) {
    X4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) { lo[e] = v[e]; hi[e] = v[4 + e]; }
    *reinterpret_cast<X4*>(&dst[row * GB_LS + col]) = lo;
    *reinterpret_cast<X4*>(&dst[row * GB_LS + col + 4]) = hi;
  };
  const X8* tp = reinterpret_cast<const X8*>(rec);
  const int t = threadIdx.x;
  // zero everything first (512 pieces), then the stored pieces
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int p = t + GB_THREADS * u;
    *reinterpret_cast<X4*>(&dst[(p >> 3) * GB_LS + 8 * (p & 7)]) = z;
    *reinterpret_cast<X4*>(&dst[(p >> 3) * GB_LS + 8 * (p & 7) + 4]) = z;
  }
  __syncthreads();
  if (t < 128) put(32 + (t >> 2), 8 * (t & 3), tp[t]);  // T21
  if (t < 2 * T_DIAG_PIECES) {
    const int blk = t >= T_DIAG_PIECES, pc = t - blk * T_DIAG_PIECES;
    int row, part;
    tri_piece(pc, row, part);
    put(32 * blk + row, 32 * blk + 8 * part, tp[128 + t]);
  }
}

// a state (or state gradient) stored by the scan as 32-column slabs in accumulator order -> K x V tile in LDS
template <typename OT>
__device__ __forceinline__ void gb_stage_state(const OT* slabs, OT* dst) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int idx = threadIdx.x + GB_THREADS * u;  // f32x4 index: ((vn * 2 + w) * 4 + q4) * 64 + lane
    const int lane = idx & 63, q4 = (idx >> 6) & 3, w = (idx >> 8) & 1, vn = idx >> 9;
    const typename OpVec<OT>::x4 t = reinterpret_cast<const typename OpVec<OT>::x4*>(slabs)[idx];
    const int row = 32 * w + 8 * q4 + 4 * (lane >> 5), col = 32 * vn + (lane & 31);
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[(row + e) * GB_LS + col] = t[e];
  }
}

// per-token factors of a chunk from its record: gamma (log2 units), beta, rk; e^gamma, e^{gamma_L - gamma}
struct GbFactors {
  float *gam, *beta, *eg, *dk, *rk, *rq;
};
__device__ __forceinline__ void gb_stage_factors(const unsigned char* rec, const GbFactors& f) {
  const float* fact = reinterpret_cast<const float*>(rec + T_BYTES);
  if (threadIdx.x < 64) {
    const int i = threadIdx.x;
    const float g = fact[i], gl = fact[63];
    f.gam[i] = g;
    f.beta[i] = fact[64 + i];
    f.rk[i] = fact[128 + i];
    f.eg[i] = __builtin_amdgcn_exp2f(g);
    f.dk[i] = __builtin_amdgcn_exp2f(gl - g);
  }
}

// M' (K x K accumulator tile: rows a = 32 tr + ..., column b = 32 tc + ln) into the 16-bit A-operand fragment order the
// scan reads; `transposed` stores the element at (b, a) instead.
template <typename OT>
__device__ __forceinline__ void gb_store_mprime(unsigned char* out, int tr, int tc, const f32x16& acc, int lane,
                                                bool transposed) {
  const int hh = lane >> 5, ln = lane & 31;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int a = 32 * tr + acc_row(r, hh), b = 32 * tc + ln;
    const int row = transposed ? b : a, col = transposed ? a : b;
    const int km = row >> 5, ks = col >> 4, c16 = col & 15;
    const int hs = (c16 >> 2) & 1, slot = 4 * (c16 >> 3) + (c16 & 3);
    *reinterpret_cast<OT*>(out + ((size_t)((km * 4 + ks) * 64 + 32 * hs + (row & 31))) * 16 + 2 * slot) = (OT)acc[r];
  }
}

// ---- maps kernel -----------------------------------------------------------------------------------------------------
// grid (chunks, HV), 256 threads. REV false: M' = -(D Kh)^T W, N = (D Kh)^T U. REV true: M'^T and
// N' = scale (E Qh)^T dO - W^T (scale P^T dO), stored at the chunk's reverse item.
template <typename T, bool REV>
__global__ void __launch_bounds__(GB_THREADS, 3)
    gdrb_maps_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const T* __restrict__ dout,
                     const unsigned char* __restrict__ recs, const int32_t* __restrict__ chunk_tok0,
                     const int32_t* __restrict__ chunk_len, const int32_t* __restrict__ chunk_item,
                     unsigned char* __restrict__ Mout, T* __restrict__ Nout, float* __restrict__ Dout, int H, int HV,
                     float scale, int l2norm) {
  using OT = T;
  extern __shared__ __align__(16) unsigned char smem[];
  OT* b_k = reinterpret_cast<OT*>(smem);
  OT* b_a = b_k + GB_TILE;      // fwd: v -> beta v;      rev: q -> scale e^gamma qh
  OT* b_t = b_a + GB_TILE;      // T;                     rev: later P
  OT* b_bk = b_t + GB_TILE;     // beta e^gamma kh, later e^{gamma_L - gamma} kh
  OT* b_w = b_bk + GB_TILE;     // W
  OT* b_u = b_w + GB_TILE;      // fwd: U;                rev: dO
  OT* b_y = b_bk;               // rev: -scale P^T dO, over the scaled k tile once M'^T is done
  float* fbase = reinterpret_cast<float*>(b_u + GB_TILE);
  GbFactors f{fbase, fbase + 64, fbase + 128, fbase + 192, fbase + 256, fbase + 320};

  const int chunk = blockIdx.x, hv = blockIdx.y, h = hv / (HV / H);
  const int tok0 = chunk_tok0[chunk], len = chunk_len[chunk], item = chunk_item[chunk];
  const unsigned char* rec = recs + ((size_t)chunk * HV + hv) * REC_BYTES;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tr = wave >> 1, tc = wave & 1, hh = lane >> 5, ln = lane & 31;

  gb_stage_factors(rec, f);
  gb_stage_T<OT>(rec, b_t);
  __syncthreads();
  gb_stage_rows<T, OT>(k + ((size_t)tok0 * H + h) * 64, (int64_t)H * 64, len, b_k, l2norm, true, nullptr, f.rk);
  if (!REV) {
    gb_stage_rows<T, OT>(v + ((size_t)tok0 * HV + hv) * 64, (int64_t)HV * 64, len, b_a, 0, false, nullptr, nullptr);
  } else {
    gb_stage_rows<T, OT>(q + ((size_t)tok0 * H + h) * 64, (int64_t)H * 64, len, b_a, l2norm, true, f.rq, nullptr);
    gb_stage_rows<T, OT>(dout + ((size_t)tok0 * HV + hv) * 64, (int64_t)HV * 64, len, b_u, 0, false, nullptr, nullptr);
  }
  __syncthreads();
  // row-scaled copies: beta e^gamma kh (and beta v in place)
  {
    using X4 = typename OpVec<OT>::x4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = threadIdx.x + GB_THREADS * u, row = p >> 4, c4 = 4 * (p & 15);
      const float fb = f.beta[row], fe = fb * f.eg[row];
      const X4 kk = *reinterpret_cast<const X4*>(&b_k[row * GB_LS + c4]);
      X4 o1;
#pragma unroll
      for (int e = 0; e < 4; ++e) o1[e] = (OT)((float)kk[e] * fe);
      *reinterpret_cast<X4*>(&b_bk[row * GB_LS + c4]) = o1;
      if (!REV) {
        const X4 vv = *reinterpret_cast<const X4*>(&b_a[row * GB_LS + c4]);
        X4 o2;
#pragma unroll
        for (int e = 0; e < 4; ++e) o2[e] = (OT)((float)vv[e] * fb);
        *reinterpret_cast<X4*>(&b_a[row * GB_LS + c4]) = o2;
      }
    }
  }
  __syncthreads();
  // W = T (beta e^gamma Kh), U = T (beta V): T is lower triangular
  {
    const f32x16 w = gb_mm<OT, false, true>(b_t, 32 * tr, b_bk, 32 * tc, 0, 32 * (tr + 1), zero16(), lane);
    gb_store<OT>(b_w, 32 * tr, 32 * tc, w, lane);
    if (!REV) {
      const f32x16 uu = gb_mm<OT, false, true>(b_t, 32 * tr, b_a, 32 * tc, 0, 32 * (tr + 1), zero16(), lane);
      gb_store<OT>(b_u, 32 * tr, 32 * tc, uu, lane);
    }
  }
  __syncthreads();
  // e^{gamma_L - gamma} kh over the scaled copy; rev: P into T's tile
  {
    using X4 = typename OpVec<OT>::x4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = threadIdx.x + GB_THREADS * u, row = p >> 4, c4 = 4 * (p & 15);
      const float fd = f.dk[row];
      const X4 kk = *reinterpret_cast<const X4*>(&b_k[row * GB_LS + c4]);
      X4 o1;
#pragma unroll
      for (int e = 0; e < 4; ++e) o1[e] = (OT)((float)kk[e] * fd);
      *reinterpret_cast<X4*>(&b_bk[row * GB_LS + c4]) = o1;
    }
  }
  if (REV) {  // P (rows i, columns j) with scale, zero above the diagonal
    f32x16 p = zero16();
    if (tr >= tc) {
      p = gb_mm<OT, false, false>(b_a, 32 * tr, b_k, 32 * tc, 0, 64, zero16(), lane);
      float gi[16];
      gb_row_factors(f.gam, 32 * tr, hh, gi);
      const float gj = f.gam[32 * tc + ln];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 32 * tr + acc_row(r, hh), j = 32 * tc + ln;
        p[r] = i >= j ? scale * p[r] * __builtin_amdgcn_exp2f(gi[r] - gj) : 0.0f;
      }
    }
    gb_store<OT>(b_t, 32 * tr, 32 * tc, p, lane);
  }
  __syncthreads();
  unsigned char* mo = Mout + ((size_t)item * HV + hv) * (64 * 64 * 2);
  OT* no = Nout + (((size_t)item * HV + hv) * 2 + tc) * (64 * 32);  // N rounded to the operand type, accumulator order
  auto store_n = [&](const f32x16& n) {
    using X4 = typename OpVec<OT>::x4;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      X4 t;
#pragma unroll
      for (int e = 0; e < 4; ++e) t[e] = (OT)n[4 * q4 + e];
      reinterpret_cast<X4*>(no)[(tr * 4 + q4) * 64 + lane] = t;
    }
  };
  if (!REV) {
    f32x16 m = gb_mm<OT, true, true>(b_bk, 32 * tr, b_w, 32 * tc, 0, 64, zero16(), lane);
#pragma unroll
    for (int r = 0; r < 16; ++r) m[r] = -m[r];
    gb_store_mprime<OT>(mo, tr, tc, m, lane, false);
    store_n(gb_mm<OT, true, true>(b_bk, 32 * tr, b_u, 32 * tc, 0, 64, zero16(), lane));
  } else {
    // M'^T = -W^T (D Kh): rows a of W^T, columns b of D Kh
    f32x16 m = gb_mm<OT, true, true>(b_w, 32 * tr, b_bk, 32 * tc, 0, 64, zero16(), lane);
#pragma unroll
    for (int r = 0; r < 16; ++r) m[r] = -m[r];
    gb_store_mprime<OT>(mo, tr, tc, m, lane, false);
    // -Y = -(scale P)^T dO: contraction over the rows i of P (i >= j)
    f32x16 y = gb_mm<OT, true, true>(b_t, 32 * tr, b_u, 32 * tc, 32 * tr, 64, zero16(), lane);
#pragma unroll
    for (int r = 0; r < 16; ++r) y[r] = -y[r];
    __syncthreads();  // every wave is past its reads of the scaled k tile (M'^T) and of qh (P)
    gb_store<OT>(b_y, 32 * tr, 32 * tc, y, lane);
    // scale e^gamma qh in place (every wave is past its reads of qh: P was stored behind the barrier above)
    {
      using X4 = typename OpVec<OT>::x4;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int p = threadIdx.x + GB_THREADS * u, row = p >> 4, c4 = 4 * (p & 15);
        const float fe = scale * f.eg[row];
        const X4 qq = *reinterpret_cast<const X4*>(&b_a[row * GB_LS + c4]);
        X4 o1;
#pragma unroll
        for (int e = 0; e < 4; ++e) o1[e] = (OT)((float)qq[e] * fe);
        *reinterpret_cast<X4*>(&b_a[row * GB_LS + c4]) = o1;
      }
    }
    __syncthreads();
    f32x16 n = gb_mm<OT, true, true>(b_a, 32 * tr, b_u, 32 * tc, 0, 64, zero16(), lane);
    n = gb_mm<OT, true, true>(b_w, 32 * tr, b_y, 32 * tc, 0, 64, n, lane);
    store_n(n);
  }
  if (threadIdx.x == 0) Dout[(size_t)item * HV + hv] = __builtin_amdgcn_exp2f(f.gam[63]);
}

// ---- scans over a level's items ------------------------------------------------------------------------------------
// Same step as the forward pass's scan kernels (S <- d S + N + M' S per item, wave w owning rows 32 w .. of a 32-column
// slab, the other wave's rows as B operand through LDS). The items of the lowest level (the chunks' maps) carry N in
// the 16-bit operand type (N16), and the states in front of the chunks are stored in that type as well (OUT16): the
// gradients kernel uses them as MFMA operands only.
template <typename OT, bool N16>
__device__ __forceinline__ void gdrb_load_n(const unsigned char* Ncomp, size_t slab, int wave, int lane, f32x4* n) {
  if constexpr (N16) {
    using X4 = typename OpVec<OT>::x4;
    const X4* N = reinterpret_cast<const X4*>(Ncomp + slab * (64 * 32 * 2));
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const X4 t = N[(wave * 4 + q4) * 64 + lane];
#pragma unroll
      for (int e = 0; e < 4; ++e) n[q4][e] = (float)t[e];
    }
  } else {
    const f32x4* N = reinterpret_cast<const f32x4*>(Ncomp + slab * (64 * 32 * 4));
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) n[q4] = N[(wave * 4 + q4) * 64 + lane];
  }
}

// The state in front of every item of a "sequence" of the level. Start state: [n, HV, K, V] rows (H0_SLABS false, may
// be NULL) or the fp32 slabs the level above left at slot `seq`.
// grid (1, sequences of the level, HV), 4 waves: waves 2 vn, 2 vn + 1 own the 32-column slab vn (both slabs in one
// workgroup read the same M' fragments, which then come from the CU's L1 the second time).
template <typename OT, bool H0_SLABS, bool N16, bool OUT16>
__global__ void __launch_bounds__(256) gdrb_scan_kernel(const int32_t* __restrict__ seg0s, const int32_t* __restrict__ nsegs,
                                                        const unsigned char* __restrict__ Mcomp,
                                                        const unsigned char* __restrict__ Ncomp,
                                                        const float* __restrict__ Dcomp, const float* __restrict__ h0,
                                                        void* __restrict__ Sinit, int HV, int spare_slot) {
  using X8 = typename OpVec<OT>::x8;
  using X4 = typename OpVec<OT>::x4;
  constexpr int KT = 64, VT = 64, NKS = KT / 16, DEPTH = 4;
  constexpr int M_BYTES = KT * KT * 2;
  __shared__ __align__(16) unsigned char s_xx[2][2][NKS * 1024];
  const int vn = threadIdx.x >> 7, seq = blockIdx.y, hv = blockIdx.z;
  const int seg0 = seg0s[seq], nseg = nsegs[seq];
  if (nseg <= 0) return;
  const int nsteps = nseg - 1;
  const int tid = threadIdx.x & 127, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  const int col = 32 * vn + ln;
  unsigned char (*s_x)[NKS * 1024] = s_xx[vn];
  f32x16 S = zero16();
  if (H0_SLABS) {
    const f32x4* src = reinterpret_cast<const f32x4*>(h0 + (((size_t)seq * HV + hv) * (VT / 32) + vn) * (KT * 32));
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const f32x4 t = src[(wave * 4 + q4) * 64 + lane];
#pragma unroll
      for (int e = 0; e < 4; ++e) S[4 * q4 + e] = t[e];
    }
  } else if (h0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = h0[(((size_t)seq * HV + hv) * KT + 32 * wave + acc_row(r, hh)) * VT + col];
  }
  X8 rm[DEPTH][NKS];
  f32x4 rn[DEPTH][4];
  float rd[DEPTH];
  auto issue = [&](int p, X8* m, f32x4* n, float& d) {
    const size_t sh = (size_t)(seg0 + p) * HV + hv;
    const X8* M = reinterpret_cast<const X8*>(Mcomp + sh * M_BYTES);
#pragma unroll
    for (int j = 0; j < NKS; ++j) m[j] = M[(wave * NKS + (2 * wave + j) % NKS) * 64 + lane];
    gdrb_load_n<OT, N16>(Ncomp, sh * (VT / 32) + vn, wave, lane, n);
    d = Dcomp[sh];
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue(max(0, min(d, nsteps - 1)), rm[d], rn[d], rd[d]);
  auto step = [&](int p, X8* m, f32x4* n, float& dd) {
    {
      const size_t slot = p <= nsteps ? (size_t)(seg0 + p) : (size_t)spare_slot;
      const size_t slab = (slot * HV + hv) * (VT / 32) + vn;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        if constexpr (OUT16) {
          X4 t;
#pragma unroll
          for (int e = 0; e < 4; ++e) t[e] = (OT)S[4 * q4 + e];
          reinterpret_cast<X4*>(reinterpret_cast<OT*>(Sinit) + slab * (KT * 32))[(wave * 4 + q4) * 64 + lane] = t;
        } else {
          f32x4 t;
#pragma unroll
          for (int e = 0; e < 4; ++e) t[e] = S[4 * q4 + e];
          reinterpret_cast<f32x4*>(reinterpret_cast<float*>(Sinit) + slab * (KT * 32))[(wave * 4 + q4) * 64 + lane] = t;
        }
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
  for (int p0 = 0; p0 <= nsteps; p0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) step(p0 + d, rm[d], rn[d], rd[d]);
  }
}

// Composite of every full group of GB_G items of a sequence but the last (which nothing follows): the step applied to
// the 64 + 64 columns [P_M | P_N] from [I | 0]; stored like an item (D = the product of the decays, M' = P_M - D I as
// 16-bit A-operand fragments, N = P_N in fp32) at slot seq * gmax + group.
// grid (gmax, n_seq, HV), 8 waves: waves 2 b, 2 b + 1 own the 32-column block b of [P_M | P_N].
template <typename OT, bool N16>
__global__ void __launch_bounds__(512, 4) gdrb_group_kernel(const int32_t* __restrict__ seg0s, const int32_t* __restrict__ nsegs,
                                                         const unsigned char* __restrict__ Msrc,
                                                         const unsigned char* __restrict__ Nsrc,
                                                         const float* __restrict__ Dsrc, unsigned char* __restrict__ Mout,
                                                         float* __restrict__ Nout, float* __restrict__ Dout, int HV,
                                                         int gmax) {
  using X8 = typename OpVec<OT>::x8;
  constexpr int KT = 64, VT = 64, NKS = KT / 16, DEPTH = 2, G = GB_G;  // (two items in flight: 128 registers)
  constexpr int M_BYTES = KT * KT * 2;
  __shared__ __align__(16) unsigned char s_xx[4][2][NKS * 1024];
  const int vn = threadIdx.x >> 7, j = blockIdx.x, seq = blockIdx.y, hv = blockIdx.z;
  const int seg0 = seg0s[seq], nseg = nsegs[seq];
  const int ngroups = (nseg + G - 1) / G;
  if (j >= ngroups - 1) return;
  const int item0 = seg0 + j * G;
  const int tid = threadIdx.x & 127, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  unsigned char (*s_x)[NKS * 1024] = s_xx[vn];
  const bool is_pm = vn < KT / 32;
  const int nblk = max(vn - KT / 32, 0);
  f32x16 S = zero16();
  if (is_pm) {
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = (32 * wave + acc_row(r, hh) == 32 * vn + ln) ? 1.0f : 0.0f;
  }
  X8 rm[DEPTH][NKS];
  f32x4 rn[DEPTH][4];
  float rd[DEPTH];
  auto issue = [&](int p, X8* m, f32x4* n, float& d) {
    const size_t sh = (size_t)(item0 + p) * HV + hv;
    const X8* M = reinterpret_cast<const X8*>(Msrc + sh * M_BYTES);
#pragma unroll
    for (int f = 0; f < NKS; ++f) m[f] = M[(wave * NKS + (2 * wave + f) % NKS) * 64 + lane];
    gdrb_load_n<OT, N16>(Nsrc, sh * (VT / 32) + nblk, wave, lane, n);
    d = Dsrc[sh];
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue(d, rm[d], rn[d], rd[d]);
  float dprod = 1.0f;
  auto step = [&](int p, X8* m, f32x4* n, float& dd) {
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
    issue(min(p + DEPTH, G - 1), m, n, dd);
  };
  for (int p0 = 0; p0 < G; p0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) step(p0 + d, rm[d], rn[d], rd[d]);
  }
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
    f32x4* out = reinterpret_cast<f32x4*>(Nout + (gh * (VT / 32) + nblk) * (KT * 32));
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f32x4 t;
#pragma unroll
      for (int e = 0; e < 4; ++e) t[e] = S[4 * q4 + e];
      out[(wave * 4 + q4) * 64 + lane] = t;
    }
  }
}

// the state a scan left in slab order at slot[seq] -> [n_seq, HV, K, V] rows (d(initial state))
template <typename OT>
__global__ void __launch_bounds__(GB_THREADS) gdrb_unslab_kernel(const OT* __restrict__ slabs,
                                                                 const int32_t* __restrict__ slot, float* __restrict__ out,
                                                                 int HV) {
  using X4 = typename OpVec<OT>::x4;
  const int seq = blockIdx.x, hv = blockIdx.y;
  const OT* src = slabs + ((size_t)slot[seq] * HV + hv) * (64 * 64);
  float* dst = out + ((size_t)seq * HV + hv) * (64 * 64);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int idx = threadIdx.x + GB_THREADS * u;
    const int lane = idx & 63, q4 = (idx >> 6) & 3, w = (idx >> 8) & 1, vn = idx >> 9;
    const X4 t = reinterpret_cast<const X4*>(src)[idx];
    const int row = 32 * w + 8 * q4 + 4 * (lane >> 5), col = 32 * vn + (lane & 31);
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[(row + e) * 64 + col] = (float)t[e];
  }
}

// ---- gradients kernel ----------------------------------------------------------------------------------------------
// grid (chunks, HV), 256 threads; H == HV (every value head has its own q / k head).
template <typename T>
__global__ void __launch_bounds__(GB_THREADS, 2)
    gdrb_grads_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const T* __restrict__ dout,
                      const unsigned char* __restrict__ recs, const int32_t* __restrict__ chunk_tok0,
                      const int32_t* __restrict__ chunk_len, const int32_t* __restrict__ item_f,
                      const int32_t* __restrict__ item_r, const T* __restrict__ Sf, const T* __restrict__ Sr,
                      T* __restrict__ dq, T* __restrict__ dk, T* __restrict__ dv, float* __restrict__ dg,
                      float* __restrict__ dbeta, int H, int HV, float scale, int l2norm) {
  using OT = T;
  extern __shared__ __align__(16) unsigned char smem[];
  OT* b_k = reinterpret_cast<OT*>(smem);
  OT* b_q = b_k + GB_TILE;
  OT* b_v = b_q + GB_TILE;    // v, then Vn
  OT* b_do = b_v + GB_TILE;
  OT* b_s = b_do + GB_TILE;   // S   [K][V]
  OT* b_g = b_s + GB_TILE;    // G'  [K][V]
  OT* b_t = b_g + GB_TILE;    // T, then N
  OT* b_r = b_t + GB_TILE;    // R, dVn, dW, Xw
  OT* b_x = b_r + GB_TILE;    // X, then M
  float* fbase = reinterpret_cast<float*>(b_x + GB_TILE);
  GbFactors f{fbase, fbase + 64, fbase + 128, fbase + 192, fbase + 256, fbase + 320};
  float* s_dgam = fbase + 384;
  float* s_dbeta = fbase + 448;
  float* s_misc = fbase + 512;  // [0] the terms of d gamma that belong to the chunk's last row
  float* f_dk = reinterpret_cast<float*>(b_v);          // at the end: d Kh and d Qh in fp32 over the dead tiles
  float* f_dq = f_dk + 64 * 64;

  const int chunk = blockIdx.x, hv = blockIdx.y, h = hv / (HV / H);
  const int tok0 = chunk_tok0[chunk], len = chunk_len[chunk];
  const unsigned char* rec = recs + ((size_t)chunk * HV + hv) * REC_BYTES;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, tr = wave >> 1, tc = wave & 1, hh = lane >> 5, ln = lane & 31;
  const T* qg = q + ((size_t)tok0 * H + h) * 64;
  const T* kg = k + ((size_t)tok0 * H + h) * 64;
  const T* vg = v + ((size_t)tok0 * HV + hv) * 64;
  const T* og = dout + ((size_t)tok0 * HV + hv) * 64;

  gb_stage_factors(rec, f);
  gb_stage_T<OT>(rec, b_t);
  if (threadIdx.x < 64) { s_dgam[threadIdx.x] = 0.0f; }
  if (threadIdx.x == 0) s_misc[0] = 0.0f;
  __syncthreads();
  gb_stage_rows<T, OT>(kg, (int64_t)H * 64, len, b_k, l2norm, true, nullptr, f.rk);
  gb_stage_rows<T, OT>(qg, (int64_t)H * 64, len, b_q, l2norm, true, f.rq, nullptr);
  gb_stage_rows<T, OT>(vg, (int64_t)HV * 64, len, b_v, 0, false, nullptr, nullptr);
  gb_stage_rows<T, OT>(og, (int64_t)HV * 64, len, b_do, 0, false, nullptr, nullptr);
  gb_stage_state<OT>(Sf + ((size_t)item_f[chunk] * HV + hv) * (64 * 64), b_s);
  gb_stage_state<OT>(Sr + ((size_t)item_r[chunk] * HV + hv) * (64 * 64), b_g);
  __syncthreads();

  float rs_g[16], rs_b[16], cs = 0.0f, gl = 0.0f;  // row sums of d gamma / d beta, column sums of d gamma, last-row terms
#pragma unroll
  for (int r = 0; r < 16; ++r) { rs_g[r] = 0.0f; rs_b[r] = 0.0f; }
  float bi[16], egi[16], gi[16];
  gb_row_factors(f.beta, 32 * tr, hh, bi);
  gb_row_factors(f.eg, 32 * tr, hh, egi);
  gb_row_factors(f.gam, 32 * tr, hh, gi);

  // (a) R = beta (v - e^gamma (Kh S))
  {
    f32x16 acc = gb_mm<OT, false, true>(b_k, 32 * tr, b_s, 32 * tc, 0, 64, zero16(), lane);
    float vv[16];
    gb_acc_view<OT>(b_v, 32 * tr, 32 * tc, lane, vv);
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = bi[r] * (vv[r] - egi[r] * acc[r]);
    gb_store<OT>(b_r, 32 * tr, 32 * tc, acc, lane);
  }
  __syncthreads();
  // (b) Vn = T R over v's tile
  {
    const f32x16 acc = gb_mm<OT, false, true>(b_t, 32 * tr, b_r, 32 * tc, 0, 32 * (tr + 1), zero16(), lane);
    gb_store<OT>(b_v, 32 * tr, 32 * tc, acc, lane);
  }
  __syncthreads();
  // (c) dVn = (scale P)^T dO + D (Kh G')   (tile: rows j = 32 tr + ..., value columns 32 tc + ...)
  {
    f32x16 acc = zero16();
    const float gjl = f.gam[32 * tr + ln];
    for (int I = tr; I < 2; ++I) {
      f32x16 p = gb_mm<OT, false, false>(b_q, 32 * I, b_k, 32 * tr, 0, 64, zero16(), lane);
      float gI[16];
      gb_row_factors(f.gam, 32 * I, hh, gI);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 32 * I + acc_row(r, hh), j = 32 * tr + ln;
        p[r] = i >= j ? scale * p[r] * __builtin_amdgcn_exp2f(gI[r] - gjl) : 0.0f;
      }
      // the tile read as an A operand is its transpose: rows j, contraction over its rows i
#pragma unroll
      for (int half = 0; half < 2; ++half)
        acc = mfma32(acc_to_op<OT>(p, 8 * half), gb_tr<OT>(b_do, 32 * tc, 32 * I + 16 * half, lane), acc);
    }
    const f32x16 a2 = gb_mm<OT, false, true>(b_k, 32 * tr, b_g, 32 * tc, 0, 64, zero16(), lane);
    float dkj[16];
    gb_row_factors(f.dk, 32 * tr, hh, dkj);
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] += dkj[r] * a2[r];
    gb_store<OT>(b_r, 32 * tr, 32 * tc, acc, lane);  // (R is dead: every wave is past (b))
  }
  __syncthreads();
  // (d) X = T^T dVn: contraction over the rows i >= j of T
  {
    const f32x16 acc = gb_mm<OT, true, true>(b_t, 32 * tr, b_r, 32 * tc, 32 * tr, 64, zero16(), lane);
    gb_store<OT>(b_x, 32 * tr, 32 * tc, acc, lane);
  }
  __syncthreads();
  {  // rows of X: dv = beta X, d beta = X . v (v read again from memory: its tile holds Vn now)
    const int row = threadIdx.x >> 2, c0 = 16 * (threadIdx.x & 3);
    float x[16], dot = 0.0f;
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const typename OpVec<OT>::x4 t = *reinterpret_cast<const typename OpVec<OT>::x4*>(&b_x[row * GB_LS + c0 + 4 * e4]);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * e4 + e] = (float)t[e];
    }
    if (row < len) {
      const typename Raw8<T>::type v0 = *reinterpret_cast<const typename Raw8<T>::type*>(vg + (size_t)row * HV * 64 + c0);
      const typename Raw8<T>::type v1 = *reinterpret_cast<const typename Raw8<T>::type*>(vg + (size_t)row * HV * 64 + c0 + 8);
      typename Raw8<T>::type o0, o1;
      const float b = f.beta[row];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        dot += x[e] * (float)v0[e] + x[8 + e] * (float)v1[e];
        o0[e] = (T)(b * x[e]);
        o1[e] = (T)(b * x[8 + e]);
      }
      T* dvp = dv + ((size_t)(tok0 + row) * HV + hv) * 64 + c0;
      *reinterpret_cast<typename Raw8<T>::type*>(dvp) = o0;
      *reinterpret_cast<typename Raw8<T>::type*>(dvp + 8) = o1;
    }
    dot += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, dot);
    dot += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, dot);
    if ((threadIdx.x & 3) == 0) s_dbeta[row] = dot;
  }
  // (g) grad A = -X Vn^T with the gating of A: M_ij = grad A_ij beta_i Gamma_ij (i > j)
  f32x16 m = zero16();
  if (tr >= tc) {
    const f32x16 da = gb_mm<OT, false, false>(b_x, 32 * tr, b_v, 32 * tc, 0, 64, zero16(), lane);
    const f32x16 kk = gb_mm<OT, false, false>(b_k, 32 * tr, b_k, 32 * tc, 0, 64, zero16(), lane);
    const float gj = f.gam[32 * tc + ln];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * tr + acc_row(r, hh), j = 32 * tc + ln;
      const float gam = i > j ? __builtin_amdgcn_exp2f(gi[r] - gj) : 0.0f;
      const float ga = -da[r], gk = kk[r] * gam;    // grad A_ij, (kh_i . kh_j) Gamma_ij
      const float a = ga * bi[r] * gk;              // grad A_ij A_ij
      rs_g[r] += a;
      cs -= a;
      rs_b[r] += ga * gk;
      m[r] = ga * bi[r] * gam;
    }
  }
  // (e) dW = -dVn S^T
  f32x16 dw = gb_mm<OT, false, false>(b_r, 32 * tr, b_s, 32 * tc, 0, 64, zero16(), lane);
#pragma unroll
  for (int r = 0; r < 16; ++r) dw[r] = -dw[r];
  __syncthreads();  // every wave is past its reads of X and dVn
  gb_store<OT>(b_x, 32 * tr, 32 * tc, m, lane);
  gb_store<OT>(b_r, 32 * tr, 32 * tc, dw, lane);
  __syncthreads();
  // (f) Xw = T^T dW
  {
    const f32x16 xw = gb_mm<OT, true, true>(b_t, 32 * tr, b_r, 32 * tc, 32 * tr, 64, zero16(), lane);
    __syncthreads();  // every wave is past its reads of dW and T
    gb_store<OT>(b_r, 32 * tr, 32 * tc, xw, lane);
  }
  // (h) grad P = scale dO Vn^T with the gating of P: N_ij = grad P_ij Gamma_ij (i >= j), into T's tile
  {
    f32x16 n = zero16();
    if (tr >= tc) {
      const f32x16 dp = gb_mm<OT, false, false>(b_do, 32 * tr, b_v, 32 * tc, 0, 64, zero16(), lane);
      const f32x16 qk = gb_mm<OT, false, false>(b_q, 32 * tr, b_k, 32 * tc, 0, 64, zero16(), lane);
      const float gj = f.gam[32 * tc + ln];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = 32 * tr + acc_row(r, hh), j = 32 * tc + ln;
        const float gam = i >= j ? __builtin_amdgcn_exp2f(gi[r] - gj) : 0.0f;
        const float gp = scale * dp[r] * gam;       // grad P_ij Gamma_ij
        const float a = gp * qk[r];                 // grad P_ij P_ij
        rs_g[r] += a;
        cs -= a;
        n[r] = gp;
      }
    }
    gb_store<OT>(b_t, 32 * tr, 32 * tc, n, lane);
  }
  __syncthreads();
  // (i) d Kh = M Kh + M^T Kh + N^T Qh + D (Vn G'^T) + beta e^gamma Xw;   d Qh = N Kh + scale e^gamma (dO S^T)
  f32x16 dkh, dqh;
  {
    f32x16 acc = gb_mm<OT, false, true>(b_x, 32 * tr, b_k, 32 * tc, 0, 32 * (tr + 1), zero16(), lane);
    acc = gb_mm<OT, true, true>(b_x, 32 * tr, b_k, 32 * tc, 32 * tr, 64, acc, lane);
    acc = gb_mm<OT, true, true>(b_t, 32 * tr, b_q, 32 * tc, 32 * tr, 64, acc, lane);
    const f32x16 a4 = gb_mm<OT, false, false>(b_v, 32 * tr, b_g, 32 * tc, 0, 64, zero16(), lane);
    float dkj[16], xw[16], khv[16];
    gb_row_factors(f.dk, 32 * tr, hh, dkj);
    gb_acc_view<OT>(b_r, 32 * tr, 32 * tc, lane, xw);
    gb_acc_view<OT>(b_k, 32 * tr, 32 * tc, lane, khv);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float t4 = dkj[r] * a4[r], t5 = bi[r] * egi[r] * xw[r];
      acc[r] += t4 + t5;
      rs_g[r] += khv[r] * (t5 - t4);
      gl += khv[r] * t4;
      rs_b[r] += khv[r] * egi[r] * xw[r];
    }
    dkh = acc;
    f32x16 aq = gb_mm<OT, false, true>(b_t, 32 * tr, b_k, 32 * tc, 0, 32 * (tr + 1), zero16(), lane);
    const f32x16 a2 = gb_mm<OT, false, false>(b_do, 32 * tr, b_s, 32 * tc, 0, 64, zero16(), lane);
    float qhv[16];
    gb_acc_view<OT>(b_q, 32 * tr, 32 * tc, lane, qhv);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float t = scale * egi[r] * a2[r];
      aq[r] += t;
      rs_g[r] += qhv[r] * t;
    }
    dqh = aq;
  }
  {  // e^{gamma_L} <G', S>
    float part = 0.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = threadIdx.x + GB_THREADS * u, row = p >> 4, c4 = 4 * (p & 15);
#pragma unroll
      for (int e = 0; e < 4; ++e) part += (float)b_s[row * GB_LS + c4 + e] * (float)b_g[row * GB_LS + c4 + e];
    }
    gl += part * __builtin_amdgcn_exp2f(f.gam[63]);
  }
  // row sums -> LDS
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float sg = gb_half_sum(rs_g[r]), sb = gb_half_sum(rs_b[r]);
    if (ln == 0) {
      atomicAdd(&s_dgam[32 * tr + acc_row(r, hh)], sg);
      atomicAdd(&s_dbeta[32 * tr + acc_row(r, hh)], sb);
    }
  }
  {
    const float c2 = cs + __shfl_xor(cs, 32);
    if (hh == 0) atomicAdd(&s_dgam[32 * tc + ln], c2);
    float g2 = gb_half_sum(gl);
    g2 += __shfl_xor(g2, 32);
    if (lane == 0) atomicAdd(&s_misc[0], g2);
  }
  __syncthreads();  // every wave is past its reads of the tiles
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    f_dk[(32 * tr + acc_row(r, hh)) * 64 + 32 * tc + ln] = dkh[r];
    f_dq[(32 * tr + acc_row(r, hh)) * 64 + 32 * tc + ln] = dqh[r];
  }
  __syncthreads();
  {  // rows: through the l2 normalisation, rounded to the input type
    const int row = threadIdx.x >> 2, c0 = 16 * (threadIdx.x & 3);
    float yk[16], yq[16], dyk[16], dyq[16], dotk = 0.0f, dotq = 0.0f;
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const typename OpVec<OT>::x4 tk = *reinterpret_cast<const typename OpVec<OT>::x4*>(&b_k[row * GB_LS + c0 + 4 * e4]);
      const typename OpVec<OT>::x4 tq = *reinterpret_cast<const typename OpVec<OT>::x4*>(&b_q[row * GB_LS + c0 + 4 * e4]);
      const f32x4 dk4 = *reinterpret_cast<const f32x4*>(&f_dk[row * 64 + c0 + 4 * e4]);
      const f32x4 dq4 = *reinterpret_cast<const f32x4*>(&f_dq[row * 64 + c0 + 4 * e4]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        yk[4 * e4 + e] = (float)tk[e];
        yq[4 * e4 + e] = (float)tq[e];
        dyk[4 * e4 + e] = dk4[e];
        dyq[4 * e4 + e] = dq4[e];
        dotk += yk[4 * e4 + e] * dyk[4 * e4 + e];
        dotq += yq[4 * e4 + e] * dyq[4 * e4 + e];
      }
    }
    dotk += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, dotk);
    dotk += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, dotk);
    dotq += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, dotq);
    dotq += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, dotq);
    if (row < len) {
      const float ck = f.rk[row], cq = f.rq[row];
      typename Raw8<T>::type ok0, ok1, oq0, oq1;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        float gk, gq;
        if (l2norm == GDR_L2_CHUNK) {
          gk = ck * (dyk[e] - yk[e] * dotk);
          gq = cq * (dyq[e] - yq[e] * dotq);
        } else if (l2norm == GDR_L2_RECURRENT) {   // c = 1 / (|x| + eps): |x| = 1 / c - eps
          gk = ck * dyk[e] - yk[e] * dotk / fmaxf(1.0f / ck - 1e-6f, 1e-30f);
          gq = cq * dyq[e] - yq[e] * dotq / fmaxf(1.0f / cq - 1e-6f, 1e-30f);
        } else {
          gk = dyk[e];
          gq = dyq[e];
        }
        if (e < 8) { ok0[e] = (T)gk; oq0[e] = (T)gq; } else { ok1[e - 8] = (T)gk; oq1[e - 8] = (T)gq; }
      }
      T* dkp = dk + ((size_t)(tok0 + row) * H + h) * 64 + c0;
      T* dqp = dq + ((size_t)(tok0 + row) * H + h) * 64 + c0;
      *reinterpret_cast<typename Raw8<T>::type*>(dkp) = ok0;
      *reinterpret_cast<typename Raw8<T>::type*>(dkp + 8) = ok1;
      *reinterpret_cast<typename Raw8<T>::type*>(dqp) = oq0;
      *reinterpret_cast<typename Raw8<T>::type*>(dqp + 8) = oq1;
    }
  }
  if (wave == 0) {  // d g = the sum of d gamma over the later rows of the chunk (gamma_i = g_0 + ... + g_i); d beta
    float x = s_dgam[lane] + (lane == len - 1 ? s_misc[0] : 0.0f);
    if (lane >= len) x = 0.0f;
    // inclusive scan from the last lane down: total - exclusive prefix
    const float incl = wave_inclusive_scan(x);
    const float total = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(incl), 63));
    if (lane < len) {
      dg[(size_t)(tok0 + lane) * HV + hv] = total - incl + x;
      dbeta[(size_t)(tok0 + lane) * HV + hv] = s_dbeta[lane];
    }
  }
}

// ---- host ----------------------------------------------------------------------------------------------------------
struct GbcWorkspace {
  int64_t recs, m, n, d, sf, sr, c1m, c1n, c1d, c2m, c2n, c2d, s2, s1, bytes;
};
static GbcWorkspace gbc_workspace(int64_t chunks, int64_t items, int n_seq, int g1, int g2, int HV) {
  GbcWorkspace w;
  int64_t off = 0;
  const int64_t MB = 64 * 64 * 2, NB = 64 * 64 * 4;
  auto take = [&](int64_t bytes) { const int64_t o = off; off += lampa_align_up(bytes > 0 ? bytes : 1, 256); return o; };
  w.recs = take(chunks * HV * (int64_t)REC_BYTES);
  w.m = take(items * HV * MB);
  w.n = take(items * HV * MB);
  w.d = take(items * HV * 4);
  w.sf = take((items + 1) * HV * MB);
  w.sr = take((items + 1) * HV * MB);
  const int64_t n1 = (int64_t)n_seq * g1, n2 = (int64_t)n_seq * g2;
  w.c1m = take(n1 * HV * MB); w.c1n = take(n1 * HV * NB); w.c1d = take(n1 * HV * 4);
  w.c2m = take(n2 * HV * MB); w.c2n = take(n2 * HV * NB); w.c2d = take(n2 * HV * 4);
  w.s2 = take((n2 + 1) * HV * NB);
  w.s1 = take((n1 + 1) * HV * NB);
  w.bytes = off;
  return w;
}

extern "C" int64_t lampa_gdr_bwd_chunk_workspace_bytes(const int32_t* plan_host, int HV) {
  if (!plan_host || HV < 1) return LAMPA_ERR_INVALID;
  return gbc_workspace(plan_host[BP_CHUNKS], plan_host[BP_ITEMS], plan_host[BP_N_SEQ], plan_host[BP_GMAX1],
                       plan_host[BP_GMAX2], HV).bytes;
}

// the states in front of every item of one direction: two levels of group composites, then three scans downwards
template <typename OT>
static void gbc_scan(const int32_t* ph, const int32_t* pd, const GbcWorkspace& w, unsigned char* ws, const float* h0,
                     OT* S_items, int HV, hipStream_t s) {
  const int n_seq = ph[BP_N_SEQ], g1 = ph[BP_GMAX1], g2 = ph[BP_GMAX2], items = ph[BP_ITEMS];
  unsigned char* M0 = ws + w.m; unsigned char* N0 = ws + w.n; float* D0 = (float*)(ws + w.d);
  unsigned char* M1 = ws + w.c1m; unsigned char* N1 = ws + w.c1n; float* D1 = (float*)(ws + w.c1d);
  unsigned char* M2 = ws + w.c2m; unsigned char* N2 = ws + w.c2n; float* D2 = (float*)(ws + w.c2d);
  float* S2 = (float*)(ws + w.s2); float* S1 = (float*)(ws + w.s1);
  const dim3 blk(256);
  if (g1 > 1) {
    hipLaunchKernelGGL((gdrb_group_kernel<OT, true>), dim3(g1, n_seq, HV), dim3(512), 0, s, pd + ph[BP_OFF_L1G],
                       pd + ph[BP_OFF_L1G] + n_seq, M0, N0, D0, M1, (float*)N1, D1, HV, g1);
    LAMPA_PROF(s, "gdrb_group_kernel<items>");
  }
  if (g2 > 1) {
    hipLaunchKernelGGL((gdrb_group_kernel<OT, false>), dim3(g2, n_seq, HV), dim3(512), 0, s, pd + ph[BP_OFF_L2G],
                       pd + ph[BP_OFF_L2G] + n_seq, M1, N1, D1, M2, (float*)N2, D2, HV, g2);
    LAMPA_PROF(s, "gdrb_group_kernel<groups>");
  }
  // the state in front of every supergroup, of every group, of every item
  hipLaunchKernelGGL((gdrb_scan_kernel<OT, false, false, false>), dim3(1, n_seq, HV), blk, 0, s, pd + ph[BP_OFF_TOP],
                     pd + ph[BP_OFF_TOP] + n_seq, M2, N2, D2, h0, (void*)S2, HV, n_seq * g2);
  LAMPA_PROF(s, "gdrb_scan_kernel<supergroups>");
  hipLaunchKernelGGL((gdrb_scan_kernel<OT, true, false, false>), dim3(1, n_seq * g2, HV), blk, 0, s, pd + ph[BP_OFF_LEAF2],
                     pd + ph[BP_OFF_LEAF2] + n_seq * g2, M1, N1, D1, (const float*)S2, (void*)S1, HV, n_seq * g1);
  LAMPA_PROF(s, "gdrb_scan_kernel<groups>");
  hipLaunchKernelGGL((gdrb_scan_kernel<OT, true, true, true>), dim3(1, n_seq * g1, HV), blk, 0, s, pd + ph[BP_OFF_LEAF1],
                     pd + ph[BP_OFF_LEAF1] + n_seq * g1, M0, N0, D0, (const float*)S1, (void*)S_items, HV, items);
  LAMPA_PROF(s, "gdrb_scan_kernel<items>");
}

template <typename T>
static int gbc_run(const void* q, const void* k, const void* v, const float* g, const float* beta, const float* h0,
                   const void* dout, const float* dht, void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
                   const int32_t* ph, const int32_t* pd, int H, int HV, float scale, int l2norm, unsigned char* ws,
                   hipStream_t s) {
  const int n_seq = ph[BP_N_SEQ], chunks = ph[BP_CHUNKS];
  const GbcWorkspace w = gbc_workspace(chunks, ph[BP_ITEMS], n_seq, ph[BP_GMAX1], ph[BP_GMAX2], HV);
  constexpr int smem_maps_f = 6 * GB_TILE * 2 + 6 * 64 * 4, smem_maps_r = smem_maps_f;
  constexpr int smem_grads = 9 * GB_TILE * 2 + (6 * 64 + 64 + 64 + 16) * 4;
  static bool attr_set[64] = {};
  static std::mutex attr_lock;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LAMPA_ERR_LAUNCH;
  {
    std::lock_guard<std::mutex> hold(attr_lock);
    if (!attr_set[dev]) {
      if (hipFuncSetAttribute((const void*)gdrb_maps_kernel<T, false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              smem_maps_f) != hipSuccess ||
          hipFuncSetAttribute((const void*)gdrb_maps_kernel<T, true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              smem_maps_r) != hipSuccess ||
          hipFuncSetAttribute((const void*)gdrb_grads_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              smem_grads) != hipSuccess)
        return LAMPA_ERR_LAUNCH;
      attr_set[dev] = true;
    }
  }
  const int32_t* tok0 = pd + ph[BP_OFF_TOK0];
  const int32_t* clen = pd + ph[BP_OFF_LEN];
  const int32_t* item_f = pd + ph[BP_OFF_ITEM_F];
  const int32_t* item_r = pd + ph[BP_OFF_ITEM_R];
  unsigned char* recs = ws + w.recs;
  T* Sf = (T*)(ws + w.sf);
  T* Sr = (T*)(ws + w.sr);
  LAMPA_PROF(s, "start");
  if (chunks > 0) {
    hipLaunchKernelGGL((gdr_local_kernel<T, T, 64>), dim3(gdr_local_grid(chunks, HV)), dim3(64), 0, s, (const T*)k, g, beta,
                       tok0, clen, recs, chunks, H, HV, l2norm);
    LAMPA_PROF(s, "gdr_local_kernel");
    hipLaunchKernelGGL((gdrb_maps_kernel<T, false>), dim3(chunks, HV), dim3(GB_THREADS), smem_maps_f, s, (const T*)q,
                       (const T*)k, (const T*)v, (const T*)dout, recs, tok0, clen, item_f, ws + w.m, (T*)(ws + w.n),
                       (float*)(ws + w.d), H, HV, scale, l2norm);
    LAMPA_PROF(s, "gdrb_maps_kernel<forward>");
  }
  gbc_scan<T>(ph, pd, w, ws, h0, Sf, HV, s);
  if (chunks > 0) {
    hipLaunchKernelGGL((gdrb_maps_kernel<T, true>), dim3(chunks, HV), dim3(GB_THREADS), smem_maps_r, s, (const T*)q,
                       (const T*)k, (const T*)v, (const T*)dout, recs, tok0, clen, item_r, ws + w.m, (T*)(ws + w.n),
                       (float*)(ws + w.d), H, HV, scale, l2norm);
    LAMPA_PROF(s, "gdrb_maps_kernel<reverse>");
  }
  gbc_scan<T>(ph, pd, w, ws, dht, Sr, HV, s);
  if (chunks > 0) {
    hipLaunchKernelGGL((gdrb_grads_kernel<T>), dim3(chunks, HV), dim3(GB_THREADS), smem_grads, s, (const T*)q, (const T*)k,
                       (const T*)v, (const T*)dout, recs, tok0, clen, item_f, item_r, Sf, Sr, (T*)dq, (T*)dk, (T*)dv, dg,
                       dbeta, H, HV, scale, l2norm);
    LAMPA_PROF(s, "gdrb_grads_kernel");
  }
  if (dh0) {
    hipLaunchKernelGGL((gdrb_unslab_kernel<T>), dim3(n_seq, HV), dim3(GB_THREADS), 0, s, (const T*)Sr,
                       pd + ph[BP_OFF_EXTRA_R], dh0, HV);
    LAMPA_PROF(s, "gdrb_unslab_kernel");
  }
  return lampa_launch_status();
}

// Gradients of the gated-delta forward in the chunked form. q, k, dq, dk [tokens, H, 64]; v, dout, dv [tokens, HV, 64]
// (dtype bf16 / fp16) with HV == H; g, beta, dg, dbeta fp32 [tokens, HV] (g <= 0); h0, dht, dh0 fp32 [n_seq, HV, 64, 64]
// (each nullable). plan_host / plan_dev: lampa_gdr_bwd_chunk_plan_fill's tables in host and in device memory.
extern "C" int lampa_gdr_bwd_chunk(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                   const float* h0, const void* dout, const float* dht, void* dq, void* dk, void* dv,
                                   float* dg, float* dbeta, float* dh0, const int32_t* plan_host, const int32_t* plan_dev,
                                   int H, int HV, int K, int V, int dtype, float scale, int l2norm, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  if (!q || !k || !v || !g || !beta || !dout || !dq || !dk || !dv || !dg || !dbeta || !plan_host || !plan_dev)
    return LAMPA_ERR_INVALID;
  if (H < 1 || HV < 1 || l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (K != 64 || V != 64 || HV != H || (dtype != GDR_BF16 && dtype != GDR_FP16)) return LAMPA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv) & 15)
    return LAMPA_ERR_INVALID;
  if (plan_host[BP_N_SEQ] < 1) return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < lampa_gdr_bwd_chunk_workspace_bytes(plan_host, HV)) return LAMPA_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  unsigned char* ws = (unsigned char*)workspace;
  if (dtype == GDR_BF16)
    return gbc_run<__bf16>(q, k, v, g, beta, h0, dout, dht, dq, dk, dv, dg, dbeta, dh0, plan_host, plan_dev, H, HV, scale,
                           l2norm, ws, s);
  return gbc_run<_Float16>(q, k, v, g, beta, h0, dout, dht, dq, dk, dv, dg, dbeta, dh0, plan_host, plan_dev, H, HV, scale,
                           l2norm, ws, s);
}

// Hierarchical (level-weighted) chunkwise gated-delta-rule forward on gfx950.
//
// Replaces chunk_h_gated_delta_rule -> hattention_kernel -> chunkwise_fwd (reference chengjiang123/Lampa,
// models/hattention/gated_delta_rule_apis.py:21-91, kernel.py:338-374, chunkwise_hgdn.py:565-791), whose
// specification is the token loop of recurrent.py:134-216: the sources s <= t of a target token t are split into
// buckets ("levels": 0 = the token itself, otherwise 1 + the position of the highest bit in which t and s differ,
// base.py:41-46), every bucket keeps a state of its own that the same gated-delta transition acts on, and
//   o_t = sum_l lambda_t[l] q_t^T S_t^(l).
//
// With chunks of 64 tokens the levels 0..6 stay inside a chunk and level 7 + j collects the earlier chunks c' of the
// sequence with highest differing chunk-index bit j. Per chunk (T, gamma, beta, rk, rq, P as in gdr_chunk_kernels.h):
//   W   = T diag(beta e^{gamma} rk) K          (the state's share of v_new is -W S)
//   Q~  = diag(scale e^{gamma} rq) Q - P W     (a state S entering the chunk adds Q~ S to the outputs)
//   S'  = e^{gamma_last} S - K^T diag(e^{gamma_last - gamma} rk) (W S)
//   N   = K^T diag(e^{gamma_last - gamma} rk) T diag(beta) V          (the chunk's own sources, at its end)
//   o_intra = ((P T diag(beta)) . Lambda) V,   Lambda_ij = lambda_i[level(i, j)]
// Kernels:
//   prep   workgroup per (chunk, head), fully parallel: W and Q~ as MFMA operand fragments, the decay factors, the
//          inter-chunk lambdas (transposed), diag(e^{gamma_last - gamma} rk) T diag(beta) V as B-operand fragments (the
//          walk multiplies it by K^T: the chunk's own state N) and o_intra go to HBM.
//   walk   workgroup per (segment of chunks, head, 32 value columns): six "chain" waves hold up to two level
//          states each in accumulator registers (level j -> wave j % 6) and walk the chunks: for every level whose
//          chunk-index bit is set, o += lambda . (Q~ S), S <- S'; after the chunk the levels below the lowest clear
//          bit and N are summed into that bit's level (the carry chain of a binary counter) through LDS. Two loader
//          waves stage the chunks' operand records and raw k tiles (K^T operands come from the tile with the
//          transposing LDS read) and one of them forms N; all eight waves add the chain waves' partial outputs to
//          o_intra, eight rows each, and store o.
//   scan   (sequences cut into segments of 2^p chunks) the same walk over whole segments with the segment
//          composites (M, N) of the plain rule: leaves every segment's entering level states.
#include "gdr_chunk_kernels.h"
#include <mutex>

// Helper stream + fork / join events for the composites that run beside the prep kernel: one set per (device, caller
// stream), created on first use and kept until the process ends, so that calls on different streams or from different
// host threads never share an event. hg_side_lock is held while a call enqueues its fork .. join section, which keeps
// the record / wait pairs of two host threads that use the same caller stream from interleaving.
struct HgSide {
  int device;
  hipStream_t caller, side;
  hipEvent_t fork, join;
};
#define HG_MAX_SIDES 32
static HgSide hg_sides[HG_MAX_SIDES];
static int hg_n_sides = 0;
static std::mutex hg_side_lock;

// (call with hg_side_lock held) the set of this device and caller stream, or nullptr: the call then runs on one stream
static HgSide* hg_side_for(hipStream_t caller) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  for (int i = 0; i < hg_n_sides; ++i)
    if (hg_sides[i].device == dev && hg_sides[i].caller == caller) return &hg_sides[i];
  if (hg_n_sides == HG_MAX_SIDES) return nullptr;
  HgSide n;
  n.device = dev;
  n.caller = caller;
  if (hipStreamCreateWithFlags(&n.side, hipStreamNonBlocking) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  if (hipEventCreateWithFlags(&n.fork, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipStreamDestroy(n.side);
    return nullptr;
  }
  if (hipEventCreateWithFlags(&n.join, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipEventDestroy(n.fork);
    (void)hipStreamDestroy(n.side);
    return nullptr;
  }
  hg_sides[hg_n_sides] = n;
  return &hg_sides[hg_n_sides++];
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define HG_CW 6                  // chain waves
#define HG_LPW 2                 // levels per chain wave
#define HG_NLV (HG_CW * HG_LPW)  // inter-chunk levels: sequences of up to 2^12 chunks
#define HG_INTRA 7               // levels 0..6 live inside a chunk

// Record of one chunk and head for the walk kernel
template <int KT>
struct HgRec {
  static constexpr int NKS = KT / 16;
  static constexpr int WF = 0;                          // W fragments   [2][NKS] KiB
  static constexpr int QF = WF + 2 * NKS * 1024;        // Q~ fragments  [2][NKS] KiB
  static constexpr int DK = QF + 2 * NKS * 1024;        // e^{gamma_last - gamma_i} rk_i, fp32 [64]
  static constexpr int LT = DK + 256;                   // lambda_i[7 + j], fp32 [HG_NLV][64]
  static constexpr int MISC = LT + HG_NLV * 256;        // e^{gamma_last}
  static constexpr int BYTES = MISC + 256;
  static constexpr int PIECES = BYTES / 16;
};

// ---- prep ---------------------------------------------------------------------------------------------------------
template <int KT, int VT>
struct HgPrepSmem {
  static constexpr int SK = KT + 8, SV = VT + 8, ST = 40, LMAX = HG_INTRA + HG_NLV + 1;
  static constexpr int OFF_K = 0;                     // raw k; later the (P T beta . Lambda) fragments and lambda
  static constexpr int OFF_Q = OFF_K + 64 * SK * 2;   // raw q; Q~ is written over it in place
  static constexpr int OFF_W = OFF_Q + 64 * SK * 2;
  static constexpr int OFF_V = OFF_W + 64 * SK * 2;
  static constexpr int OFF_T = OFF_V + 64 * SV * 2;
  static constexpr int OFF_P = OFF_T + 3 * 32 * ST * 2;
  static constexpr int OFF_LAM = OFF_K + 6 * 1024;           // levels 0..6, written once the k tile is done with
  static constexpr int OFF_F = OFF_P + 6 * 1024;             // gamma, beta, rk, qsc, qs, dk, bek
  static constexpr int BYTES = OFF_F + 7 * 64 * 4;           // 51.25 KiB at K = V = 64: three workgroups per CU
  static_assert(6 * 1024 + HG_INTRA * 64 * 4 <= 64 * SK * 2, "fragments + lambda fit in the k tile");
};

template <typename T, int KT, int VT>
__global__ void __launch_bounds__(256)
    hgdn_prep_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                     const void* __restrict__ lam, int lam_dtype, float lam_div,
                     const int32_t* __restrict__ chunk_tok0,
                     const int32_t* __restrict__ chunk_len, const unsigned char* __restrict__ tmat,
                     unsigned char* __restrict__ wrec, unsigned char* __restrict__ Ub_out, float* __restrict__ Oi,
                     float* __restrict__ hstates, int chunks_per_seq, int H, int HV, int L, float scale, int l2norm) {
  using SM = HgPrepSmem<KT, VT>;
  using REC = HgRec<KT>;
  constexpr int SK = SM::SK, SV = SM::SV, ST = SM::ST, NKS = KT / 16;
  extern __shared__ __align__(16) unsigned char smem[];
  __bf16* s_k = reinterpret_cast<__bf16*>(smem + SM::OFF_K);
  __bf16* s_q = reinterpret_cast<__bf16*>(smem + SM::OFF_Q);
  __bf16* s_qt = s_q;
  __bf16* s_w = reinterpret_cast<__bf16*>(smem + SM::OFF_W);
  __bf16* s_v = reinterpret_cast<__bf16*>(smem + SM::OFF_V);
  __bf16* s_t = reinterpret_cast<__bf16*>(smem + SM::OFF_T);
  unsigned char* s_P = smem + SM::OFF_P;
  unsigned char* s_PL = smem + SM::OFF_K;
  float* s_lam = reinterpret_cast<float*>(smem + SM::OFF_LAM);
  float* s_gamma = reinterpret_cast<float*>(smem + SM::OFF_F);
  float* s_beta = s_gamma + 64;
  float* s_rk = s_gamma + 128;
  float* s_qsc = s_gamma + 192;  // scale rq_i
  float* s_qs = s_gamma + 256;   // scale e^{gamma_i} rq_i
  float* s_dk = s_gamma + 320;   // e^{gamma_last - gamma_i} rk_i
  float* s_bek = s_gamma + 384;  // beta_i e^{gamma_i} rk_i

  const int chunk = blockIdx.x, hv = blockIdx.y;
  const int h = hv / (HV / H);
  const int tok0 = chunk_tok0[chunk], len = chunk_len[chunk];
  const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  const size_t ch = (size_t)chunk * HV + hv;
  const unsigned char* rec_in = tmat + ch * REC_BYTES;
  unsigned char* rec = wrec + ch * REC::BYTES;

  // lambda rows (at most LMAX levels: five values per thread); the intra-chunk levels wait in registers until the
  // k tile's space is free
  constexpr int NLAM = (64 * SM::LMAX + 255) / 256;
  const int Lc = min(L, SM::LMAX);
  float lv[NLAM];
  {  // ---- stage the tiles: thread = (row, quarter of the row)
    const int row = tid >> 2, part = tid & 3;
    const bool live = row < len;
    const int rr = min(row, len - 1);
    constexpr int KU = KT / 32, VU = VT / 32;  // 16-byte pieces per thread
    typename Raw8<T>::type rk_[KU], rq_[KU], rv_[VU], zero;
#pragma unroll
    for (int e = 0; e < 8; ++e) zero[e] = (T)0.0f;
    const T* kp = k + ((size_t)(tok0 + rr) * H + h) * KT + part * (KT / 4);
    const T* qp = q + ((size_t)(tok0 + rr) * H + h) * KT + part * (KT / 4);
    const T* vp = v + ((size_t)(tok0 + rr) * HV + hv) * VT + part * (VT / 4);
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      rk_[u] = *reinterpret_cast<const typename Raw8<T>::type*>(kp + 8 * u);
      rq_[u] = *reinterpret_cast<const typename Raw8<T>::type*>(qp + 8 * u);
    }
#pragma unroll
    for (int u = 0; u < VU; ++u) rv_[u] = *reinterpret_cast<const typename Raw8<T>::type*>(vp + 8 * u);
    const float* fact = reinterpret_cast<const float*>(rec_in + T_BYTES);
    const float gv = fact[row], g_last = fact[63], bv = fact[64 + row];
    // every global load of the stage is issued before the first use: T blocks and the lambda rows, indices
    // clamped instead of branches
    bf16x8 tp0, tp1;
    {
      const bf16x8* tp = reinterpret_cast<const bf16x8*>(rec_in);
      // T21 (128 pieces) | T11 packed (80) | T22 packed (80): every thread takes piece tid (T21, T11, the first 48 of
      // T22), threads 0 .. 31 also the last 32 of T22 (the others repeat them); unconditional loads
      tp0 = tp[tid];
      tp1 = tp[256 + (tid & 31)];
      size_t li[NLAM];
#pragma unroll
      for (int j = 0; j < NLAM; ++j) {
        const int idx = min(tid + 256 * j, 64 * Lc - 1), r = idx / Lc, lvl = idx - r * Lc;
        li[j] = ((size_t)(tok0 + min(r, len - 1)) * HV + hv) * L + lvl;
      }
      // (one branch around all the loads of a type, so that they are in flight together)
      if (lam_dtype == GDR_FP32) {
#pragma unroll
        for (int j = 0; j < NLAM; ++j) lv[j] = reinterpret_cast<const float*>(lam)[li[j]];
      } else if (lam_dtype == GDR_BF16) {
        __bf16 t[NLAM];
#pragma unroll
        for (int j = 0; j < NLAM; ++j) t[j] = reinterpret_cast<const __bf16*>(lam)[li[j]];
#pragma unroll
        for (int j = 0; j < NLAM; ++j) lv[j] = (float)t[j];
      } else {
        _Float16 t[NLAM];
#pragma unroll
        for (int j = 0; j < NLAM; ++j) t[j] = reinterpret_cast<const _Float16*>(lam)[li[j]];
#pragma unroll
        for (int j = 0; j < NLAM; ++j) lv[j] = (float)t[j];
      }
    }
    {
      // the pieces to their rows of the LDS tile (rows 0-31 T11, 32-63 T21, 64-95 T22); the 48 pieces above the
      // diagonal of either packed block are zero
      int r0, c0, r1, c1;
      if (tid < 128) {  // a piece of T21
        r0 = 32 + (tid >> 2);
        c0 = tid & 3;
      } else {
        const int d = tid - 128;  // among the 160 packed pieces
        tri_piece(d < T_DIAG_PIECES ? d : d - T_DIAG_PIECES, r0, c0);
        r0 += d < T_DIAG_PIECES ? 0 : 64;
      }
      tri_piece(128 + (tid & 31) - T_DIAG_PIECES, r1, c1);
      *reinterpret_cast<bf16x8*>(&s_t[r0 * ST + 8 * c0]) = tp0;
      *reinterpret_cast<bf16x8*>(&s_t[(64 + r1) * ST + 8 * c1]) = tp1;
      if (tid < 128 - T_DIAG_PIECES) {
        int ur, up;
        tri_upper_piece(tid, ur, up);
        bf16x8 z8;
#pragma unroll
        for (int e = 0; e < 8; ++e) z8[e] = (__bf16)0.0f;
        *reinterpret_cast<bf16x8*>(&s_t[ur * ST + 8 * up]) = z8;
        *reinterpret_cast<bf16x8*>(&s_t[(64 + ur) * ST + 8 * up]) = z8;
      }
    }
    const bool want_ss = l2norm != GDR_L2_NONE;
    bf16x8 kb[KU], qb[KU];
    float kss = 0.0f, qss = 0.0f;
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      kb[u] = raw_to_bf16<T>(live ? rk_[u] : zero, kss, want_ss);
      qb[u] = raw_to_bf16<T>(live ? rq_[u] : zero, qss, want_ss);
      *reinterpret_cast<bf16x8*>(&s_k[row * SK + part * (KT / 4) + 8 * u]) = kb[u];
      *reinterpret_cast<bf16x8*>(&s_q[row * SK + part * (KT / 4) + 8 * u]) = qb[u];
    }
    kss += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, kss);
    kss += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, kss);
    qss += dpp_f32<GDR_DPP_QUAD_XOR1, 0xF>(0.0f, qss);
    qss += dpp_f32<GDR_DPP_QUAD_XOR2, 0xF>(0.0f, qss);
    const float rk = l2_factor(kss, l2norm), rq = l2_factor(qss, l2norm);
    const float eg = __builtin_amdgcn_exp2f(gv);
    const float bek = bv * eg * rk;
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      float unused = 0.0f;
      *reinterpret_cast<bf16x8*>(&s_v[row * SV + part * (VT / 4) + 8 * u]) =
          raw_to_bf16<T>(live ? rv_[u] : zero, unused, false);
    }
    if (part == 0) {
      const float dk = __builtin_amdgcn_exp2f(g_last - gv) * rk;
      s_gamma[row] = gv;
      s_beta[row] = bv;
      s_rk[row] = rk;
      s_qsc[row] = scale * rq;
      s_qs[row] = scale * eg * rq;
      s_dk[row] = dk;
      s_bek[row] = bek;
      reinterpret_cast<float*>(rec + REC::DK)[row] = dk;
      if (row == 0) reinterpret_cast<float*>(rec + REC::MISC)[0] = __builtin_amdgcn_exp2f(g_last);
    }
    // lambda, transposed ([level][row]): the inter-chunk levels go to the record
    if (lam_div != 1.0f) {  // lambda / scale, rounded to lambda's own type as the element-wise division would
#pragma unroll
      for (int j = 0; j < NLAM; ++j) {
        const float x = __fdiv_rn(lv[j], lam_div);
        lv[j] = lam_dtype == GDR_FP32 ? x : lam_dtype == GDR_BF16 ? (float)(__bf16)x : (float)(_Float16)x;
      }
    }
    float* lt = reinterpret_cast<float*>(rec + REC::LT);
#pragma unroll
    for (int j = 0; j < NLAM; ++j) {
      const int idx = tid + 256 * j, r = idx / Lc, lvl = idx - r * Lc;
      if (idx < 64 * Lc) {
        if (lvl >= HG_INTRA && lvl < HG_INTRA + HG_NLV) lt[(lvl - HG_INTRA) * 64 + r] = lv[j];
      }
    }
    for (int idx = tid; idx < HG_NLV * 64; idx += 256)
      if (HG_INTRA + idx / 64 >= L) lt[idx] = 0.0f;
  }
  __syncthreads();

  auto t_frag = [&](int tm, int ks) {  // A operand of T: rows 32 tm + ln, contraction step ks (tokens 16 ks ..)
    const int blk = tm == 0 ? 0 : (ks < 2 ? 1 : 2);
    return ld_kappa(s_t + blk * 32 * ST, ST, ln, 16 * (ks & 1), hh);
  };
  // the same with column j scaled by fac[j] (T diag(fac)): the per-token factor of a product's right-hand rows goes
  // onto T, so that the right-hand operand is the raw tile
  auto t_frag_scaled = [&](int tm, int ks, const float* fac) {
    const bf16x8 t = t_frag(tm, ks);
    const f32x4 lo = *reinterpret_cast<const f32x4*>(&fac[16 * ks + 4 * hh]);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(&fac[16 * ks + 8 + 4 * hh]);
    bf16x8 out;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[e] = (__bf16)((float)t[e] * lo[e]);
      out[4 + e] = (__bf16)((float)t[4 + e] * hi[e]);
    }
    return out;
  };
  auto w_tile = [&](int tm, int ct) {  // W rows 32 tm .., columns 32 ct ..
    f32x16 acc = zero16();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
      if (ks < 2 * (tm + 1)) acc = mfma32(t_frag_scaled(tm, ks, s_bek), ld_kappa_tr(s_k, SK, 32 * ct, 16 * ks, lane), acc);
#pragma unroll
    for (int r = 0; r < 16; ++r) s_w[(32 * tm + acc_row(r, hh)) * SK + 32 * ct + ln] = (__bf16)acc[r];
  };
  auto p_tile = [&](int t) {  // P^T tile: rows j (k tile jm), columns i (q tile tn) -> P fragments
    const int jm = t == 2 ? 1 : 0, tn = t == 0 ? 0 : 1;
    f32x16 acc = zero16();
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      acc = mfma32(*reinterpret_cast<const bf16x8*>(&s_k[(32 * jm + ln) * SK + 16 * ks + 8 * hh]),
                   *reinterpret_cast<const bf16x8*>(&s_q[(32 * tn + ln) * SK + 16 * ks + 8 * hh]), acc);
    const int i = 32 * tn + ln;
    const float gi = s_gamma[i], fi = s_qsc[i];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 32 * jm + acc_row(r, hh);
      acc[r] *= fi * s_rk[j] * __builtin_amdgcn_exp2f(i >= j ? gi - s_gamma[j] : -1e30f);
    }
    const int f0 = tn == 0 ? 0 : 2 + 2 * jm;
    frag_store(s_P, f0, lane, acc_to_operand(acc, 0));
    frag_store(s_P, f0 + 1, lane, acc_to_operand(acc, 8));
  };
  auto un_tile = [&](int vt) {  // dk . U with U = (T diag(beta)) V for 32 value columns, as B-operand fragments
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      f32x16 acc = zero16();
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        if (ks < 2 * (tm + 1)) acc = mfma32(t_frag_scaled(tm, ks, s_beta), ld_kappa_tr(s_v, SV, 32 * vt, 16 * ks, lane), acc);
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] *= s_dk[32 * tm + acc_row(r, hh)];
      unsigned char* out = Ub_out + (ch * (VT / 32) + vt) * 4096;
      frag_store(out, 2 * tm, lane, acc_to_operand(acc, 0));
      frag_store(out, 2 * tm + 1, lane, acc_to_operand(acc, 8));
    }
  };
  // The last chunk of a sequence, when the caller wants the level states after the last token (HState.states of
  // the reference, [B, HV, K, V, L]): level l < 7 holds the chunk's own sources j with level(63, j) = l, carried to
  // the end of the chunk -- N with beta masked to that bucket (the mask acts on the sources, i.e. on T's columns).
  const bool want_tail = hstates != nullptr && (chunk % chunks_per_seq) == chunks_per_seq - 1;
  auto tail_tile = [&](int vt, int lvl) {
    bf16x8 Ub[4];
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      f32x16 acc = zero16();
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        if (ks >= 2 * (tm + 1)) continue;
        const bf16x8 t = t_frag(tm, ks);
        bf16x8 ts;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int j = 16 * ks + kappa(hh, e);
          const int lj = j == 63 ? 0 : 32 - __builtin_clz(63 ^ j);
          ts[e] = (__bf16)(lj == lvl ? (float)t[e] * s_beta[j] : 0.0f);
        }
        acc = mfma32(ts, ld_kappa_tr(s_v, SV, 32 * vt, 16 * ks, lane), acc);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] *= s_dk[32 * tm + acc_row(r, hh)];
      Ub[2 * tm] = acc_to_operand(acc, 0);
      Ub[2 * tm + 1] = acc_to_operand(acc, 8);
    }
    float* out = hstates + ((size_t)(chunk / chunks_per_seq) * HV + hv) * KT * VT * L + lvl;
#pragma unroll
    for (int km = 0; km < KT / 32; ++km) {
      f32x16 acc = zero16();
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) acc = mfma32(ld_kappa_tr(s_k, SK, 32 * km, 16 * ks, lane), Ub[ks], acc);
#pragma unroll
      for (int r = 0; r < 16; ++r) out[((size_t)(32 * km + acc_row(r, hh)) * VT + 32 * vt + ln) * L] = acc[r];
    }
  };
  // ---- W, P, the scaled U of the chunk's own state (tasks spread over the four waves)
  constexpr int NW = 2 * (KT / 32), NU = VT / 32;
  const int n_tail = want_tail ? NU * HG_INTRA : 0;
  for (int task = wave; task < NW + 3 + NU + n_tail; task += 4) {
    if (task < NW) w_tile(task / (KT / 32), task % (KT / 32));
    else if (task < NW + 3) p_tile(task - NW);
    else if (task < NW + 3 + NU) un_tile(task - NW - 3);
    else {
      const int f = task - NW - 3 - NU;
      tail_tile(f / HG_INTRA, f % HG_INTRA);
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NLAM; ++j) {
    const int idx = tid + 256 * j, r = idx / Lc, lvl = idx - r * Lc;
    if (idx < 64 * Lc && lvl < HG_INTRA) s_lam[lvl * 64 + r] = lv[j];
  }
  __syncthreads();

  auto q_tile = [&](int tm, int ct) {  // Q~ = qs Q - P W
    f32x16 acc = zero16();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
      if (ks < 2 * (tm + 1))
        acc = mfma32(frag_load(s_P, 2 * tm + ks, lane), ld_kappa_tr(s_w, SK, 32 * ct, 16 * ks, lane), acc);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 32 * tm + acc_row(r, hh);
      s_qt[row * SK + 32 * ct + ln] = (__bf16)(s_qs[row] * (float)s_q[row * SK + 32 * ct + ln] - acc[r]);
    }
  };
  auto a_tile = [&](int t) {  // ((P T diag(beta)) . Lambda)^T tile: rows j' (tile tj), columns i (tile ti)
    const int tj = t == 2 ? 1 : 0, ti = t == 0 ? 0 : 1;
    f32x16 acc = zero16();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks / 2 < tj || ks / 2 > ti) continue;  // T[j][j'] = 0 for j < j', P[i][j] = 0 for j > i
      const int blk = ks < 2 ? 0 : (tj == 0 ? 1 : 2);
      acc = mfma32(ld_kappa_tr(s_t + blk * 32 * ST, ST, 0, 16 * (ks & 1), lane), frag_load(s_P, 2 * ti + ks, lane), acc);
    }
    const int i = 32 * ti + ln;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 32 * tj + acc_row(r, hh);
      const int lvl = i == j ? 0 : 32 - __builtin_clz(i ^ j);
      acc[r] = j <= i ? acc[r] * s_beta[j] * s_lam[lvl * 64 + i] : 0.0f;
    }
    const int f0 = ti == 0 ? 0 : 2 + 2 * tj;
    frag_store(s_PL, f0, lane, acc_to_operand(acc, 0));
    frag_store(s_PL, f0 + 1, lane, acc_to_operand(acc, 8));
  };
  for (int task = wave; task < NW + 3; task += 4) {
    if (task < NW) q_tile(task / (KT / 32), task % (KT / 32));
    else a_tile(task - NW);
  }
  __syncthreads();

  // ---- o_intra and the W / Q~ fragments
  for (int task = wave; task < 2 * NU + 4 * NKS; task += 4) {
    if (task < 2 * NU) {
      const int tm = task / NU, vt = task % NU;
      f32x16 acc = zero16();
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        if (ks < 2 * (tm + 1))
          acc = mfma32(frag_load(s_PL, 2 * tm + ks, lane), ld_kappa_tr(s_v, SV, 32 * vt, 16 * ks, lane), acc);
      float* out = Oi + ch * (64 * VT) + 32 * vt + ln;
#pragma unroll
      for (int r = 0; r < 16; ++r) out[(32 * tm + acc_row(r, hh)) * VT] = acc[r];
    } else {
      const int f = task - 2 * NU, which = f / (2 * NKS), g = f % (2 * NKS);  // fragment (tm, ks) = (g / NKS, g % NKS)
      const bf16x8 fr = ld_kappa(which == 0 ? s_w : s_qt, SK, 32 * (g / NKS) + ln, 16 * (g % NKS), hh);
      frag_store(rec + (which == 0 ? REC::WF : REC::QF), g, lane, fr);
    }
  }
}

// ---- walk ---------------------------------------------------------------------------------------------------------
template <int KT>
struct HgWalkSmem {
  static constexpr int SP = 36;  // row stride of a partial output tile (fp32)
  static constexpr int SK = KT + 8;  // row stride of the k tile
  static constexpr int OFF_REC = 0;
  static constexpr int OFF_KT = 2 * HgRec<KT>::BYTES;          // raw k tile (row-major), double-buffered
  static constexpr int OFF_PART = OFF_KT + 2 * 64 * SK * 2;
  static constexpr int OFF_ACC = OFF_PART + HG_CW * 64 * SP * 4;
  static constexpr int BYTES = OFF_ACC + KT * 32 * 4;
};

// accumulator-order slab (KT x 32 fp32) <-> registers
template <int KT>
__device__ __forceinline__ void slab_load(const float* p, int lane, f32x16* S) {
  const f32x4* s = reinterpret_cast<const f32x4*>(p);
#pragma unroll
  for (int km = 0; km < KT / 32; ++km)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const f32x4 t = s[(km * 4 + q4) * 64 + lane];
#pragma unroll
      for (int e = 0; e < 4; ++e) S[km][4 * q4 + e] = t[e];
    }
}
template <int KT>
__device__ __forceinline__ void slab_store(float* p, int lane, const f32x16* S) {
  f32x4* s = reinterpret_cast<f32x4*>(p);
#pragma unroll
  for (int km = 0; km < KT / 32; ++km)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f32x4 t;
#pragma unroll
      for (int e = 0; e < 4; ++e) t[e] = S[km][4 * q4 + e];
      s[(km * 4 + q4) * 64 + lane] = t;
    }
}
template <int KT>
__device__ __forceinline__ void slab_add(float* p, int lane, const f32x16* S) {
  f32x4* s = reinterpret_cast<f32x4*>(p);
#pragma unroll
  for (int km = 0; km < KT / 32; ++km)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f32x4 t = s[(km * 4 + q4) * 64 + lane];
#pragma unroll
      for (int e = 0; e < 4; ++e) t[e] += S[km][4 * q4 + e];
      s[(km * 4 + q4) * 64 + lane] = t;
    }
}

// The carry chain after chunk cs (index in its sequence): the levels below the lowest clear bit z of cs are all
// occupied; they and the new state already in s_acc are summed, in level order, and become level z. One barrier
// per level (uniform over the workgroup); a wave that owns none of the levels only takes part in the barriers.
template <int KT>
__device__ __forceinline__ void hg_merge(int cs, int lvl0, int wave, bool chain, int lane, float* s_acc,
                                         f32x16 (*S)[KT / 32]) {
  const int z = __builtin_ctz(~cs);
  for (int j = lvl0; j < z; ++j) {
    if (chain) {
#pragma unroll
      for (int slot = 0; slot < HG_LPW; ++slot)
        if (slot * HG_CW + wave == j) {
          slab_add<KT>(s_acc, lane, S[slot]);
#pragma unroll
          for (int km = 0; km < KT / 32; ++km) S[slot][km] = zero16();
        }
    }
    lds_barrier();
  }
  if (chain) {
#pragma unroll
    for (int slot = 0; slot < HG_LPW; ++slot)
      if (slot * HG_CW + wave == z) slab_load<KT>(s_acc, lane, S[slot]);
  }
}

template <typename T, int KT, int VT>
__global__ void __launch_bounds__(64 * (HG_CW + 2))
    hgdn_walk_kernel(const GdrPlanView pv, const int32_t* __restrict__ chunk_tok0, const int32_t* __restrict__ chunk_len,
                     const T* __restrict__ k, int H, const unsigned char* __restrict__ wrec, const unsigned char* __restrict__ Ub_in,
                     const float* __restrict__ Oi, const float* __restrict__ Xinit, T* __restrict__ o,
                     float* __restrict__ hstates, int L, int HV) {
  using REC = HgRec<KT>;
  using SM = HgWalkSmem<KT>;
  constexpr int NKS = KT / 16, SP = SM::SP;
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_part = reinterpret_cast<float*>(smem + SM::OFF_PART);
  float* s_acc = reinterpret_cast<float*>(smem + SM::OFF_ACC);

  const int seg = blockIdx.x, hv = blockIdx.y, vslab = blockIdx.z;
  const int c0 = pv.seg_chunk0[seg], nc = pv.seg_nchunks[seg], c1 = c0 + nc;
  if (nc <= 0) return;
  const int cs0 = c0 - pv.seg_chunk0[pv.seq_seg0[pv.seg_seq[seg]]];  // index of the first chunk in its sequence
  const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63, hh = lane >> 5, ln = lane & 31;

  // Output of a chunk: every wave of the workgroup sums eight rows of the chain waves' partial tiles and the intra-chunk
  // part (read one chunk ahead), rounds and stores them -- lane = (row, four columns).
  const int orow = 8 * wave + (lane >> 3), ocol = 4 * (lane & 7);
  auto oi_load = [&](int c) __attribute__((always_inline)) {
    return *reinterpret_cast<const f32x4*>(Oi + ((size_t)uniform(c) * HV + hv) * (64 * VT) + orow * VT + 32 * vslab + ocol);
  };
  auto out_rows = [&](int tok0, int len, f32x4 a) __attribute__((always_inline)) {
#pragma unroll
    for (int w = 0; w < HG_CW; ++w) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(&s_part[w * 64 * SP + orow * SP + ocol]);
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] += t[i];
    }
    typedef T T4 __attribute__((ext_vector_type(4)));
    T4 pk;
#pragma unroll
    for (int i = 0; i < 4; ++i) pk[i] = GdrElem<T>::from_float(a[i]);
    if (orow < len) *reinterpret_cast<T4*>(o + ((size_t)(tok0 + orow) * HV + hv) * VT + 32 * vslab + ocol) = pk;
  };
  static_assert(HG_CW + 2 == 8, "eight waves share the 64 output rows");

  if (wave >= HG_CW) {
    // ================================================ loader ================================================
    const int ltid = tid - 64 * HG_CW;
    constexpr int NP = (REC::PIECES + 127) / 128, KU = KT / 16;  // 16-byte pieces per thread: record; half a k row
    const int h = hv / (HV / H);
    const int krow = ltid >> 1, khalf = ltid & 1;
    const bool nwave = wave == HG_CW;  // the loader wave that also turns (dk U) into the chunk's own state
    struct Set {
      u32x4 rec[NP];
      typename Raw8<T>::type kk[KU];
      bf16x8 ub[4];
    };
    Set sA, sB;
    auto load_rec = [&](int c, Set& st) __attribute__((always_inline)) {  // record and k tile of chunk c
      const u32x4* src = reinterpret_cast<const u32x4*>(wrec + ((size_t)uniform(c) * HV + hv) * REC::BYTES);
#pragma unroll
      for (int j = 0; j < NP; ++j) st.rec[j] = src[min(ltid + 128 * j, REC::PIECES - 1)];
      const T* kp = k + ((size_t)(chunk_tok0[uniform(c)] + krow) * H + h) * KT + khalf * (KT / 2);
#pragma unroll
      for (int u = 0; u < KU; ++u) st.kk[u] = *reinterpret_cast<const typename Raw8<T>::type*>(kp + 8 * u);
    };
    auto store_rec = [&](int par, const Set& st) __attribute__((always_inline)) {
      u32x4* dst = reinterpret_cast<u32x4*>(smem + SM::OFF_REC + par * REC::BYTES);
#pragma unroll
      for (int j = 0; j < NP; ++j)
        if (ltid + 128 * j < REC::PIECES) dst[ltid + 128 * j] = st.rec[j];
      __bf16* kt = reinterpret_cast<__bf16*>(smem + SM::OFF_KT) + par * (64 * SM::SK);
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        float unused = 0.0f;
        *reinterpret_cast<bf16x8*>(&kt[krow * SM::SK + khalf * (KT / 2) + 8 * u]) = raw_to_bf16<T>(st.kk[u], unused, false);
      }
    };
    auto load_set = [&](int c, Set& st) __attribute__((always_inline)) {  // what chunk c issues
      load_rec(min(c + 2, c1 - 1), st);
      const unsigned char* ub = Ub_in + (((size_t)uniform(min(c + 1, c1 - 1)) * HV + hv) * (VT / 32) + vslab) * 4096;
#pragma unroll
      for (int f = 0; f < 4; ++f) st.ub[f] = frag_load(ub, f, lane);  // (used by one wave; the other's copy is dropped)
    };
    load_rec(c0, sA);
    store_rec(0, sA);
    load_set(c0 - 1, sA);  // record and k (c0 + 1), scaled U (c0)
    f32x4 oi_cur = oi_load(c0);
    auto one_chunk = [&](int c, const Set& held, Set& next) __attribute__((always_inline)) {
      lds_barrier();  // T(c): record and k (c) are staged; their buffers (c+1)&1, s_acc and the partial tiles are free
      const int tok0 = chunk_tok0[uniform(c)], len = chunk_len[uniform(c)];  // (scalar loads: early, so that they land)
      store_rec((c - c0 + 1) & 1, held);
      if (nwave) {  // N = K^T (dk U): the chunk's own sources at its end, into s_acc in accumulator order
        const __bf16* kt = reinterpret_cast<const __bf16*>(smem + SM::OFF_KT) + ((c - c0) & 1) * (64 * SM::SK);
#pragma unroll
        for (int km = 0; km < KT / 32; ++km) {
          f32x16 acc = zero16();
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) acc = mfma32(ld_kappa_tr(kt, SM::SK, 32 * km, 16 * ks, lane), held.ub[ks], acc);
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            f32x4 t;
#pragma unroll
            for (int e = 0; e < 4; ++e) t[e] = acc[4 * q4 + e];
            reinterpret_cast<f32x4*>(s_acc)[(km * 4 + q4) * 64 + lane] = t;
          }
        }
      }
      load_set(c, next);
      const f32x4 oi_next = oi_load(min(c + 1, c1 - 1));
      lds_barrier();  // M0(c): the chain waves' partial tiles are complete
      out_rows(tok0, len, oi_cur);
      if (c + 1 < c1) hg_merge<KT>(cs0 + (c - c0), 0, wave, false, lane, nullptr, nullptr);
      oi_cur = oi_next;
    };
    for (int c = c0; c < c1; c += 2) {
      one_chunk(c, sA, sB);
      if (c + 1 < c1) one_chunk(c + 1, sB, sA);
    }
    return;
  }

  // ================================================== chain ==================================================
  f32x16 S[HG_LPW][KT / 32];
#pragma unroll
  for (int slot = 0; slot < HG_LPW; ++slot) {
    const int lvl = slot * HG_CW + wave;
#pragma unroll
    for (int km = 0; km < KT / 32; ++km) S[slot][km] = zero16();
    if (Xinit && ((cs0 >> lvl) & 1))
      slab_load<KT>(Xinit + ((((size_t)seg * HG_NLV + lvl) * HV + hv) * (VT / 32) + vslab) * (KT * 32), lane, S[slot]);
  }
  f32x4 oi_cur = oi_load(c0);
  for (int c = c0; c < c1; ++c) {
    const int cs = cs0 + (c - c0);
    lds_barrier();  // T(c)
    const int tok0 = chunk_tok0[uniform(c)], len = chunk_len[uniform(c)];
    const f32x4 oi_next = oi_load(min(c + 1, c1 - 1));
    const unsigned char* rec = smem + SM::OFF_REC + ((c - c0) & 1) * REC::BYTES;
    const __bf16* s_kt = reinterpret_cast<const __bf16*>(smem + SM::OFF_KT) + ((c - c0) & 1) * (64 * SM::SK);
    const float* s_dk = reinterpret_cast<const float*>(rec + REC::DK);
    const float* s_lt = reinterpret_cast<const float*>(rec + REC::LT);
    const float dec = reinterpret_cast<const float*>(rec + REC::MISC)[0];
    f32x16 O[2] = {zero16(), zero16()};
#pragma unroll
    for (int slot = 0; slot < HG_LPW; ++slot) {
      const int lvl = slot * HG_CW + wave;
      if (!((cs >> lvl) & 1)) continue;
      // The fragments of a stage are read from LDS as one batch ahead of its MFMAs (lds_fence() pins that order; left
      // alone the compiler fetches each fragment right before its MFMA and pays the LDS latency every time), and the
      // two accumulation chains of a stage are interleaved.
      bf16x8 fr[2 * NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        fr[ks] = frag_load(rec + REC::WF, ks, lane);
        fr[NKS + ks] = frag_load(rec + REC::QF, ks, lane);
      }
      bf16x8 Sb[NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) Sb[ks] = acc_to_operand(S[slot][ks / 2], 8 * (ks % 2));
      bf16x8 Zb[4];
#pragma unroll
      for (int tm = 0; tm < 2; ++tm) {
        f32x4 dk[4], lm[4];
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          dk[b4] = *reinterpret_cast<const f32x4*>(&s_dk[32 * tm + 8 * b4 + 4 * hh]);
          lm[b4] = *reinterpret_cast<const f32x4*>(&s_lt[lvl * 64 + 32 * tm + 8 * b4 + 4 * hh]);
        }
        lds_fence();
        f32x16 z = zero16(), a = zero16();
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          z = mfma32(fr[ks], Sb[ks], z);
          a = mfma32(fr[NKS + ks], Sb[ks], a);
        }
        // the next stage's fragments: row tile 1 of W and Q~, then K^T
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          if (tm == 0) {
            fr[ks] = frag_load(rec + REC::WF, NKS + ks, lane);
            fr[NKS + ks] = frag_load(rec + REC::QF, NKS + ks, lane);
          } else if (ks < 4) {
#pragma unroll
            for (int km = 0; km < KT / 32; ++km) fr[km * 4 + ks] = ld_kappa_tr(s_kt, SM::SK, 32 * km, 16 * ks, lane);
          }
        }
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            z[4 * b4 + e] *= -dk[b4][e];
            O[tm][4 * b4 + e] = __builtin_fmaf(lm[b4][e], a[4 * b4 + e], O[tm][4 * b4 + e]);
          }
        Zb[2 * tm] = acc_to_operand(z, 0);
        Zb[2 * tm + 1] = acc_to_operand(z, 8);
      }
#pragma unroll
      for (int km = 0; km < KT / 32; ++km)
#pragma unroll
        for (int r = 0; r < 16; ++r) S[slot][km][r] *= dec;
      lds_fence();
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int km = 0; km < KT / 32; ++km) S[slot][km] = mfma32(fr[km * 4 + ks], Zb[ks], S[slot][km]);
    }
    {
      float* part = s_part + wave * 64 * SP;
#pragma unroll
      for (int tm = 0; tm < 2; ++tm)
#pragma unroll
        for (int r = 0; r < 16; ++r) part[(32 * tm + acc_row(r, hh)) * SP + ln] = O[tm][r];
    }
    lds_barrier();  // M0(c)
    out_rows(tok0, len, oi_cur);
    if (c + 1 < c1) hg_merge<KT>(cs, 0, wave, true, lane, s_acc, S);
    oi_cur = oi_next;
  }
  // the level states after the sequence's last token (before any carry): level 7 + j for the occupied inter-chunk levels
  if (hstates && (pv.seg_flags[seg] & SEG_LAST)) {
    const int cs = cs0 + nc - 1;
    float* out = hstates + ((size_t)pv.seg_seq[seg] * HV + hv) * KT * VT * L;
#pragma unroll
    for (int slot = 0; slot < HG_LPW; ++slot) {
      const int lvl = slot * HG_CW + wave;
      if (!((cs >> lvl) & 1) || HG_INTRA + lvl >= L) continue;
#pragma unroll
      for (int km = 0; km < KT / 32; ++km)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          out[((size_t)(32 * km + acc_row(r, hh)) * VT + 32 * vslab + ln) * L + HG_INTRA + lvl] = S[slot][km][r];
    }
  }
}

// ---- scan over the segments --------------------------------------------------------------------------------------
// grid (VT/32, n_seq, HV), HG_CW waves. Segments hold G = 2^p chunks, so at a segment's first chunk only levels >= p
// can be occupied; they are carried from segment to segment with the segment's composite map of the plain rule
// (S -> d S + M' S; its N is the sum of everything the segment's own chunks contribute) and merged by the same carry
// chain. Xinit[seg][level] receives every occupied level's state at the segment's first chunk.
template <int KT, int VT>
__global__ void __launch_bounds__(64 * HG_CW)
    hgdn_scan_kernel(const GdrPlanView pv, const unsigned char* __restrict__ Mcomp, const unsigned char* __restrict__ Ncomp,
                     const float* __restrict__ Dcomp, float* __restrict__ Xinit, int HV, int p) {
  constexpr int NKS = KT / 16, M_BYTES = KT * KT * 2, N_BYTES = KT * 32 * 4;
  __shared__ __align__(16) float s_acc[KT * 32];
  const int vslab = blockIdx.x, seq = blockIdx.y, hv = blockIdx.z;
  const int seg0 = pv.seq_seg0[seq], nseg = pv.seq_nseg[seq];
  const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
  f32x16 S[HG_LPW][KT / 32];
#pragma unroll
  for (int slot = 0; slot < HG_LPW; ++slot)
#pragma unroll
    for (int km = 0; km < KT / 32; ++km) S[slot][km] = zero16();
  // composite of the coming segment: loaded one step ahead (two register sets that swap roles)
  constexpr int NM = (KT / 32) * NKS, NPT = KT / 32;
  bf16x8 mA[NM], mB[NM];
  f32x4 nA[NPT], nB[NPT];
  float dA = 0.0f, dB = 0.0f;
  auto issue = [&](int i, bf16x8* m, f32x4* n, float& d) __attribute__((always_inline)) {
    const size_t sh = (size_t)(seg0 + max(0, min(i, nseg - 2))) * HV + hv;
    const bf16x8* M = reinterpret_cast<const bf16x8*>(Mcomp + sh * M_BYTES);
    const f32x4* N = reinterpret_cast<const f32x4*>(Ncomp + (sh * (VT / 32) + vslab) * N_BYTES);
#pragma unroll
    for (int f = 0; f < NM; ++f) m[f] = M[f * 64 + lane];
#pragma unroll
    for (int j = 0; j < NPT; ++j) n[j] = N[tid + 64 * HG_CW * j];
    d = Dcomp[sh];
  };
  auto step = [&](int i, const bf16x8* m, const f32x4* n, float d, bf16x8* m2, f32x4* n2, float& d2)
                  __attribute__((always_inline)) {
    const int seg = seg0 + i, cs = i << p;
#pragma unroll
    for (int slot = 0; slot < HG_LPW; ++slot) {
      const int lvl = slot * HG_CW + wave;
      if ((cs >> lvl) & 1)
        slab_store<KT>(Xinit + ((((size_t)seg * HG_NLV + lvl) * HV + hv) * (VT / 32) + vslab) * (KT * 32), lane, S[slot]);
    }
    if (i == nseg - 1) return;
    issue(i + 1, m2, n2, d2);
#pragma unroll
    for (int slot = 0; slot < HG_LPW; ++slot) {
      const int lvl = slot * HG_CW + wave;
      if (!((cs >> lvl) & 1)) continue;
      bf16x8 Sb[NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) Sb[ks] = acc_to_operand(S[slot][ks / 2], 8 * (ks % 2));
#pragma unroll
      for (int km = 0; km < KT / 32; ++km) {
#pragma unroll
        for (int r = 0; r < 16; ++r) S[slot][km][r] *= d;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) S[slot][km] = mfma32(m[km * NKS + ks], Sb[ks], S[slot][km]);
      }
    }
    lds_barrier();  // the level that took the last carry has read s_acc
#pragma unroll
    for (int j = 0; j < NPT; ++j) reinterpret_cast<f32x4*>(s_acc)[tid + 64 * HG_CW * j] = n[j];
    lds_barrier();
    hg_merge<KT>(cs + (1 << p) - 1, p, wave, true, lane, s_acc, S);
  };
  if (nseg > 1) issue(0, mA, nA, dA);
  for (int i = 0; i < nseg; i += 2) {
    step(i, mA, nA, dA, mB, nB, dB);
    if (i + 1 < nseg) step(i + 1, mB, nB, dB, mA, nA, dA);
  }
}

// ---- host side ------------------------------------------------------------------------------------------------
struct HgWorkspace {
  int64_t off_t, off_m, off_n, off_d, off_rec, off_nc, off_oi, off_x, bytes;
};

static HgWorkspace hg_workspace(int64_t chunks, int64_t segs, int HV, int K, int V) {
  HgWorkspace w;
  const int64_t rec_bytes = K == 64 ? HgRec<64>::BYTES : HgRec<128>::BYTES;
  int64_t off = 0;
  w.off_t = off;   off += lampa_align_up(chunks * HV * (int64_t)REC_BYTES, 256);
  w.off_m = off;   off += lampa_align_up(segs * HV * (int64_t)K * K * 2, 256);
  w.off_n = off;   off += lampa_align_up(segs * HV * (int64_t)K * V * 4, 256);
  w.off_d = off;   off += lampa_align_up(segs * HV * 4, 256);
  w.off_rec = off; off += lampa_align_up(chunks * HV * rec_bytes, 256);
  w.off_nc = off;  off += lampa_align_up(chunks * HV * (int64_t)(V / 32) * 4096, 256);  // dk . U fragments
  w.off_oi = off;  off += lampa_align_up(chunks * HV * (int64_t)64 * V * 4, 256);
  w.off_x = off;   off += lampa_align_up(segs * HG_NLV * HV * (int64_t)K * V * 4, 256);
  w.bytes = off > 0 ? off : 256;
  return w;
}

static bool hg_supported(int K, int V) { return K == 64 && (V == 64 || V == 128); }

extern "C" int64_t lampa_hgdn_chunk_workspace_bytes(int64_t total_chunks, int64_t n_segments, int HV, int K, int V) {
  if (total_chunks < 0 || n_segments < 0 || HV < 1) return LAMPA_ERR_INVALID;
  if (!hg_supported(K, V)) return LAMPA_ERR_UNSUPPORTED;
  return hg_workspace(total_chunks, n_segments, HV, K, V).bytes;
}

template <typename T, int KT, int VT>
static int hg_launch(const void* q, const void* k, const void* v, const float* g, const float* beta, const void* lam,
                     int lam_dtype, float lam_div, void* o, float* hstates, int chunks_per_seq, const GdrPlanView pv, int n_seq, int chunks, int segs, int p, int H, int HV, int L,
                     float scale, int l2norm, unsigned char* ws, hipStream_t s) {
  const HgWorkspace w = hg_workspace(chunks, segs, HV, KT, VT);
  unsigned char* tf = ws + w.off_t;
  unsigned char* Mc = ws + w.off_m;
  unsigned char* Nm = ws + w.off_n;
  float* Dc = (float*)(ws + w.off_d);
  unsigned char* rec = ws + w.off_rec;
  unsigned char* Ubw = ws + w.off_nc;
  float* Oi = (float*)(ws + w.off_oi);
  float* Xi = (float*)(ws + w.off_x);
  constexpr int smem_a = GdrSegSmem<KT, VT, false, false>::BYTES, smem_p = HgPrepSmem<KT, VT>::BYTES,
                smem_w = HgWalkSmem<KT>::BYTES;
  static bool attr_set_dev[64];  // the attribute belongs to the device's copy of the kernel
  int cur_dev = 0;
  if (hipGetDevice(&cur_dev) != hipSuccess || cur_dev < 0 || cur_dev >= 64) return LAMPA_ERR_LAUNCH;
  bool& attr_set = attr_set_dev[cur_dev];
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)gdr_segment_kernel<T, KT, VT, false, false, __bf16>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, smem_a) != hipSuccess ||
        hipFuncSetAttribute((const void*)hgdn_prep_kernel<T, KT, VT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            smem_p) != hipSuccess ||
        hipFuncSetAttribute((const void*)hgdn_walk_kernel<T, KT, VT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            smem_w) != hipSuccess)
      return LAMPA_ERR_LAUNCH;
    attr_set = true;
  }
  LAMPA_PROF(s, "start");
  if (chunks == 0) return LAMPA_OK;
  // (the hierarchical kernels keep bf16 operands whatever the input type)
  hipLaunchKernelGGL((gdr_local_kernel<T, __bf16, KT>), dim3(gdr_local_grid(chunks, HV)), dim3(64), 0, s, (const T*)k, g,
                     beta, pv.chunk_tok0, pv.chunk_len, tf, chunks, H, HV, l2norm);
  LAMPA_PROF(s, "gdr_local_kernel");
  const bool split = segs > n_seq;
  // The segment composites and their scan depend on T only, like the prep kernel, and are latency bound on a few
  // workgroups: they run on a second stream (default priority) beside the prep kernel (launched first, which
  // measured slightly better than the other order) and join before the walk.
  // With a profile recording open everything stays on the caller's stream, so that the intervals mean one kernel each.
  bool overlap = split && !lampa_prof_recording();
  std::unique_lock<std::mutex> hold(hg_side_lock, std::defer_lock);
  HgSide* sd = nullptr;
  if (overlap) {
    hold.lock();
    sd = hg_side_for(s);
    if (!sd) { overlap = false; hold.unlock(); }
  }
  hipStream_t side = sd ? sd->side : s;
  hipEvent_t ev_fork = sd ? sd->fork : nullptr, ev_join = sd ? sd->join : nullptr;
  hipStream_t cs = s;  // the stream of the composites
  if (overlap) {
    if (hipEventRecord(ev_fork, s) != hipSuccess || hipStreamWaitEvent(side, ev_fork, 0) != hipSuccess) return LAMPA_ERR_LAUNCH;
    cs = side;
  }
  hipLaunchKernelGGL((hgdn_prep_kernel<T, KT, VT>), dim3(chunks, HV), dim3(256), smem_p, s, (const T*)q, (const T*)k,
                     (const T*)v, lam, lam_dtype, lam_div, pv.chunk_tok0, pv.chunk_len, tf, rec, Ubw, Oi, hstates, chunks_per_seq, H, HV, L,
                     scale, l2norm);
  LAMPA_PROF(s, "hgdn_prep_kernel");
  if (split) {
    hipLaunchKernelGGL((gdr_segment_kernel<T, KT, VT, false, false, __bf16>), dim3(segs, HV),
                       dim3(64 * GdrSegShape<KT, VT, false>::WAVES), smem_a, cs, (const T*)q, (const T*)k, (const T*)v, g,
                       beta, pv, pv.chunk_tok0, pv.chunk_len, tf, (const float*)nullptr, Mc, Nm, Dc, (T*)nullptr,
                       (float*)nullptr, H, HV, scale, l2norm, (const unsigned char*)nullptr,
                       (const unsigned char*)nullptr, (const float*)nullptr, (const float*)nullptr, 0);
    LAMPA_PROF(s, "gdr_segment_kernel<composite>");
    hipLaunchKernelGGL((hgdn_scan_kernel<KT, VT>), dim3(VT / 32, n_seq, HV), dim3(64 * HG_CW), 0, cs, pv, Mc, Nm, Dc, Xi,
                       HV, p);
    LAMPA_PROF(s, "hgdn_scan_kernel");
    if (overlap && hipEventRecord(ev_join, side) != hipSuccess) return LAMPA_ERR_LAUNCH;
  }
  if (overlap) {
    if (hipStreamWaitEvent(s, ev_join, 0) != hipSuccess) return LAMPA_ERR_LAUNCH;
    hold.unlock();
  }
  hipLaunchKernelGGL((hgdn_walk_kernel<T, KT, VT>), dim3(segs, HV, VT / 32), dim3(64 * (HG_CW + 2)), smem_w, s, pv,
                     pv.chunk_tok0, pv.chunk_len, (const T*)k, H, rec, Ubw, Oi, split ? (const float*)Xi : (const float*)nullptr, (T*)o,
                     hstates, L, HV);
  LAMPA_PROF(s, "hgdn_walk_kernel");
  return lampa_launch_status();
}

// Hierarchical chunkwise forward. q, k [total_tokens, H, K]; v, o [total_tokens, HV, V] (dtype 0 bf16 / 1 fp16);
// g, beta fp32 [total_tokens, HV]; lam [total_tokens, HV, L] of type lam_dtype (0 bf16 / 1 fp16 / 2 fp32): the level
// weights; the kernel uses lam / lam_div rounded to lam's type (the reference divides the weights by `scale`, which
// multiplies q, before its kernel; lam_div = 1 takes them as they are). The plan's chunks_per_segment must be a
// power of two (or at least the longest sequence's chunk count: one segment per sequence); every sequence may hold at
// most 2^12 chunks, every sequence length must be a multiple of 64 and L must cover 7 + the number of chunk-index bits
// of the longest sequence.
// level_states (nullable): fp32 [n_seq, HV, K, V, L], ZEROED by the caller; receives the occupied levels' states after
// the last token of every sequence (the reference's HState.states); needs sequences of equal length, a multiple of 64.
extern "C" int lampa_hgdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                    const void* lam, int lam_dtype, float lam_div, void* o, float* level_states,
                                    const int32_t* plan_host, const int32_t* plan_dev, int H, int HV, int K, int V, int L,
                                    int dtype, float scale, int l2norm, void* workspace, int64_t workspace_bytes,
                                    void* stream) {
  if (!q || !k || !v || !g || !beta || !lam || !o || !plan_host || !plan_dev) return LAMPA_ERR_INVALID;
  if (H < 1 || HV < H || HV % H != 0 || l2norm < 0 || l2norm > 2 || L < HG_INTRA) return LAMPA_ERR_INVALID;
  if (lam_dtype < 0 || lam_dtype > 2 || !(lam_div > 0.0f)) return LAMPA_ERR_INVALID;
  if (!hg_supported(K, V) || (dtype != GDR_BF16 && dtype != GDR_FP16)) return LAMPA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15) return LAMPA_ERR_INVALID;
  const int n_seq = plan_host[PLAN_N_SEQ], chunks = plan_host[PLAN_TOTAL_CHUNKS], segs = plan_host[PLAN_N_SEGMENTS];
  const int cps = plan_host[PLAN_CHUNKS_PER_SEGMENT];
  if (n_seq < 1 || segs < n_seq) return LAMPA_ERR_INVALID;
  int p = 0;
  if (segs > n_seq) {
    if (cps & (cps - 1)) return LAMPA_ERR_INVALID;
    while ((1 << p) < cps) ++p;
  }
  int max_nc = 0;
  for (int i = 0; i < n_seq; ++i) {
    const int s0 = plan_host[plan_host[PLAN_OFF_SEQ_SEG0] + i], ns = plan_host[plan_host[PLAN_OFF_SEQ_NSEG] + i];
    int nc = 0;
    for (int j = 0; j < ns; ++j) nc += plan_host[plan_host[PLAN_OFF_SEG_NCHUNKS] + s0 + j];
    max_nc = nc > max_nc ? nc : max_nc;
  }
  if (max_nc > (1 << HG_NLV)) return LAMPA_ERR_UNSUPPORTED;
  // whole chunks only, as the reference demands (chunkwise_hgdn.py:598-601)
  if ((int64_t)chunks * GDR_C != plan_host[PLAN_TOTAL_TOKENS]) return LAMPA_ERR_INVALID;
  if (level_states) {  // every sequence: the same whole number of chunks
    if (max_nc < 1 || (int64_t)max_nc * n_seq != chunks) return LAMPA_ERR_INVALID;
  }
  int bits = 0;
  while ((1 << bits) < max_nc) ++bits;
  if (HG_INTRA + bits > L) return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < hg_workspace(chunks, segs, HV, K, V).bytes) return LAMPA_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  unsigned char* ws = (unsigned char*)workspace;
  const GdrPlanView pv = gdr_plan_view(plan_host, plan_dev);
#define HG_CASE(TT, KK, VV) \
  return hg_launch<TT, KK, VV>(q, k, v, g, beta, lam, lam_dtype, lam_div, o, level_states, max_nc, pv, n_seq, chunks, segs, p, H, HV, L, scale, l2norm, ws, s)
  if (dtype == GDR_BF16) {
    if (V == 64) HG_CASE(__bf16, 64, 64);
    if (V == 128) HG_CASE(__bf16, 64, 128);
  } else {
    if (V == 64) HG_CASE(_Float16, 64, 64);
    if (V == 128) HG_CASE(_Float16, 64, 128);
  }
#undef HG_CASE
  return LAMPA_ERR_UNSUPPORTED;
}

// One token of the hierarchical (level-weighted) gated delta rule on explicit level states.
//
// Replaces hattention_step (reference chengjiang123/Lampa, models/hattention/kernel.py:577-633) with
// step_state / step_output (recurrent.py:134-166) and HState.cascade_weak / insert (recurrent.py:44-97):
//   cascade   the full levels 0 .. z-1 are added into level z and emptied (lowest first);
//   gate      S_l <- a (S_l - b k (k^T S_l)) for every level, a = e^g;
//   insert    S_0 <- b k v^T;
//   output    o = q^T sum_l lambda_l S_l      (q l2-normalised and scaled, k l2-normalised, kernel.py:613-616).
// The level states are the reference's HState.states: fp32 [B, HV, K, V, L] with the level index fastest. Which levels
// are full depends only on the number of tokens seen, so the caller passes z (0 = nothing to merge).
// Workgroup per (sequence, value head, 16 value columns), 256 threads = 16 row groups x 16 columns: every thread walks
// the rows i = group, group + 16, ... of its column twice (k^T S_l first, summed over the groups through LDS, then the
// update); a row's L level values are contiguous, 16 columns of a row are one contiguous piece.
#include "gdr_common.h"

#define HGS_LMAX 32

#define HGS_COLS 16
#define HGS_GROUPS 16
#define HGS_LOADS 6  // 16-byte loads a thread of the LDS-staged form keeps in flight
#define HGS_ROWS 4   // rows of a thread's position whose LDS reads are in flight together
#define HGS_LDS_LIMIT (144 * 1024)  // dynamic LDS of the LDS-staged form at most (a CU has 160 KB)

template <typename T, int LM>
__global__ void __launch_bounds__(256)
    hgdn_step_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                     const float* __restrict__ g, const float* __restrict__ beta, const void* __restrict__ lam,
                     int lam_dtype, float lam_div, float* __restrict__ states, T* __restrict__ o, int H, int HV, int K,
                     int V, int L, int z, float scale, int l2norm) {
  extern __shared__ float s_qk[];  // q [K], k [K], lambda [HGS_LMAX], norm scratch [8], partial sums
  float* s_q = s_qk;
  float* s_k = s_qk + K;
  float* s_l = s_qk + 2 * K;
  float* s_red = s_l + HGS_LMAX;
  float* s_part = s_red + 8;  // [HGS_GROUPS][HGS_COLS][HGS_LMAX + 1]
  float* s_tot = s_part + HGS_GROUPS * HGS_COLS * (HGS_LMAX + 1);  // [HGS_COLS][HGS_LMAX + 1]
  float* s_m = s_tot + HGS_COLS * (HGS_LMAX + 1);                  // cascade coefficients, 3 x [HGS_LMAX]
  const int b = blockIdx.x / HV, hv = blockIdx.x % HV, h = hv / (HV / H);
  const int tid = threadIdx.x;
  const T* qp = q + ((size_t)b * H + h) * K;
  const T* kp = k + ((size_t)b * H + h) * K;
  float qs = 0.0f, ks = 0.0f;
  for (int i = tid; i < K; i += blockDim.x) {
    const float qi = GdrElem<T>::to_float(qp[i]), ki = GdrElem<T>::to_float(kp[i]);
    s_q[i] = qi;
    s_k[i] = ki;
    qs = __builtin_fmaf(qi, qi, qs);
    ks = __builtin_fmaf(ki, ki, ks);
  }
  for (int off = 32; off > 0; off >>= 1) {
    qs += __shfl_xor(qs, off);
    ks += __shfl_xor(ks, off);
  }
  if ((tid & 63) == 0) {
    s_red[2 * (tid >> 6)] = qs;
    s_red[2 * (tid >> 6) + 1] = ks;
  }
  if (tid < HGS_LMAX) {
    float x = 0.0f;  // levels past L weigh nothing
    if (tid < L) {
      const size_t li = ((size_t)b * HV + hv) * L + tid;
      x = lam_dtype == GDR_FP32   ? reinterpret_cast<const float*>(lam)[li]
          : lam_dtype == GDR_BF16 ? (float)reinterpret_cast<const __bf16*>(lam)[li]
                                  : (float)reinterpret_cast<const _Float16*>(lam)[li];
      if (lam_div != 1.0f) {  // lambda / scale, rounded to lambda's own type as the element-wise division would
        x = __fdiv_rn(x, lam_div);
        x = lam_dtype == GDR_FP32 ? x : lam_dtype == GDR_BF16 ? (float)(__bf16)x : (float)(_Float16)x;
      }
    }
    s_l[tid] = x;
    // the cascade as arithmetic on 0 / 1 coefficients (no branches in the row loops): the full levels below z are
    // summed, level z takes the sum, levels past L (loaded from a clamped index) are dropped
    s_m[tid] = (tid < L && tid < z) ? 1.0f : 0.0f;                 // enters the sum
    s_m[HGS_LMAX + tid] = (tid < L && tid >= z) ? 1.0f : 0.0f;     // keeps its value
    s_m[2 * HGS_LMAX + tid] = (z > 0 && tid == z) ? 1.0f : 0.0f;   // receives the sum
  }
  __syncthreads();
  qs = 0.0f;
  ks = 0.0f;
  for (int w = 0; w < 4; ++w) {
    qs += s_red[2 * w];
    ks += s_red[2 * w + 1];
  }
  float rq = scale, rk = 1.0f;
  if (l2norm == GDR_L2_CHUNK) {
    rq = scale / __fsqrt_rn(qs + 1e-6f);
    rk = 1.0f / __fsqrt_rn(ks + 1e-6f);
  } else if (l2norm == GDR_L2_RECURRENT) {
    rq = scale / (__fsqrt_rn(qs) + 1e-6f);
    rk = 1.0f / (__fsqrt_rn(ks) + 1e-6f);
  }
  const int grp = tid / HGS_COLS, jl = tid % HGS_COLS;
  const int j = blockIdx.y * HGS_COLS + jl;
  const bool live = j < V;
  const int jc = live ? j : V - 1;  // (idle threads shadow the last column and store nothing)
  const float a = __expf(g[(size_t)b * HV + hv]), bt = beta[(size_t)b * HV + hv];
  const float vj = GdrElem<T>::to_float(v[((size_t)b * HV + hv) * V + jc]);
  float* col = states + (((size_t)b * HV + hv) * K * V + jc) * L;  // row i of this column: col + i * V * L
  const size_t rs = (size_t)V * L;

  // A row's level values: LM unconditional loads (indices past L - 1 re-read the last level and are dropped), so that
  // all of them -- and those of the second row of a pair -- are in flight together; then the cascade.
  auto load_row = [&](const float* p, float* S) {
#pragma unroll
    for (int l = 0; l < LM; ++l) S[l] = p[min(l, L - 1)];
  };
  float m_sum[LM], m_keep[LM], m_take[LM];
#pragma unroll
  for (int l = 0; l < LM; ++l) {
    m_sum[l] = s_m[l];
    m_keep[l] = s_m[HGS_LMAX + l];
    m_take[l] = s_m[2 * HGS_LMAX + l];
  }
  auto cascade = [&](float* S) {
    float acc = m_sum[0] * S[0];
#pragma unroll
    for (int l = 1; l < LM; ++l) acc = __builtin_fmaf(m_sum[l], S[l], acc);  // S_1 + S_0, then + S_2 ...: exact 0 / 1 factors
#pragma unroll
    for (int l = 0; l < LM; ++l) S[l] = __builtin_fmaf(m_take[l], acc, m_keep[l] * S[l]);
  };
  float d[LM];
#pragma unroll
  for (int l = 0; l < LM; ++l) d[l] = 0.0f;
  for (int i = grp; i < K; i += 2 * HGS_GROUPS) {
    const int i2 = i + HGS_GROUPS;
    const bool two = i2 < K;
    float S[LM], S2[LM];
    load_row(col + i * rs, S);
    load_row(col + (two ? i2 : i) * rs, S2);
    cascade(S);
    cascade(S2);
    const float ki = s_k[i] * rk, ki2 = two ? s_k[i2] * rk : 0.0f;
#pragma unroll
    for (int l = 1; l < LM; ++l) d[l] = __builtin_fmaf(ki2, S2[l], __builtin_fmaf(ki, S[l], d[l]));
  }
  float* mine = s_part + (grp * HGS_COLS + jl) * (HGS_LMAX + 1);
  mine[0] = 0.0f;
#pragma unroll
  for (int l = 1; l < LM; ++l) mine[l] = d[l];
  __syncthreads();
  // sums over the row groups: one (column, level) pair per thread and round, then every thread takes its column's
  for (int pair = tid; pair < HGS_COLS * LM; pair += 256) {
    const int pc = pair / LM, pl = pair % LM;
    float t = 0.0f;
#pragma unroll
    for (int gq = 0; gq < HGS_GROUPS; ++gq) t += s_part[(gq * HGS_COLS + pc) * (HGS_LMAX + 1) + pl];
    s_tot[pc * (HGS_LMAX + 1) + pl] = t;
  }
  __syncthreads();
#pragma unroll
  for (int l = 1; l < LM; ++l) d[l] = s_tot[jl * (HGS_LMAX + 1) + l];
  float acc_o = 0.0f;
  auto update_row = [&](int i, float* S) {
    const float ki = s_k[i] * rk, qi = s_q[i] * rq;
    float sl = 0.0f;
    S[0] = bt * ki * vj;
#pragma unroll
    for (int l = 1; l < LM; ++l) S[l] = a * (S[l] - bt * ki * d[l]);
#pragma unroll
    for (int l = 0; l < LM; ++l) sl = __builtin_fmaf(s_l[l], S[l], sl);
    if (live) {
#pragma unroll
      for (int l = 0; l < LM; ++l)
        if (l < L) col[i * rs + l] = S[l];
    }
    acc_o = __builtin_fmaf(qi, sl, acc_o);
  };
  for (int i = grp; i < K; i += 2 * HGS_GROUPS) {
    const int i2 = i + HGS_GROUPS;
    const bool two = i2 < K;
    float S[LM], S2[LM];
    load_row(col + i * rs, S);
    load_row(col + (two ? i2 : i) * rs, S2);
    cascade(S);
    cascade(S2);
    update_row(i, S);
    if (two) update_row(i2, S2);
  }
  __syncthreads();  // every thread is done with the k^T S sums
  mine[0] = acc_o;
  __syncthreads();
  if (grp == 0 && live) {
    float t = 0.0f;
    for (int gq = 0; gq < HGS_GROUPS; ++gq) t += s_part[(gq * HGS_COLS + jl) * (HGS_LMAX + 1)];
    o[((size_t)b * HV + hv) * V + j] = GdrElem<T>::from_float(t);
  }
}

// The same token with the workgroup's part of the state staged in LDS: COLS value columns of every row are one
// contiguous piece of COLS * L floats, so the K pieces are read once with 16-byte accesses, worked on in LDS and written
// back once with 16-byte accesses. The cascade runs with a thread per (row, column) -- the only step that couples the
// levels of a row -- then a thread owns one (column, level) position of the piece and walks the rows
// i = group, group + 256 / (COLS * L), ...; k^T S_l and the output are sums of per-thread partial sums through LDS.
// Needs COLS * L <= 256, V * L a multiple of 4 floats, V a multiple of COLS and the pieces to fit in LDS; the kernel
// above covers the rest.
template <typename T, int COLS>
__global__ void __launch_bounds__(256)
    hgdn_step_lds_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                         const float* __restrict__ g, const float* __restrict__ beta, const void* __restrict__ lam,
                         int lam_dtype, float lam_div, float* __restrict__ states, T* __restrict__ o, int H, int HV,
                         int K, int V, int L, int z, float scale, int l2norm) {
  extern __shared__ float4 s_raw4[];
  const int PW = COLS * L;
  float* s_slab = reinterpret_cast<float*>(s_raw4);  // [K][PW], 16-byte aligned
  float* s_q = s_slab + K * PW;
  float* s_k = s_q + K;
  float* s_red = s_k + K;     // [8]
  float* s_part = s_red + 8;  // [256] partial sums of k^T S_l, then of the output
  const int b = blockIdx.x / HV, hv = blockIdx.x % HV, h = hv / (HV / H);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int groups = 256 / PW;
  const bool active = tid < groups * PW;
  const int grp = tid / PW, c = tid - grp * PW, jl = c / L, l = c - jl * L;
  // the token's own values first (short loads, in flight together with the pieces)
  const T* qp = q + ((size_t)b * H + h) * K;
  const T* kp = k + ((size_t)b * H + h) * K;
  float q0 = 0.0f, k0 = 0.0f, lam_l = 0.0f, vj = 0.0f;
  if (tid < K) {
    q0 = GdrElem<T>::to_float(qp[tid]);
    k0 = GdrElem<T>::to_float(kp[tid]);
  }
  if (active) {
    const size_t li = ((size_t)b * HV + hv) * L + l;
    lam_l = lam_dtype == GDR_FP32   ? reinterpret_cast<const float*>(lam)[li]
            : lam_dtype == GDR_BF16 ? (float)reinterpret_cast<const __bf16*>(lam)[li]
                                    : (float)reinterpret_cast<const _Float16*>(lam)[li];
    vj = GdrElem<T>::to_float(v[((size_t)b * HV + hv) * V + blockIdx.y * COLS + jl]);
  }
  const float g_tok = g[(size_t)b * HV + hv], bt = beta[(size_t)b * HV + hv];
  float* base = states + (((size_t)b * HV + hv) * K * V + (size_t)blockIdx.y * COLS) * L;  // row i: base + i * V * L
  const size_t rs = (size_t)V * L;
  const int p4 = PW / 4, n4 = K * p4;
  // the piece loads of a batch are all issued before the first is stored to LDS (one round trip per batch)
  for (int e0 = tid; e0 < n4; e0 += 256 * HGS_LOADS) {
    float4 r[HGS_LOADS];
#pragma unroll
    for (int u = 0; u < HGS_LOADS; ++u) {
      const int e = e0 + 256 * u;
      if (e < n4) {
        const int i = e / p4, c4 = e - i * p4;
        r[u] = reinterpret_cast<const float4*>(base + i * rs)[c4];
      }
    }
#pragma unroll
    for (int u = 0; u < HGS_LOADS; ++u) {
      const int e = e0 + 256 * u;
      if (e < n4) reinterpret_cast<float4*>(s_slab)[e] = r[u];
    }
  }
  float qs = q0 * q0, ks = k0 * k0;
  if (tid < K) {
    s_q[tid] = q0;
    s_k[tid] = k0;
  }
  for (int i = tid + 256; i < K; i += 256) {
    const float qi = GdrElem<T>::to_float(qp[i]), ki = GdrElem<T>::to_float(kp[i]);
    s_q[i] = qi;
    s_k[i] = ki;
    qs = __builtin_fmaf(qi, qi, qs);
    ks = __builtin_fmaf(ki, ki, ks);
  }
  for (int off = 32; off > 0; off >>= 1) {
    qs += __shfl_xor(qs, off);
    ks += __shfl_xor(ks, off);
  }
  if (lane == 0) {
    s_red[2 * wave] = qs;
    s_red[2 * wave + 1] = ks;
  }
  if (lam_div != 1.0f) {  // lambda / scale, rounded to lambda's own type as the element-wise division would
    lam_l = __fdiv_rn(lam_l, lam_div);
    lam_l = lam_dtype == GDR_FP32 ? lam_l : lam_dtype == GDR_BF16 ? (float)(__bf16)lam_l : (float)(_Float16)lam_l;
  }
  const float a = __expf(g_tok);
  __syncthreads();
  qs = 0.0f;
  ks = 0.0f;
  for (int w = 0; w < 4; ++w) {
    qs += s_red[2 * w];
    ks += s_red[2 * w + 1];
  }
  float rq = scale, rk = 1.0f;
  if (l2norm == GDR_L2_CHUNK) {
    rq = scale / __fsqrt_rn(qs + 1e-6f);
    rk = 1.0f / __fsqrt_rn(ks + 1e-6f);
  } else if (l2norm == GDR_L2_RECURRENT) {
    rq = scale / (__fsqrt_rn(qs) + 1e-6f);
    rk = 1.0f / (__fsqrt_rn(ks) + 1e-6f);
  }
  // cascade, a (row, column) pair per thread: the full levels below z are summed (S_1 + S_0, then + S_2 ...) into
  // level z and emptied
  if (z > 0) {
    for (int pr = tid; pr < K * COLS; pr += 256) {
      float* lv = s_slab + (pr / COLS) * PW + (pr % COLS) * L;
      float acc = lv[0];
      lv[0] = 0.0f;
      for (int m = 1; m < z; ++m) {
        acc += lv[m];
        lv[m] = 0.0f;
      }
      lv[z] += acc;
    }
    __syncthreads();
  }
  // k^T S_l on the unscaled key (the key's norm enters through the coefficients below); a thread's rows in batches
  // whose LDS reads are all issued before the first is used, the last rows one by one
  const int stride = groups * PW;
  const int n_rows = active ? (K - grp + groups - 1) / groups : 0;  // rows grp, grp + groups, ...
  float d = 0.0f;
  {
    const float* kr = s_k + grp;
    const float* sr = s_slab + grp * PW + c;
    int n = n_rows;
    for (; n >= HGS_ROWS; n -= HGS_ROWS, kr += HGS_ROWS * groups, sr += HGS_ROWS * stride) {
      float kk[HGS_ROWS], sv[HGS_ROWS];
#pragma unroll
      for (int u = 0; u < HGS_ROWS; ++u) {
        kk[u] = kr[u * groups];
        sv[u] = sr[u * stride];
      }
#pragma unroll
      for (int u = 0; u < HGS_ROWS; ++u) d = __builtin_fmaf(kk[u], sv[u], d);
    }
    for (; n > 0; --n, kr += groups, sr += stride) d = __builtin_fmaf(kr[0], sr[0], d);
  }
  s_part[tid] = d;
  __syncthreads();
  d = 0.0f;
  for (int gq = 0; gq < groups; ++gq) d += s_part[gq * PW + c];
  __syncthreads();  // every thread has its sum before the partial sums are used again
  // gate, insert, output: S <- c_a (c_m S + k_i c_b), with the coefficients of the thread's level
  //   l > 0: a (S - b k_i rk (rk d))      l = 0: b k_i rk v_j
  const float c_a = l == 0 ? 1.0f : a, c_m = l == 0 ? 0.0f : 1.0f, c_b = l == 0 ? bt * rk * vj : -(bt * rk) * (rk * d);
  float acc_o = 0.0f;
  {
    const float* kr = s_k + grp;
    const float* qr = s_q + grp;
    float* sr = s_slab + grp * PW + c;
    int n = n_rows;
    for (; n >= HGS_ROWS; n -= HGS_ROWS, kr += HGS_ROWS * groups, qr += HGS_ROWS * groups, sr += HGS_ROWS * stride) {
      float kk[HGS_ROWS], qq[HGS_ROWS], sv[HGS_ROWS];
#pragma unroll
      for (int u = 0; u < HGS_ROWS; ++u) {
        kk[u] = kr[u * groups];
        qq[u] = qr[u * groups];
        sv[u] = sr[u * stride];
      }
#pragma unroll
      for (int u = 0; u < HGS_ROWS; ++u) {
        const float x = c_a * __builtin_fmaf(kk[u], c_b, c_m * sv[u]);
        sr[u * stride] = x;
        acc_o = __builtin_fmaf(qq[u], x, acc_o);
      }
    }
    for (; n > 0; --n, kr += groups, qr += groups, sr += stride) {
      const float x = c_a * __builtin_fmaf(kr[0], c_b, c_m * sr[0]);
      sr[0] = x;
      acc_o = __builtin_fmaf(qr[0], x, acc_o);
    }
  }
  acc_o *= rq;
  s_part[tid] = lam_l * acc_o;
  __syncthreads();  // the updated rows and the output's partial sums are in LDS
  if (tid < COLS) {
    float t = 0.0f;
    for (int gq = 0; gq < groups; ++gq)
      for (int m = 0; m < L; ++m) t += s_part[gq * PW + tid * L + m];
    o[((size_t)b * HV + hv) * V + blockIdx.y * COLS + tid] = GdrElem<T>::from_float(t);
  }
  for (int e = tid; e < n4; e += 256) {
    const int i = e / p4, c4 = e - i * p4;
    reinterpret_cast<float4*>(base + i * rs)[c4] = reinterpret_cast<const float4*>(s_slab)[e];
  }
}

struct HgsArgs {
  const void *q, *k, *v;
  const float *g, *beta;
  const void* lam;
  int lam_dtype;
  float lam_div;
  float* states;
  void* o;
  int B, H, HV, K, V, L, z;
  float scale;
  int l2norm;
};

// One instantiation of the LDS-staged form: raises its dynamic LDS limit on the current device (set_attr) and launches
// it when it is the one picked.
template <typename TT, int CC>
static bool hgs_lds_one(const HgsArgs& a, bool set_attr, bool launch, size_t smem, hipStream_t s) {
  if (set_attr && hipFuncSetAttribute((const void*)hgdn_step_lds_kernel<TT, CC>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, HGS_LDS_LIMIT) != hipSuccess)
    return false;
  if (launch)
    hipLaunchKernelGGL((hgdn_step_lds_kernel<TT, CC>), dim3(a.B * a.HV, a.V / CC), dim3(256), smem, s, (const TT*)a.q,
                       (const TT*)a.k, (const TT*)a.v, a.g, a.beta, a.lam, a.lam_dtype, a.lam_div, a.states, (TT*)a.o,
                       a.H, a.HV, a.K, a.V, a.L, a.z, a.scale, a.l2norm);
  return true;
}

template <typename TT>
static bool hgs_lds_type(const HgsArgs& a, bool set_attr, bool mine, int cols, size_t smem, hipStream_t s) {
  return hgs_lds_one<TT, 4>(a, set_attr, mine && cols == 4, smem, s) &&
         hgs_lds_one<TT, 8>(a, set_attr, mine && cols == 8, smem, s);
}

// q, k [B, H, K]; v, o [B, HV, V] (dtype 0 bf16 / 1 fp16 / 2 fp32); g (log decay), beta fp32 [B, HV]; lam [B, HV, L] of
// lam_dtype, used as lam / lam_div rounded to its type; states fp32 [B, HV, K, V, L], updated in place;
// z: the levels 0 .. z-1 are full and cascade into level z (0: the state is empty). L <= 32.
extern "C" int lampa_hgdn_step(const void* q, const void* k, const void* v, const float* g, const float* beta,
                               const void* lam, int lam_dtype, float lam_div, float* states, void* o, int B, int H, int HV,
                               int K, int V, int L, int z, int dtype, float scale, int l2norm, void* stream) {
  if (!q || !k || !v || !g || !beta || !lam || !states || !o) return LAMPA_ERR_INVALID;
  if (B < 0 || H < 1 || HV < H || HV % H != 0 || K < 1 || V < 1 || L < 1 || z < 0 || z >= L) return LAMPA_ERR_INVALID;
  if (l2norm < 0 || l2norm > 2 || lam_dtype < 0 || lam_dtype > 2 || !(lam_div > 0.0f)) return LAMPA_ERR_INVALID;
  if (V > 1024 || L > HGS_LMAX || K > 4096 || dtype < 0 || dtype > 2) return LAMPA_ERR_UNSUPPORTED;
  if (B == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  LAMPA_PROF(s, "start");
  // the LDS-staged form where its layout conditions hold: 4 columns per workgroup (most workgroups, shortest loads)
  // unless the launch is large enough to fill the device with 8
  auto lds_bytes = [&](int cols) { return ((size_t)K * cols * L + 2 * (size_t)K + 8 + 256) * sizeof(float); };
  auto fits = [&](int cols) {
    return V % cols == 0 && cols * L <= 256 && ((size_t)V * L) % 4 == 0 &&
           (reinterpret_cast<uintptr_t>(states) & 15) == 0 && lds_bytes(cols) <= HGS_LDS_LIMIT;
  };
  const int cols = ((size_t)B * HV * (V / 4) > 8192 && fits(8)) ? 8 : fits(4) ? 4 : 0;
  if (cols) {
    static bool attr_set[64] = {};  // per device: the dynamic LDS limit of every instantiation (a repeated set is harmless)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LAMPA_ERR_LAUNCH;
    const HgsArgs a = {q, k, v, g, beta, lam, lam_dtype, lam_div, states, o, B, H, HV, K, V, L, z, scale, l2norm};
    const bool set_attr = !attr_set[dev];
    if (!hgs_lds_type<__bf16>(a, set_attr, dtype == GDR_BF16, cols, lds_bytes(cols), s) ||
        !hgs_lds_type<_Float16>(a, set_attr, dtype == GDR_FP16, cols, lds_bytes(cols), s) ||
        !hgs_lds_type<float>(a, set_attr, dtype == GDR_FP32, cols, lds_bytes(cols), s))
      return LAMPA_ERR_LAUNCH;
    attr_set[dev] = true;
    LAMPA_PROF(s, "hgdn_step_lds_kernel");
    return lampa_launch_status();
  }
  const size_t smem = (2 * (size_t)K + 4 * HGS_LMAX + 8 + (HGS_GROUPS + 1) * HGS_COLS * (HGS_LMAX + 1)) * sizeof(float);
#define HGS_LAUNCH(TT, LM)                                                                                         \
  hipLaunchKernelGGL((hgdn_step_kernel<TT, LM>), dim3(B * HV, (V + HGS_COLS - 1) / HGS_COLS), dim3(256), smem, s,  \
                     (const TT*)q, (const TT*)k, (const TT*)v, g, beta, lam, lam_dtype, lam_div, states, (TT*)o, H, \
                     HV, K, V, L, z, scale, l2norm)
#define HGS_CASE(TT)                    \
  do {                                  \
    if (L <= 16) HGS_LAUNCH(TT, 16);    \
    else if (L <= 24) HGS_LAUNCH(TT, 24); \
    else HGS_LAUNCH(TT, 32);            \
  } while (0)
  if (dtype == GDR_BF16) HGS_CASE(__bf16);
  else if (dtype == GDR_FP16) HGS_CASE(_Float16);
  else HGS_CASE(float);
#undef HGS_CASE
#undef HGS_LAUNCH
  LAMPA_PROF(s, "hgdn_step_kernel");
  return lampa_launch_status();
}

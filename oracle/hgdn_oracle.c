/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the hierarchical (level-weighted) gated-delta-rule forward.
 * Nothing in the shipped package may link or call this file.
 *
 * Restates (reference = chengjiang123/Lampa):
 *   models/hattention/recurrent.py:44-56    HState.cascade_weak: level j holds at most 2^j tokens; a full level is
 *                                           added into the next one and emptied, lowest level first
 *   models/hattention/recurrent.py:84-97    HState.insert: cascade, apply the gate to EVERY level, put the new
 *                                           token's value into level 0
 *   models/hattention/recurrent.py:134-155  step_state: gate = a (I - b k k^T), value = b k v^T
 *   models/hattention/recurrent.py:158-166  step_output: o = q^T sum_l lambda_l S_l
 *   models/hattention/kernel.py:100-101     q = l2norm(q) * scale, k = l2norm(k) (chunk-path l2norm,
 *                                           l2norm.py:100-101)
 * Per (sequence, head value-head), L level states S_l [K,V] and their token counts, for each token t:
 *   cascade; S_l <- a_t (S_l - b_t k (k^T S_l)) for all l; S_0 <- b_t k v^T; o_t = sum_l lam[t,l] q^T S_l
 * Pins (tests/test_oracle_hgdn.py): all lambda = 1 equals the plain gated-delta oracle; the quadratic form with
 * the level of a (target, source) pair taken from the recursion of base.py:41-46; one-hot lambda.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* states_in / states_out: optional level states [n_seq, HV, K, V, L] (L fastest, the reference's HState.states layout,
 * recurrent.py:33-36); counts_in / counts_out: optional token counts per level [L] (shared by all sequences and heads,
 * recurrent.py:37-40). */
void oracle_hgdn_recurrent_state_f64(const float* q, const float* k, const float* v, const float* g, const float* beta,
                                     const float* lam, const int64_t* cu_seqlens, int n_seq, int H, int HV, int K, int V,
                                     int L, float scale, int l2norm, const float* states_in, const int32_t* counts_in,
                                     float* o, float* states_out, int32_t* counts_out) {
  const size_t KV = (size_t)K * V;
  double* S = (double*)malloc(sizeof(double) * KV * L);
  int64_t* cnt = (int64_t*)malloc(sizeof(int64_t) * L);
  double* qn = (double*)malloc(sizeof(double) * K);
  double* kn = (double*)malloc(sizeof(double) * K);
  double* d = (double*)malloc(sizeof(double) * V);
  const int rep = HV / H;
  for (int s = 0; s < n_seq; ++s)
    for (int hv = 0; hv < HV; ++hv) {
      const int h = hv / rep;
      memset(S, 0, sizeof(double) * KV * L);
      memset(cnt, 0, sizeof(int64_t) * L);
      if (states_in)
        for (int l = 0; l < L; ++l)
          for (size_t i = 0; i < KV; ++i) S[(size_t)l * KV + i] = states_in[(((size_t)s * HV + hv) * KV + i) * L + l];
      if (counts_in)
        for (int l = 0; l < L; ++l) cnt[l] = counts_in[l];
      for (int64_t t = cu_seqlens[s]; t < cu_seqlens[s + 1]; ++t) {
        const float* qt = q + (t * H + h) * K;
        const float* kt = k + (t * H + h) * K;
        const float* vt = v + (t * HV + hv) * V;
        double qs = 0, ks = 0;
        for (int i = 0; i < K; ++i) { qs += (double)qt[i] * qt[i]; ks += (double)kt[i] * kt[i]; }
        double qi = 1, ki = 1;
        if (l2norm == 1) { qi = 1 / sqrt(qs + 1e-6); ki = 1 / sqrt(ks + 1e-6); }
        for (int i = 0; i < K; ++i) { qn[i] = (double)qt[i] * qi * (double)scale; kn[i] = (double)kt[i] * ki; }
        /* cascade_weak */
        for (int l = 0; l < L; ++l) {
          const int64_t cap = (int64_t)1 << l;
          if (cnt[l] == cap) {
            if (l + 1 < L) {
              for (size_t i = 0; i < KV; ++i) S[(size_t)(l + 1) * KV + i] += S[(size_t)l * KV + i];
              cnt[l + 1] += cnt[l];
            }
            memset(S + (size_t)l * KV, 0, sizeof(double) * KV);
            cnt[l] = 0;
          } else {
            break;
          }
        }
        const double a = exp((double)g[t * HV + hv]), b = (double)beta[t * HV + hv];
        for (int l = 1; l < L; ++l) {
          if (cnt[l] == 0) continue;
          double* Sl = S + (size_t)l * KV;
          for (int j = 0; j < V; ++j) d[j] = 0;
          for (int i = 0; i < K; ++i)
            for (int j = 0; j < V; ++j) d[j] += Sl[(size_t)i * V + j] * kn[i];
          for (int i = 0; i < K; ++i)
            for (int j = 0; j < V; ++j) Sl[(size_t)i * V + j] = a * (Sl[(size_t)i * V + j] - b * kn[i] * d[j]);
        }
        for (int i = 0; i < K; ++i)
          for (int j = 0; j < V; ++j) S[(size_t)i * V + j] = b * kn[i] * (double)vt[j];
        cnt[0] = 1;
        float* ot = o + (t * HV + hv) * V;
        const float* lt = lam + (t * HV + hv) * L;
        for (int j = 0; j < V; ++j) d[j] = 0;
        for (int l = 0; l < L; ++l) {
          if (cnt[l] == 0) continue;
          const double* Sl = S + (size_t)l * KV;
          const double w = (double)lt[l];
          for (int i = 0; i < K; ++i) {
            const double qw = qn[i] * w;
            for (int j = 0; j < V; ++j) d[j] += qw * Sl[(size_t)i * V + j];
          }
        }
        for (int j = 0; j < V; ++j) ot[j] = (float)d[j];
      }
      if (states_out)
        for (int l = 0; l < L; ++l)
          for (size_t i = 0; i < KV; ++i) states_out[(((size_t)s * HV + hv) * KV + i) * L + l] = (float)S[(size_t)l * KV + i];
      if (counts_out)
        for (int l = 0; l < L; ++l) counts_out[l] = (int32_t)cnt[l];
    }
  free(S); free(cnt); free(qn); free(kn); free(d);
}

void oracle_hgdn_recurrent_f64(const float* q, const float* k, const float* v, const float* g, const float* beta,
                               const float* lam, const int64_t* cu_seqlens, int n_seq, int H, int HV, int K, int V,
                               int L, float scale, int l2norm, float* o) {
  oracle_hgdn_recurrent_state_f64(q, k, v, g, beta, lam, cu_seqlens, n_seq, H, HV, K, V, L, scale, l2norm, 0, 0, o, 0, 0);
}

/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the gated-delta-rule forward (token-serial form).
 * Nothing in the shipped package may link or call this file.
 *
 * Restates (reference = chengjiang123/Lampa):
 *   models/hattention/gated_delta_rule_ori.py:430-453  (fused recurrent kernel: order of the operations,
 *                                                       scale applied to q, optional in-kernel l2norm)
 *   models/hattention/recurrent.py:134-155             (S_t = a_t (I - b_t k_t k_t^T) S_{t-1} + b_t k_t v_t^T)
 *   models/hattention/l2norm.py:97-103                 (chunk path l2norm: x / sqrt(sum x^2 + 1e-6))
 * Per (sequence, head), state S [K,V] row-major (K-major rows), for each token t:
 *   S   <- exp(g_t) * S
 *   d   =  beta_t * (v_t - S^T k_t)
 *   S   <- S + k_t d^T
 *   o_t =  S^T (scale * q_t)
 * Grouped value heads (HV >= H, HV % H == 0): value head hv reads q/k head hv / (HV / H).
 * beta_headwise != 0: beta is [tokens, HV, V], one value per value column (IS_BETA_HEADWISE,
 * gated_delta_rule_ori.py:415-418,444-448); otherwise [tokens, HV].
 * Pins (tests/test_oracle_gdr.py): T=1 closed form, beta=0 pure decay, orthonormal-key recall and
 * overwrite, equality with the quadratic (materialised) form and with the chunk form for several chunk
 * sizes -- all evaluated by the independent numpy/torch restatements in oracle/gated_delta.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define DEFINE_GDR(NAME, REAL, EXP, SQRT)                                                                  \
  void NAME(const float* q, const float* k, const float* v, const float* g, const float* beta,             \
            const int64_t* cu_seqlens, int n_seq, int H, int HV, int K, int V, float scale, int l2norm,    \
            const float* h0, float* o, float* ht, int beta_headwise) {                                     \
    REAL* S = (REAL*)malloc(sizeof(REAL) * (size_t)K * V);                                                 \
    REAL* qn = (REAL*)malloc(sizeof(REAL) * (size_t)K);                                                    \
    REAL* kn = (REAL*)malloc(sizeof(REAL) * (size_t)K);                                                    \
    REAL* d = (REAL*)malloc(sizeof(REAL) * (size_t)V);                                                     \
    int rep = HV / H;                                                                                      \
    for (int s = 0; s < n_seq; ++s)                                                                        \
      for (int hv = 0; hv < HV; ++hv) {                                                                    \
        int h = hv / rep;                                                                                  \
        for (int i = 0; i < K * V; ++i)                                                                    \
          S[i] = h0 ? (REAL)h0[((int64_t)s * HV + hv) * K * V + i] : (REAL)0;                              \
        for (int64_t t = cu_seqlens[s]; t < cu_seqlens[s + 1]; ++t) {                                      \
          const float* qt = q + (t * H + h) * K;                                                           \
          const float* kt = k + (t * H + h) * K;                                                           \
          const float* vt = v + (t * HV + hv) * V;                                                         \
          REAL qs = 0, ks = 0;                                                                             \
          for (int i = 0; i < K; ++i) { qs += (REAL)qt[i] * qt[i]; ks += (REAL)kt[i] * kt[i]; }            \
          REAL qi = 1, ki = 1;                                                                             \
          if (l2norm == 1) { qi = 1 / SQRT(qs + (REAL)1e-6); ki = 1 / SQRT(ks + (REAL)1e-6); }             \
          if (l2norm == 2) { qi = 1 / (SQRT(qs) + (REAL)1e-6); ki = 1 / (SQRT(ks) + (REAL)1e-6); }         \
          for (int i = 0; i < K; ++i) { qn[i] = (REAL)qt[i] * qi * (REAL)scale; kn[i] = (REAL)kt[i] * ki; }\
          REAL decay = EXP((REAL)g[t * HV + hv]);                                                          \
          const float* bt = beta_headwise ? beta + (t * HV + hv) * V : beta + (t * HV + hv);               \
          for (int j = 0; j < V; ++j) d[j] = 0;                                                            \
          for (int i = 0; i < K; ++i)                                                                      \
            for (int j = 0; j < V; ++j) { S[i * V + j] *= decay; d[j] += S[i * V + j] * kn[i]; }           \
          for (int j = 0; j < V; ++j) d[j] = (REAL)bt[beta_headwise ? j : 0] * ((REAL)vt[j] - d[j]);       \
          float* ot = o + (t * HV + hv) * V;                                                               \
          for (int j = 0; j < V; ++j) {                                                                    \
            REAL acc = 0;                                                                                  \
            for (int i = 0; i < K; ++i) {                                                                  \
              S[i * V + j] += kn[i] * d[j];                                                                \
              acc += S[i * V + j] * qn[i];                                                                 \
            }                                                                                              \
            ot[j] = (float)acc;                                                                            \
          }                                                                                                \
        }                                                                                                  \
        if (ht)                                                                                            \
          for (int i = 0; i < K * V; ++i) ht[((int64_t)s * HV + hv) * K * V + i] = (float)S[i];            \
      }                                                                                                    \
    free(S); free(qn); free(kn); free(d);                                                                  \
  }

DEFINE_GDR(oracle_gdr_recurrent_f64, double, exp, sqrt)
DEFINE_GDR(oracle_gdr_recurrent_f32, float, expf, sqrtf)

/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the LSH stage (hash, bucket-id packing, stable sort,
 * gather/scatter of hit features).  Nothing in the shipped package may link or call this file; it exists
 * so that tests, the smoke check and the CPU-baseline leg of the benchmark have an independent statement
 * of the algorithm to compare the HIP kernels against.
 *
 * What it restates (reference = chengjiang123/Lampa):
 *   - projection            models/model_utils/hash_utils.py:368-371 (E2LSH.forward: bmm(vecs, alpha))
 *                           models/baselines/full_mamba2.py:136-141 (single-head variant)
 *   - range of the hashes   models/model_utils/hash_utils.py:334-340 (max - min over the hits)
 *   - mixed-radix key       models/attention/hept.py:79-88 (key = hash + index * shift, shift = hash range)
 *   - LSHOrdering key       models/baselines/full_mamba2.py:181-208 (sum_h 2^h * proj_h, norm pre-sort,
 *                           stable sort by key)
 *   - gather / inverse perm models/model_utils/hash_utils.py:46-57,83-93
 * The reference never quantises its projections (beta ~ U(0,r) is allocated but unused); the bucket id
 * floor((a.x + b) / w) is the textbook E2LSH of Datar et al. 2004 written on the reference's own
 * parameters (alpha, beta, r = w).
 *
 * Arithmetic contract shared with the HIP kernels (this is what makes bit-exact parity possible):
 *   p   = fmaf(x[D-1], a[D-1], ... fmaf(x[1], a[1], fmaf(x[0], a[0], 0.0f)))      (left to right)
 *   t   = (p + b) * inv_w            with inv_w = 1.0f / w computed once in fp32 on the host
 *   id  = floorf(t) saturated to int32, NaN -> INT32_MAX
 * Pins (tests/test_oracle_lsh.py): projection against torch.bmm / float64 dot, ids against
 * floor((p+b)/w) in float64 away from bucket edges, packing against Python integers, sort against
 * torch.sort(stable=True) and sorted(), gather against torch.gather.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LSH_MAX_PROJ 8

/* proj[c*N + n] = <coords[n,:], alpha[:,c]>; coords [N,D] row-major, alpha [D,C] row-major. */
void oracle_lsh_project(const float* coords, int64_t N, int D, const float* alpha, int C, float* proj) {
  for (int c = 0; c < C; ++c)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int d = 0; d < D; ++d) acc = fmaf(coords[n * D + d], alpha[d * C + c], acc);
      proj[(int64_t)c * N + n] = acc;
    }
}

static int32_t quantise(float p, float b, float inv_w) {
  float t = (p + b) * inv_w;
  if (t != t) return INT32_MAX;
  float f = floorf(t);
  if (f >= 2147483648.0f) return INT32_MAX;
  if (f <= -2147483648.0f) return INT32_MIN;
  return (int32_t)f;
}

/* ids[c*N + n] = floor((proj + beta[c]) * inv_w), C = n_tables * n_proj columns. */
void oracle_lsh_bucket_ids(const float* coords, int64_t N, int D, const float* alpha, const float* beta,
                           int C, float inv_w, int32_t* ids) {
  for (int c = 0; c < C; ++c)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int d = 0; d < D; ++d) acc = fmaf(coords[n * D + d], alpha[d * C + c], acc);
      ids[(int64_t)c * N + n] = quantise(acc, beta[c], inv_w);
    }
}

/*
 * Mixed-radix packing of the J ids of each table into one int32 key.
 * ids [T, J, N]; hits n >= n_valid are padding and receive key = total (one past the largest valid key)
 * so that they sort last.  meta [T, 2J+3] = lo[J], range[J], total, key_bits, overflow.
 *   lo_j = min_n id_j, range_j = max_n id_j - lo_j + 1, stride_0 = 1, stride_j = stride_{j-1} * range_{j-1}
 *   key  = sum_j (id_j - lo_j) * stride_j,  total = prod_j range_j
 * overflow = 1 when total exceeds INT32_MAX (keys are then reduced modulo 2^32 and not meaningful).
 */
void oracle_lsh_pack_keys(const int32_t* ids, int T, int J, int64_t N, int64_t n_valid, int32_t* keys,
                          int32_t* meta) {
  for (int t = 0; t < T; ++t) {
    int32_t lo[LSH_MAX_PROJ], hi[LSH_MAX_PROJ];
    int64_t range[LSH_MAX_PROJ], stride[LSH_MAX_PROJ];
    for (int j = 0; j < J; ++j) {
      lo[j] = INT32_MAX;
      hi[j] = INT32_MIN;
      const int32_t* col = ids + ((int64_t)t * J + j) * N;
      for (int64_t n = 0; n < n_valid; ++n) {
        if (col[n] < lo[j]) lo[j] = col[n];
        if (col[n] > hi[j]) hi[j] = col[n];
      }
      if (n_valid == 0) lo[j] = hi[j] = 0;
    }
    int overflow = 0;
    uint64_t total = 1; /* saturates at 2^31 once it no longer fits an int32 */
    for (int j = 0; j < J; ++j) {
      range[j] = (int64_t)hi[j] - (int64_t)lo[j] + 1;
      stride[j] = (int64_t)total;
      total *= (uint64_t)range[j]; /* <= 2^31 * 2^32, fits */
      if (total > (uint64_t)INT32_MAX) { overflow = 1; total = (uint64_t)INT32_MAX + 1; }
    }
    for (int64_t n = 0; n < N; ++n) {
      uint32_t key = 0;
      if (n < n_valid) {
        for (int j = 0; j < J; ++j) {
          uint32_t digit = (uint32_t)ids[((int64_t)t * J + j) * N + n] - (uint32_t)lo[j];
          key += digit * (uint32_t)stride[j];
        }
      } else {
        key = (uint32_t)total;
      }
      keys[(int64_t)t * N + n] = (int32_t)key;
    }
    int32_t* m = meta + (int64_t)t * (2 * J + 3);
    for (int j = 0; j < J; ++j) {
      m[j] = lo[j];
      m[J + j] = range[j] > INT32_MAX ? INT32_MAX : (int32_t)range[j];
    }
    uint64_t top = (n_valid < N) ? total : total - 1; /* largest key value present */
    int bits = 1;
    while (bits < 32 && (top >> bits) != 0) ++bits;
    if (overflow) bits = 32;
    m[2 * J] = total > (uint64_t)INT32_MAX ? INT32_MAX : (int32_t)total;
    m[2 * J + 1] = bits;
    m[2 * J + 2] = overflow;
  }
}

/* Order-preserving map of the three key kinds onto uint32 (ascending). */
enum { KEY_U32 = 0, KEY_I32 = 1, KEY_F32 = 2 };

static uint32_t ordered_bits(uint32_t raw, int kind) {
  if (kind == KEY_I32) return raw ^ 0x80000000u;
  if (kind == KEY_F32) {
    float f;
    memcpy(&f, &raw, 4);
    if (f != f) return 0xFFFFFFFFu;          /* NaN sorts last, as torch.sort does */
    if (f == 0.0f) raw = 0;                  /* -0.0 and +0.0 compare equal */
    return (raw & 0x80000000u) ? ~raw : (raw | 0x80000000u);
  }
  return raw;
}

/* Stable ascending argsort of S independent segments of length N (bottom-up merge sort on indices).
 * vals_in (optional, [S,N]) are the payload carried through the sort; NULL means 0..N-1. */
void oracle_stable_argsort(const uint32_t* keys, int S, int64_t N, int kind, const int32_t* vals_in,
                           int32_t* perm_out, uint32_t* keys_out) {
  uint32_t* ka = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)(N > 0 ? N : 1));
  int32_t* a = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
  int32_t* b = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
  for (int s = 0; s < S; ++s) {
    const uint32_t* k = keys + (int64_t)s * N;
    for (int64_t n = 0; n < N; ++n) { ka[n] = ordered_bits(k[n], kind); a[n] = (int32_t)n; }
    for (int64_t width = 1; width < N; width *= 2) {
      for (int64_t lo = 0; lo < N; lo += 2 * width) {
        int64_t mid = lo + width < N ? lo + width : N, hi = lo + 2 * width < N ? lo + 2 * width : N;
        int64_t i = lo, j = mid, o = lo;
        while (i < mid && j < hi) b[o++] = (ka[a[j]] < ka[a[i]]) ? a[j++] : a[i++];
        while (i < mid) b[o++] = a[i++];
        while (j < hi) b[o++] = a[j++];
      }
      int32_t* tmp = a; a = b; b = tmp;
    }
    for (int64_t n = 0; n < N; ++n) {
      int32_t src = a[n];
      perm_out[(int64_t)s * N + n] = vals_in ? vals_in[(int64_t)s * N + src] : src;
      if (keys_out) keys_out[(int64_t)s * N + n] = k[src];
    }
  }
  free(ka); free(a); free(b);
}

/* dst[s, n, :] = src[(s or 0), idx[s, n], :]; rows of row_bytes bytes. */
void oracle_gather_rows(const uint8_t* src, int src_segments, const int32_t* idx, int S, int64_t N,
                        int64_t row_bytes, uint8_t* dst) {
  for (int s = 0; s < S; ++s) {
    const uint8_t* base = src + (src_segments > 1 ? (int64_t)s * N * row_bytes : 0);
    for (int64_t n = 0; n < N; ++n)
      memcpy(dst + ((int64_t)s * N + n) * row_bytes, base + (int64_t)idx[(int64_t)s * N + n] * row_bytes,
             (size_t)row_bytes);
  }
}

/* dst[s, idx[s, n], :] = src[s, n, :] (the "unsort" by scatter). */
void oracle_scatter_rows(const uint8_t* src, const int32_t* idx, int S, int64_t N, int64_t row_bytes,
                         uint8_t* dst) {
  for (int s = 0; s < S; ++s)
    for (int64_t n = 0; n < N; ++n)
      memcpy(dst + ((int64_t)s * N + idx[(int64_t)s * N + n]) * row_bytes,
             src + ((int64_t)s * N + n) * row_bytes, (size_t)row_bytes);
}

/* inv[s, perm[s, n]] = n */
void oracle_invert_perm(const int32_t* perm, int S, int64_t N, int32_t* inv) {
  for (int s = 0; s < S; ++s)
    for (int64_t n = 0; n < N; ++n) inv[(int64_t)s * N + perm[(int64_t)s * N + n]] = (int32_t)n;
}

/* LSHOrdering keys: key[n] = ((p_0*1 + p_1*2) + p_2*4 ...) and norm[n] = sqrt(sum_d x_d^2), both by the
 * left-to-right fp32 chains stated in the header. proj [H, N]. */
void oracle_lsh_ordering_keys(const float* coords, int64_t N, int D, const float* alpha, int H, float* key,
                              float* norm) {
  for (int64_t n = 0; n < N; ++n) {
    float k = 0.0f, ss = 0.0f, w = 1.0f;
    for (int h = 0; h < H; ++h) {
      float acc = 0.0f;
      for (int d = 0; d < D; ++d) acc = fmaf(coords[n * D + d], alpha[d * H + h], acc);
      float term = acc * w; /* exact: w is a power of two */
      k = (h == 0) ? term : k + term;
      w *= 2.0f;
    }
    for (int d = 0; d < D; ++d) ss = fmaf(coords[n * D + d], coords[n * D + d], ss);
    key[n] = k;
    norm[n] = sqrtf(ss);
  }
}

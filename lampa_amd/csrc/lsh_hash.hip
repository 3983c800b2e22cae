// E2LSH hashing of detector hits on gfx950.
//
// Arithmetic contract (bit-exact against the CPU oracle): the projection is the left-to-right chain
// p = fmaf(x[d], a[d], p) starting from 0, the quantisation is floorf((p + b) * inv_w) saturated to int32 with
// NaN -> INT32_MAX.  Only explicit fmaf / single operations are used so that compiler contraction cannot
// change a result.
//
// Replaces (reference chengjiang123/Lampa): E2LSH.forward  models/model_utils/hash_utils.py:368-371,
// the hash range of lsh_mapping  hash_utils.py:334-340, the mixed-radix key idiom of get_geo_shift
// models/attention/hept.py:79-88, and the key/norm of LSHOrdering  models/baselines/full_mamba2.py:181-203.
#include "lsh_device.h"

// ---- pass 1: per-block min / max of every id column over the valid hits -------------------------------
// A block covers LSH_MM_ITEMS * 256 hits (all coordinate loads of a thread are independent). partial
// [gridDim.x, n_cols, 2] (min, max) per event; no atomics, no initialisation needed.
#define LSH_MM_ITEMS 8
#define LSH_PK_ITEMS 4
template <int DIM>
__global__ void __launch_bounds__(LSH_BLOCK) lsh_minmax_kernel(const float* __restrict__ coords, int64_t n_hits,
                                                              int64_t n_valid,
                                                              const int32_t* __restrict__ n_valid_dev, int dim,
                                                              const float* __restrict__ alpha,
                                                              const float* __restrict__ beta, int n_cols,
                                                              float inv_w, int32_t* __restrict__ partial) {
  __shared__ int32_t s_min[LSH_BLOCK / 64][LSH_MAX_COLS];
  __shared__ int32_t s_max[LSH_BLOCK / 64][LSH_MAX_COLS];
  // the projections are read from LDS (one broadcast read per use) instead of scalar loads inside the column loop
  __shared__ float s_alpha[LSH_MAX_DIM * LSH_MAX_COLS], s_beta[LSH_MAX_COLS];
  for (int i = threadIdx.x; i < dim * n_cols; i += LSH_BLOCK) s_alpha[i] = alpha[i];
  for (int i = threadIdx.x; i < n_cols; i += LSH_BLOCK) s_beta[i] = beta[i];
  // blockIdx.z = event of a batch: its own coords, valid count and partials
  coords += (int64_t)blockIdx.z * n_hits * dim;
  partial += (int64_t)blockIdx.z * gridDim.x * n_cols * 2;
  if (n_valid_dev) n_valid = max((int64_t)0, min(n_hits, (int64_t)n_valid_dev[blockIdx.z]));  // a count outside the event is cut
  float x[LSH_MM_ITEMS][LSH_MAX_DIM];
  bool valid[LSH_MM_ITEMS];
#pragma unroll
  for (int i = 0; i < LSH_MM_ITEMS; ++i) {
    const int64_t n = ((int64_t)blockIdx.x * LSH_MM_ITEMS + i) * LSH_BLOCK + threadIdx.x;
    valid[i] = n < n_valid;
    lsh_load_coords<DIM>(coords, valid[i] ? n : 0, dim, x[i]);
  }
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  // The kernel is bound by its arithmetic (hits x columns), so the extremes are taken on the scaled projections and
  // only they are quantised: the quantisation is monotone, NaNs (id INT32_MAX) are ignored by fminf / fmaxf and noted
  // separately. Invalid items hold the coordinates of hit 0, a valid hit, so they need no masking (with no valid hit
  // at all the packing kernel ignores the partials).
  for (int c = 0; c < n_cols; ++c) {
    const float b = s_beta[c];
    float tlo = INFINITY, thi = -INFINITY;
    bool nan_seen = false;
#pragma unroll
    for (int i = 0; i < LSH_MM_ITEMS; ++i) {
      const float t = lsh_scaled(lsh_dot<DIM>(x[i], s_alpha, dim, n_cols, c), b, inv_w);
      tlo = fminf(tlo, t);
      thi = fmaxf(thi, t);
      nan_seen = nan_seen || t != t;
    }
    int32_t lo = lsh_quantise_scaled(tlo), hi = nan_seen ? INT32_MAX : lsh_quantise_scaled(thi);
    lo = lsh_wave_extreme<false>(lo);
    hi = lsh_wave_extreme<true>(hi);
    if (lane_id() == 63) { s_min[wave][c] = lo; s_max[wave][c] = hi; }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < n_cols; c += LSH_BLOCK) {
    int32_t lo = s_min[0][c], hi = s_max[0][c];
    for (int w = 1; w < LSH_BLOCK / 64; ++w) { lo = min(lo, s_min[w][c]); hi = max(hi, s_max[w][c]); }
    partial[((int64_t)blockIdx.x * n_cols + c) * 2 + 0] = lo;
    partial[((int64_t)blockIdx.x * n_cols + c) * 2 + 1] = hi;
  }
}

// ---- pass 2: reduce the partials, derive the mixed-radix strides, pack the keys of every table ---------
// grid (ceil(N / (256 * LSH_PK_ITEMS)), 1, events): a hit's coordinates are read once for all tables.
// meta [n_tables, 2J+3] = lo[J], range[J], total, key_bits, overflow.
template <int DIM>
__global__ void __launch_bounds__(LSH_BLOCK) lsh_pack_kernel(const float* __restrict__ coords, int64_t n_hits,
                                                            int64_t n_valid,
                                                            const int32_t* __restrict__ n_valid_dev, int dim,
                                                            const float* __restrict__ alpha,
                                                            const float* __restrict__ beta, int n_tables,
                                                            int n_proj, float inv_w,
                                                            const int32_t* __restrict__ partial, int n_partial,
                                                            int32_t* __restrict__ ids, int32_t* __restrict__ keys,
                                                            int32_t* __restrict__ meta) {
  const int n_cols = n_tables * n_proj;
  // blockIdx.z = event of a batch
  coords += (int64_t)blockIdx.z * n_hits * dim;
  partial += (int64_t)blockIdx.z * n_partial * n_cols * 2;
  if (ids) ids += (int64_t)blockIdx.z * n_cols * n_hits;
  keys += (int64_t)blockIdx.z * n_tables * n_hits;
  meta += (int64_t)blockIdx.z * n_tables * (2 * n_proj + 3);
  if (n_valid_dev) n_valid = max((int64_t)0, min(n_hits, (int64_t)n_valid_dev[blockIdx.z]));  // a count outside the event is cut
  __shared__ int32_t s_lo[LSH_MAX_COLS], s_hi[LSH_MAX_COLS];
  __shared__ uint32_t s_stride[LSH_MAX_COLS];
  __shared__ uint32_t s_total[LSH_MAX_COLS];  // per table
  __shared__ float s_alpha[LSH_MAX_DIM * LSH_MAX_COLS], s_beta[LSH_MAX_COLS];  // (as in the min / max kernel)
  for (int i = threadIdx.x; i < dim * n_cols; i += LSH_BLOCK) s_alpha[i] = alpha[i];
  for (int i = threadIdx.x; i < n_cols; i += LSH_BLOCK) s_beta[i] = beta[i];
  // column c is reduced by the four threads 4c .. 4c+3 (n_cols <= 64)
  {
    const int c = threadIdx.x >> 2, part = threadIdx.x & 3;
    int32_t lo = INT32_MAX, hi = INT32_MIN;
    if (c < n_cols)
      for (int b = part; b < n_partial; b += 4) {
        lo = min(lo, partial[((int64_t)b * n_cols + c) * 2 + 0]);
        hi = max(hi, partial[((int64_t)b * n_cols + c) * 2 + 1]);
      }
    lo = min(lo, __shfl_xor(lo, 1)); hi = max(hi, __shfl_xor(hi, 1));
    lo = min(lo, __shfl_xor(lo, 2)); hi = max(hi, __shfl_xor(hi, 2));
    if (c < n_cols && part == 0) { s_lo[c] = n_valid == 0 ? 0 : lo; s_hi[c] = n_valid == 0 ? 0 : hi; }
  }
  __syncthreads();
  if ((int)threadIdx.x < n_tables) {
    const int table = threadIdx.x;
    uint64_t total = 1;
    int overflow = 0;
    int32_t* m = meta + (int64_t)table * (2 * n_proj + 3);
    for (int j = 0; j < n_proj; ++j) {
      const int c = table * n_proj + j;
      const int64_t range = (int64_t)s_hi[c] - (int64_t)s_lo[c] + 1;
      s_stride[c] = (uint32_t)total;
      total *= (uint64_t)range;
      if (total > (uint64_t)INT32_MAX) { overflow = 1; total = (uint64_t)INT32_MAX + 1; }
      if (blockIdx.x == 0) {
        m[j] = s_lo[c];
        m[n_proj + j] = range > INT32_MAX ? INT32_MAX : (int32_t)range;
      }
    }
    s_total[table] = (uint32_t)total;
    if (blockIdx.x == 0) {
      uint64_t top = (n_valid < n_hits) ? total : total - 1;
      int bits = 1;
      while (bits < 32 && (top >> bits) != 0) ++bits;
      if (overflow) bits = 32;
      m[2 * n_proj] = total > (uint64_t)INT32_MAX ? INT32_MAX : (int32_t)total;
      m[2 * n_proj + 1] = bits;
      m[2 * n_proj + 2] = overflow;
    }
  }
  __syncthreads();
  // LSH_PK_ITEMS hits per thread: the reduction above is paid once per block, and the coordinate loads of a thread
  // are independent
  float x[LSH_PK_ITEMS][LSH_MAX_DIM];
#pragma unroll
  for (int i = 0; i < LSH_PK_ITEMS; ++i) {
    const int64_t n = ((int64_t)blockIdx.x * LSH_PK_ITEMS + i) * LSH_BLOCK + threadIdx.x;
    lsh_load_coords<DIM>(coords, n < n_valid ? n : 0, dim, x[i]);
  }
  for (int table = 0; table < n_tables; ++table) {
    uint32_t key[LSH_PK_ITEMS];
#pragma unroll
    for (int i = 0; i < LSH_PK_ITEMS; ++i) key[i] = s_total[table];
    for (int j = 0; j < n_proj; ++j) {
      const int c = table * n_proj + j;
      const float b = s_beta[c];
      const uint32_t lo = (uint32_t)s_lo[c], stride = s_stride[c];
#pragma unroll
      for (int i = 0; i < LSH_PK_ITEMS; ++i) {
        const int64_t n = ((int64_t)blockIdx.x * LSH_PK_ITEMS + i) * LSH_BLOCK + threadIdx.x;
        const bool valid = n < n_valid;
        const int32_t id = valid ? lsh_quantise(lsh_dot<DIM>(x[i], s_alpha, dim, n_cols, c), b, inv_w) : 0;
        if (j == 0 && valid) key[i] = 0u;
        if (valid) key[i] += ((uint32_t)id - lo) * stride;
        if (ids && n < n_hits) ids[(int64_t)c * n_hits + n] = id;
      }
    }
#pragma unroll
    for (int i = 0; i < LSH_PK_ITEMS; ++i) {
      const int64_t n = ((int64_t)blockIdx.x * LSH_PK_ITEMS + i) * LSH_BLOCK + threadIdx.x;
      if (n < n_hits) keys[(int64_t)table * n_hits + n] = (int32_t)key[i];
    }
  }
}

// ---- plain projection (the reference's E2LSH.forward, a batched [N,dim] x [dim,n_hashes] product) -----
// vecs [n_heads, N, dim], alpha [n_heads, dim, n_cols]; out element (c, head, n) at
// c * stride_c + head * stride_h + n * stride_n.
__global__ void __launch_bounds__(LSH_BLOCK) lsh_project_kernel(const float* __restrict__ vecs, int64_t n_hits,
                                                               int dim, const float* __restrict__ alpha,
                                                               int n_cols, float* __restrict__ out,
                                                               int64_t stride_c, int64_t stride_h,
                                                               int64_t stride_n) {
  const int head = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * LSH_BLOCK + threadIdx.x;
  if (n >= n_hits) return;
  const float* x = vecs + ((int64_t)head * n_hits + n) * dim;
  const float* a = alpha + (int64_t)head * dim * n_cols;
  for (int c = 0; c < n_cols; ++c) {
    float acc = 0.0f;
    for (int d = 0; d < dim; ++d) acc = __builtin_fmaf(x[d], a[d * n_cols + c], acc);
    out[c * stride_c + head * stride_h + n * stride_n] = acc;
  }
}

// ---- LSHOrdering sort keys: key = ((p_0 + 2 p_1) + 4 p_2) + ..., norm = sqrt(sum x^2) ------------------
__global__ void __launch_bounds__(LSH_BLOCK) lsh_ordering_keys_kernel(const float* __restrict__ coords,
                                                                     int64_t n_hits, int dim,
                                                                     const float* __restrict__ alpha,
                                                                     int n_hashes, float* __restrict__ key,
                                                                     float* __restrict__ norm) {
  const int64_t n = (int64_t)blockIdx.x * LSH_BLOCK + threadIdx.x;
  if (n >= n_hits) return;
  const float* x = coords + n * dim;
  float k = 0.0f, w = 1.0f;
  for (int h = 0; h < n_hashes; ++h) {
    float acc = 0.0f;
    for (int d = 0; d < dim; ++d) acc = __builtin_fmaf(x[d], alpha[d * n_hashes + h], acc);
    float term = acc * w;
    k = (h == 0) ? term : k + term;
    w *= 2.0f;
  }
  float ss = 0.0f;
  for (int d = 0; d < dim; ++d) ss = __builtin_fmaf(x[d], x[d], ss);
  key[n] = k;
  norm[n] = __fsqrt_rn(ss);
}

// ---- host entry points ----------------------------------------------------------------------------------
extern "C" int64_t lampa_lsh_bucket_workspace_bytes(int64_t n_hits, int n_tables, int n_proj) {
  if (n_hits < 0 || n_tables <= 0 || n_proj <= 0) return LAMPA_ERR_INVALID;
  int64_t blocks = (n_hits + LSH_BLOCK - 1) / LSH_BLOCK;
  if (blocks < 1) blocks = 1;
  return lampa_align_up(blocks * n_tables * n_proj * 2 * (int64_t)sizeof(int32_t), 256);
}

// ids, keys and meta of n_events events of n_hits hits each (event e at offset e * n_hits rows); the valid count of
// an event is n_valid_dev[e] (device) when given, else n_valid for all of them.
static int lsh_bucket_keys_batch(const float* coords, int n_events, int64_t n_hits, int64_t n_valid,
                                 const int32_t* n_valid_dev, int dim, const float* alpha, const float* beta,
                                 int n_tables, int n_proj, float w, int32_t* ids_out, int32_t* keys_out,
                                 int32_t* meta_out, void* workspace, int64_t workspace_bytes, hipStream_t s) {
  if (!coords || !alpha || !beta || !keys_out || !meta_out) return LAMPA_ERR_INVALID;
  if (n_events < 1 || n_events > 65535 || n_hits < 0 || n_valid < 0 || n_valid > n_hits || n_hits > INT32_MAX)
    return LAMPA_ERR_INVALID;
  if (dim < 1 || dim > LSH_MAX_DIM || n_tables < 1 || n_proj < 1 || n_proj > LSH_MAX_PROJ ||
      n_tables * n_proj > LSH_MAX_COLS || !(w > 0.0f))
    return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < n_events * lampa_lsh_bucket_workspace_bytes(n_hits, n_tables, n_proj))
    return LAMPA_ERR_WORKSPACE;
  if (n_hits == 0) return LAMPA_OK;
  const float inv_w = 1.0f / w;
  const int n_cols = n_tables * n_proj;
  int32_t* partial = (int32_t*)workspace;
  // with per-event counts on the device every block of the event takes part (blocks past the count contribute
  // the neutral elements)
  const int64_t per_block = (int64_t)LSH_BLOCK * LSH_MM_ITEMS;
  int blocks_valid = (int)(((n_valid_dev ? n_hits : n_valid) + per_block - 1) / per_block);
  if (blocks_valid < 1) blocks_valid = 1;
  const int blocks_all = (int)((n_hits + LSH_BLOCK * LSH_PK_ITEMS - 1) / (LSH_BLOCK * LSH_PK_ITEMS));
  LAMPA_PROF(s, "start");
  if (dim == 4) {
    hipLaunchKernelGGL(lsh_minmax_kernel<4>, dim3(blocks_valid, 1, n_events), dim3(LSH_BLOCK), 0, s, coords, n_hits,
                       n_valid, n_valid_dev, dim, alpha, beta, n_cols, inv_w, partial);
    LAMPA_PROF(s, "lsh_minmax_kernel");
    hipLaunchKernelGGL(lsh_pack_kernel<4>, dim3(blocks_all, 1, n_events), dim3(LSH_BLOCK), 0, s, coords, n_hits,
                       n_valid, n_valid_dev, dim, alpha, beta, n_tables, n_proj, inv_w, partial, blocks_valid, ids_out,
                       keys_out, meta_out);
  } else {
    hipLaunchKernelGGL(lsh_minmax_kernel<0>, dim3(blocks_valid, 1, n_events), dim3(LSH_BLOCK), 0, s, coords, n_hits,
                       n_valid, n_valid_dev, dim, alpha, beta, n_cols, inv_w, partial);
    LAMPA_PROF(s, "lsh_minmax_kernel");
    hipLaunchKernelGGL(lsh_pack_kernel<0>, dim3(blocks_all, 1, n_events), dim3(LSH_BLOCK), 0, s, coords, n_hits,
                       n_valid, n_valid_dev, dim, alpha, beta, n_tables, n_proj, inv_w, partial, blocks_valid, ids_out,
                       keys_out, meta_out);
  }
  LAMPA_PROF(s, "lsh_pack_kernel");
  return lampa_launch_status();
}

extern "C" int lampa_lsh_bucket_keys(const float* coords, int64_t n_hits, int64_t n_valid, int dim,
                                     const float* alpha, const float* beta, int n_tables, int n_proj, float w,
                                     int32_t* ids_out, int32_t* keys_out, int32_t* meta_out, void* workspace,
                                     int64_t workspace_bytes, void* stream) {
  return lsh_bucket_keys_batch(coords, 1, n_hits, n_valid, nullptr, dim, alpha, beta, n_tables, n_proj, w, ids_out,
                               keys_out, meta_out, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int lampa_lsh_project_f32(const float* vecs, int n_heads, int64_t n_hits, int dim, const float* alpha,
                                     int n_cols, float* out, int64_t stride_c, int64_t stride_h, int64_t stride_n,
                                     void* stream) {
  if (!vecs || !alpha || !out || n_heads < 1 || n_hits < 0 || dim < 1 || n_cols < 1) return LAMPA_ERR_INVALID;
  if (n_hits == 0) return LAMPA_OK;
  const int blocks = (int)((n_hits + LSH_BLOCK - 1) / LSH_BLOCK);
  hipLaunchKernelGGL(lsh_project_kernel, dim3(blocks, n_heads), dim3(LSH_BLOCK), 0, (hipStream_t)stream, vecs,
                     n_hits, dim, alpha, n_cols, out, stride_c, stride_h, stride_n);
  return lampa_launch_status();
}

extern "C" int lampa_lsh_ordering_keys(const float* coords, int64_t n_hits, int dim, const float* alpha,
                                       int n_hashes, float* key_out, float* norm_out, void* stream) {
  if (!coords || !alpha || !key_out || !norm_out || n_hits < 0 || dim < 1 || n_hashes < 1) return LAMPA_ERR_INVALID;
  if (n_hits == 0) return LAMPA_OK;
  const int blocks = (int)((n_hits + LSH_BLOCK - 1) / LSH_BLOCK);
  hipLaunchKernelGGL(lsh_ordering_keys_kernel, dim3(blocks), dim3(LSH_BLOCK), 0, (hipStream_t)stream, coords,
                     n_hits, dim, alpha, n_hashes, key_out, norm_out);
  return lampa_launch_status();
}

// ---- per-row min / max of hashed values (the range used as a radix stride, hash_utils.py:334-340) -----------
// x [rows, n]; out [rows, 2] = (min, max). NaNs are ignored unless the whole row is NaN.
__global__ void __launch_bounds__(LSH_BLOCK) lsh_row_minmax_kernel(const float* __restrict__ x, int64_t n,
                                                                  float* __restrict__ out) {
  __shared__ float s_lo[LSH_BLOCK / 64], s_hi[LSH_BLOCK / 64];
  const float* row = x + (int64_t)blockIdx.x * n;
  float lo = INFINITY, hi = -INFINITY;
  for (int64_t i = threadIdx.x; i < n; i += LSH_BLOCK) {
    const float v = row[i];
    lo = fminf(lo, v);
    hi = fmaxf(hi, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, off));
    hi = fmaxf(hi, __shfl_xor(hi, off));
  }
  if (lane_id() == 0) { s_lo[threadIdx.x >> 6] = lo; s_hi[threadIdx.x >> 6] = hi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < LSH_BLOCK / 64; ++w) { lo = fminf(lo, s_lo[w]); hi = fmaxf(hi, s_hi[w]); }
    out[blockIdx.x * 2 + 0] = lo;
    out[blockIdx.x * 2 + 1] = hi;
  }
}

extern "C" int lampa_row_minmax_f32(const float* x, int rows, int64_t n, float* out, void* stream) {
  if (!x || !out || rows < 1 || n < 1) return LAMPA_ERR_INVALID;
  hipLaunchKernelGGL(lsh_row_minmax_kernel, dim3(rows), dim3(LSH_BLOCK), 0, (hipStream_t)stream, x, n, out);
  return lampa_launch_status();
}

// ---- whole bucketing stage of one event in one call ---------------------------------------------------------------
extern "C" int64_t lampa_sort_workspace_bytes(int n_segments, int64_t n);
extern "C" int lampa_sort_pairs(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments, int64_t n,
                                int key_bits, const int32_t* key_bits_dev, int key_bits_stride, int n_passes,
                                int32_t* vals_out, void* workspace, int64_t workspace_bytes, void* stream);
int lampa_gather_rows_grouped(const void* src, int src_segments, int group, int64_t n_src, const void* idx,
                              int idx_bytes, int n_segments, int64_t n, int64_t row_bytes, void* dst, void* stream);

// the one-launch form of the stage (lsh_stage.hip)
int64_t lsh_fused_workspace_bytes(int n_events, int64_t n_hits, int n_tables);
int lsh_fused_launch(const float* coords, int n_events, int64_t n_hits, int64_t n_valid, const int32_t* n_valid_dev,
                     int dim, const float* alpha, const float* beta, int n_tables, int n_proj, float w,
                     int32_t* ids_out, int32_t* keys_out, int32_t* meta_out, int32_t* perm_out, const void* feats,
                     int64_t feat_row_bytes, void* feats_out, void* workspace, int64_t workspace_bytes,
                     hipStream_t s);

// Enough for either form of the stage: the one-launch kernel, or the separate kernels (key packing + sort).
extern "C" int64_t lampa_lsh_bucket_sort_batch_workspace_bytes(int n_events, int64_t n_hits, int n_tables, int n_proj) {
  if (n_events < 1 || n_tables < 1) return LAMPA_ERR_INVALID;
  const int64_t a = lampa_lsh_bucket_workspace_bytes(n_hits, n_tables, n_proj);
  const int64_t b = lampa_sort_workspace_bytes(n_events * n_tables, n_hits);
  if (a < 0 || b < 0) return LAMPA_ERR_INVALID;
  const int64_t separate = n_events * a + b, fused = lsh_fused_workspace_bytes(n_events, n_hits, n_tables);
  return separate > fused ? separate : fused;
}

// Argument checks of the stage (those of the key kernels and of the sort), so that both forms refuse the same calls.
static int lsh_stage_check(const float* coords, int n_events, int64_t n_hits, int64_t n_valid, int dim,
                           const float* alpha, const float* beta, int n_tables, int n_proj, float w,
                           const int32_t* keys_out, const int32_t* meta_out, const int32_t* perm_out, const void* feats,
                           int64_t feat_row_bytes, const void* feats_out, int n_passes) {
  if (!perm_out || (feats && (!feats_out || feat_row_bytes < 1)) || n_events < 1) return LAMPA_ERR_INVALID;
  if (!coords || !alpha || !beta || !keys_out || !meta_out) return LAMPA_ERR_INVALID;
  if (n_events > 65535 || n_hits < 0 || n_valid < 0 || n_valid > n_hits || n_hits > INT32_MAX)
    return LAMPA_ERR_INVALID;
  if (dim < 1 || dim > LSH_MAX_DIM || n_tables < 1 || n_proj < 1 || n_proj > LSH_MAX_PROJ ||
      n_tables * n_proj > LSH_MAX_COLS || !(w > 0.0f))
    return LAMPA_ERR_INVALID;
  if (n_passes != 0 && n_passes != 3 && n_passes != 4) return LAMPA_ERR_INVALID;  // 32-bit keys, 11-bit digits
  return LAMPA_OK;
}

extern "C" int64_t lampa_lsh_bucket_sort_workspace_bytes(int64_t n_hits, int n_tables, int n_proj) {
  return lampa_lsh_bucket_sort_batch_workspace_bytes(1, n_hits, n_tables, n_proj);
}

// A batch of events in one set of launches: coords [n_events, n_hits, dim]; n_valid_dev: device int32 [n_events]
// (NULL = every hit valid); outputs as for one event with a leading event dimension: ids [E, T*J, N], keys / perm
// [E, T, N], meta [E, T, 2J+3], feats [E, N, row] -> feats_out [E, T, N, row]. Events are independent
// (each has its own id ranges and key width); the sort runs over E*T segments.
extern "C" int lampa_lsh_bucket_sort_batch(const float* coords, int n_events, int64_t n_hits,
                                           const int32_t* n_valid_dev, int dim, const float* alpha, const float* beta,
                                           int n_tables, int n_proj, float w, int32_t* ids_out, int32_t* keys_out,
                                           int32_t* meta_out, int32_t* perm_out, const void* feats,
                                           int64_t feat_row_bytes, void* feats_out, int n_passes, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  int rc = lsh_stage_check(coords, n_events, n_hits, n_hits, dim, alpha, beta, n_tables, n_proj, w, keys_out, meta_out,
                           perm_out, feats, feat_row_bytes, feats_out, n_passes);
  if (rc != LAMPA_OK) return rc;
  const int64_t a = lampa_lsh_bucket_workspace_bytes(n_hits, n_tables, n_proj);
  if (a < 0) return LAMPA_ERR_INVALID;
  const int64_t b = lampa_sort_workspace_bytes(n_events * n_tables, n_hits);
  if (b < 0) return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < lampa_lsh_bucket_sort_batch_workspace_bytes(n_events, n_hits, n_tables, n_proj))
    return LAMPA_ERR_WORKSPACE;
  if (n_hits == 0) return LAMPA_OK;
  rc = lsh_fused_launch(coords, n_events, n_hits, n_hits, n_valid_dev, dim, alpha, beta, n_tables, n_proj, w, ids_out,
                        keys_out, meta_out, perm_out, feats, feat_row_bytes, feats_out, workspace, workspace_bytes,
                        (hipStream_t)stream);
  if (rc != 1) return rc;  // launched (or failed); 1 = this call needs the separate kernels
  rc = lsh_bucket_keys_batch(coords, n_events, n_hits, n_hits, n_valid_dev, dim, alpha, beta, n_tables, n_proj, w,
                                 ids_out, keys_out, meta_out, workspace, n_events * a, (hipStream_t)stream);
  if (rc != LAMPA_OK) return rc;
  const int stride = 2 * n_proj + 3;
  rc = lampa_sort_pairs(keys_out, /*KEY_U32*/ 0, nullptr, n_events * n_tables, n_hits, 32, meta_out + 2 * n_proj + 1,
                        stride, n_passes, perm_out, (char*)workspace + n_events * a, b, stream);
  if (rc != LAMPA_OK) return rc;
  if (feats)
    rc = lampa_gather_rows_grouped(feats, n_events, n_tables, n_hits, perm_out, 4, n_events * n_tables, n_hits,
                                   feat_row_bytes, feats_out, stream);
  return rc;
}

// ids + keys + meta (lampa_lsh_bucket_keys), stable sort permutation of every table (lampa_sort_pairs on the packed
// keys, digit width taken from meta on the device) and, when feats is given, the hit features in sorted order
// (lampa_gather_rows): perm_out [n_tables, n_hits] int32, feats_out [n_tables, n_hits, feat_row_bytes].
extern "C" int lampa_lsh_bucket_sort(const float* coords, int64_t n_hits, int64_t n_valid, int dim, const float* alpha,
                                     const float* beta, int n_tables, int n_proj, float w, int32_t* ids_out,
                                     int32_t* keys_out, int32_t* meta_out, int32_t* perm_out, const void* feats,
                                     int64_t feat_row_bytes, void* feats_out, int n_passes, void* workspace,
                                     int64_t workspace_bytes, void* stream) {
  int rc = lsh_stage_check(coords, 1, n_hits, n_valid, dim, alpha, beta, n_tables, n_proj, w, keys_out, meta_out, perm_out,
                           feats, feat_row_bytes, feats_out, n_passes);
  if (rc != LAMPA_OK) return rc;
  const int64_t a = lampa_lsh_bucket_workspace_bytes(n_hits, n_tables, n_proj);
  const int64_t b = lampa_sort_workspace_bytes(n_tables, n_hits);
  if (a < 0 || b < 0) return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < lampa_lsh_bucket_sort_workspace_bytes(n_hits, n_tables, n_proj))
    return LAMPA_ERR_WORKSPACE;
  if (n_hits == 0) return LAMPA_OK;
  rc = lsh_fused_launch(coords, 1, n_hits, n_valid, nullptr, dim, alpha, beta, n_tables, n_proj, w, ids_out, keys_out,
                        meta_out, perm_out, feats, feat_row_bytes, feats_out, workspace, workspace_bytes,
                        (hipStream_t)stream);
  if (rc != 1) return rc;  // launched (or failed); 1 = this call needs the separate kernels
  rc = lampa_lsh_bucket_keys(coords, n_hits, n_valid, dim, alpha, beta, n_tables, n_proj, w, ids_out, keys_out,
                                 meta_out, workspace, a, stream);
  if (rc != LAMPA_OK) return rc;
  const int stride = 2 * n_proj + 3;
  rc = lampa_sort_pairs(keys_out, /*KEY_U32*/ 0, nullptr, n_tables, n_hits, 32, meta_out + 2 * n_proj + 1, stride,
                        n_passes, perm_out, (char*)workspace + a, b, stream);
  if (rc != LAMPA_OK) return rc;
  if (feats)
    rc = lampa_gather_rows_grouped(feats, 1, 1, n_hits, perm_out, 4, n_tables, n_hits, feat_row_bytes, feats_out, stream);
  return rc;
}

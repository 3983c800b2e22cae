// Region (AND-hash) front end of the HEPT bucketing on gfx950: quantile regions of the eta / phi order, the
// region shift of every (hash, head) row, and the fused sort key. Pure HBM-bound element-wise work.
//
// Replaces (reference chengjiang123/Lampa): quantile_partition  models/model_utils/hash_utils.py:14-26,
// get_geo_shift  models/attention/hept.py:78-88, and the key arithmetic between lsh_mapping and argsort in
// HEPTAttention.forward  hept.py:127-139.
//
// Arithmetic contract (float32, one rounding per operation, no contraction):
//   region_size = ceilf((float)n / regions)                       hash_utils.py:16
//   region      = floorf((float)rank / region_size) + 1           hash_utils.py:24-25 (rank = inverse of the sort)
//   shift       = (region_phi * hash_shift) * (ceilf(regions_eta) + 1) + region_eta * hash_shift     hept.py:82-86
//   key         = hashed + shift, hashed = +inf for hits at or beyond n_raw                          hept.py:130-136
// rank < 2^24 keeps (float)rank exact and the float floor division equal to the integer one.
#include "common.h"

#define HR_BLOCK 256
#define HR_ITEMS 4

template <typename IdxT>
__device__ __forceinline__ float hr_rank(const void* rank, int64_t i) {
  return (float)reinterpret_cast<const IdxT*>(rank)[i];
}

__device__ __forceinline__ float hr_region(float rank, float region_size) {
  return floorf(__fdiv_rn(rank, region_size)) + 1.0f;
}

// Two products and a sum, each rounded on its own: contraction into a fused multiply-add is switched off here.
__device__ __forceinline__ float hr_shift(float reg_eta, float reg_phi, float hash_shift, float phi_mult) {
#pragma clang fp contract(off)
  const float a = (reg_phi * hash_shift) * phi_mult;
  const float b = reg_eta * hash_shift;
  return a + b;
}

template <typename IdxT>
__global__ void __launch_bounds__(HR_BLOCK) hr_quantile_kernel(const void* __restrict__ rank, int64_t n,
                                                              const float* __restrict__ regions,
                                                              float* __restrict__ out) {
  const int row = blockIdx.y;
  const float region_size = ceilf(__fdiv_rn((float)n, regions[row]));
  const int64_t base = ((int64_t)blockIdx.x * HR_BLOCK + threadIdx.x) * HR_ITEMS;
#pragma unroll
  for (int j = 0; j < HR_ITEMS; ++j) {
    const int64_t i = base + j;
    if (i < n) out[(int64_t)row * n + i] = hr_region(hr_rank<IdxT>(rank, i), region_size);
  }
}

__global__ void __launch_bounds__(HR_BLOCK) hr_geo_shift_kernel(const float* __restrict__ region_eta,
                                                               const float* __restrict__ region_phi,
                                                               const float* __restrict__ hash_shift,
                                                               const float* __restrict__ regions_eta, int64_t n,
                                                               float* __restrict__ out) {
  const int row = blockIdx.y;
  const float shift = hash_shift[row];
  const float mult = ceilf(regions_eta[row]) + 1.0f;
  const int64_t base = ((int64_t)blockIdx.x * HR_BLOCK + threadIdx.x) * HR_ITEMS;
#pragma unroll
  for (int j = 0; j < HR_ITEMS; ++j) {
    const int64_t i = base + j, at = (int64_t)row * n + i;
    if (i < n) out[at] = hr_shift(region_eta[at], region_phi[at], shift, mult);
  }
}

// One thread makes the keys of HR_ITEMS consecutive hits of one (hash, head) row; the two rank arrays are shared
// by all rows and stay in L2.
__global__ void __launch_bounds__(HR_BLOCK) hr_sort_keys_kernel(const float* __restrict__ hashed,
                                                               const int32_t* __restrict__ rank_eta,
                                                               const int32_t* __restrict__ rank_phi,
                                                               const float* __restrict__ regions,
                                                               const float* __restrict__ hash_shift, int n_rows,
                                                               int64_t n, int64_t n_raw, float* __restrict__ keys) {
  const int row = blockIdx.y;
  const float r_eta = regions[row], r_phi = regions[n_rows + row];
  const float size_eta = ceilf(__fdiv_rn((float)n, r_eta)), size_phi = ceilf(__fdiv_rn((float)n, r_phi));
  const float shift = hash_shift[row];
  const float mult = ceilf(r_eta) + 1.0f;
  const int64_t base = ((int64_t)blockIdx.x * HR_BLOCK + threadIdx.x) * HR_ITEMS;
  if (base >= n) return;
  const int64_t at = (int64_t)row * n + base;
  float h[HR_ITEMS];
  int32_t re[HR_ITEMS], rp[HR_ITEMS];
  const bool full = base + HR_ITEMS <= n && (at % HR_ITEMS) == 0;
  if (full) {
    const float4 hv = *reinterpret_cast<const float4*>(hashed + at);
    const int4 ev = *reinterpret_cast<const int4*>(rank_eta + base);
    const int4 pv = *reinterpret_cast<const int4*>(rank_phi + base);
    h[0] = hv.x; h[1] = hv.y; h[2] = hv.z; h[3] = hv.w;
    re[0] = ev.x; re[1] = ev.y; re[2] = ev.z; re[3] = ev.w;
    rp[0] = pv.x; rp[1] = pv.y; rp[2] = pv.z; rp[3] = pv.w;
  } else {
#pragma unroll
    for (int j = 0; j < HR_ITEMS; ++j) {
      const bool ok = base + j < n;
      h[j] = ok ? hashed[at + j] : 0.0f;
      re[j] = ok ? rank_eta[base + j] : 0;
      rp[j] = ok ? rank_phi[base + j] : 0;
    }
  }
  float k[HR_ITEMS];
#pragma unroll
  for (int j = 0; j < HR_ITEMS; ++j) {
    const float hj = base + j < n_raw ? h[j] : __builtin_inff();
    k[j] = hj + hr_shift(hr_region((float)re[j], size_eta), hr_region((float)rp[j], size_phi), shift, mult);
  }
  if (full) {
    *reinterpret_cast<float4*>(keys + at) = make_float4(k[0], k[1], k[2], k[3]);
  } else {
#pragma unroll
    for (int j = 0; j < HR_ITEMS; ++j)
      if (base + j < n) keys[at + j] = k[j];
  }
}

static dim3 hr_grid(int64_t n, int n_rows) {
  const int64_t per_block = (int64_t)HR_BLOCK * HR_ITEMS;
  return dim3((unsigned)((n + per_block - 1) / per_block), n_rows);
}

// out [n_rows, n] float32: 1-based quantile region of every hit for each row's number of regions.
// rank [n] (int32 or int64): position of the hit in the coordinate-sorted order; regions [n_rows] device float32 > 0.
extern "C" int lampa_quantile_regions(const void* rank, int idx_bytes, int64_t n, const float* regions, int n_rows,
                                      float* out, void* stream) {
  if (!rank || !regions || !out || n < 0 || n_rows < 1 || n_rows > 65535) return LAMPA_ERR_INVALID;
  if (idx_bytes != 4 && idx_bytes != 8) return LAMPA_ERR_INVALID;
  if (n > (1 << 24)) return LAMPA_ERR_UNSUPPORTED;
  if (n == 0) return LAMPA_OK;
  LAMPA_PROF((hipStream_t)stream, "start");
  if (idx_bytes == 4)
    hipLaunchKernelGGL(hr_quantile_kernel<int32_t>, hr_grid(n, n_rows), dim3(HR_BLOCK), 0, (hipStream_t)stream, rank, n,
                       regions, out);
  else
    hipLaunchKernelGGL(hr_quantile_kernel<int64_t>, hr_grid(n, n_rows), dim3(HR_BLOCK), 0, (hipStream_t)stream, rank, n,
                       regions, out);
  LAMPA_PROF((hipStream_t)stream, "hr_quantile_kernel");
  return lampa_launch_status();
}

// out [n_rows, n] = (region_phi * hash_shift) * (ceil(regions_eta) + 1) + region_eta * hash_shift.
// region_eta, region_phi [n_rows, n]; hash_shift, regions_eta [n_rows] (device float32).
extern "C" int lampa_geo_shift(const float* region_eta, const float* region_phi, const float* hash_shift,
                               const float* regions_eta, int n_rows, int64_t n, float* out, void* stream) {
  if (!region_eta || !region_phi || !hash_shift || !regions_eta || !out) return LAMPA_ERR_INVALID;
  if (n < 0 || n_rows < 1 || n_rows > 65535) return LAMPA_ERR_INVALID;
  if (n == 0) return LAMPA_OK;
  LAMPA_PROF((hipStream_t)stream, "start");
  hipLaunchKernelGGL(hr_geo_shift_kernel, hr_grid(n, n_rows), dim3(HR_BLOCK), 0, (hipStream_t)stream, region_eta,
                     region_phi, hash_shift, regions_eta, n, out);
  LAMPA_PROF((hipStream_t)stream, "hr_geo_shift_kernel");
  return lampa_launch_status();
}

// keys [n_rows, n] = hashed (+inf at or beyond n_raw) + region shift, without materialising the region indices.
// hashed [n_rows, n]; rank_eta, rank_phi [n] int32; regions [2, n_rows] (eta row, phi row); hash_shift [n_rows].
extern "C" int lampa_hept_sort_keys(const float* hashed, const int32_t* rank_eta, const int32_t* rank_phi,
                                    const float* regions, const float* hash_shift, int n_rows, int64_t n, int64_t n_raw,
                                    float* keys, void* stream) {
  if (!hashed || !rank_eta || !rank_phi || !regions || !hash_shift || !keys) return LAMPA_ERR_INVALID;
  if (n < 0 || n_raw < 0 || n_raw > n || n_rows < 1 || n_rows > 65535) return LAMPA_ERR_INVALID;
  if (n > (1 << 24)) return LAMPA_ERR_UNSUPPORTED;
  if (n == 0) return LAMPA_OK;
  LAMPA_PROF((hipStream_t)stream, "start");
  hipLaunchKernelGGL(hr_sort_keys_kernel, hr_grid(n, n_rows), dim3(HR_BLOCK), 0, (hipStream_t)stream, hashed, rank_eta,
                     rank_phi, regions, hash_shift, n_rows, n, n_raw, keys);
  LAMPA_PROF((hipStream_t)stream, "hr_sort_keys_kernel");
  return lampa_launch_status();
}

// ---------------------------------------------------------------------------------------------- prep_qk
// scale[h, c] = sqrt(2 * qw[h, max(c - 1, 0)]), qw[h, r] = sum_k exp(min(sum_d w[h, d, r, k], 50))   (hept.py:55-58)
__global__ void hr_prep_scale_kernel(const float* __restrict__ w, int H, int d, int R, int Kw, float* __restrict__ scale) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= H * (R + 1)) return;
  const int h = i / (R + 1), c = i % (R + 1), r = c > 0 ? c - 1 : 0;
  float qw = 0.0f;
  for (int k = 0; k < Kw; ++k) {
    float sum = 0.0f;
    for (int j = 0; j < d; ++j) sum += w[(((int64_t)h * d + j) * R + r) * Kw + k];
    qw += expf(fminf(sum, 50.0f));
  }
  scale[i] = sqrtf(2.0f * qw);
}

// out[(n, h) or (h, n)][j] = x[n, h, j] for j < d, scale[h, j - d] * coords[n, j - d] for the R + 1 appended columns;
// rows at or beyond n_raw are zero. blockIdx.y selects query / key.
__global__ void __launch_bounds__(HR_BLOCK) hr_prep_qk_kernel(const float* __restrict__ query, const float* __restrict__ key,
                                                             const float* __restrict__ coords, const float* __restrict__ scale,
                                                             int64_t n, int64_t n_raw, int H, int d, int C, int heads_first,
                                                             float* __restrict__ q_hat, float* __restrict__ k_hat) {
  const int D = d + C;
  const int64_t i = (int64_t)blockIdx.x * HR_BLOCK + threadIdx.x;
  if (i >= n * H * D) return;
  const int j = (int)(i % D);
  const int64_t nh = i / D;
  const int h = (int)(nh % H);
  const int64_t t = nh / H;
  const float* x = blockIdx.y == 0 ? query : key;
  float* out = blockIdx.y == 0 ? q_hat : k_hat;
  float v = 0.0f;
  if (t < n_raw) v = j < d ? x[(t * H + h) * d + j] : __fmul_rn(scale[h * C + (j - d)], coords[t * C + (j - d)]);
  out[heads_first ? ((int64_t)h * n + t) * D + j : i] = v;
}

// query, key [n, H, d] fp32; w [H, d, R, Kw] fp32; coords [n, R + 1] fp32; scale_ws: R + 1 floats per head (device).
// q_hat, k_hat [n, H, d + R + 1] (heads_first 0) or [H, n, d + R + 1] (heads_first 1); rows from n_raw on are zero.
// Replaces prep_qk and the rearrange + zeroing that follows it (models/attention/hept.py:54-62,118-128).
extern "C" int lampa_hept_prep_qk(const float* query, const float* key, const float* w, const float* coords, int64_t n,
                                  int64_t n_raw, int H, int d, int R, int Kw, int heads_first, float* scale_ws, float* q_hat,
                                  float* k_hat, void* stream) {
  if (!query || !key || !w || !coords || !scale_ws || !q_hat || !k_hat) return LAMPA_ERR_INVALID;
  if (n < 0 || n_raw < 0 || n_raw > n || H < 1 || d < 1 || R < 1 || Kw < 1) return LAMPA_ERR_INVALID;
  hipStream_t s = (hipStream_t)stream;
  const int C = R + 1;
  hipLaunchKernelGGL(hr_prep_scale_kernel, dim3((H * C + 63) / 64), dim3(64), 0, s, w, H, d, R, Kw, scale_ws);
  if (n == 0) return lampa_launch_status();
  const int64_t items = n * H * (d + C);
  LAMPA_PROF(s, "start");
  hipLaunchKernelGGL(hr_prep_qk_kernel, dim3((unsigned)((items + HR_BLOCK - 1) / HR_BLOCK), 2), dim3(HR_BLOCK), 0, s, query,
                     key, coords, scale_ws, n, n_raw, H, d, C, heads_first, q_hat, k_hat);
  LAMPA_PROF(s, "hr_prep_qk_kernel");
  return lampa_launch_status();
}

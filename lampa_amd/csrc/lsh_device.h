// Device helpers of the E2LSH hash.
// Arithmetic contract: p = fmaf(x[d], a[d], p) left to right from 0; id = floorf((p + b) * inv_w) saturated to
// int32, NaN -> INT32_MAX. Only explicit fmaf / single operations, so compiler contraction cannot change a bit.
#pragma once
#include "common.h"

#define LSH_MAX_DIM 8
#define LSH_MAX_COLS 64
#define LSH_MAX_PROJ 8
#define LSH_BLOCK 256

// bucket id of the scaled projection t = (p + b) * inv_w. Monotone non-decreasing on the non-NaN floats (so the
// smallest / largest id of a set is the id of its smallest / largest t).
__device__ __forceinline__ int32_t lsh_quantise_scaled(float t) {
  if (t != t) return INT32_MAX;
  float f = floorf(t);
  if (f >= 2147483648.0f) return INT32_MAX;
  if (f <= -2147483648.0f) return INT32_MIN;
  return (int32_t)f;
}
__device__ __forceinline__ float lsh_scaled(float p, float b, float inv_w) { return (p + b) * inv_w; }
__device__ __forceinline__ int32_t lsh_quantise(float p, float b, float inv_w) {
  return lsh_quantise_scaled(lsh_scaled(p, b, inv_w));
}

template <int DIM>
__device__ __forceinline__ void lsh_load_coords(const float* __restrict__ coords, int64_t n, int dim, float* x) {
  if (DIM == 4) {
    float4 c = *reinterpret_cast<const float4*>(coords + n * 4);
    x[0] = c.x; x[1] = c.y; x[2] = c.z; x[3] = c.w;
  } else {
#pragma unroll
    for (int d = 0; d < LSH_MAX_DIM; ++d) x[d] = d < dim ? coords[n * dim + d] : 0.0f;
  }
}

template <int DIM>
__device__ __forceinline__ float lsh_dot(const float* x, const float* __restrict__ alpha, int dim, int n_cols, int c) {
  float acc = 0.0f;
  if (DIM == 4) {
#pragma unroll
    for (int d = 0; d < 4; ++d) acc = __builtin_fmaf(x[d], alpha[d * n_cols + c], acc);
  } else {
#pragma unroll
    for (int d = 0; d < LSH_MAX_DIM; ++d)
      if (d < dim) acc = __builtin_fmaf(x[d], alpha[d * n_cols + c], acc);
  }
  return acc;
}


// Wave-wide min / max on the VALU data-parallel-primitive path (no LDS round trips); the result is valid in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int32_t lsh_dpp(int32_t x) {
  return __builtin_amdgcn_update_dpp(x, x, CTRL, ROW_MASK, 0xF, false);  // lanes without a source keep their own x
}
template <bool MAX>
__device__ __forceinline__ int32_t lsh_wave_extreme(int32_t v) {
#define LSH_STEP(CTRL, ROWS)                      \
  {                                               \
    const int32_t o = lsh_dpp<CTRL, ROWS>(v);     \
    v = MAX ? max(v, o) : min(v, o);              \
  }
  LSH_STEP(0xB1, 0xF)   // quad_perm [1,0,3,2]
  LSH_STEP(0x4E, 0xF)   // quad_perm [2,3,0,1]
  LSH_STEP(0x141, 0xF)  // row_half_mirror
  LSH_STEP(0x140, 0xF)  // row_mirror: every lane of a row of 16 holds the row's extreme
  LSH_STEP(0x142, 0xA)  // row_bcast15 into rows 1 and 3
  LSH_STEP(0x143, 0xC)  // row_bcast31 into rows 2 and 3
#undef LSH_STEP
  return v;
}

// Device helpers of the E2LSH hash shared by the separate kernels and the fused single-launch kernel.
// Arithmetic contract: p = fmaf(x[d], a[d], p) left to right from 0; id = floorf((p + b) * inv_w) saturated to
// int32, NaN -> INT32_MAX. Only explicit fmaf / single operations, so compiler contraction cannot change a bit.
#pragma once
#include "common.h"

#define LSH_MAX_DIM 8
#define LSH_MAX_COLS 64
#define LSH_MAX_PROJ 8
#define LSH_BLOCK 256

__device__ __forceinline__ int32_t lsh_quantise(float p, float b, float inv_w) {
  float t = (p + b) * inv_w;
  if (t != t) return INT32_MAX;
  float f = floorf(t);
  if (f >= 2147483648.0f) return INT32_MAX;
  if (f <= -2147483648.0f) return INT32_MIN;
  return (int32_t)f;
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


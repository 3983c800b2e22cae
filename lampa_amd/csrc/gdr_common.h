// Types and small device helpers shared by the gated-delta kernels (gfx950, wave64, MFMA 32x32x16 bf16).
#pragma once
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

enum { GDR_BF16 = 0, GDR_FP16 = 1, GDR_FP32 = 2 };
enum { GDR_L2_NONE = 0, GDR_L2_CHUNK = 1, GDR_L2_RECURRENT = 2 };

// D = A (32x16) * B (16x32) + C on one wave.  Lane l = 32*hh + ln supplies A[row ln][k 8hh..8hh+7] and
// B[k 8hh..8hh+7][col ln]; accumulator register r of lane l is element (row 8*(r/4) + 4*hh + r%4, col ln).
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// The 8 accumulator registers [base, base+8) of a lane, rounded to bf16, form that lane's share of an MFMA
// operand whose 16-wide contraction step covers accumulator rows 16*(base/8) .. +15 in the order
// slot s -> row 8*(s/4) + 4*hh + s%4.  Any operand built from memory for the other side of such a product
// must use the same slot order (see kappa()).
__device__ __forceinline__ bf16x8 acc_to_operand(const f32x16& acc, int base) {
  bf16x8 out;
#pragma unroll
  for (int s = 0; s < 8; ++s) out[s] = (__bf16)acc[base + s];
  return out;
}

// Offset inside a 16-wide contraction step of slot s for lane half hh.
__device__ __forceinline__ int kappa(int hh, int s) { return 8 * (s / 4) + 4 * hh + (s % 4); }

__device__ __forceinline__ float bf16_bits_to_float(unsigned short b) { return __uint_as_float((uint32_t)b << 16); }

template <typename T>
struct GdrElem;
template <>
struct GdrElem<__bf16> {
  static __device__ __forceinline__ float to_float(__bf16 x) { return (float)x; }
  static __device__ __forceinline__ __bf16 from_float(float x) { return (__bf16)x; }
};
template <>
struct GdrElem<_Float16> {
  static __device__ __forceinline__ float to_float(_Float16 x) { return (float)x; }
  static __device__ __forceinline__ _Float16 from_float(float x) { return (_Float16)x; }
};
template <>
struct GdrElem<float> {
  static __device__ __forceinline__ float to_float(float x) { return x; }
  static __device__ __forceinline__ float from_float(float x) { return x; }
};

// Loads 8 consecutive elements (the pointer must be aligned to 8 elements) and widens them to fp32.
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* out) {
  if constexpr (sizeof(T) == 2) {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    vec8 v = *reinterpret_cast<const vec8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = GdrElem<T>::to_float(v[i]);
  } else {
    f32x4 a = *reinterpret_cast<const f32x4*>(p);
    f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { out[i] = a[i]; out[4 + i] = b[i]; }
  }
}

// Lane exchanges on the VALU data-parallel-primitive path (no LDS round trip, unlike __shfl*).
// dpp_f32<CTRL, ROW_MASK>(old, x): lane i receives x of the lane CTRL selects; lanes whose row is not in ROW_MASK
// or whose source lies outside their row of 16 keep `old`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32(float old, float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(x), CTRL, ROW_MASK, 0xF, false));
}
#define GDR_DPP_QUAD_XOR1 0xB1   /* quad_perm [1,0,3,2] */
#define GDR_DPP_QUAD_XOR2 0x4E   /* quad_perm [2,3,0,1] */
#define GDR_DPP_ROW_SHR(n) (0x110 + (n))
#define GDR_DPP_ROW_BCAST15 0x142 /* lane 15 of each row -> every lane of the next row */
#define GDR_DPP_ROW_BCAST31 0x143 /* lane 31 -> rows 2 and 3 */

// Inclusive prefix sum over the 64 lanes of a wave: Hillis-Steele inside each row of 16, then the row totals.
__device__ __forceinline__ float wave_inclusive_scan(float x) {
  x += dpp_f32<GDR_DPP_ROW_SHR(1), 0xF>(0.0f, x);
  x += dpp_f32<GDR_DPP_ROW_SHR(2), 0xF>(0.0f, x);
  x += dpp_f32<GDR_DPP_ROW_SHR(4), 0xF>(0.0f, x);
  x += dpp_f32<GDR_DPP_ROW_SHR(8), 0xF>(0.0f, x);
  x += dpp_f32<GDR_DPP_ROW_BCAST15, 0xA>(0.0f, x);
  x += dpp_f32<GDR_DPP_ROW_BCAST31, 0xC>(0.0f, x);
  return x;
}

// Inclusive running minimum / maximum over the 64 lanes (same data movement as the prefix sum; exact).
__device__ __forceinline__ float wave_inclusive_min(float x) {
  const float inf = __builtin_inff();
  x = fminf(x, dpp_f32<GDR_DPP_ROW_SHR(1), 0xF>(inf, x));
  x = fminf(x, dpp_f32<GDR_DPP_ROW_SHR(2), 0xF>(inf, x));
  x = fminf(x, dpp_f32<GDR_DPP_ROW_SHR(4), 0xF>(inf, x));
  x = fminf(x, dpp_f32<GDR_DPP_ROW_SHR(8), 0xF>(inf, x));
  x = fminf(x, dpp_f32<GDR_DPP_ROW_BCAST15, 0xA>(inf, x));
  x = fminf(x, dpp_f32<GDR_DPP_ROW_BCAST31, 0xC>(inf, x));
  return x;
}
__device__ __forceinline__ float wave_inclusive_max(float x) { return -wave_inclusive_min(-x); }

// In-chunk cumulative log-decay of a wave's 64 tokens (lane = token). A tree-shaped prefix sum is not monotone in
// floating point: with every g <= 0 a later lane can still come out an ulp ABOVE an earlier one, and the decay ratios
// e^{gamma_i - gamma_j} are masked wherever that difference is positive (safe_exp), which would drop whole terms.
// So the non-positive and the positive parts of g are summed separately and each prefix is made exactly monotone by a
// running minimum / maximum: for g <= 0 the result never increases from one token to the next.
__device__ __forceinline__ float wave_cumulative_decay(float g) {
  if (__ballot(g != g)) return wave_inclusive_scan(g);  // a NaN decay poisons everything after it, as in the reference
  float cum = wave_inclusive_min(wave_inclusive_scan(fminf(g, 0.0f)));
  if (__ballot(g > 0.0f)) cum += wave_inclusive_max(wave_inclusive_scan(fmaxf(g, 0.0f)));
  return cum;
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every outstanding global load
// and store of the wave (vmcnt(0)), which would serialise the software prefetch of the next chunk behind each
// barrier; here only the LDS / scalar counter is drained.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Waits for this wave's outstanding LDS reads and keeps the compiler from moving LDS accesses across this point.
__device__ __forceinline__ void lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// Pieces of the segmented token-serial forward (gdr_recurrent.hip) that the backward pass (gdr_backward.hip) runs on
// their own: every segment's affine map [M | N] (mn [n_seg, HV, K, K + V], fp32), and the serial product of the maps
// over each sequence's segments (sinit [n_seg, HV, K, V]: the state each segment starts from; h0 nullable), for a few
// long sequences in three launches over groups of segments (`groups`: scratch of gdr_scan_group_floats floats or NULL).
int gdr_segment_maps(const void* k, const void* v, const float* g, const float* beta, const int64_t* cu_seg, int n_seg,
                     int H, int HV, int K, int V, int dtype, int l2norm, float* mn, hipStream_t s);
int gdr_segment_scan(const float* mn, const float* h0, const int32_t* seq_seg0, int n_seq, int n_seg, int HV, int K,
                     int V, float* sinit, float* groups, hipStream_t s);
// floats of the `groups` area (the groups' maps and start states of the scan's three-launch form; 0: not used at this
// size, pass NULL)
int64_t gdr_scan_group_floats(int n_seg, int HV, int K, int V);

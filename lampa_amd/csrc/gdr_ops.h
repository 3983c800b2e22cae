// MFMA operand helpers of the chunkwise gated-delta kernels, generic in the 16-bit operand type (bf16 or fp16).
//
// bf16 inputs run on v_mfma_f32_32x32x16_bf16, fp16 inputs on v_mfma_f32_32x32x16_f16: every operand that the kernels
// derive (T, W, U, P, the state as operand ...) is rounded to the INPUT type, as the reference's Triton kernels do
// (b_h.to(b_k.dtype), models/hattention/chunk_delta_h.py:133-151; its caller feeds fp16,
// models/hattention/modeling_gated_deltaproduct.py:583-587).
#pragma once
#include "gdr_common.h"

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

template <typename T>
struct OpVec {
  typedef T x8 __attribute__((ext_vector_type(8)));
  typedef T x4 __attribute__((ext_vector_type(4)));
  typedef T x2 __attribute__((ext_vector_type(2)));
};

// 8 accumulator registers [base, base + 8) of a lane, rounded to T: the lane's share of an MFMA operand whose 16-wide
// contraction step covers accumulator rows 16 (base / 8) .. + 15 in slot order (see acc_to_operand in gdr_common.h).
// Read as the B operand it is (rows of the accumulator tile = contraction, lane's column = operand column); read as
// the A operand it is the TRANSPOSE of the tile (operand row = the lane's column).
template <typename T>
__device__ __forceinline__ typename OpVec<T>::x8 acc_to_op(const f32x16& acc, int base) {
  typename OpVec<T>::x8 out;
#pragma unroll
  for (int s = 0; s < 8; ++s) out[s] = (T)acc[base + s];
  return out;
}

template <typename T>
__device__ __forceinline__ typename OpVec<T>::x8 op_frag_load(const unsigned char* base, int frag, int lane) {
  return *reinterpret_cast<const typename OpVec<T>::x8*>(base + (size_t)frag * 1024 + lane * 16);
}
template <typename T>
__device__ __forceinline__ void op_frag_store(unsigned char* base, int frag, int lane, typename OpVec<T>::x8 v) {
  *reinterpret_cast<typename OpVec<T>::x8*>(base + (size_t)frag * 1024 + lane * 16) = v;
}

// A-operand fragment of rows row0 .. row0 + 31 (lane's row = `row`) of a row-major array with `stride` elements per
// row, contraction step starting at column col0, in accumulator slot order.
template <typename T>
__device__ __forceinline__ typename OpVec<T>::x8 op_ld_kappa(const T* arr, int stride, int row, int col0, int hh) {
  const typename OpVec<T>::x4 lo = *reinterpret_cast<const typename OpVec<T>::x4*>(arr + row * stride + col0 + 4 * hh);
  const typename OpVec<T>::x4 hi = *reinterpret_cast<const typename OpVec<T>::x4*>(arr + row * stride + col0 + 8 + 4 * hh);
  typename OpVec<T>::x8 out;
#pragma unroll
  for (int s = 0; s < 4; ++s) { out[s] = lo[s]; out[4 + s] = hi[s]; }
  return out;
}

// Swizzled row-major tiles. The lane's share of a 16-wide contraction step in accumulator slot order is elements
// 4 hh .. + 3 and 8 + 4 hh .. + 3 of the 16: two 8-byte LDS reads, and the 32 lanes of a half-wave hit every bank pair
// twice whatever 16-byte aligned row stride the tile has. Tiles that feed such operands are therefore stored with the
// two middle groups of four of every 16 columns swapped ([0-3 | 8-11 | 4-7 | 12-15]): the share becomes ONE aligned
// 16-byte piece at column 8 hh of the group (a ds_read_b128, served 16 lanes at a time without conflicts). The writer
// holds both 8-element pieces of a group in registers, so the swap is a renaming of registers.
template <typename T>
__device__ __forceinline__ void op_swizzle16(typename OpVec<T>::x8& a, typename OpVec<T>::x8& b) {
  typename OpVec<T>::x8 na, nb;
#pragma unroll
  for (int s = 0; s < 4; ++s) { na[s] = a[s]; na[4 + s] = b[s]; nb[s] = a[4 + s]; nb[4 + s] = b[4 + s]; }
  a = na;
  b = nb;
}
template <typename T>
__device__ __forceinline__ typename OpVec<T>::x8 op_ld_kappa_swz(const T* arr, int stride, int row, int col0, int hh) {
  return *reinterpret_cast<const typename OpVec<T>::x8*>(arr + row * stride + col0 + 8 * hh);
}

// ds_read_b64_tr_b16: lane i of every block of 16 lanes receives element (i % 4) of the four 8-byte rows that lanes
// i/4, i/4 + 4, i/4 + 8 and i/4 + 12 of its block point at. Must be issued with every lane enabled.
template <typename T>
__device__ __forceinline__ typename OpVec<T>::x4 op_lds_read_tr4(const T* p) {
  typedef short s16x4v __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) s16x4v lds_s16x4;
  return __builtin_bit_cast(typename OpVec<T>::x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p));
}

// Four consecutive rows row0 + 4 hh .. + 3 of column col0 + (lane % 32) of a row-major tile: lane L of a block of 16
// points at row L / 4, column group L % 4 of the block's 16 columns.
template <typename T>
__device__ __forceinline__ typename OpVec<T>::x4 op_ld_col4(const T* arr, int stride, int col0, int row0, int lane) {
  const int L = lane & 15, blk = (lane >> 4) & 1, hh = lane >> 5;
  return op_lds_read_tr4<T>(arr + (row0 + 4 * hh + (L >> 2)) * stride + col0 + 16 * blk + 4 * (L & 3));
}

// Fragment of the TRANSPOSE of a row-major tile: operand row (A) / column (B) = tile column col0 + (lane % 32),
// contraction over the tile rows row0 .. row0 + 15 in accumulator slot order.
// SWZ: the tile is stored swizzled (above): logical column group g of a 16 sits at position [0, 2, 1, 3][g].
template <typename T, bool SWZ = false>
__device__ __forceinline__ typename OpVec<T>::x8 op_ld_kappa_tr(const T* arr, int stride, int col0, int row0, int lane) {
  const int L = lane & 15, blk = (lane >> 4) & 1, hh = lane >> 5;
  const int g = SWZ ? (((L & 1) << 1) | ((L >> 1) & 1)) : (L & 3);
  const T* p = arr + (row0 + 4 * hh + (L >> 2)) * stride + col0 + 16 * blk + 4 * g;
  const typename OpVec<T>::x4 lo = op_lds_read_tr4<T>(p), hi = op_lds_read_tr4<T>(p + 8 * stride);
  typename OpVec<T>::x8 out;
#pragma unroll
  for (int s = 0; s < 4; ++s) { out[s] = lo[s]; out[4 + s] = hi[s]; }
  return out;
}

// ---- 16 x 16 x 32 products ("narrow" chain waves: 16 columns of the state per wave) ------------------------------------
// D = A (16 x 32) * B (32 x 16) + C on one wave. Lane l = 16 g + i supplies A[row i][k 8 g .. 8 g + 7] and
// B[k 8 g .. 8 g + 7][col i]; accumulator register r of lane l is element (row 4 g + r, col i).
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Two accumulator tiles that cover rows 0-15 and 16-31 of a 32-row block, rounded to T: the lane's share of an operand
// whose 32-wide contraction step visits those rows in the order slot s -> row 16 (s / 4) + 4 g + s % 4 ("slot order
// of the narrow shape"). Read as the B operand it is the block itself (the lane's column = operand column), read as the
// A operand its transpose (operand row = the lane's column).
template <typename T>
__device__ __forceinline__ typename OpVec<T>::x8 acc2_to_op(const f32x4& lo, const f32x4& hi) {
  typename OpVec<T>::x8 out;
#pragma unroll
  for (int s = 0; s < 4; ++s) { out[s] = (T)lo[s]; out[4 + s] = (T)hi[s]; }
  return out;
}

// Row-major tiles that feed such products from memory keep every group of 32 columns in the order
// [0-3 | 16-19 | 4-7 | 20-23 | 8-11 | 24-27 | 12-15 | 28-31]: the lane's share of a 32-wide step in the slot order above
// (columns 4 g .. + 3 and 16 + 4 g .. + 3) is then ONE aligned 16-byte piece at position 8 g of the group. A writer that
// holds the four 8-element pieces of a group renames registers:
template <typename T>
__device__ __forceinline__ void op_perm32(typename OpVec<T>::x8& p0, typename OpVec<T>::x8& p1, typename OpVec<T>::x8& p2,
                                          typename OpVec<T>::x8& p3) {
  typename OpVec<T>::x8 d0, d1, d2, d3;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    d0[s] = p0[s];     d0[4 + s] = p2[s];
    d1[s] = p0[4 + s]; d1[4 + s] = p2[4 + s];
    d2[s] = p1[s];     d2[4 + s] = p3[s];
    d3[s] = p1[4 + s]; d3[4 + s] = p3[4 + s];
  }
  p0 = d0; p1 = d1; p2 = d2; p3 = d3;
}
// position (in elements) inside such a tile row of the 4-column group that starts at logical column c (c % 4 == 0)
__device__ __forceinline__ int op_perm32_col(int c) {
  const int q = (c >> 2) & 7;  // group within its 32
  return (c & ~31) + 4 * (q < 4 ? 2 * q : 2 * (q - 4) + 1);
}
// where the two 8-byte halves of the 8-column piece `part` (0..3) of a 32-column group go: the first at 4 * slot, the
// second 8 elements further on
__device__ __forceinline__ int op_perm32_piece(int part) { return 4 * (part < 2 ? 4 * part : 4 * (part - 2) + 1); }

// Fragment of the TRANSPOSE of such a tile for the narrow shape: operand row (A) = tile column col0 + i, contraction
// over the tile rows row0 .. row0 + 31 in the slot order above. PERM: the tile's columns are stored in the order above.
template <typename T, bool PERM>
__device__ __forceinline__ typename OpVec<T>::x8 op_ld_tr16(const T* arr, int stride, int col0, int row0, int lane) {
  const int L = lane & 15, g = lane >> 4;
  const int c = col0 + 4 * (L & 3);
  const T* p = arr + (row0 + 4 * g + (L >> 2)) * stride + (PERM ? op_perm32_col(c) : c);
  const typename OpVec<T>::x4 lo = op_lds_read_tr4<T>(p), hi = op_lds_read_tr4<T>(p + 16 * stride);
  typename OpVec<T>::x8 out;
#pragma unroll
  for (int s = 0; s < 4; ++s) { out[s] = lo[s]; out[4 + s] = hi[s]; }
  return out;
}

// sum of squares of a 16-byte piece of the input type, accumulated in fp32
template <typename T>
__device__ __forceinline__ float op_sumsq(typename OpVec<T>::x8 v, float ss) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float f = (float)v[e];
    ss = __builtin_fmaf(f, f, ss);
  }
  return ss;
}

// Row gather / scatter / inverse permutation for the LSH stage on gfx950 (pure HBM-bound data movement).
//
// Replaces (reference chengjiang123/Lampa): batched_index_select  models/model_utils/hash_utils.py:83-93
// (gather with an index tensor expanded over the feature dimension), sort_to_buckets / unsort_from_buckets
// models/attention/hept.py:9-19, invert_permutation  hash_utils.py:46-57, and the gather / argsort-unsort of
// LSHOrdering's caller  models/baselines/full_mamba2.py:213-216,678-682.
#include "common.h"

#define GS_BLOCK 256

template <typename IdxT>
__device__ __forceinline__ int64_t gs_index(const void* idx, int64_t i) {
  return (int64_t)reinterpret_cast<const IdxT*>(idx)[i];
}

// One thread moves GS_UNROLL VEC-byte pieces of rows, a block's worth apart: all their indices are loaded first, then
// all their source pieces, then they are stored, so a thread has GS_UNROLL independent loads in flight (the kernel is a
// chain of three dependent memory operations per piece and is bound by how many bytes the chip has in flight, not by
// the bus). dst[s, n, :] = src[s or 0, idx[s, n], :] when GATHER, dst[s, idx[s, n], :] = src[s, n, :] otherwise.
#define GS_UNROLL 4
template <typename VecT, typename IdxT, bool GATHER>
__global__ void __launch_bounds__(GS_BLOCK) gs_rows_kernel(const char* __restrict__ src, int64_t src_seg_stride,
                                                          int src_segments, int group, const void* __restrict__ idx, int64_t n,
                                                          int64_t n_src, int vec_per_row, char* __restrict__ dst) {
  const int seg = blockIdx.y;
  const int64_t limit = GATHER ? n_src : n;
  const int64_t row_bytes = (int64_t)vec_per_row * (int64_t)sizeof(VecT);
  const char* src_seg = src + ((seg / group) % src_segments) * src_seg_stride;
  char* dst_seg = dst + (int64_t)seg * n * row_bytes;
  int64_t row[GS_UNROLL], other[GS_UNROLL];
  int piece[GS_UNROLL];
  bool live[GS_UNROLL], inside[GS_UNROLL];
#pragma unroll
  for (int u = 0; u < GS_UNROLL; ++u) {
    const int64_t item = ((int64_t)blockIdx.x * GS_UNROLL + u) * GS_BLOCK + threadIdx.x;
    row[u] = item / vec_per_row;
    piece[u] = (int)(item - row[u] * vec_per_row);
    live[u] = row[u] < n;
    other[u] = live[u] ? gs_index<IdxT>(idx, (int64_t)seg * n + row[u]) : 0;
  }
  VecT val[GS_UNROLL];
#pragma unroll
  for (int u = 0; u < GS_UNROLL; ++u) {
    // an index outside the source: a gathered row reads as zeros (never as whatever the output buffer held), a
    // scattered row is dropped
    inside[u] = live[u] && other[u] >= 0 && other[u] < limit;
    const int64_t from = GATHER ? other[u] : row[u];
    val[u] = inside[u] ? reinterpret_cast<const VecT*>(src_seg + from * row_bytes)[piece[u]] : VecT{};
  }
#pragma unroll
  for (int u = 0; u < GS_UNROLL; ++u) {
    const int64_t to = GATHER ? row[u] : other[u];
    if (inside[u] || (GATHER && live[u])) {
      VecT* at = reinterpret_cast<VecT*>(dst_seg + to * row_bytes) + piece[u];
      if constexpr (GATHER && sizeof(VecT) == 16) {
        // rows in output order: written once, in order, not read here -- a non-temporal store leaves the L2 to the
        // source rows, which the other tables of the event read again (batch of 32 events: 378 -> 369 us)
        typedef unsigned int gs_u32x4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(*reinterpret_cast<const gs_u32x4*>(&val[u]), reinterpret_cast<gs_u32x4*>(at));
      } else {
        *at = val[u];
      }
    }
  }
}

template <typename IdxT>
__global__ void __launch_bounds__(GS_BLOCK) gs_invert_kernel(const IdxT* __restrict__ perm, int64_t n,
                                                            IdxT* __restrict__ inv) {
  const int seg = blockIdx.y;
  const int64_t i = (int64_t)blockIdx.x * GS_BLOCK + threadIdx.x;
  if (i >= n) return;
  const int64_t p = (int64_t)perm[(int64_t)seg * n + i];
  if (p >= 0 && p < n) inv[(int64_t)seg * n + p] = (IdxT)i;
}

template <typename IdxT, bool GATHER>
static int gs_launch(const void* src, int64_t src_seg_stride, int src_segments, int group, const void* idx, int n_segments, int64_t n,
                     int64_t n_src, int64_t row_bytes, void* dst, hipStream_t s) {
  const bool a16 = row_bytes % 16 == 0 && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0) &&
                   src_seg_stride % 16 == 0;
  const bool a4 = row_bytes % 4 == 0 && ((uintptr_t)src % 4 == 0) && ((uintptr_t)dst % 4 == 0) &&
                  src_seg_stride % 4 == 0;
  const int vec = a16 ? 16 : (a4 ? 4 : 1);
  const int vec_per_row = (int)(row_bytes / vec);
  const int64_t items = n * vec_per_row;
  const int64_t per_block = (int64_t)GS_BLOCK * GS_UNROLL;
  const dim3 grid((unsigned)((items + per_block - 1) / per_block), n_segments), block(GS_BLOCK);
  LAMPA_PROF(s, "start");
  if (vec == 16)
    hipLaunchKernelGGL((gs_rows_kernel<uint4, IdxT, GATHER>), grid, block, 0, s, (const char*)src, src_seg_stride, src_segments,
                       group, idx, n, n_src, vec_per_row, (char*)dst);
  else if (vec == 4)
    hipLaunchKernelGGL((gs_rows_kernel<uint32_t, IdxT, GATHER>), grid, block, 0, s, (const char*)src, src_seg_stride,
                       src_segments, group, idx, n, n_src, vec_per_row, (char*)dst);
  else
    hipLaunchKernelGGL((gs_rows_kernel<uint8_t, IdxT, GATHER>), grid, block, 0, s, (const char*)src, src_seg_stride,
                       src_segments, group, idx, n, n_src, vec_per_row, (char*)dst);
  LAMPA_PROF(s, "gs_rows_kernel");
  return lampa_launch_status();
}

// dst [S, n, row_bytes] = rows of src selected by idx [S, n]. src is [src_segments, n_src, row_bytes] and segment s
// reads source segment s % src_segments (src_segments == S: one source per segment; a divisor of S: the sources
// are shared round-robin, which is how a [1, batch, ...] tensor broadcasts over [n_hashes, batch, ...] indices). idx_bytes is 4 (int32) or 8 (int64). A row whose
// index lies outside the source is written as zeros.
// Segment s reads source segment (s / group) % src_segments (group = 1: the exported behaviour; group = tables per
// event: a batch of events whose tables share the event's rows).
int lampa_gather_rows_grouped(const void* src, int src_segments, int group, int64_t n_src, const void* idx,
                              int idx_bytes, int n_segments, int64_t n, int64_t row_bytes, void* dst, void* stream) {
  if (!src || !idx || !dst || n_segments < 1 || n < 0 || n_src < 0 || row_bytes < 1 || group < 1) return LAMPA_ERR_INVALID;
  if (src_segments < 1 || n_segments % src_segments != 0) return LAMPA_ERR_INVALID;
  if (idx_bytes != 4 && idx_bytes != 8) return LAMPA_ERR_INVALID;
  if (n == 0) return LAMPA_OK;
  const int64_t stride = n_src * row_bytes;
  if (idx_bytes == 4)
    return gs_launch<int32_t, true>(src, stride, src_segments, group, idx, n_segments, n, n_src, row_bytes, dst, (hipStream_t)stream);
  return gs_launch<int64_t, true>(src, stride, src_segments, group, idx, n_segments, n, n_src, row_bytes, dst, (hipStream_t)stream);
}

extern "C" int lampa_gather_rows(const void* src, int src_segments, int64_t n_src, const void* idx, int idx_bytes,
                                 int n_segments, int64_t n, int64_t row_bytes, void* dst, void* stream) {
  return lampa_gather_rows_grouped(src, src_segments, 1, n_src, idx, idx_bytes, n_segments, n, row_bytes, dst, stream);
}

// dst [S, n, row_bytes]: dst[s, idx[s, i]] = src[s, i] (idx is a permutation of 0..n-1 per segment).
extern "C" int lampa_scatter_rows(const void* src, const void* idx, int idx_bytes, int n_segments, int64_t n,
                                  int64_t row_bytes, void* dst, void* stream) {
  if (!src || !idx || !dst || n_segments < 1 || n < 0 || row_bytes < 1) return LAMPA_ERR_INVALID;
  if (idx_bytes != 4 && idx_bytes != 8) return LAMPA_ERR_INVALID;
  if (n == 0) return LAMPA_OK;
  const int64_t stride = n * row_bytes;
  if (idx_bytes == 4)
    return gs_launch<int32_t, false>(src, stride, n_segments, 1, idx, n_segments, n, n, row_bytes, dst, (hipStream_t)stream);
  return gs_launch<int64_t, false>(src, stride, n_segments, 1, idx, n_segments, n, n, row_bytes, dst, (hipStream_t)stream);
}

// inv[s, perm[s, i]] = i
extern "C" int lampa_invert_perm(const void* perm, int idx_bytes, int n_segments, int64_t n, void* inv, void* stream) {
  if (!perm || !inv || n_segments < 1 || n < 0) return LAMPA_ERR_INVALID;
  if (idx_bytes != 4 && idx_bytes != 8) return LAMPA_ERR_INVALID;
  if (n == 0) return LAMPA_OK;
  const dim3 grid((unsigned)((n + GS_BLOCK - 1) / GS_BLOCK), n_segments), block(GS_BLOCK);
  if (idx_bytes == 4)
    hipLaunchKernelGGL(gs_invert_kernel<int32_t>, grid, block, 0, (hipStream_t)stream, (const int32_t*)perm, n,
                       (int32_t*)inv);
  else
    hipLaunchKernelGGL(gs_invert_kernel<int64_t>, grid, block, 0, (hipStream_t)stream, (const int64_t*)perm, n,
                       (int64_t*)inv);
  return lampa_launch_status();
}

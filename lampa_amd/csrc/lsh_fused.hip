// Single-launch E2LSH bucket sort of one event: bucket ids, mixed-radix keys, three LSD radix passes and the
// feature gather in ONE persistent kernel whose phases are separated by grid-wide barriers.
//
// Why: at N = 60000 hits the stage moves only ~40 MB, so eight dependent launches (each ~10 us of launch gap and
// tail on this part) dominate; a persistent grid of (tables x tiles) <= 192 co-resident workgroups pays a
// device-scope barrier (~2-3 us) per phase instead. Results are bit-identical to the multi-kernel path
// (lampa_lsh_bucket_keys + lampa_sort_pairs + lampa_gather_rows), which remains the path for larger events.
//
// Replaces the same reference steps as those entry points: hash + range + key (models/model_utils/hash_utils.py:
// 333-371, models/attention/hept.py:79-88), argsort (hept.py:138-139), sort_to_buckets gather (hept.py:9-14).
#include "lsh_device.h"

#define LF_BLOCK 256
#define LF_WAVES 4
#define LF_ITEMS 8
#define LF_TILE (LF_BLOCK * LF_ITEMS)
#define LF_MAX_BINS 2048
#define LF_MAX_GRID 192
#define LF_SPIN_LIMIT (1 << 22)  // polls before a barrier gives up (sets the error flag; every wave still exits)

struct LfCtrl {
  unsigned int arrive;   // grid barrier counter
  unsigned int error;    // set when a barrier timed out
  int32_t minmax[LSH_MAX_COLS][2];
};

__global__ void lf_init_kernel(LfCtrl* ctrl, int n_cols) {
  const int c = threadIdx.x;
  if (c == 0) { ctrl->arrive = 0; ctrl->error = 0; }
  if (c < n_cols) { ctrl->minmax[c][0] = INT32_MAX; ctrl->minmax[c][1] = INT32_MIN; }
}

// All workgroups of the grid meet here. Co-residency is guaranteed by the host (grid <= LF_MAX_GRID, one workgroup
// per CU fits); the spin is bounded so that a scheduling surprise ends in an error flag, not in a hang.
__device__ __forceinline__ void lf_grid_barrier(LfCtrl* ctrl, unsigned int target) {
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    atomicAdd(&ctrl->arrive, 1u);
    int spins = 0;
    while (__hip_atomic_load(&ctrl->arrive, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      __builtin_amdgcn_s_sleep(1);
      if (++spins > LF_SPIN_LIMIT) { atomicExch(&ctrl->error, 1u); break; }
    }
    __threadfence();
  }
  __syncthreads();
}

struct LfArgs {
  const float* coords; const float* alpha; const float* beta;
  int64_t n_hits, n_valid;
  int dim, n_tables, n_proj, n_tiles;
  float inv_w;
  int32_t* ids; int32_t* keys; int32_t* meta; int32_t* perm;
  const uint4* feats; uint4* feats_out; int feat_vecs;  // feature rows in 16-byte pieces
  LfCtrl* ctrl; uint32_t* hist; uint32_t* kbuf; int32_t* vbuf;  // hist [T, n_tiles, LF_MAX_BINS]; k/v [2, T, N]
};

template <int DIM>
__global__ void __launch_bounds__(LF_BLOCK) lf_bucket_sort_kernel(LfArgs a) {
  __shared__ uint32_t s_bin[LF_WAVES][LF_MAX_BINS];
  __shared__ uint32_t s_total[LF_MAX_BINS];
  __shared__ uint32_t s_wsum[LF_WAVES];
  __shared__ int32_t s_red[2][LSH_MAX_PROJ][LF_WAVES];
  __shared__ int32_t s_lo[LSH_MAX_PROJ];
  __shared__ uint32_t s_stride[LSH_MAX_PROJ];
  __shared__ uint32_t s_tot, s_bits;

  const int table = blockIdx.x / a.n_tiles, tile = blockIdx.x % a.n_tiles;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n_cols = a.n_tables * a.n_proj;
  const int64_t N = a.n_hits;
  const int64_t wbase = (int64_t)tile * LF_TILE + wave * (LF_TILE / LF_WAVES);
  unsigned int epoch = 0;

  // ---- phase 0: min / max of this table's id columns over the valid hits ----
  {
    int32_t lo[LSH_MAX_PROJ], hi[LSH_MAX_PROJ];
#pragma unroll
    for (int j = 0; j < LSH_MAX_PROJ; ++j) { lo[j] = INT32_MAX; hi[j] = INT32_MIN; }
#pragma unroll
    for (int i = 0; i < LF_ITEMS; ++i) {
      const int64_t n = wbase + i * 64 + lane;
      if (n < a.n_valid) {
        float x[LSH_MAX_DIM];
        lsh_load_coords<DIM>(a.coords, n, a.dim, x);
#pragma unroll
        for (int j = 0; j < LSH_MAX_PROJ; ++j)
          if (j < a.n_proj) {
            const int c = table * a.n_proj + j;
            const int32_t id = lsh_quantise(lsh_dot<DIM>(x, a.alpha, a.dim, n_cols, c), a.beta[c], a.inv_w);
            lo[j] = min(lo[j], id);
            hi[j] = max(hi[j], id);
          }
      }
    }
#pragma unroll
    for (int j = 0; j < LSH_MAX_PROJ; ++j)
      if (j < a.n_proj) {
        int32_t l = lo[j], h = hi[j];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
          l = min(l, __shfl_xor(l, off));
          h = max(h, __shfl_xor(h, off));
        }
        if (lane == 0) { s_red[0][j][wave] = l; s_red[1][j][wave] = h; }
      }
    __syncthreads();
    if (tid < a.n_proj) {
      int32_t l = s_red[0][tid][0], h = s_red[1][tid][0];
      for (int w = 1; w < LF_WAVES; ++w) { l = min(l, s_red[0][tid][w]); h = max(h, s_red[1][tid][w]); }
      atomicMin(&a.ctrl->minmax[table * a.n_proj + tid][0], l);
      atomicMax(&a.ctrl->minmax[table * a.n_proj + tid][1], h);
    }
  }
  lf_grid_barrier(a.ctrl, ++epoch * gridDim.x);

  // ---- phase 1: strides, keys, meta ----
  if (tid == 0) {
    uint64_t total = 1;
    int overflow = 0;
    int32_t lo_j[LSH_MAX_PROJ];
    int64_t range_j[LSH_MAX_PROJ];
    for (int j = 0; j < a.n_proj; ++j) {
      int32_t lo = __hip_atomic_load(&a.ctrl->minmax[table * a.n_proj + j][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      int32_t hi = __hip_atomic_load(&a.ctrl->minmax[table * a.n_proj + j][1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (a.n_valid == 0) { lo = 0; hi = 0; }
      lo_j[j] = lo;
      range_j[j] = (int64_t)hi - (int64_t)lo + 1;
      s_lo[j] = lo;
      s_stride[j] = (uint32_t)total;
      total *= (uint64_t)range_j[j];
      if (total > (uint64_t)INT32_MAX) { overflow = 1; total = (uint64_t)INT32_MAX + 1; }
    }
    s_tot = (uint32_t)total;
    const uint64_t top = (a.n_valid < N) ? total : total - 1;
    int bits = 1;
    while (bits < 32 && (top >> bits) != 0) ++bits;
    if (overflow) bits = 32;
    s_bits = bits;
    if (tile == 0) {
      int32_t* m = a.meta + (int64_t)table * (2 * a.n_proj + 3);
      for (int j = 0; j < a.n_proj; ++j) {
        m[j] = lo_j[j];
        m[a.n_proj + j] = range_j[j] > INT32_MAX ? INT32_MAX : (int32_t)range_j[j];
      }
      m[2 * a.n_proj] = total > (uint64_t)INT32_MAX ? INT32_MAX : (int32_t)total;
      m[2 * a.n_proj + 1] = bits;
      m[2 * a.n_proj + 2] = overflow;
    }
  }
  __syncthreads();
  const int key_bits = (int)s_bits;
  const int width = (key_bits + 2) / 3;  // three passes, as the multi-kernel path does for device-side bit counts

  uint32_t key[LF_ITEMS];
  int32_t val[LF_ITEMS];
  bool valid[LF_ITEMS];
#pragma unroll
  for (int i = 0; i < LF_ITEMS; ++i) {
    const int64_t n = wbase + i * 64 + lane;
    valid[i] = n < N;
    val[i] = (int32_t)n;
    uint32_t kk = s_tot;
    if (n < a.n_valid) {
      float x[LSH_MAX_DIM];
      lsh_load_coords<DIM>(a.coords, n, a.dim, x);
      kk = 0;
#pragma unroll
      for (int j = 0; j < LSH_MAX_PROJ; ++j)
        if (j < a.n_proj) {
          const int c = table * a.n_proj + j;
          const int32_t id = lsh_quantise(lsh_dot<DIM>(x, a.alpha, a.dim, n_cols, c), a.beta[c], a.inv_w);
          kk += ((uint32_t)id - (uint32_t)s_lo[j]) * s_stride[j];
          if (a.ids) a.ids[(int64_t)c * N + n] = id;
        }
    } else if (valid[i] && a.ids) {
      for (int j = 0; j < a.n_proj; ++j) a.ids[(int64_t)(table * a.n_proj + j) * N + n] = 0;
    }
    key[i] = kk;
    if (valid[i]) a.keys[(int64_t)table * N + n] = (int32_t)kk;
  }

  // ---- three radix passes: histogram | barrier | scatter | barrier ----
  uint32_t* hist_t = a.hist + (int64_t)table * a.n_tiles * LF_MAX_BINS;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int pass = 0; pass < 3; ++pass) {
    const int shift = min(pass * width, 31);
    const int nbits = max(0, min(width, key_bits - pass * width));
    const int bins = 1 << nbits;
    const uint32_t mask = (uint32_t)bins - 1u;
    if (pass > 0) {  // reload this tile from the previous pass's output
      const uint32_t* kin = a.kbuf + ((int64_t)((pass - 1) & 1) * a.n_tables + table) * N;
      const int32_t* vin = a.vbuf + ((int64_t)((pass - 1) & 1) * a.n_tables + table) * N;
#pragma unroll
      for (int i = 0; i < LF_ITEMS; ++i) {
        const int64_t n = wbase + i * 64 + lane;
        key[i] = valid[i] ? kin[n] : 0xFFFFFFFFu;
        val[i] = valid[i] ? vin[n] : 0;
      }
    }
    // per-wave ranks (match-any over the digit bits, stable: items in order, lanes in order) and wave histograms
    for (int d = tid; d < bins; d += LF_BLOCK) {
#pragma unroll
      for (int w = 0; w < LF_WAVES; ++w) s_bin[w][d] = 0;
    }
    __syncthreads();
    uint32_t rank[LF_ITEMS];
#pragma unroll
    for (int i = 0; i < LF_ITEMS; ++i) {
      const uint32_t d = (key[i] >> shift) & mask;
      uint64_t peers = __ballot(valid[i]);
      for (int b = 0; b < nbits; ++b) {
        const uint64_t bal = __ballot((d >> b) & 1u);
        peers &= ((d >> b) & 1u) ? bal : ~bal;
      }
      if (!valid[i]) peers = 0;
      const int leader = peers ? (__ffsll((unsigned long long)peers) - 1) : lane;
      uint32_t old = 0;
      if (valid[i] && lane == leader) old = atomicAdd(&s_bin[wave][d], (uint32_t)__popcll(peers));
      old = __shfl(old, leader);
      rank[i] = old + (uint32_t)__popcll(peers & lt_mask);
    }
    __syncthreads();
    for (int d = tid; d < bins; d += LF_BLOCK) {  // this tile's histogram for the other tiles of the table
      uint32_t c = 0;
#pragma unroll
      for (int w = 0; w < LF_WAVES; ++w) c += s_bin[w][d];
      hist_t[(int64_t)tile * LF_MAX_BINS + d] = c;
    }
    lf_grid_barrier(a.ctrl, ++epoch * gridDim.x);

    for (int d = tid; d < bins; d += LF_BLOCK) {
      uint32_t all = 0, before = 0;
      for (int t = 0; t < a.n_tiles; ++t) {
        const uint32_t c = hist_t[(int64_t)t * LF_MAX_BINS + d];
        all += c;
        before += (t < tile) ? c : 0u;
      }
      s_total[d] = all;
      uint32_t run = before;
#pragma unroll
      for (int w = 0; w < LF_WAVES; ++w) {
        const uint32_t c = s_bin[w][d];
        s_bin[w][d] = run;
        run += c;
      }
    }
    __syncthreads();
    {
      const int per = (bins + LF_BLOCK - 1) / LF_BLOCK;
      const int d0 = tid * per;
      uint32_t local = 0;
      for (int j = 0; j < per; ++j) local += (d0 + j < bins) ? s_total[d0 + j] : 0u;
      uint32_t incl = local;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
      }
      if (lane == 63) s_wsum[wave] = incl;
      __syncthreads();
      uint32_t woff = 0;
      for (int w = 0; w < wave; ++w) woff += s_wsum[w];
      uint32_t run = woff + incl - local;
      for (int j = 0; j < per; ++j)
        if (d0 + j < bins) {
          const uint32_t c = s_total[d0 + j];
          s_total[d0 + j] = run;
          run += c;
        }
    }
    __syncthreads();
    const bool last = pass == 2;
    uint32_t* kout = a.kbuf + ((int64_t)(pass & 1) * a.n_tables + table) * N;
    int32_t* vout = last ? a.perm + (int64_t)table * N : a.vbuf + ((int64_t)(pass & 1) * a.n_tables + table) * N;
#pragma unroll
    for (int i = 0; i < LF_ITEMS; ++i)
      if (valid[i]) {
        const uint32_t d = (key[i] >> shift) & mask;
        const uint32_t pos = s_total[d] + s_bin[wave][d] + rank[i];
        if (!last) kout[pos] = key[i];
        vout[pos] = val[i];
        if (last && a.feats) {  // the hit's features go straight to their sorted position
          const uint4* src = a.feats + (int64_t)val[i] * a.feat_vecs;
          uint4* dst = a.feats_out + ((int64_t)table * N + pos) * a.feat_vecs;
          for (int q = 0; q < a.feat_vecs; ++q) dst[q] = src[q];
        }
      }
    if (!last) lf_grid_barrier(a.ctrl, ++epoch * gridDim.x);
  }
}

extern "C" int64_t lampa_lsh_fused_workspace_bytes(int64_t n_hits, int n_tables, int n_proj) {
  if (n_hits < 0 || n_tables < 1 || n_proj < 1) return LAMPA_ERR_INVALID;
  const int64_t n_tiles = (n_hits + LF_TILE - 1) / LF_TILE > 0 ? (n_hits + LF_TILE - 1) / LF_TILE : 1;
  return lampa_align_up(sizeof(LfCtrl), 256) + lampa_align_up(n_tables * n_tiles * LF_MAX_BINS * 4, 256) +
         2 * lampa_align_up(2 * n_tables * n_hits * 4, 256);
}

// 1 when the single-launch kernel can take this event (grid fits on the chip, 16-byte feature rows), else 0.
extern "C" int lampa_lsh_fused_supported(int64_t n_hits, int n_tables, int n_proj, int dim, int64_t feat_row_bytes) {
  if (n_hits < 1 || n_tables < 1 || n_proj < 1 || n_proj > LSH_MAX_PROJ || n_tables * n_proj > LSH_MAX_COLS) return 0;
  if (dim < 1 || dim > LSH_MAX_DIM || n_hits > INT32_MAX) return 0;
  if (feat_row_bytes % 16 != 0) return 0;
  const int64_t n_tiles = (n_hits + LF_TILE - 1) / LF_TILE;
  return n_tables * n_tiles <= LF_MAX_GRID ? 1 : 0;
}

// Same outputs as lampa_lsh_bucket_sort (three radix passes), from one persistent kernel.
extern "C" int lampa_lsh_bucket_sort_fused(const float* coords, int64_t n_hits, int64_t n_valid, int dim,
                                           const float* alpha, const float* beta, int n_tables, int n_proj, float w,
                                           int32_t* ids_out, int32_t* keys_out, int32_t* meta_out, int32_t* perm_out,
                                           const void* feats, int64_t feat_row_bytes, void* feats_out, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  if (!coords || !alpha || !beta || !keys_out || !meta_out || !perm_out) return LAMPA_ERR_INVALID;
  if (n_valid < 0 || n_valid > n_hits || !(w > 0.0f)) return LAMPA_ERR_INVALID;
  if (feats && !feats_out) return LAMPA_ERR_INVALID;
  if (!lampa_lsh_fused_supported(n_hits, n_tables, n_proj, dim, feats ? feat_row_bytes : 16)) return LAMPA_ERR_UNSUPPORTED;
  if (((uintptr_t)feats | (uintptr_t)feats_out) & 15) return LAMPA_ERR_UNSUPPORTED;
  if (!workspace || workspace_bytes < lampa_lsh_fused_workspace_bytes(n_hits, n_tables, n_proj)) return LAMPA_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const int n_tiles = (int)((n_hits + LF_TILE - 1) / LF_TILE);
  char* ws = (char*)workspace;
  LfArgs a;
  a.coords = coords; a.alpha = alpha; a.beta = beta;
  a.n_hits = n_hits; a.n_valid = n_valid;
  a.dim = dim; a.n_tables = n_tables; a.n_proj = n_proj; a.n_tiles = n_tiles;
  a.inv_w = 1.0f / w;
  a.ids = ids_out; a.keys = keys_out; a.meta = meta_out; a.perm = perm_out;
  a.feats = (const uint4*)feats; a.feats_out = (uint4*)feats_out; a.feat_vecs = feats ? (int)(feat_row_bytes / 16) : 0;
  a.ctrl = (LfCtrl*)ws;
  int64_t off = lampa_align_up(sizeof(LfCtrl), 256);
  a.hist = (uint32_t*)(ws + off); off += lampa_align_up((int64_t)n_tables * n_tiles * LF_MAX_BINS * 4, 256);
  a.kbuf = (uint32_t*)(ws + off); off += lampa_align_up(2 * (int64_t)n_tables * n_hits * 4, 256);
  a.vbuf = (int32_t*)(ws + off);
  LAMPA_PROF(s, "start");
  hipLaunchKernelGGL(lf_init_kernel, dim3(1), dim3(64), 0, s, a.ctrl, n_tables * n_proj);
  LAMPA_PROF(s, "lf_init_kernel");
  if (dim == 4)
    hipLaunchKernelGGL(lf_bucket_sort_kernel<4>, dim3(n_tables * n_tiles), dim3(LF_BLOCK), 0, s, a);
  else
    hipLaunchKernelGGL(lf_bucket_sort_kernel<0>, dim3(n_tables * n_tiles), dim3(LF_BLOCK), 0, s, a);
  LAMPA_PROF(s, "lf_bucket_sort_kernel");
  return lampa_launch_status();
}

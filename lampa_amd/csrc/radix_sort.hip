// Stable segmented LSD radix sort of (32-bit key, int32 payload) pairs on gfx950.
//
// S independent segments of equal length N are sorted ascending; ties keep their input order, so the payload
// of an index sort is bit-identical to torch.sort(stable=True).indices.  Replaces the ATen sorts of the
// reference: q_hashed.argsort(dim=-1)  models/attention/hept.py:138-139, norm.argsort() and
// bk.sort(stable=True)  models/baselines/full_mamba2.py:203,207, perm.argsort(dim=1)  full_mamba2.py:678.
//
// Each pass = a histogram kernel (LDS histogram per tile of 2048 keys, written to HBM per tile), an offsets kernel
// (per digit: prefix of the tile counts over the tiles of the segment, and the digit's total) and a scatter kernel
// (scan of the digit totals, per-wave ranks through a match table in LDS, both added to the tile's offsets).  The number of
// passes is fixed by the host; the digit width of a segment is at most 11 bits. key_bits may live in device memory
// (written by the key-packing kernel) so that no host synchronisation is needed: then the host launches the worst
// case and each segment uses only the launches its keys need (see rs_digit).
#include "common.h"
#include <mutex>

#define RS_BLOCK 256
#define RS_WAVES (RS_BLOCK / 64)
#define RS_ITEMS 8
#define RS_TILE (RS_BLOCK * RS_ITEMS)
#define RS_MAX_DIGIT_BITS 11
#define RS_MAX_BINS (1 << RS_MAX_DIGIT_BITS)

enum { KEY_U32 = 0, KEY_I32 = 1, KEY_F32 = 2 };

__device__ __forceinline__ uint32_t rs_ordered(uint32_t raw, int kind) {
  if (kind == KEY_I32) return raw ^ 0x80000000u;
  if (kind == KEY_F32) {
    float f = __uint_as_float(raw);
    if (f != f) return 0xFFFFFFFFu;  // NaN last
    if (f == 0.0f) raw = 0;          // -0.0 == +0.0
    return (raw & 0x80000000u) ? ~raw : (raw | 0x80000000u);
  }
  return raw;
}

struct RsDigit {
  int shift;
  int nbits;
  bool skip;   // this launch has nothing to do for the segment
  bool first;  // this launch reads the caller's keys / payload, not the ping-pong buffers
};

// Digit of launch `pass` out of `n_passes`. With the bit count in device memory the host cannot size the passes, so
// it launches the worst case and the segment decides: only the last ceil(bits / 11) launches work, the earlier ones
// return at once and the first working one reads the original input.
__device__ __forceinline__ RsDigit rs_digit(const int32_t* bits_dev, int bits_stride, int host_bits, int seg,
                                            int pass, int n_passes) {
  int bits = bits_dev ? bits_dev[(int64_t)seg * bits_stride] : host_bits;
  bits = max(1, min(32, bits));
  int eff = n_passes;
  if (bits_dev) eff = max(1, min(n_passes, (bits + RS_MAX_DIGIT_BITS - 1) / RS_MAX_DIGIT_BITS));
  const int skipped = n_passes - eff, e = pass - skipped;
  const int width = (bits + eff - 1) / eff;
  RsDigit d;
  d.skip = e < 0;
  d.first = e == 0;
  d.shift = max(e, 0) * width;
  d.nbits = max(0, min(width, bits - d.shift));
  if (d.shift > 31) d.shift = 31;
  return d;
}

// Block -> (segment, tile) for the 1-D grids of the histogram and scatter kernels. Workgroups go to the 8 XCDs round
// robin by their linear id, and each XCD has its own L2: with 8 or more segments all tiles of a segment are given to
// one XCD, so that the scattered 4-byte writes into the segment's output range meet in one L2 and leave it as full
// lines. Fewer segments are spread over all XCDs instead. Returns false for the padding blocks of the grid.
#define RS_XCDS 8
static int rs_grid_blocks(int n_tiles, int n_segments) {
  if (n_segments < RS_XCDS) return n_tiles * n_segments;
  return RS_XCDS * ((n_segments + RS_XCDS - 1) / RS_XCDS) * n_tiles;
}
__device__ __forceinline__ bool rs_block_to_tile(int n_tiles, int n_segments, int& seg, int& tile) {
  const int b = blockIdx.x;
  if (n_segments < RS_XCDS) {
    seg = b / n_tiles;
    tile = b - seg * n_tiles;
    return true;
  }
  const int xcd = b % RS_XCDS, i = b / RS_XCDS;
  seg = xcd + RS_XCDS * (i / n_tiles);
  tile = i % n_tiles;
  return seg < n_segments;
}

// 1-D grid of rs_grid_blocks(n_tiles, S) blocks. hist [S, n_tiles, RS_MAX_BINS] (only the first 2^nbits entries of a row are used).
__global__ void __launch_bounds__(RS_BLOCK) rs_histogram_kernel(const uint32_t* __restrict__ keys_orig,
                                                               const uint2* __restrict__ pairs_buf, int64_t n,
                                                               int kind_orig, const int32_t* bits_dev, int bits_stride,
                                                               int host_bits, int pass, int n_passes, int n_tiles,
                                                               int n_segments, uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[RS_MAX_BINS];
  int seg, tile;
  if (!rs_block_to_tile(n_tiles, n_segments, seg, tile)) return;
  const RsDigit dg = rs_digit(bits_dev, bits_stride, host_bits, seg, pass, n_passes);
  if (dg.skip) return;
  const int bins = 1 << dg.nbits;
  const uint32_t mask = (uint32_t)bins - 1u;
  for (int d = threadIdx.x; d < bins; d += RS_BLOCK) s_hist[d] = 0;
  __syncthreads();
  const int64_t base = (int64_t)seg * n, first = (int64_t)tile * RS_TILE;
  // a whole tile of a 16-byte aligned segment is read 16 bytes per lane (the order inside a tile does not matter here)
  const bool wide = (n & 3) == 0 && first + RS_TILE <= n &&
                    ((dg.first ? (uintptr_t)keys_orig : (uintptr_t)pairs_buf) & 15) == 0;
  if (wide && dg.first) {
    const uint4* src = reinterpret_cast<const uint4*>(keys_orig + base + first);
    uint4 v[RS_ITEMS / 4];
#pragma unroll
    for (int i = 0; i < RS_ITEMS / 4; ++i) v[i] = src[i * RS_BLOCK + threadIdx.x];
#pragma unroll
    for (int i = 0; i < RS_ITEMS / 4; ++i) {
      atomicAdd(&s_hist[(rs_ordered(v[i].x, kind_orig) >> dg.shift) & mask], 1u);
      atomicAdd(&s_hist[(rs_ordered(v[i].y, kind_orig) >> dg.shift) & mask], 1u);
      atomicAdd(&s_hist[(rs_ordered(v[i].z, kind_orig) >> dg.shift) & mask], 1u);
      atomicAdd(&s_hist[(rs_ordered(v[i].w, kind_orig) >> dg.shift) & mask], 1u);
    }
  } else if (wide) {
    const uint4* src = reinterpret_cast<const uint4*>(pairs_buf + base + first);  // two (key, payload) pairs
    uint4 v[RS_ITEMS / 2];
#pragma unroll
    for (int i = 0; i < RS_ITEMS / 2; ++i) v[i] = src[i * RS_BLOCK + threadIdx.x];
#pragma unroll
    for (int i = 0; i < RS_ITEMS / 2; ++i) {
      atomicAdd(&s_hist[(v[i].x >> dg.shift) & mask], 1u);
      atomicAdd(&s_hist[(v[i].z >> dg.shift) & mask], 1u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
      const int64_t idx = first + i * RS_BLOCK + threadIdx.x;
      if (idx < n) {
        // the ping-pong buffers hold (ordered key, payload) pairs
        const uint32_t k = dg.first ? rs_ordered(keys_orig[base + idx], kind_orig) : pairs_buf[base + idx].x;
        atomicAdd(&s_hist[(k >> dg.shift) & mask], 1u);
      }
    }
  }
  __syncthreads();
  uint32_t* out = hist + ((int64_t)seg * n_tiles + tile) * RS_MAX_BINS;
  for (int d = threadIdx.x; d < bins; d += RS_BLOCK) out[d] = s_hist[d];
}

// grid (RS_MAX_BINS / RS_BLOCK, S). One thread per digit: exclusive prefix of the digit's counts over the tiles of the
// segment, in place (hist[tile][d] <- keys with digit d in earlier tiles), and the digit's total to tot[seg][d].
// The scan of the totals over the digits is left to the scatter kernel, so this kernel is one short chain of
// independent, coalesced loads per thread.
__global__ void __launch_bounds__(RS_BLOCK) rs_offsets_kernel(const int32_t* bits_dev, int bits_stride, int host_bits,
                                                             int pass, int n_passes, int n_tiles,
                                                             uint32_t* __restrict__ hist, uint32_t* __restrict__ tot) {
  const int seg = blockIdx.y;
  const RsDigit dg = rs_digit(bits_dev, bits_stride, host_bits, seg, pass, n_passes);
  if (dg.skip) return;
  const int d = blockIdx.x * RS_BLOCK + threadIdx.x;
  if (d >= (1 << dg.nbits)) return;
  uint32_t* hcol = hist + (int64_t)seg * n_tiles * RS_MAX_BINS + d;
  uint32_t run = 0;
  // 32 tiles at a time, every load requested before the first is used: a segment of 60 000 keys (30 tiles) is one
  // round trip to memory instead of four
  constexpr int OB = 32;
  for (int t0 = 0; t0 < n_tiles; t0 += OB) {
    uint32_t c[OB];
#pragma unroll
    for (int u = 0; u < OB; ++u) c[u] = hcol[(int64_t)min(t0 + u, n_tiles - 1) * RS_MAX_BINS];
#pragma unroll
    for (int u = 0; u < OB; ++u)
      if (t0 + u < n_tiles) {
        hcol[(int64_t)(t0 + u) * RS_MAX_BINS] = run;
        run += c[u];
      }
  }
  tot[(int64_t)seg * RS_MAX_BINS + d] = run;
}

// 1-D grid of rs_grid_blocks(n_tiles, S) blocks. Element order inside a tile: wave w owns [w*512, (w+1)*512), item i
// of lane l is at w*512 + i*64 + l, so (item, lane) order within a wave is input order and the scatter is stable.
//
// A key's output position = (keys of the segment with a smaller digit) + (keys with its digit in earlier tiles)
// [s_base, 32 bits per digit] + (keys with its digit in earlier waves of the tile) [s_cnt, 16 bits per wave and digit:
// a wave holds 512 keys, a tile 2048] + its rank among the wave's keys with its digit. Ranks: lanes of a wave with the
// same digit find each other through two small tables of the wave in LDS -- every lane writes its number to tab[d] and
// reads back the one that stayed (the group's speaker), sets its bit in the speaker's 64-bit word, reads the word
// (= the group) and clears it; the speaker adds the group's size to the wave's 16-bit count of the digit and hands the
// old count to the group. The LDS executes the instructions of one wave in order, so these steps need no waits between
// them; relaxed atomic accesses keep the compiler from forwarding a lane's own store to its load. A key beyond the
// segment's end carries the largest digit and comes last in (wave, item, lane) order: it changes no rank and only
// counts that no real key's position depends on.
__global__ void __launch_bounds__(RS_BLOCK) rs_scatter_kernel(const uint32_t* __restrict__ keys_orig,
                                                             const int32_t* __restrict__ vals_orig,
                                                             const uint2* __restrict__ pairs_in, int64_t n,
                                                             int kind_orig, const int32_t* bits_dev, int bits_stride,
                                                             int host_bits, int pass, int n_passes, int n_tiles,
                                                             int n_segments, const uint32_t* __restrict__ hist,
                                                             const uint32_t* __restrict__ tot,
                                                             uint2* __restrict__ pairs_out,
                                                             int32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_base[RS_MAX_BINS];
  __shared__ uint32_t s_cnt[RS_WAVES][RS_MAX_BINS / 2];  // two 16-bit counts per word: digits 2j (low half) and 2j + 1
  __shared__ uint8_t s_tab[RS_WAVES][RS_MAX_BINS];
  __shared__ unsigned long long s_grp[RS_WAVES][64];
  __shared__ uint32_t s_wsum[RS_WAVES];
  int seg, tile;
  if (!rs_block_to_tile(n_tiles, n_segments, seg, tile)) return;
  const int wave = threadIdx.x >> 6, lane = lane_id();
  const RsDigit dg = rs_digit(bits_dev, bits_stride, host_bits, seg, pass, n_passes);
  if (dg.skip) return;
  const int bins = 1 << dg.nbits;
  const uint32_t mask = (uint32_t)bins - 1u;

  // digit totals of the segment: thread t owns digits 8t .. 8t+7; entries beyond the digit range are stale
  constexpr int DPT = RS_MAX_BINS / RS_BLOCK;
  uint32_t dt[DPT];
  {
    const uint32_t* trow = tot + (int64_t)seg * RS_MAX_BINS + threadIdx.x * DPT;
    const bool live = (int)threadIdx.x * DPT < bins;
    const uint4 a = live ? *reinterpret_cast<const uint4*>(trow) : make_uint4(0, 0, 0, 0);
    const uint4 b = live ? *reinterpret_cast<const uint4*>(trow + 4) : make_uint4(0, 0, 0, 0);
    dt[0] = a.x; dt[1] = a.y; dt[2] = a.z; dt[3] = a.w; dt[4] = b.x; dt[5] = b.y; dt[6] = b.z; dt[7] = b.w;
#pragma unroll
    for (int j = 0; j < DPT; ++j)
      if ((int)threadIdx.x * DPT + j >= bins) dt[j] = 0;
  }

  const int64_t sbase = (int64_t)seg * n;
  const int64_t wbase = (int64_t)tile * RS_TILE + wave * (RS_TILE / RS_WAVES);
  uint32_t key[RS_ITEMS], rank[RS_ITEMS];
  int32_t val[RS_ITEMS];
  bool valid[RS_ITEMS];
  if (dg.first) {  // the caller's keys and payload (or the position): every load is requested before the key mapping
                   // (whose branches on the key kind would otherwise sit between the loads and wait for each of them)
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
      const int64_t idx = wbase + i * 64 + lane;
      valid[i] = idx < n;
      key[i] = valid[i] ? keys_orig[sbase + idx] : 0xFFFFFFFFu;
      val[i] = (int32_t)idx;
    }
    if (vals_orig) {
#pragma unroll
      for (int i = 0; i < RS_ITEMS; ++i) val[i] = valid[i] ? vals_orig[sbase + wbase + i * 64 + lane] : 0;
    }
    if (kind_orig != KEY_U32) {
#pragma unroll
      for (int i = 0; i < RS_ITEMS; ++i) key[i] = valid[i] ? rs_ordered(key[i], kind_orig) : 0xFFFFFFFFu;
    }
  } else {  // (ordered key, payload) pairs of the previous pass
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
      const int64_t idx = wbase + i * 64 + lane;
      valid[i] = idx < n;
      const uint2 kv = valid[i] ? pairs_in[sbase + idx] : make_uint2(0xFFFFFFFFu, 0u);
      key[i] = kv.x;
      val[i] = (int32_t)kv.y;
    }
  }
  // this tile's offsets within each digit (written by rs_offsets_kernel), for the digit pairs of the words this thread
  // turns into bases after the ranking: words t, t + 256, ...
  constexpr int WPT = RS_MAX_BINS / 2 / RS_BLOCK;
  const uint32_t* hrow = hist + ((int64_t)seg * n_tiles + tile) * RS_MAX_BINS;
  uint2 hoff[WPT];
#pragma unroll
  for (int j = 0; j < WPT; ++j) {
    const int w2 = threadIdx.x + j * RS_BLOCK;
    hoff[j] = 2 * w2 < bins ? *reinterpret_cast<const uint2*>(hrow + 2 * w2) : make_uint2(0u, 0u);
  }

  // exclusive scan of the digit totals over the block -> s_base; the waves' counts start at zero
  {
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < DPT; ++j) mine += dt[j];
    uint32_t incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) s_wsum[wave] = incl;
    for (int w2 = threadIdx.x; 2 * w2 < bins; w2 += RS_BLOCK) {
#pragma unroll
      for (int w = 0; w < RS_WAVES; ++w) s_cnt[w][w2] = 0;
    }
    s_grp[wave][lane] = 0ull;
    __syncthreads();
    uint32_t run = incl - mine;
#pragma unroll
    for (int w = 0; w < RS_WAVES; ++w) run += w < wave ? s_wsum[w] : 0u;
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
      if ((int)threadIdx.x * DPT + j < bins) s_base[threadIdx.x * DPT + j] = run;
      run += dt[j];
    }
  }

  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  uint32_t dd[RS_ITEMS];
  {
    uint8_t* tab = s_tab[wave];
    unsigned long long* grp = s_grp[wave];
    uint32_t* cnt = s_cnt[wave];
    const unsigned long long bit = 1ull << lane;
    uint32_t spk[RS_ITEMS], old[RS_ITEMS];
    uint64_t peers[RS_ITEMS];
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
      dd[i] = (key[i] >> dg.shift) & mask;
      __hip_atomic_store(&tab[dd[i]], (uint8_t)lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
      spk[i] = __hip_atomic_load(&tab[dd[i]], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    }
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
      __hip_atomic_fetch_or(&grp[spk[i]], bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
      peers[i] = __hip_atomic_load(&grp[spk[i]], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
      __hip_atomic_store(&grp[spk[i]], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    }
    // in item order: the value a speaker gets back is the number of the wave's earlier keys with this digit
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
      const int sh = 16 * (dd[i] & 1u);
      old[i] = 0;
      if ((uint32_t)lane == spk[i])
        old[i] = (atomicAdd(&cnt[dd[i] >> 1], (uint32_t)__popcll(peers[i]) << sh) >> sh) & 0xFFFFu;
    }
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i)
      rank[i] = (uint32_t)__shfl((int)old[i], (int)spk[i]) + (uint32_t)__popcll(peers[i] & lt_mask);
  }
  __syncthreads();

  // the waves' counts become the keys of the tile's earlier waves with the digit (both halves of a word at once: no
  // sum exceeds the 2048 keys of a tile); the tile's offset joins the digit's base
#pragma unroll
  for (int j = 0; j < WPT; ++j) {
    const int w2 = threadIdx.x + j * RS_BLOCK;
    if (2 * w2 < bins) {
      uint32_t run = 0;
#pragma unroll
      for (int w = 0; w < RS_WAVES; ++w) {
        const uint32_t c = s_cnt[w][w2];
        s_cnt[w][w2] = run;
        run += c;
      }
      s_base[2 * w2] += hoff[j].x;
      if (2 * w2 + 1 < bins) s_base[2 * w2 + 1] += hoff[j].y;
    }
  }
  __syncthreads();

  // one scattered store per key: an 8-byte (key, payload) pair between passes, the payload alone after the last
  const uint16_t* wpre = reinterpret_cast<const uint16_t*>(s_cnt[wave]);
#pragma unroll
  for (int i = 0; i < RS_ITEMS; ++i) {
    if (valid[i]) {
      const int64_t pos = sbase + s_base[dd[i]] + wpre[dd[i]] + rank[i];
      if (pairs_out) pairs_out[pos] = make_uint2(key[i], (uint32_t)val[i]);
      else vals_out[pos] = val[i];
    }
  }
}

extern "C" int64_t lampa_sort_workspace_bytes(int n_segments, int64_t n) {
  if (n_segments < 1 || n < 0) return LAMPA_ERR_INVALID;
  const int64_t n_tiles = (n + RS_TILE - 1) / RS_TILE > 0 ? (n + RS_TILE - 1) / RS_TILE : 1;
  const int64_t pairs = lampa_align_up((int64_t)n_segments * n * 4, 256);
  const int64_t hist = lampa_align_up((int64_t)n_segments * (n_tiles + 1) * RS_MAX_BINS * 4, 256);  // + digit totals
  return 4 * pairs + hist;
}

// Enqueues the passes of one sort; `workspace` holds lampa_sort_workspace_bytes(n_segments, n) bytes (checked by the
// callers). Nothing in it has to start at zero: every histogram row and total that a pass reads is written by that pass.
static int rs_sort_enqueue(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments, int64_t n,
                           int key_bits, const int32_t* key_bits_dev, int key_bits_stride, int n_passes,
                           int32_t* vals_out, void* workspace, hipStream_t s) {
  const int n_tiles = (int)((n + RS_TILE - 1) / RS_TILE);
  const int64_t pairs = lampa_align_up((int64_t)n_segments * n * 4, 256);
  char* ws = (char*)workspace;
  uint2* pbuf[2] = {(uint2*)ws, (uint2*)(ws + 2 * pairs)};
  uint32_t* hist = (uint32_t*)(ws + 4 * pairs);
  uint32_t* tot = hist + (int64_t)n_segments * n_tiles * RS_MAX_BINS;
  const dim3 grid(rs_grid_blocks(n_tiles, n_segments)), block(RS_BLOCK);
  LAMPA_PROF(s, "start");
  for (int p = 0; p < n_passes; ++p) {
    const uint2* pairs_in = pbuf[(p + 1) & 1];  // written by the previous launch (never read by the first)
    const bool last = p == n_passes - 1;
    hipLaunchKernelGGL(rs_histogram_kernel, grid, block, 0, s, (const uint32_t*)keys_in, pairs_in, n, key_kind,
                       key_bits_dev, key_bits_stride, key_bits, p, n_passes, n_tiles, n_segments, hist);
    LAMPA_PROF(s, "rs_histogram_kernel");
    hipLaunchKernelGGL(rs_offsets_kernel, dim3(RS_MAX_BINS / RS_BLOCK, n_segments), block, 0, s, key_bits_dev,
                       key_bits_stride, key_bits, p, n_passes, n_tiles, hist, tot);
    LAMPA_PROF(s, "rs_offsets_kernel");
    hipLaunchKernelGGL(rs_scatter_kernel, grid, block, 0, s, (const uint32_t*)keys_in, vals_in, pairs_in, n,
                       key_kind, key_bits_dev, key_bits_stride, key_bits, p, n_passes, n_tiles, n_segments, hist, tot,
                       last ? (uint2*)nullptr : pbuf[p & 1], vals_out);
    LAMPA_PROF(s, "rs_scatter_kernel");
  }
  return lampa_launch_status();
}

// Argument checks shared by the two entry points; resolves the automatic pass count.
static int rs_check_args(const void* keys_in, int key_kind, int n_segments, int64_t n, int& key_bits,
                         const int32_t*& key_bits_dev, int& n_passes, const int32_t* vals_out) {
  if (!keys_in || !vals_out || n_segments < 1 || n < 0 || n > INT32_MAX) return LAMPA_ERR_INVALID;
  if (key_kind != KEY_U32 && key_kind != KEY_I32 && key_kind != KEY_F32) return LAMPA_ERR_INVALID;
  if (key_kind != KEY_U32) { key_bits = 32; key_bits_dev = nullptr; }
  if (!key_bits_dev && (key_bits < 1 || key_bits > 32)) return LAMPA_ERR_INVALID;
  const int max_bits = key_bits_dev ? 32 : key_bits;
  if (n_passes == 0) n_passes = key_bits_dev ? 3 : (max_bits + RS_MAX_DIGIT_BITS - 1) / RS_MAX_DIGIT_BITS;
  if (n_passes < 1 || n_passes > 4 || (max_bits + n_passes - 1) / n_passes > RS_MAX_DIGIT_BITS)
    return LAMPA_ERR_INVALID;
  return LAMPA_OK;
}

// keys_in [S, n] (raw 32-bit keys of kind key_kind), vals_in [S, n] or NULL (payload = position), vals_out [S, n].
// key_bits_dev (nullable): per-segment number of significant key bits in device memory, element s at
// key_bits_dev[s * key_bits_stride]; otherwise key_bits (host, 1..32) applies to all segments. Signed and float
// keys always need 32 bits. n_passes in 1..4 with ceil(bits / n_passes) <= 11; 0 picks ceil(key_bits / 11)
// for host bits and 3 for device bits.
extern "C" int lampa_sort_pairs(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments, int64_t n,
                                int key_bits, const int32_t* key_bits_dev, int key_bits_stride, int n_passes,
                                int32_t* vals_out, void* workspace, int64_t workspace_bytes, void* stream) {
  const int rc = rs_check_args(keys_in, key_kind, n_segments, n, key_bits, key_bits_dev, n_passes, vals_out);
  if (rc != LAMPA_OK) return rc;
  if (!workspace || workspace_bytes < lampa_sort_workspace_bytes(n_segments, n)) return LAMPA_ERR_WORKSPACE;
  if (n == 0) return LAMPA_OK;
  return rs_sort_enqueue(keys_in, key_kind, vals_in, n_segments, n, key_bits, key_bits_dev, key_bits_stride, n_passes,
                         vals_out, workspace, (hipStream_t)stream);
}

// ---- the sort for callers that cannot allocate -------------------------------------------------------------------
// Same sort, same kernels, but the ping-pong buffers and histograms live in a fixed array of device memory that is
// part of the library image (every GPU the library runs on holds its own copy until the process ends). The array's
// name is only a host-side handle: its device address is looked up once per device with hipGetSymbolAddress and that
// pointer is what the kernels receive.
#define RS_STATIC_SCRATCH_BYTES (8 << 20)
#define RS_MAX_DEVICES 64
static __device__ __align__(256) unsigned char rs_static_scratch[RS_STATIC_SCRATCH_BYTES];
static void* rs_scratch_ptr[RS_MAX_DEVICES];
static std::mutex rs_scratch_lock;

// Device address of the current device's copy of the array (nullptr on failure).
static void* rs_static_scratch_address() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= RS_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> hold(rs_scratch_lock);
  if (!rs_scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(rs_static_scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    rs_scratch_ptr[dev] = p;
  }
  return rs_scratch_ptr[dev];
}

extern "C" int64_t lampa_sort_pairs_static_max_bytes(void) { return RS_STATIC_SCRATCH_BYTES; }

extern "C" int lampa_sort_pairs_static(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments,
                                       int64_t n, int key_bits, const int32_t* key_bits_dev, int key_bits_stride,
                                       int n_passes, int32_t* vals_out, void* stream) {
  const int rc = rs_check_args(keys_in, key_kind, n_segments, n, key_bits, key_bits_dev, n_passes, vals_out);
  if (rc != LAMPA_OK) return rc;
  if (lampa_sort_workspace_bytes(n_segments, n) > RS_STATIC_SCRATCH_BYTES) return LAMPA_ERR_WORKSPACE;
  if (n == 0) return LAMPA_OK;
  void* scratch = rs_static_scratch_address();
  if (!scratch) return LAMPA_ERR_LAUNCH;
  return rs_sort_enqueue(keys_in, key_kind, vals_in, n_segments, n, key_bits, key_bits_dev, key_bits_stride, n_passes,
                         vals_out, scratch, (hipStream_t)stream);
}

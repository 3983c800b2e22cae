// Stable segmented LSD radix sort of (32-bit key, int32 payload) pairs on gfx950.
//
// S independent segments of equal length N are sorted ascending; ties keep their input order, so the payload
// of an index sort is bit-identical to torch.sort(stable=True).indices.  Replaces the ATen sorts of the
// reference: q_hashed.argsort(dim=-1)  models/attention/hept.py:138-139, norm.argsort() and
// bk.sort(stable=True)  models/baselines/full_mamba2.py:203,207, perm.argsort(dim=1)  full_mamba2.py:678.
//
// Each pass = a histogram kernel (LDS histogram per tile of 2048 keys, written to HBM per tile), an offsets kernel
// (per-tile histograms -> output offsets, one block per segment) and a scatter kernel (per-wave ranks from wavefront
// ballots added to the tile's offsets).  The number of
// passes is fixed by the host; the digit width of a segment is at most 11 bits. key_bits may live in device memory
// (written by the key-packing kernel) so that no host synchronisation is needed: then the host launches the worst
// case and each segment uses only the launches its keys need (see rs_digit).
#include "common.h"

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

// grid (n_tiles, S). hist [S, n_tiles, RS_MAX_BINS] (only the first 2^nbits entries of a row are used).
__global__ void __launch_bounds__(RS_BLOCK) rs_histogram_kernel(const uint32_t* __restrict__ keys_orig,
                                                               const uint32_t* __restrict__ keys_buf, int64_t n,
                                                               int kind_orig, const int32_t* bits_dev, int bits_stride,
                                                               int host_bits, int pass, int n_passes,
                                                               uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[RS_MAX_BINS];
  const int seg = blockIdx.y, tile = blockIdx.x, n_tiles = gridDim.x;
  const RsDigit dg = rs_digit(bits_dev, bits_stride, host_bits, seg, pass, n_passes);
  if (dg.skip) return;
  const uint32_t* keys = dg.first ? keys_orig : keys_buf;
  const int kind = dg.first ? kind_orig : KEY_U32;  // the buffers hold ordered keys
  const int bins = 1 << dg.nbits;
  const uint32_t mask = (uint32_t)bins - 1u;
  for (int d = threadIdx.x; d < bins; d += RS_BLOCK) s_hist[d] = 0;
  __syncthreads();
  const uint32_t* kseg = keys + (int64_t)seg * n;
  const int64_t base = (int64_t)tile * RS_TILE;
#pragma unroll
  for (int i = 0; i < RS_ITEMS; ++i) {
    const int64_t idx = base + i * RS_BLOCK + threadIdx.x;
    if (idx < n) atomicAdd(&s_hist[(rs_ordered(kseg[idx], kind) >> dg.shift) & mask], 1u);
  }
  __syncthreads();
  uint32_t* out = hist + ((int64_t)seg * n_tiles + tile) * RS_MAX_BINS;
  for (int d = threadIdx.x; d < bins; d += RS_BLOCK) out[d] = s_hist[d];
}

// grid (S), 1024 threads. Turns the per-tile histograms of a segment into output offsets, in place:
// hist[tile][d] <- (keys of the segment with a smaller digit) + (keys with digit d in earlier tiles).
// One pass over the [n_tiles, bins] counts per segment; without it every tile of the scatter would have to re-read
// all of them (n_tiles times the traffic and a chain of dependent loads per tile).
#define RS_OFFS_BLOCK 1024
__global__ void __launch_bounds__(RS_OFFS_BLOCK) rs_offsets_kernel(const int32_t* bits_dev, int bits_stride, int host_bits,
                                                                  int pass, int n_passes, int n_tiles,
                                                                  uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_wsum[RS_OFFS_BLOCK / 64];
  const int seg = blockIdx.x;
  const RsDigit dg = rs_digit(bits_dev, bits_stride, host_bits, seg, pass, n_passes);
  if (dg.skip) return;
  const int bins = 1 << dg.nbits;
  uint32_t* hseg = hist + (int64_t)seg * n_tiles * RS_MAX_BINS;
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  // each thread owns digits d0 = tid and d1 = tid + 1024 (bins <= 2048): exclusive prefix over the tiles
  uint32_t tot[2] = {0, 0};
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int d = threadIdx.x + h * RS_OFFS_BLOCK;
    if (d < bins) {
      uint32_t run = 0;
      for (int t0 = 0; t0 < n_tiles; t0 += 8) {
        uint32_t c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = hseg[(int64_t)min(t0 + u, n_tiles - 1) * RS_MAX_BINS + d];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (t0 + u < n_tiles) {
            hseg[(int64_t)(t0 + u) * RS_MAX_BINS + d] = run;
            run += c[u];
          }
      }
      tot[h] = run;
    }
  }
  // exclusive scan of the digit totals over d = 0 .. bins-1 (digit order: first all d0 of the block, then all d1)
  uint32_t base[2];
  uint32_t carry = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint32_t incl = tot[h];
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    __syncthreads();
    if (lane == 63) s_wsum[wave] = incl;
    __syncthreads();
    uint32_t woff = 0, all = 0;
    for (int w = 0; w < RS_OFFS_BLOCK / 64; ++w) {
      const uint32_t v = s_wsum[w];
      woff += w < wave ? v : 0u;
      all += v;
    }
    base[h] = carry + woff + incl - tot[h];
    carry += all;
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int d = threadIdx.x + h * RS_OFFS_BLOCK;
    if (d < bins)
      for (int t = 0; t < n_tiles; ++t) hseg[(int64_t)t * RS_MAX_BINS + d] += base[h];
  }
}

// grid (n_tiles, S). Element order inside a tile: wave w owns [w*512, (w+1)*512), item i of lane l is at
// w*512 + i*64 + l, so (item, lane) order within a wave is input order and the scatter is stable.
__global__ void __launch_bounds__(RS_BLOCK) rs_scatter_kernel(const uint32_t* __restrict__ keys_orig,
                                                             const int32_t* __restrict__ vals_orig,
                                                             const uint32_t* __restrict__ keys_buf,
                                                             const int32_t* __restrict__ vals_buf, int64_t n,
                                                             int kind_orig, const int32_t* bits_dev, int bits_stride,
                                                             int host_bits, int pass, int n_passes,
                                                             const uint32_t* __restrict__ hist,
                                                             uint32_t* __restrict__ keys_out,
                                                             int32_t* __restrict__ vals_out) {
  __shared__ uint32_t s_bin[RS_WAVES][RS_MAX_BINS];  // per-wave counts, then per-wave output bases
  const int seg = blockIdx.y, tile = blockIdx.x, n_tiles = gridDim.x;
  const int wave = threadIdx.x >> 6, lane = lane_id();
  const RsDigit dg = rs_digit(bits_dev, bits_stride, host_bits, seg, pass, n_passes);
  if (dg.skip) return;
  const uint32_t* keys_in = dg.first ? keys_orig : keys_buf;
  const int32_t* vals_in = dg.first ? vals_orig : vals_buf;
  const int kind = dg.first ? kind_orig : KEY_U32;
  const int bins = 1 << dg.nbits;
  const uint32_t mask = (uint32_t)bins - 1u;

  for (int d = threadIdx.x; d < bins; d += RS_BLOCK) {
#pragma unroll
    for (int w = 0; w < RS_WAVES; ++w) s_bin[w][d] = 0;
  }
  __syncthreads();

  const uint32_t* kseg = keys_in + (int64_t)seg * n;
  const int32_t* vseg = vals_in ? vals_in + (int64_t)seg * n : nullptr;
  const int64_t wbase = (int64_t)tile * RS_TILE + wave * (RS_TILE / RS_WAVES);
  uint32_t key[RS_ITEMS], rank[RS_ITEMS];
  int32_t val[RS_ITEMS];
  bool valid[RS_ITEMS];
#pragma unroll
  for (int i = 0; i < RS_ITEMS; ++i) {
    const int64_t idx = wbase + i * 64 + lane;
    valid[i] = idx < n;
    key[i] = valid[i] ? rs_ordered(kseg[idx], kind) : 0xFFFFFFFFu;
    val[i] = valid[i] ? (vseg ? vseg[idx] : (int32_t)idx) : 0;
  }
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int i = 0; i < RS_ITEMS; ++i) {
    const uint32_t d = (key[i] >> dg.shift) & mask;
    uint64_t peers = __ballot(valid[i]);
    for (int b = 0; b < dg.nbits; ++b) {
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

  // output base of every digit for this tile (rs_offsets_kernel), then of every wave of the tile
  const uint32_t* hrow = hist + ((int64_t)seg * n_tiles + tile) * RS_MAX_BINS;
  for (int d = threadIdx.x; d < bins; d += RS_BLOCK) {
    uint32_t run = hrow[d];
#pragma unroll
    for (int w = 0; w < RS_WAVES; ++w) {
      const uint32_t c = s_bin[w][d];
      s_bin[w][d] = run;
      run += c;
    }
  }
  __syncthreads();

  uint32_t* kout = keys_out ? keys_out + (int64_t)seg * n : nullptr;
  int32_t* vout = vals_out + (int64_t)seg * n;
#pragma unroll
  for (int i = 0; i < RS_ITEMS; ++i) {
    if (valid[i]) {
      const uint32_t d = (key[i] >> dg.shift) & mask;
      const uint32_t pos = s_bin[wave][d] + rank[i];
      if (kout) kout[pos] = key[i];
      vout[pos] = val[i];
    }
  }
}

extern "C" int64_t lampa_sort_workspace_bytes(int n_segments, int64_t n) {
  if (n_segments < 1 || n < 0) return LAMPA_ERR_INVALID;
  const int64_t n_tiles = (n + RS_TILE - 1) / RS_TILE > 0 ? (n + RS_TILE - 1) / RS_TILE : 1;
  const int64_t pairs = lampa_align_up((int64_t)n_segments * n * 4, 256);
  const int64_t hist = lampa_align_up((int64_t)n_segments * n_tiles * RS_MAX_BINS * 4, 256);
  return 4 * pairs + hist;
}

// keys_in [S, n] (raw 32-bit keys of kind key_kind), vals_in [S, n] or NULL (payload = position), vals_out [S, n].
// key_bits_dev (nullable): per-segment number of significant key bits in device memory, element s at
// key_bits_dev[s * key_bits_stride]; otherwise key_bits (host, 1..32) applies to all segments. Signed and float
// keys always need 32 bits. n_passes in 1..4 with ceil(bits / n_passes) <= 11; 0 picks ceil(key_bits / 11)
// for host bits and 3 for device bits.
extern "C" int lampa_sort_pairs(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments, int64_t n,
                                int key_bits, const int32_t* key_bits_dev, int key_bits_stride, int n_passes,
                                int32_t* vals_out, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!keys_in || !vals_out || n_segments < 1 || n < 0 || n > INT32_MAX) return LAMPA_ERR_INVALID;
  if (key_kind != KEY_U32 && key_kind != KEY_I32 && key_kind != KEY_F32) return LAMPA_ERR_INVALID;
  if (key_kind != KEY_U32) { key_bits = 32; key_bits_dev = nullptr; }
  if (!key_bits_dev && (key_bits < 1 || key_bits > 32)) return LAMPA_ERR_INVALID;
  const int max_bits = key_bits_dev ? 32 : key_bits;
  if (n_passes == 0) n_passes = key_bits_dev ? 3 : (max_bits + RS_MAX_DIGIT_BITS - 1) / RS_MAX_DIGIT_BITS;
  if (n_passes < 1 || n_passes > 4 || (max_bits + n_passes - 1) / n_passes > RS_MAX_DIGIT_BITS)
    return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < lampa_sort_workspace_bytes(n_segments, n)) return LAMPA_ERR_WORKSPACE;
  if (n == 0) return LAMPA_OK;
  hipStream_t s = (hipStream_t)stream;
  const int n_tiles = (int)((n + RS_TILE - 1) / RS_TILE);
  const int64_t pairs = lampa_align_up((int64_t)n_segments * n * 4, 256);
  char* ws = (char*)workspace;
  uint32_t* kbuf[2] = {(uint32_t*)ws, (uint32_t*)(ws + pairs)};
  int32_t* vbuf[2] = {(int32_t*)(ws + 2 * pairs), (int32_t*)(ws + 3 * pairs)};
  uint32_t* hist = (uint32_t*)(ws + 4 * pairs);
  const dim3 grid(n_tiles, n_segments), block(RS_BLOCK);
  LAMPA_PROF(s, "start");
  for (int p = 0; p < n_passes; ++p) {
    const uint32_t* kbuf_in = p == 0 ? (const uint32_t*)keys_in : kbuf[(p - 1) & 1];
    const int32_t* vbuf_in = p == 0 ? vals_in : vbuf[(p - 1) & 1];
    const bool last = p == n_passes - 1;
    hipLaunchKernelGGL(rs_histogram_kernel, grid, block, 0, s, (const uint32_t*)keys_in, kbuf_in, n, key_kind,
                       key_bits_dev, key_bits_stride, key_bits, p, n_passes, hist);
    LAMPA_PROF(s, "rs_histogram_kernel");
    hipLaunchKernelGGL(rs_offsets_kernel, dim3(n_segments), dim3(RS_OFFS_BLOCK), 0, s, key_bits_dev, key_bits_stride,
                       key_bits, p, n_passes, n_tiles, hist);
    LAMPA_PROF(s, "rs_offsets_kernel");
    hipLaunchKernelGGL(rs_scatter_kernel, grid, block, 0, s, (const uint32_t*)keys_in, vals_in, kbuf_in, vbuf_in, n,
                       key_kind, key_bits_dev, key_bits_stride, key_bits, p, n_passes, hist,
                       last ? (uint32_t*)nullptr : kbuf[p & 1], last ? vals_out : vbuf[p & 1]);
    LAMPA_PROF(s, "rs_scatter_kernel");
  }
  return lampa_launch_status();
}

// The whole E2LSH bucketing stage (hash -> key ranges -> packed keys -> stable radix sort -> feature gather) of one
// event, or of a few, in ONE kernel launch on gfx950.
//
// Why one kernel: for one event of 60 000 hits every step is a few microseconds of work, and a dependent kernel
// launch costs about as much as the step itself. Here the tiles of a segment (a table of an event: its own key
// ranges, its own sort) hand their results to each other inside the kernel instead, and a segment's keys go from the
// packing step into the first sort pass in registers. Everything that is handed over moves through device-scope relaxed
// atomic stores and loads: such a store is written through, such a load never reads a CU's L1. Small values (min / max
// partials, digit counts, prefixes, totals) are 64-bit words that carry a tag of the launch and the step, and the reader
// polls the word itself (lf_put / lf_get): one trip to memory per exchange. The scattered (key, payload) pairs and the
// permutation have no room for a tag: after each radix pass's scatter there is a barrier over the segment's tiles (a
// flag per tile, raised after the tile's stores have completed; two to four microseconds). No fence is used: on this
// GPU a device-scope release writes back a whole L2 and an acquire invalidates one, several microseconds each
// (measured), which is more than a step costs.
//
// Every tile of every segment of the call is a workgroup, and all of them must be on the GPU at once (a tile waits
// for the other tiles of its segment): the launcher checks the grid against what the GPU holds and otherwise leaves
// the call to the separate kernels, which are the better form for large batches anyway (bandwidth, not latency).
// Every wait is bounded; a tile whose wait runs out marks the segment's meta row (overflow field, bit 1) and goes on
// with what it has, with every store kept in range.
//
// Replaces (reference chengjiang123/Lampa), fused: E2LSH.forward  models/model_utils/hash_utils.py:368-371, the hash
// range of lsh_mapping  hash_utils.py:334-340, the mixed-radix key of get_geo_shift  models/attention/hept.py:79-88,
// q_hashed.argsort(dim=-1)  hept.py:138-139 and sort_to_buckets  hept.py:9-14. Same arithmetic contract as
// lsh_hash.hip (explicit fmaf chain, floorf, saturation) and the same stable order as radix_sort.hip.
#include "lsh_device.h"
#include <atomic>
#include <chrono>
#include <mutex>

#define LF_MAX_DIGIT_BITS 11
#define LF_MAX_BINS (1 << LF_MAX_DIGIT_BITS)
#define LF_SPIN_LIMIT (1 << 22)
#define LF_PARTIAL_STRIDE (2 * LSH_MAX_PROJ)

struct LshFusedArgs {
  const float* coords; int64_t n_hits; int64_t n_valid; const int32_t* n_valid_dev; int dim;
  const float* alpha; const float* beta; int n_tables; int n_proj; float inv_w;
  int32_t* ids; int32_t* keys; int32_t* meta; int32_t* perm;
  const char* feats; int vec_per_row; char* feats_out;   // rows of vec_per_row 16-byte pieces
  int n_events; int n_tiles;
  uint64_t* flags; uint64_t* partial; uint64_t* rows; uint64_t* totals; uint2* pairs0; uint2* pairs1;
  uint32_t* failed;     // one word per segment: holds `gen` once a tile of the segment has given up a wait in this call
  uint32_t gen;
  int spin_limit;       // polls a tile spends in one wait before it gives up
};

__device__ __forceinline__ void lf_flag_store(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t lf_flag_load(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Data that tiles exchange inside the kernel goes through device-scope relaxed atomics as well: such a store is
// written through to the point where all CUs agree, such a load never reads a CU's L1.
template <typename W>
__device__ __forceinline__ W lf_load(const W* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename W>
__device__ __forceinline__ void lf_store(W* p, W v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint2 lf_load_pair(const uint2* p) {
  const uint64_t v = lf_load(reinterpret_cast<const uint64_t*>(p));
  return make_uint2((uint32_t)v, (uint32_t)(v >> 32));
}
__device__ __forceinline__ void lf_store_pair(uint2* p, uint32_t key, uint32_t val) {
  lf_store(reinterpret_cast<uint64_t*>(p), (uint64_t)key | ((uint64_t)val << 32));
}

// Small values that tiles hand to each other (min / max partials, digit counts, prefixes, totals) travel as 64-bit
// words that carry their own tag: value | tag << 32, the tag naming the launch and the step. The reader polls the word
// itself until the tag is there, so such an exchange costs one trip to memory instead of the three of "stores, wait for
// them, raise a flag | poll the flag, load" -- five of the kernel's seven barriers became exchanges of this kind.
// The waits are bounded as the barriers' are: `budget` polls per thread and wait (none at all when the limit is 0 or the
// tile has already given up: the value is then meaningless and `ok` false).
__device__ __forceinline__ void lf_put(uint64_t* p, uint32_t tag, uint32_t value) {
  lf_flag_store(p, (uint64_t)value | ((uint64_t)tag << 32));
}
__device__ __forceinline__ uint32_t lf_get(const uint64_t* p, uint32_t tag, int limit, bool healthy, bool& ok) {
  uint64_t v = lf_flag_load(p);
  if (!healthy || limit <= 0) { ok = false; return (uint32_t)v; }
  for (int spins = 0; (uint32_t)(v >> 32) != tag; ++spins) {
    if (spins >= limit) { ok = false; break; }
    __builtin_amdgcn_s_sleep(1);
    v = lf_flag_load(p);
  }
  return (uint32_t)v;
}

// Barrier over the n_tiles workgroups of a segment: a flag per tile, every tile polls all of them. Before the flag is
// raised every thread has waited for its own (written-through) stores to complete. `want` grows by one per barrier; a
// neighbour can be at most one barrier ahead. Returns false when the bounded wait ran out (after `limit` polls). A
// tile that has already given up a wait (`healthy` false) still raises its flag, so that the others do not wait for
// it, and polls no more: one starved call costs one wait, not one per barrier.
__device__ __forceinline__ bool lf_barrier(uint64_t* gf, int tile, int n_tiles, uint64_t want, int limit, bool healthy) {
  __shared__ int s_ok;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x < 64) {
    if (threadIdx.x == 0) lf_flag_store(gf + tile, want);
    int spins = 0;
    bool done = false;
    for (; healthy && limit > 0;) {  // (a limit of 0 gives up at once, whatever the other tiles have done)
      bool ok = true;
      for (int c = threadIdx.x; c < n_tiles; c += 64) {
        const uint64_t v = lf_flag_load(gf + c);
        ok = ok && (v == want || v == want + 1);
      }
      done = __all(ok);
      if (done || ++spins > limit) break;
      __builtin_amdgcn_s_sleep(1);
    }
    if (threadIdx.x == 0) s_ok = done ? 1 : 0;
  }
  __syncthreads();
  return s_ok != 0;
}

__device__ __forceinline__ uint32_t lf_wave_inclusive(uint32_t v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(v, off);
    if (lane >= off) v += up;
  }
  return v;
}

// grid = segments * n_tiles workgroups: workgroup b is tile b % n_tiles of segment b / n_tiles (segment =
// event * n_tables + table). A tile is BLOCK * ITEMS hits; element order inside a tile as in the radix sort: wave w owns
// 64 * ITEMS consecutive hits, item k of lane l is at 64 * ITEMS * w + k * 64 + l. Every step of the kernel is latency
// bound: small tiles (more CUs) and many waves per tile (less serial work per thread) are what one event needs.
template <int DIM, int BLOCK, int ITEMS>
__global__ void __launch_bounds__(BLOCK) lsh_fused_kernel(const LshFusedArgs a) {
  constexpr int WAVES = BLOCK / 64;
  // per-wave digit counts, later the keys of the tile's earlier waves with the digit: 16 bits each (a wave holds
  // 64 * ITEMS keys, a tile at most 2048), digits 2j and 2j + 1 in one word
  __shared__ uint32_t s_cnt[WAVES][LF_MAX_BINS / 2];
  __shared__ uint32_t s_base[LF_MAX_BINS];           // keys of the segment with a smaller digit (+ of earlier tiles)
  __shared__ uint32_t s_tot[LF_MAX_BINS];            // digit totals of the segment; later the tile's permutation
  __shared__ uint8_t s_tab[WAVES][LF_MAX_BINS];      // the ranking's match tables (see below)
  __shared__ unsigned long long s_grp[WAVES][64];
  __shared__ int32_t s_mm[WAVES][LF_PARTIAL_STRIDE];
  __shared__ int32_t s_lo[LSH_MAX_PROJ], s_hi[LSH_MAX_PROJ];
  __shared__ uint32_t s_stride[LSH_MAX_PROJ];
  __shared__ float s_alpha[LSH_MAX_DIM][LSH_MAX_PROJ], s_beta[LSH_MAX_PROJ];  // the table's projections
  __shared__ uint32_t s_total;
  __shared__ int s_bits, s_over;
  __shared__ uint32_t s_wsum[WAVES];
  constexpr int XD = DIM ? DIM : LSH_MAX_DIM;
  constexpr int DPT = (LF_MAX_BINS + BLOCK - 1) / BLOCK;
  constexpr int TILE = BLOCK * ITEMS;
  static_assert(TILE <= LF_MAX_BINS, "the tile's permutation is staged in s_tot");

  const int tile = blockIdx.x % a.n_tiles, seg = blockIdx.x / a.n_tiles;
  const int n_tiles = a.n_tiles, J = a.n_proj, T = a.n_tables, n_cols = J * T;
  const int n_hits = (int)a.n_hits, dim = DIM ? DIM : a.dim;
  const int wave = threadIdx.x >> 6, lane = lane_id();
  uint64_t* gf = a.flags + (int64_t)seg * n_tiles;
  uint64_t* partial = a.partial + (int64_t)seg * n_tiles * LF_PARTIAL_STRIDE;
  uint64_t* rows = a.rows + (int64_t)seg * n_tiles * LF_MAX_BINS;
  uint64_t* totals = a.totals + (int64_t)seg * LF_MAX_BINS;
  uint2* pairs[2] = {a.pairs0 + (int64_t)seg * n_hits, a.pairs1 + (int64_t)seg * n_hits};
  uint64_t phase = (uint64_t)a.gen << 32;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  const int ibase = tile * TILE + wave * (TILE / WAVES) + lane;

  {
    const int ev = seg / T, table = seg - ev * T;
    const float* coords = a.coords + (int64_t)ev * n_hits * a.dim;
    const int n_valid = max(0, min(n_hits, a.n_valid_dev ? a.n_valid_dev[ev] : (int)a.n_valid));  // a count outside the event is cut
    bool healthy = true;
    // barrier number `want` of the segment; the first wait that runs out is made known to the segment's other tiles
    // (the word is written through before this tile raises its next flag, which the others wait for)
    auto lf_sync = [&](uint64_t want) -> bool {
      const bool ok = lf_barrier(gf, tile, n_tiles, want, a.spin_limit, healthy);
      if (healthy && !ok && threadIdx.x == 0) lf_store(a.failed + seg, a.gen);
      return ok;
    };
    // tag of the words of exchange k (0 .. 3) of radix pass e (the partials: pass 0, exchange 3)
    auto lf_tag = [&](int e, int k) -> uint32_t { return (a.gen << 4) | (uint32_t)(e << 2 | k); };
    // closes an exchange: did every thread of the tile get its words? (workgroup barrier inside)
    auto lf_got = [&](bool ok) -> bool {
      const bool all = __syncthreads_and(ok ? 1 : 0) != 0;
      if (healthy && !all && threadIdx.x == 0) lf_store(a.failed + seg, a.gen);
      return healthy && all;
    };

    // ---- hash the tile's hits for this table: min / max of every projection's bucket id ----
    if ((int)threadIdx.x < LSH_MAX_DIM * LSH_MAX_PROJ) {
      const int d = threadIdx.x / LSH_MAX_PROJ, j = threadIdx.x % LSH_MAX_PROJ;
      s_alpha[d][j] = (d < dim && j < J) ? a.alpha[d * n_cols + table * J + j] : 0.0f;
      if (d == 0) s_beta[j] = j < J ? a.beta[table * J + j] : 0.0f;
    }
    float x[ITEMS][XD];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int idx = ibase + 64 * k;
      lsh_load_coords<DIM>(coords, idx < n_valid ? idx : 0, a.dim, x[k]);
    }
    __syncthreads();
    // scaled projection of item k for column j: the chain p = fmaf(x[d], a[d], p) from 0, as everywhere in this
    // library, then (p + b) * inv_w; its bucket id is lsh_quantise_scaled of it
    auto scaled = [&](int k, int j) -> float {
      float acc = 0.0f;
#pragma unroll
      for (int d = 0; d < XD; ++d)
        if (DIM || d < dim) acc = __builtin_fmaf(x[k][d], s_alpha[d][j], acc);
      return lsh_scaled(acc, s_beta[j], a.inv_w);
    };
    auto bucket_id = [&](int k, int j) -> int32_t { return lsh_quantise_scaled(scaled(k, j)); };
    // extremes on the scaled projections, quantised once (the quantisation is monotone; NaNs, id INT32_MAX, are
    // ignored by fminf / fmaxf and noted separately); items past the valid count hold hit 0, a valid hit
    for (int j = 0; j < J; ++j) {
      float tlo = INFINITY, thi = -INFINITY;
      bool nan_seen = false;
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        const float t = scaled(k, j);
        tlo = fminf(tlo, t);
        thi = fmaxf(thi, t);
        nan_seen = nan_seen || t != t;
      }
      int32_t lo = lsh_quantise_scaled(tlo), hi = nan_seen ? INT32_MAX : lsh_quantise_scaled(thi);
      lo = lsh_wave_extreme<false>(lo);
      hi = lsh_wave_extreme<true>(hi);
      if (lane == 63) { s_mm[wave][2 * j] = lo; s_mm[wave][2 * j + 1] = hi; }
    }
    __syncthreads();
    if ((int)threadIdx.x < 2 * J) {
      const int q = threadIdx.x;
      int32_t v = s_mm[0][q];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) v = (q & 1) ? max(v, s_mm[w][q]) : min(v, s_mm[w][q]);
      lf_put(partial + tile * LF_PARTIAL_STRIDE + q, lf_tag(0, 3), (uint32_t)v);
    }

    // ---- ranges, mixed-radix strides, key width (every tile computes them; tile 0 writes the meta row) ----
    {  // thread t reduces value t % 16 over tiles t / 16, t / 16 + 16, ...: independent loads, one round trip
      const int q = threadIdx.x & 15;
      int32_t v = (q & 1) ? INT32_MIN : INT32_MAX;
      bool got = true;
      if (q < 2 * J) {
#pragma unroll 4
        for (int p = threadIdx.x >> 4; p < n_tiles; p += BLOCK / 16) {
          const int32_t o = (int32_t)lf_get(partial + p * LF_PARTIAL_STRIDE + q, lf_tag(0, 3), a.spin_limit, healthy, got);
          v = (q & 1) ? max(v, o) : min(v, o);
        }
      }
      healthy = lf_got(got);
      int32_t o = __shfl_xor(v, 16);
      v = (q & 1) ? max(v, o) : min(v, o);
      o = __shfl_xor(v, 32);
      v = (q & 1) ? max(v, o) : min(v, o);
      if (lane < 16) s_mm[wave][lane] = v;
      __syncthreads();
      if ((int)threadIdx.x < 2 * J) {
        v = s_mm[0][q];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v = (q & 1) ? max(v, s_mm[w][q]) : min(v, s_mm[w][q]);
        if (n_valid == 0) v = 0;
        if (q & 1) s_hi[q >> 1] = v; else s_lo[q >> 1] = v;
      }
    }
    __syncthreads();
    int32_t* m = a.meta + (int64_t)seg * (2 * J + 3);
    if (threadIdx.x == 0) {
      uint64_t total = 1;
      int overflow = 0;
      for (int j = 0; j < J; ++j) {
        const int64_t range = (int64_t)s_hi[j] - (int64_t)s_lo[j] + 1;
        s_stride[j] = (uint32_t)total;
        total *= (uint64_t)range;
        if (total > (uint64_t)INT32_MAX) { overflow = 1; total = (uint64_t)INT32_MAX + 1; }
        if (tile == 0) {
          m[j] = s_lo[j];
          m[J + j] = range > INT32_MAX ? INT32_MAX : (int32_t)range;
        }
      }
      const uint64_t top = (n_valid < n_hits) ? total : total - 1;
      int bits = min(32, max(1, 64 - (int)__clzll((unsigned long long)top)));  // significant bits of the largest key
      if (overflow) bits = 32;
      s_total = (uint32_t)total;
      s_bits = bits;
      s_over = overflow;
      if (tile == 0) {
        m[2 * J] = total > (uint64_t)INT32_MAX ? INT32_MAX : (int32_t)total;
        m[2 * J + 1] = bits;
        m[2 * J + 2] = overflow;
      }
    }
    __syncthreads();

    // ---- bucket ids and packed keys of the tile's hits (padding hits: ids 0, key = total, so they sort last) ----
    uint32_t key[ITEMS], rank[ITEMS];
    int32_t val[ITEMS];
    bool inside[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int idx = ibase + 64 * k;
      inside[k] = idx < n_hits;
      const bool valid = idx < n_valid;
      uint32_t kk = valid ? 0u : s_total;
      for (int j = 0; j < J; ++j) {
        int32_t id = 0;
        if (valid) {
          id = bucket_id(k, j);
          kk += ((uint32_t)id - (uint32_t)s_lo[j]) * s_stride[j];
        }
        if (a.ids && inside[k]) a.ids[((int64_t)ev * n_cols + table * J + j) * n_hits + idx] = id;
      }
      if (inside[k]) a.keys[(int64_t)seg * n_hits + idx] = (int32_t)kk;
      key[k] = inside[k] ? kk : 0xFFFFFFFFu;
      val[k] = idx;
    }

    // ---- stable LSD radix sort of the segment: ceil(bits / 11) passes of equal digit width ----
    const int bits = s_bits;
    const int eff = (bits + LF_MAX_DIGIT_BITS - 1) / LF_MAX_DIGIT_BITS, width = (bits + eff - 1) / eff;
    int32_t* perm = a.perm + (int64_t)seg * n_hits;
    for (int e = 0; e < eff; ++e) {
      const int shift = e * width, nbits = min(width, bits - shift), bins = 1 << nbits;
      const uint32_t mask = (uint32_t)bins - 1u;
      const bool last = e == eff - 1;
      for (int d2 = threadIdx.x; 2 * d2 < bins; d2 += BLOCK) {
#pragma unroll
        for (int w = 0; w < WAVES; ++w) s_cnt[w][d2] = 0;
      }
      __syncthreads();
      {
        // Ranks within the wave. Lanes with the same digit find each other through two tables of the wave in LDS:
        // every lane writes its number to tab[d] and reads back the one
        // that stayed (the group's speaker), sets its bit in the speaker's 64-bit word, reads the word (= the group)
        // and clears it; the speaker then adds the group's size to the wave's count of the digit. The LDS executes
        // the instructions of one wave in order, so the steps need no wait between them, and the relaxed atomic
        // accesses keep the compiler from forwarding a lane's own store to its load. (Eleven wavefront ballots per
        // key did the same in three times the instructions: 62.3 -> 58.7 us for one event.) A hit beyond the event's
        // end carries the largest digit and comes last in (item, lane) order: it changes no rank, only the count of
        // the largest digit in the segment's last tile, which no other key's position depends on.
        uint8_t* tab = s_tab[wave];
        unsigned long long* grp = s_grp[wave];
        grp[lane] = 0ull;
        const unsigned long long bit = 1ull << lane;
        uint32_t dd[ITEMS], spk[ITEMS], old[ITEMS];
        uint64_t peers[ITEMS];
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
          dd[k] = (key[k] >> shift) & mask;
          __hip_atomic_store(&tab[dd[k]], (uint8_t)lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
          spk[k] = __hip_atomic_load(&tab[dd[k]], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        }
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
          __hip_atomic_fetch_or(&grp[spk[k]], bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
          peers[k] = __hip_atomic_load(&grp[spk[k]], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
          __hip_atomic_store(&grp[spk[k]], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        }
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
          const int sh = 16 * (dd[k] & 1u);
          old[k] = 0;
          if ((uint32_t)lane == spk[k])
            old[k] = (atomicAdd(&s_cnt[wave][dd[k] >> 1], (uint32_t)__popcll(peers[k]) << sh) >> sh) & 0xFFFFu;
        }
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
          rank[k] = (uint32_t)__shfl((int)old[k], (int)spk[k]) + (uint32_t)__popcll(peers[k] & lt_mask);
      }
      __syncthreads();
      // the tile's digit counts for the other tiles of the segment
      for (int d = threadIdx.x; d < bins; d += BLOCK) {
        uint32_t c = 0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) c += (s_cnt[w][d >> 1] >> (16 * (d & 1))) & 0xFFFFu;
        lf_put(rows + tile * LF_MAX_BINS + d, lf_tag(e, 0), c);
      }
      // Tile t turns the counts of digits t*per .. (t+1)*per - 1 of ALL tiles into prefixes over the tiles (in place)
      // and their sum into the segment's totals: every tile reads n_tiles * per words instead of n_tiles rows. A wave
      // takes a digit, its lanes the tiles (128 at a time); four digits per wave are in flight, all loads first.
      {
        const int per = (bins + n_tiles - 1) / n_tiles, d0 = tile * per;
        const int steps = (per + WAVES - 1) / WAVES;
        bool got = true;
        for (int s0 = 0; s0 < steps; s0 += 4) {
          uint32_t carry[4] = {0, 0, 0, 0};
          for (int p0 = 0; p0 < n_tiles; p0 += 128) {
            uint32_t c[4][2];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int dd = (s0 + u) * WAVES + wave, d = d0 + dd;
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const int p = p0 + 64 * h + lane;
                c[u][h] = (dd < per && d < bins && p < n_tiles)
                              ? lf_get(rows + p * LF_MAX_BINS + d, lf_tag(e, 0), a.spin_limit, healthy, got) : 0u;
              }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int dd = (s0 + u) * WAVES + wave, d = d0 + dd;
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const int p = p0 + 64 * h + lane;
                const uint32_t incl = lf_wave_inclusive(c[u][h], lane);
                if (dd < per && d < bins && p < n_tiles)
                  lf_put(rows + p * LF_MAX_BINS + d, lf_tag(e, 1), carry[u] + incl - c[u][h]);
                carry[u] += __shfl(incl, 63);
              }
            }
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int dd = (s0 + u) * WAVES + wave, d = d0 + dd;
            if (lane == 0 && dd < per && d < bins) lf_put(totals + d, lf_tag(e, 1), carry[u]);
          }
        }
        healthy = lf_got(got);
      }
      // thread t owns digits t, t + BLOCK, ...: keys of the digit in the tiles before this one, and in the segment
      uint32_t excl[DPT];
      {
        bool got = true;
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
          const int d = threadIdx.x + j * BLOCK;
          excl[j] = d < bins ? lf_get(rows + tile * LF_MAX_BINS + d, lf_tag(e, 1), a.spin_limit, healthy, got) : 0u;
          if (d < bins) s_tot[d] = lf_get(totals + d, lf_tag(e, 1), a.spin_limit, healthy, got);
        }
        healthy = lf_got(got);
      }
      {  // exclusive scan of the digit totals: thread t scans digits 8t .. 8t+7
        uint32_t dt[DPT], mine = 0;
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
          const int d = threadIdx.x * DPT + j;
          dt[j] = d < bins ? s_tot[d] : 0u;
          mine += dt[j];
        }
        uint32_t incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
          const uint32_t up = __shfl_up(incl, off);
          if (lane >= off) incl += up;
        }
        if (lane == 63) s_wsum[wave] = incl;
        __syncthreads();
        uint32_t run = incl - mine;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) run += w < wave ? s_wsum[w] : 0u;
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
          const int d = threadIdx.x * DPT + j;
          if (d < bins) s_base[d] = run;
          run += dt[j];
        }
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < DPT; ++j) {  // per digit: the tile's base, and the keys of the tile's earlier waves
        const int d = threadIdx.x + j * BLOCK;
        if (d < bins) {
          s_base[d] += excl[j];
          uint32_t run = 0;
#pragma unroll
          for (int w = 0; w < WAVES; ++w) {
            uint16_t* half = reinterpret_cast<uint16_t*>(s_cnt[w]) + d;
            const uint32_t c = *half;
            *half = (uint16_t)run;
            run += c;
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        if (inside[k]) {
          const uint32_t d = (key[k] >> shift) & mask;
          const uint32_t pos = s_base[d] + reinterpret_cast<const uint16_t*>(s_cnt[wave])[d] + rank[k];
          if (pos < (uint32_t)n_hits) {  // always, unless a wait was abandoned
            if (last) { if (healthy) lf_store(perm + pos, val[k]); }
            else lf_store_pair(pairs[e & 1] + pos, key[k], (uint32_t)val[k]);
          }
        }
      }
      healthy = lf_sync(++phase);
      if (!last) {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
          const int idx = ibase + 64 * k;
          const uint2 kv = inside[k] ? lf_load_pair(pairs[e & 1] + idx) : make_uint2(0xFFFFFFFFu, 0u);
          key[k] = kv.x;
          val[k] = (int32_t)kv.y;
        }
      }
    }

    // A wait that ran out, here or (seen through the segment's word after the last barrier) in another tile: the
    // segment's order cannot be trusted. Every tile that knows then writes -1 over the segment's WHOLE permutation
    // (other tiles scatter into every part of it, and a tile that has given up scatters into it no more, so the tile
    // that finishes last leaves it all -1) and zeros over its own rows of the sorted features, so that the failure
    // shows in the outputs themselves and not only in the meta row. (Only a tile that had already left the last
    // barrier when another gave up at that same barrier does not know; all scatters were complete by then.)
    const bool poisoned = !healthy || lf_load(a.failed + seg) == a.gen;
    const int row0 = tile * TILE, n_rows = max(0, min(TILE, n_hits - row0));
    if (poisoned)
      for (int r = threadIdx.x; r < n_hits; r += BLOCK) lf_store(perm + r, (int32_t)-1);

    // ---- the hit features in sorted order: rows tile*TILE .. of the segment's output ----
    if (a.feats) {
      for (int r = threadIdx.x; r < n_rows; r += BLOCK)
        s_tot[r] = poisoned ? 0xFFFFFFFFu : (uint32_t)lf_load(perm + row0 + r);
      __syncthreads();
      const int vpr = a.vec_per_row, items = n_rows * vpr;
      const uint4* src = reinterpret_cast<const uint4*>(a.feats) + (int64_t)ev * n_hits * vpr;
      uint4* dst = reinterpret_cast<uint4*>(a.feats_out) + ((int64_t)seg * n_hits + row0) * vpr;
      constexpr int GU = 12;  // 16-byte loads in flight per thread: the reads are random rows, a memory latency each
      for (int it0 = 0; it0 < items; it0 += GU * BLOCK) {
        uint4 v[GU];
#pragma unroll
        for (int u = 0; u < GU; ++u) {
          const int it = it0 + u * BLOCK + threadIdx.x;
          v[u] = make_uint4(0, 0, 0, 0);
          if (it < items) {
            const int r = it / vpr, piece = it - r * vpr;
            const uint32_t from = s_tot[r];
            if (from < (uint32_t)n_hits) v[u] = src[(int64_t)from * vpr + piece];
          }
        }
#pragma unroll
        for (int u = 0; u < GU; ++u) {
          const int it = it0 + u * BLOCK + threadIdx.x;
          if (it < items) dst[it] = v[u];
        }
      }
    }
    // a wait that ran out: say so in the segment's meta row (after tile 0's write of the overflow field, which
    // happened before the first sort barrier)
    if (poisoned && threadIdx.x == 0) m[2 * J + 2] = s_over | 2;
  }
}

// ---- host side ---------------------------------------------------------------------------------------------------
#define LF_MAX_DEVICES 64
// The forms of the kernel that are built: threads per workgroup x hits per thread (tile = their product).
struct LfForm { int block, items; };
static const LfForm lf_forms[] = {{512, 2}, {768, 1}};
#define LF_FORMS ((int)(sizeof(lf_forms) / sizeof(lf_forms[0])))
#define LF_MIN_TILE 768
struct LfDevice {
  int state;                    // 0 unknown, 1 known
  int cus;                      // compute units
  int capacity[2][LF_FORMS];    // workgroups the GPU holds at once: [generic dim, dim 4][form]
};
static LfDevice lf_dev[LF_MAX_DEVICES];
static std::mutex lf_lock;

// A value that no earlier call of this process has left in a workspace (the flags are compared for equality with
// generation << 32 | barrier number, so they need no clearing), started from the clock so that a workspace written by
// another process is no more likely to match.
static uint32_t lf_next_generation() {
  static std::atomic<uint32_t> counter{(uint32_t)std::chrono::steady_clock::now().time_since_epoch().count()};
  return counter.fetch_add(1) + 1;
}

// Process-wide switches of the one-launch form (lampa_lsh_one_launch_config): whether it is used at all (0 / 1, or
// 100 + i: form i for every call that fits), and the number of polls a tile spends in one wait (< 0: LF_SPIN_LIMIT).
static std::atomic<int> lf_enabled{1};
static std::atomic<int64_t> lf_wait_limit{-1};

extern "C" int lampa_lsh_one_launch_config(int enabled, int64_t wait_limit) {
  lf_enabled.store(enabled >= 100 && enabled < 100 + LF_FORMS ? enabled : (enabled ? 1 : 0));
  lf_wait_limit.store(wait_limit);
  return LAMPA_OK;
}

template <int DIM, int BLOCK, int ITEMS>
static int lf_occupancy() {
  int occ = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, lsh_fused_kernel<DIM, BLOCK, ITEMS>, BLOCK, 0) != hipSuccess) {
    (void)hipGetLastError();
    occ = 0;
  }
  return occ;
}

// How many workgroups of each form of the kernel the current GPU holds at once (CUs x workgroups per CU), looked up
// once per device.
static const LfDevice* lf_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LF_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> hold(lf_lock);
  LfDevice& d = lf_dev[dev];
  if (d.state == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    d.cus = cus;
    d.capacity[0][0] = cus * lf_occupancy<0, 512, 2>(); d.capacity[1][0] = cus * lf_occupancy<4, 512, 2>();
    d.capacity[0][1] = cus * lf_occupancy<0, 768, 1>(); d.capacity[1][1] = cus * lf_occupancy<4, 768, 1>();
    d.state = 1;
  }
  return &d;
}

static int64_t lf_tiles(int64_t n_hits, int tile) { return n_hits > 0 ? (n_hits + tile - 1) / tile : 1; }

// The fused kernel is for calls of at most this many segments (events x tables): beyond it the call cannot fit the
// GPU at once whatever the event size.
#define LF_MAX_SEGMENTS 64

// Workspace of the fused kernel: flags | partials | digit counts and totals | two pair buffers, sized for the
// smallest tile. Zero when the call is too large for the fused kernel.
int64_t lsh_fused_workspace_bytes(int n_events, int64_t n_hits, int n_tables) {
  const int64_t segs = (int64_t)n_events * n_tables, tiles = lf_tiles(n_hits, LF_MIN_TILE);
  if (segs > LF_MAX_SEGMENTS || segs * lf_tiles(n_hits, 1024) > 4096) return 0;
  return lampa_align_up(segs * tiles * 8, 256) + lampa_align_up(segs * tiles * LF_PARTIAL_STRIDE * 8, 256) +
         lampa_align_up(segs * (tiles + 1) * LF_MAX_BINS * 8, 256) + 2 * lampa_align_up(segs * n_hits * 8, 256) +
         lampa_align_up(segs * 4, 256);
}

// Launches the fused kernel when it applies: returns LAMPA_OK after a launch, 1 when the caller has to take the
// separate kernels (the tiles of the call do not all fit the GPU at once, rows that are not 16-byte pieces), or an
// error.
int lsh_fused_launch(const float* coords, int n_events, int64_t n_hits, int64_t n_valid, const int32_t* n_valid_dev,
                     int dim, const float* alpha, const float* beta, int n_tables, int n_proj, float w,
                     int32_t* ids_out, int32_t* keys_out, int32_t* meta_out, int32_t* perm_out, const void* feats,
                     int64_t feat_row_bytes, void* feats_out, void* workspace, int64_t workspace_bytes,
                     hipStream_t s) {
  const int64_t segs = (int64_t)n_events * n_tables;
  if (!lf_enabled.load()) return 1;
  if (n_hits < 1 || n_hits > (1 << 24) || segs > LF_MAX_SEGMENTS) return 1;
  if (feats && (feat_row_bytes % 16 != 0 || feat_row_bytes / 16 > (1 << 16) || ((uintptr_t)feats % 16) != 0 ||
                ((uintptr_t)feats_out % 16) != 0))
    return 1;
  const int64_t need = lsh_fused_workspace_bytes(n_events, n_hits, n_tables);
  if (need == 0) return 1;
  if (workspace_bytes < need) return LAMPA_ERR_WORKSPACE;
  const LfDevice* d = lf_device();
  if (!d) return 1;
  // Which form, if any. Every step of this kernel is latency bound: more waves per tile shorten the steps (a tile of
  // 1 024 hits: 60.5 us with 256 threads, 49.7 us with 512, for one event of 60 000 hits), smaller tiles do too as long as
  // a CU runs one of them and a table does not get too many (the barriers run over a table's tiles), and a CU that runs
  // two tiles takes 1.3-1.7 times as long for each, while the separate kernels grow by only 0.145 us per 1 000 hits.
  // Measured, us per call: separate kernels | 256 threads x 4 hits | 256 x 3 | 512 x 2 | 1 024 x 1 | 768 x 1 (- = the
  // workgroups do not fit the GPU at once):
  //   60 000 hits x 1 event   65.7 | 60.5 | 56.2 | 49.7 | 50.0 | 51.1      30 000 x 1   60.3 | 58.6 | 51.0 | 45.5 | 43.7 | 43.4
  //            x 2 events     72.4 | 74.8 | 77.7 | 69.1 |  -   |  -                x 2   62.3 | 61.1 | 55.1 | 50.1 | 48.7 | 48.5
  //            x 3            82.5 | 87.1 | 99.6 |  -   |  -   |  -                x 3   67.4 | 64.9 | 67.0 | 57.3 |  -   |  -
  //            x 4            90.9 | 102.9 | -   |  -   |  -   |  -                x 4   72.1 | 72.1 | 71.0 | 66.7 |  -   |  -
  // Built: 512 x 2 and 768 x 1. The latter when it gives at most one workgroup per CU and at most 48 tiles per table,
  // else the former when its workgroups fit the GPU at once (two per CU), else the separate kernels.
  // lampa_lsh_one_launch_config(100 / 101, ...) forces a form for every call that fits.
  const int dsel = dim == 4 ? 1 : 0;
  const int forced = lf_enabled.load();
  int pick = -1;
  if (forced >= 100) {
    const int i = forced - 100;
    if (segs * lf_tiles(n_hits, lf_forms[i].block * lf_forms[i].items) <= d->capacity[dsel][i]) pick = i;
  } else {
    const int64_t t768 = lf_tiles(n_hits, 768), t1024 = lf_tiles(n_hits, 1024);
    if (segs * t768 <= d->cus && segs * t768 <= d->capacity[dsel][1] && t768 <= 48) pick = 1;
    else if (segs * t1024 <= d->capacity[dsel][0]) pick = 0;
  }
  if (pick < 0) return 1;
  const int tile_hits = lf_forms[pick].block * lf_forms[pick].items;
  const int64_t tiles = lf_tiles(n_hits, tile_hits);
  LshFusedArgs a;
  a.coords = coords; a.n_hits = n_hits; a.n_valid = n_valid; a.n_valid_dev = n_valid_dev; a.dim = dim;
  a.alpha = alpha; a.beta = beta; a.n_tables = n_tables; a.n_proj = n_proj; a.inv_w = 1.0f / w;
  a.ids = ids_out; a.keys = keys_out; a.meta = meta_out; a.perm = perm_out;
  a.feats = (const char*)feats; a.vec_per_row = feats ? (int)(feat_row_bytes / 16) : 0; a.feats_out = (char*)feats_out;
  a.n_events = n_events; a.n_tiles = (int)tiles;
  char* p = (char*)workspace;
  a.flags = (uint64_t*)p;   p += lampa_align_up(segs * tiles * 8, 256);
  a.partial = (uint64_t*)p; p += lampa_align_up(segs * tiles * LF_PARTIAL_STRIDE * 8, 256);
  a.rows = (uint64_t*)p;    a.totals = a.rows + segs * tiles * LF_MAX_BINS;
  p += lampa_align_up(segs * (tiles + 1) * LF_MAX_BINS * 8, 256);
  a.pairs0 = (uint2*)p;     p += lampa_align_up(segs * n_hits * 8, 256);
  a.pairs1 = (uint2*)p;     p += lampa_align_up(segs * n_hits * 8, 256);
  a.failed = (uint32_t*)p;
  a.gen = lf_next_generation();
  const int64_t limit = lf_wait_limit.load();
  a.spin_limit = limit < 0 ? LF_SPIN_LIMIT : (int)(limit > LF_SPIN_LIMIT ? LF_SPIN_LIMIT : limit);
  const dim3 grid((unsigned)(segs * tiles)), block(lf_forms[pick].block);
  LAMPA_PROF(s, "start");
#define LF_LAUNCH(DIM, BLOCK, ITEMS) hipLaunchKernelGGL((lsh_fused_kernel<DIM, BLOCK, ITEMS>), grid, block, 0, s, a)
#define LF_LAUNCH_DIM(DIM)                                                                        \
  switch (pick) {                                                                                 \
    case 0: LF_LAUNCH(DIM, 512, 2); break;                                                        \
    default: LF_LAUNCH(DIM, 768, 1); break;                                                       \
  }
  if (dim == 4) { LF_LAUNCH_DIM(4) } else { LF_LAUNCH_DIM(0) }
#undef LF_LAUNCH_DIM
#undef LF_LAUNCH
  LAMPA_PROF(s, "lsh_fused_kernel");
  return lampa_launch_status();
}

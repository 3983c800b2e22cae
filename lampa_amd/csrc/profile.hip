// Per-kernel timing of the library's own launches with HIP events recorded on the launch stream.
// A profiling aid for the benchmark: one recording at a time, not thread-safe, adds a few event records per call.
#include "common.h"

#include <string.h>

#define PROF_MAX 4096

static bool g_recording = false;
static int g_count = 0;
static hipEvent_t g_events[PROF_MAX];
static const char* g_names[PROF_MAX];

bool lampa_prof_recording() { return g_recording; }

void lampa_prof_mark(hipStream_t stream, const char* name) {
  if (!g_recording || g_count >= PROF_MAX) return;
  if (hipEventCreate(&g_events[g_count]) != hipSuccess) return;
  (void)hipEventRecord(g_events[g_count], stream);
  g_names[g_count] = name;
  ++g_count;
}

// Starts recording the kernels launched by subsequent library calls (on whatever stream they use).
extern "C" int lampa_profile_begin() {
  if (g_recording) return LAMPA_ERR_INVALID;
  g_count = 0;
  g_recording = true;
  return LAMPA_OK;
}

// Stops recording, waits for the recorded work and returns the number of kernel intervals n (<= max_entries):
// ms[i] is the time between the previous mark and the mark after kernel i, names[i] points to a static string.
extern "C" int lampa_profile_end(int max_entries, float* ms, const char** names) {
  if (!g_recording) return LAMPA_ERR_INVALID;
  g_recording = false;
  int n = 0;
  if (g_count > 0) (void)hipEventSynchronize(g_events[g_count - 1]);
  for (int i = 1; i < g_count; ++i) {
    if (strcmp(g_names[i], "start") == 0) continue;
    float t = 0.0f;
    (void)hipEventElapsedTime(&t, g_events[i - 1], g_events[i]);
    if (n < max_entries) {
      if (ms) ms[n] = t;
      if (names) names[n] = g_names[i];
      ++n;
    }
  }
  for (int i = 0; i < g_count; ++i) (void)hipEventDestroy(g_events[i]);
  g_count = 0;
  return n;
}

// ---- memory-only twin of the output pass ----------------------------------------------------------------------------
// The loads and stores of the chunk pipeline's output pass (K = V = 64, 2-byte elements, one dense sequence of whole
// chunks) with no arithmetic at all: per (segment, head) workgroup and chunk, 128 threads fetch the chunk's k, v and q
// rows (128 bytes per row and head, rows one token apart) and the 4.5 KiB of T in its record one chunk ahead, the other 128
// threads store the o rows. Its duration is what this access pattern costs on the memory system alone, i.e. the
// practical floor of the output pass (the algorithmic roofline assumes 8 TB/s for any pattern).
typedef unsigned int prof_u32x4 __attribute__((ext_vector_type(4)));
#define PROBE_REC_U4 336  // 5376-byte record of a chunk and head, in 16-byte units (the first 288 are read: T)

// WALK: before its first chunk the workgroup also reads what the output pass reads for the second level of the two-level
// scan -- the composites of the groups of 8 segments before its group, then of the segments before it inside its group:
// per step and wave the 8 KiB of M' and the wave's 8 KiB slab of N, two steps ahead, as the kernel does.
#define PROBE_COMP_U4 1536  // composite of a segment (or group) and head: M' 8 KiB, then N 16 KiB, in 16-byte units
template <bool WALK>
__global__ void __launch_bounds__(256, 2)
    gdr_traffic_probe_kernel(const prof_u32x4* __restrict__ q, const prof_u32x4* __restrict__ k,
                             const prof_u32x4* __restrict__ v, const prof_u32x4* __restrict__ rec,
                             const prof_u32x4* __restrict__ comp, prof_u32x4* __restrict__ o, int n_chunks, int H,
                             int cps) {
  const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int c0 = seg * cps, c1 = min(c0 + cps, n_chunks);
  if (tid < 128) {
    const int row = tid >> 1, half = tid & 1;
    prof_u32x4 buf[15], acc = {0, 0, 0, 0};
    auto issue = [&](int c) __attribute__((always_inline)) {
      c = min(c, c1 - 1);
      const size_t base = ((size_t)(c * 64 + row) * H + h) * 8 + half * 4;
#pragma unroll
      for (int u = 0; u < 4; ++u) { buf[u] = k[base + u]; buf[4 + u] = v[base + u]; buf[8 + u] = q[base + u]; }
      const prof_u32x4* rp = rec + ((size_t)c * H + h) * PROBE_REC_U4;
#pragma unroll
      for (int j = 0; j < 3; ++j) buf[12 + j] = rp[min(tid + 128 * j, 287)];  // (threads past the end repeat the last piece)
    };
    issue(c0);
    for (int c = c0; c < c1; ++c) {
#pragma unroll
      for (int u = 0; u < 15; ++u) acc += buf[u];
      issue(c + 1);
      __syncthreads();
    }
    if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) o[0] = acc;  // keeps the loads alive; never true in practice
  } else {
    const int t = tid - 128;
    if constexpr (WALK) {
      const int segs = gridDim.x, lane = t & 63, slab = t >> 6;
      const int lead = seg / 8, nst = lead + seg % 8, item0 = seg - seg % 8;
      prof_u32x4 ring[2][16], acc = {0, 0, 0, 0};
      auto issue = [&](int p, prof_u32x4* r) __attribute__((always_inline)) {
        p = max(0, min(p, nst - 1));
        const int item = p < lead ? segs + p : item0 + (p - lead);  // (the groups' composites follow the segments')
        const prof_u32x4* base = comp + ((size_t)item * H + h) * PROBE_COMP_U4;
#pragma unroll
        for (int f = 0; f < 8; ++f) { r[f] = base[f * 64 + lane]; r[8 + f] = base[512 + slab * 512 + f * 64 + lane]; }
      };
      if (nst > 0) {
        issue(0, ring[0]);
        issue(1, ring[1]);
        for (int p = 0; p < nst; p += 2) {
#pragma unroll
          for (int f = 0; f < 16; ++f) acc += ring[0][f];
          issue(p + 2, ring[0]);
          if (p + 1 < nst) {
#pragma unroll
            for (int f = 0; f < 16; ++f) acc += ring[1][f];
          }
          issue(p + 3, ring[1]);
        }
      }
      if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) o[1] = acc;  // keeps the loads alive; never true in practice
    }
    for (int c = c0; c < c1; ++c) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int piece = t + 128 * j, row = piece >> 3, part = piece & 7;
        const prof_u32x4 val = {(unsigned)c, (unsigned)row, (unsigned)part, 0u};
        __builtin_nontemporal_store(val, &o[((size_t)(c * 64 + row) * H + h) * 8 + part]);  // as the output pass stores o
      }
      __syncthreads();
    }
  }
}

// q, k, v, o: [n_chunks * 64, H, 64] 2-byte elements; records: n_chunks * H * 5376 bytes (any content). o is
// overwritten with a pattern. One launch = one pass.
extern "C" int lampa_gdr_traffic_probe(const void* q, const void* k, const void* v, const void* records, void* o,
                                       int n_chunks, int H, int chunks_per_segment, void* stream) {
  if (!q || !k || !v || !records || !o || n_chunks < 1 || H < 1 || chunks_per_segment < 1) return LAMPA_ERR_INVALID;
  const int segs = (n_chunks + chunks_per_segment - 1) / chunks_per_segment;
  hipLaunchKernelGGL(gdr_traffic_probe_kernel<false>, dim3(segs, H), dim3(256), 0, (hipStream_t)stream,
                     (const prof_u32x4*)q, (const prof_u32x4*)k, (const prof_u32x4*)v, (const prof_u32x4*)records,
                     (const prof_u32x4*)nullptr, (prof_u32x4*)o, n_chunks, H, chunks_per_segment);
  return hipGetLastError() == hipSuccess ? LAMPA_OK : LAMPA_ERR_LAUNCH;
}

// The same with the reads of the walk over the earlier composites that the output pass does before its first chunk when
// the scan runs in two levels. composites: (segments + ceil(segments / 8)) * H * 24576 bytes of any content (the
// segments' composites, then the groups').
extern "C" int lampa_gdr_traffic_probe_walk(const void* q, const void* k, const void* v, const void* records,
                                            const void* composites, void* o, int n_chunks, int H,
                                            int chunks_per_segment, void* stream) {
  if (!q || !k || !v || !records || !composites || !o || n_chunks < 1 || H < 1 || chunks_per_segment < 1)
    return LAMPA_ERR_INVALID;
  const int segs = (n_chunks + chunks_per_segment - 1) / chunks_per_segment;
  hipLaunchKernelGGL(gdr_traffic_probe_kernel<true>, dim3(segs, H), dim3(256), 0, (hipStream_t)stream,
                     (const prof_u32x4*)q, (const prof_u32x4*)k, (const prof_u32x4*)v, (const prof_u32x4*)records,
                     (const prof_u32x4*)composites, (prof_u32x4*)o, n_chunks, H, chunks_per_segment);
  return hipGetLastError() == hipSuccess ? LAMPA_OK : LAMPA_ERR_LAUNCH;
}

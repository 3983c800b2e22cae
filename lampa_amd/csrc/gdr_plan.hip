// Host-side construction of the plan (see gdr_plan.h). No device code.
#include "gdr_plan.h"

static int64_t plan_counts(const int64_t* cu, int n_seq, int cps, int64_t* n_chunks, int64_t* n_segments) {
  int64_t chunks = 0, segs = 0;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t len = cu[s + 1] - cu[s];
    if (len < 0) return -1;
    const int64_t nc = (len + GDR_C - 1) / GDR_C;
    chunks += nc;
    segs += nc == 0 ? 1 : (nc + cps - 1) / cps;  // an empty sequence still owns one (empty) segment
  }
  *n_chunks = chunks;
  *n_segments = segs;
  return 0;
}

// Number of int32 entries of the plan for these sequences (negative on error).
extern "C" int64_t lampa_gdr_plan_size(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment) {
  if (!cu_seqlens_host || n_seq < 1 || chunks_per_segment < 1) return LAMPA_ERR_INVALID;
  int64_t chunks, segs;
  if (plan_counts(cu_seqlens_host, n_seq, chunks_per_segment, &chunks, &segs) != 0) return LAMPA_ERR_INVALID;
  if (cu_seqlens_host[n_seq] > INT32_MAX) return LAMPA_ERR_UNSUPPORTED;
  return PLAN_HEADER + 2 * chunks + 4 * segs + 2 * (int64_t)n_seq;
}

// Fills plan_host (lampa_gdr_plan_size entries). The caller copies it to the device and passes that pointer on.
extern "C" int lampa_gdr_plan_fill(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment,
                                   int32_t* plan_host) {
  if (!plan_host) return LAMPA_ERR_INVALID;
  const int64_t size = lampa_gdr_plan_size(cu_seqlens_host, n_seq, chunks_per_segment);
  if (size < 0) return (int)size;
  int64_t chunks, segs;
  plan_counts(cu_seqlens_host, n_seq, chunks_per_segment, &chunks, &segs);
  int32_t* p = plan_host;
  for (int i = 0; i < PLAN_HEADER; ++i) p[i] = 0;
  p[PLAN_N_SEQ] = n_seq;
  p[PLAN_TOTAL_CHUNKS] = (int32_t)chunks;
  p[PLAN_N_SEGMENTS] = (int32_t)segs;
  p[PLAN_CHUNKS_PER_SEGMENT] = chunks_per_segment;
  p[PLAN_TOTAL_TOKENS] = (int32_t)cu_seqlens_host[n_seq];
  int64_t off = PLAN_HEADER;
  p[PLAN_OFF_CHUNK_TOK0] = (int32_t)off; off += chunks;
  p[PLAN_OFF_CHUNK_LEN] = (int32_t)off; off += chunks;
  p[PLAN_OFF_SEG_CHUNK0] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEG_NCHUNKS] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEG_SEQ] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEG_FLAGS] = (int32_t)off; off += segs;
  p[PLAN_OFF_SEQ_SEG0] = (int32_t)off; off += n_seq;
  p[PLAN_OFF_SEQ_NSEG] = (int32_t)off; off += n_seq;
  int64_t c = 0, g = 0;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t bos = cu_seqlens_host[s], len = cu_seqlens_host[s + 1] - bos;
    const int64_t nc = (len + GDR_C - 1) / GDR_C;
    const int64_t ns = nc == 0 ? 1 : (nc + chunks_per_segment - 1) / chunks_per_segment;
    p[p[PLAN_OFF_SEQ_SEG0] + s] = (int32_t)g;
    p[p[PLAN_OFF_SEQ_NSEG] + s] = (int32_t)ns;
    for (int64_t i = 0; i < ns; ++i) {
      const int64_t c0 = i * chunks_per_segment;
      const int64_t cn = nc - c0 < chunks_per_segment ? nc - c0 : chunks_per_segment;
      p[p[PLAN_OFF_SEG_CHUNK0] + g] = (int32_t)(c + c0);
      p[p[PLAN_OFF_SEG_NCHUNKS] + g] = (int32_t)(cn < 0 ? 0 : cn);
      p[p[PLAN_OFF_SEG_SEQ] + g] = s;
      p[p[PLAN_OFF_SEG_FLAGS] + g] = (i == 0 ? SEG_FIRST : 0) | (i == ns - 1 ? SEG_LAST : 0);
      ++g;
    }
    for (int64_t i = 0; i < nc; ++i) {
      p[p[PLAN_OFF_CHUNK_TOK0] + c] = (int32_t)(bos + i * GDR_C);
      p[p[PLAN_OFF_CHUNK_LEN] + c] = (int32_t)(len - i * GDR_C < GDR_C ? len - i * GDR_C : GDR_C);
      ++c;
    }
  }
  return LAMPA_OK;
}


// Host-side construction of the plan (see gdr_plan.h). No device code.
#include "gdr_plan.h"
#include <algorithm>
#include <vector>

// Segments per sequence. cps > 0: segments of cps chunks (the last one of a sequence may be shorter).
// cps == 0: `target` segments in all, dealt out so that the longest segment is as short as possible (every sequence
// starts with one segment and the next segment always goes to the sequence whose segments are longest); a sequence's
// segments then differ by at most one chunk. An empty sequence still owns one (empty) segment.
// cps < 0: the caller's own segment lengths (`lens`, `target` of them: sequence after sequence, every sequence's
// lengths adding up to its chunks; an empty sequence takes one length of 0).
static int plan_segments(const int64_t* cu, int n_seq, int cps, int64_t target, std::vector<int64_t>& ns,
                         int64_t* n_chunks, int64_t* n_segments, const int32_t* lens = nullptr) {
  ns.assign(n_seq, 1);
  if (cps < 0) {
    int64_t chunks = 0, at = 0;
    for (int s = 0; s < n_seq; ++s) {
      const int64_t len = cu[s + 1] - cu[s];
      if (len < 0) return -1;
      const int64_t nc = (len + GDR_C - 1) / GDR_C;
      int64_t sum = 0, cnt = 0;
      do {
        if (at >= target || lens[at] < 0 || (nc > 0 && lens[at] == 0)) return -1;
        sum += lens[at++];
        ++cnt;
      } while (sum < nc);
      if (sum != nc) return -1;
      ns[s] = cnt;
      chunks += nc;
    }
    if (at != target) return -1;
    *n_chunks = chunks;
    *n_segments = target;
    return 0;
  }
  int64_t chunks = 0, segs = 0;
  std::vector<int64_t> nc(n_seq);
  for (int s = 0; s < n_seq; ++s) {
    const int64_t len = cu[s + 1] - cu[s];
    if (len < 0) return -1;
    nc[s] = (len + GDR_C - 1) / GDR_C;
    chunks += nc[s];
    if (cps > 0 && nc[s] > 0) ns[s] = (nc[s] + cps - 1) / cps;
    segs += ns[s];
  }
  if (cps == 0) {
    for (; segs < target; ++segs) {
      int best = -1;
      for (int s = 0; s < n_seq; ++s) {  // longest segments = largest nc / ns, compared without division
        if (nc[s] <= ns[s]) continue;    // already one chunk per segment
        if (best < 0 || nc[s] * ns[best] > nc[best] * ns[s]) best = s;
      }
      if (best < 0) break;
      ++ns[best];
    }
  }
  *n_chunks = chunks;
  *n_segments = segs;
  return 0;
}

static int64_t plan_size(const int64_t* cu, int n_seq, int cps, int64_t target) {
  std::vector<int64_t> ns;
  int64_t chunks, segs;
  if (plan_segments(cu, n_seq, cps, target, ns, &chunks, &segs) != 0) return LAMPA_ERR_INVALID;
  if (cu[n_seq] > INT32_MAX) return LAMPA_ERR_UNSUPPORTED;
  return PLAN_HEADER + 2 * chunks + 5 * segs + 2 * (int64_t)n_seq;
}

// Number of int32 entries of the plan for these sequences (negative on error).
extern "C" int64_t lampa_gdr_plan_size(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment) {
  if (!cu_seqlens_host || n_seq < 1 || chunks_per_segment < 1) return LAMPA_ERR_INVALID;
  return plan_size(cu_seqlens_host, n_seq, chunks_per_segment, 0);
}
extern "C" int64_t lampa_gdr_plan_size_balanced(const int64_t* cu_seqlens_host, int n_seq, int total_segments) {
  if (!cu_seqlens_host || n_seq < 1 || total_segments < 1) return LAMPA_ERR_INVALID;
  return plan_size(cu_seqlens_host, n_seq, 0, total_segments);
}

static int plan_fill(const int64_t* cu_seqlens_host, int n_seq, int cps, int64_t target, int32_t* plan_host,
                     const int32_t* lens = nullptr) {
  std::vector<int64_t> seq_ns;
  int64_t chunks, segs;
  if (plan_segments(cu_seqlens_host, n_seq, cps, target, seq_ns, &chunks, &segs, lens) != 0) return LAMPA_ERR_INVALID;
  if (cu_seqlens_host[n_seq] > INT32_MAX) return LAMPA_ERR_UNSUPPORTED;
  int32_t* p = plan_host;
  for (int i = 0; i < PLAN_HEADER; ++i) p[i] = 0;
  p[PLAN_N_SEQ] = n_seq;
  p[PLAN_TOTAL_CHUNKS] = (int32_t)chunks;
  p[PLAN_N_SEGMENTS] = (int32_t)segs;
  p[PLAN_CHUNKS_PER_SEGMENT] = cps > 0 ? cps : 0;  // 0: segments of unequal length
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
  p[PLAN_OFF_SEG_ORDER] = (int32_t)off; off += segs;
  int64_t c = 0, g = 0;
  for (int s = 0; s < n_seq; ++s) {
    const int64_t bos = cu_seqlens_host[s], len = cu_seqlens_host[s + 1] - bos;
    const int64_t nc = (len + GDR_C - 1) / GDR_C;
    const int64_t ns = seq_ns[s];
    p[p[PLAN_OFF_SEQ_SEG0] + s] = (int32_t)g;
    p[p[PLAN_OFF_SEQ_NSEG] + s] = (int32_t)ns;
    // segments of cps chunks, or (cps == 0) the first nc % ns segments one chunk longer than the others
    const int64_t lo = nc / ns, longer = nc % ns;
    int64_t c0 = 0;
    for (int64_t i = 0; i < ns; ++i) {
      int64_t cn = cps > 0 ? (nc - c0 < cps ? nc - c0 : cps) : cps < 0 ? lens[g] : lo + (i < longer ? 1 : 0);
      p[p[PLAN_OFF_SEG_CHUNK0] + g] = (int32_t)(c + c0);
      p[p[PLAN_OFF_SEG_NCHUNKS] + g] = (int32_t)(cn < 0 ? 0 : cn);
      p[p[PLAN_OFF_SEG_SEQ] + g] = s;
      p[p[PLAN_OFF_SEG_FLAGS] + g] = (i == 0 ? SEG_FIRST : 0) | (i == ns - 1 ? SEG_LAST : 0);
      c0 += cn < 0 ? 0 : cn;
      ++g;
    }
    for (int64_t i = 0; i < nc; ++i) {
      p[p[PLAN_OFF_CHUNK_TOK0] + c] = (int32_t)(bos + i * GDR_C);
      p[p[PLAN_OFF_CHUNK_LEN] + c] = (int32_t)(len - i * GDR_C < GDR_C ? len - i * GDR_C : GDR_C);
      ++c;
    }
  }
  // Workgroups start in the order of their index, and a batch may need several rounds of them: with the long segments
  // first and the short ones last, the workgroups of the last round end together (the first free slots, those of the
  // shortest segments, take the longest of the next head).
  int32_t* order = p + p[PLAN_OFF_SEG_ORDER];
  const int32_t* len = p + p[PLAN_OFF_SEG_NCHUNKS];
  for (int64_t i = 0; i < segs; ++i) order[i] = (int32_t)i;
  std::stable_sort(order, order + segs, [len](int32_t a, int32_t b) { return len[a] > len[b]; });
  return LAMPA_OK;
}

// Fills plan_host (lampa_gdr_plan_size entries). The caller copies it to the device and passes that pointer on.
extern "C" int lampa_gdr_plan_fill(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment,
                                   int32_t* plan_host) {
  if (!plan_host || !cu_seqlens_host || n_seq < 1 || chunks_per_segment < 1) return LAMPA_ERR_INVALID;
  return plan_fill(cu_seqlens_host, n_seq, chunks_per_segment, 0, plan_host);
}
// The same tables with total_segments segments of nearly equal length over all sequences (more when there are more
// sequences than that, fewer when there are fewer chunks): for batches whose workgroups take several rounds on the chip.
extern "C" int lampa_gdr_plan_fill_balanced(const int64_t* cu_seqlens_host, int n_seq, int total_segments,
                                            int32_t* plan_host) {
  if (!plan_host || !cu_seqlens_host || n_seq < 1 || total_segments < 1) return LAMPA_ERR_INVALID;
  return plan_fill(cu_seqlens_host, n_seq, 0, total_segments, plan_host);
}
// The same tables with the caller's own segment lengths: seg_chunks[n_segments], the segments of sequence 0 first, every
// sequence's lengths adding up to its number of 64-token chunks (an empty sequence takes one segment of 0 chunks).
extern "C" int64_t lampa_gdr_plan_size_lengths(const int64_t* cu_seqlens_host, int n_seq, const int32_t* seg_chunks,
                                               int n_segments) {
  if (!cu_seqlens_host || !seg_chunks || n_seq < 1 || n_segments < n_seq) return LAMPA_ERR_INVALID;
  std::vector<int64_t> ns;
  int64_t chunks, segs;
  if (plan_segments(cu_seqlens_host, n_seq, -1, n_segments, ns, &chunks, &segs, seg_chunks) != 0) return LAMPA_ERR_INVALID;
  if (cu_seqlens_host[n_seq] > INT32_MAX) return LAMPA_ERR_UNSUPPORTED;
  return PLAN_HEADER + 2 * chunks + 5 * segs + 2 * (int64_t)n_seq;
}
extern "C" int lampa_gdr_plan_fill_lengths(const int64_t* cu_seqlens_host, int n_seq, const int32_t* seg_chunks,
                                           int n_segments, int32_t* plan_host) {
  if (!plan_host || !cu_seqlens_host || !seg_chunks || n_seq < 1 || n_segments < n_seq) return LAMPA_ERR_INVALID;
  return plan_fill(cu_seqlens_host, n_seq, -1, n_segments, plan_host, seg_chunks);
}

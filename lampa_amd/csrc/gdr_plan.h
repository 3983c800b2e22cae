// Chunk / segment tables ("plan") of the chunkwise gated-delta forward, built on the host.
//
// Replaces prepare_chunk_indices / prepare_chunk_offsets (reference chengjiang123/Lampa,
// models/hattention/index.py:69-83): chunks of 64 tokens never straddle a sequence; on top of that the plan cuts
// every sequence into segments of `chunks_per_segment` chunks for the split-sequence scan.
#pragma once
#include "common.h"

#define GDR_C 64  // chunk length

// layout of the plan (int32 entries)
enum {
  PLAN_N_SEQ = 0,
  PLAN_TOTAL_CHUNKS = 1,
  PLAN_N_SEGMENTS = 2,
  PLAN_CHUNKS_PER_SEGMENT = 3,
  PLAN_OFF_CHUNK_TOK0 = 4,
  PLAN_OFF_CHUNK_LEN = 5,
  PLAN_OFF_SEG_CHUNK0 = 6,
  PLAN_OFF_SEG_NCHUNKS = 7,
  PLAN_OFF_SEG_SEQ = 8,
  PLAN_OFF_SEG_FLAGS = 9,
  PLAN_OFF_SEQ_SEG0 = 10,
  PLAN_OFF_SEQ_NSEG = 11,
  PLAN_TOTAL_TOKENS = 12,
  PLAN_OFF_SEG_ORDER = 13,  // the segments from the longest to the shortest: the order the segment kernels take them in
  PLAN_HEADER = 16
};
#define SEG_FIRST 1
#define SEG_LAST 2


// Host side of the chunkwise gated-delta-rule forward: workspace layout, launch sequence and the C entry points.
// The kernels (and the description of the algorithm) are in gdr_chunk_kernels.h.
#include "gdr_chunk_kernels.h"
#include <atomic>
#include <mutex>

struct GdrWorkspace {
  int64_t off_t, off_m, off_n, off_d, off_sinit, off_gm, off_gn, off_gd, max_groups, bytes;
};

static GdrWorkspace gdr_workspace(int64_t chunks, int64_t segs, int HV, int K, int V) {
  GdrWorkspace w;
  int64_t off = 0;
  w.off_t = off;     off += lampa_align_up(chunks * HV * (int64_t)REC_BYTES, 256);
  w.off_m = off;     off += lampa_align_up(segs * HV * (int64_t)K * K * 2, 256);
  w.off_n = off;     off += lampa_align_up(segs * HV * (int64_t)K * V * 4, 256);
  w.off_d = off;     off += lampa_align_up(segs * HV * 4, 256);
  w.off_sinit = off; off += lampa_align_up((segs + 1) * HV * (int64_t)K * V * 4, 256);  // + a spare slot (scan)
  // two-level scan: composites of the groups of GDR_SCAN_GROUP segments
  w.max_groups = segs / GDR_SCAN_GROUP + 2;
  w.off_gm = off;    off += lampa_align_up(w.max_groups * HV * (int64_t)K * K * 2, 256);
  w.off_gn = off;    off += lampa_align_up(w.max_groups * HV * (int64_t)K * V * 4, 256);
  w.off_gd = off;    off += lampa_align_up(w.max_groups * HV * 4, 256);
  w.bytes = off > 0 ? off : 256;
  return w;
}

// Output pass with narrow chain waves (16 value columns per wave on the 16x16x32 MFMA; built for K >= 64).
// 0: never, 1: where it is the faster form (heads wider than 64 x 64), 2: wherever it is built.
static std::atomic<int> gdr_narrow_output{1};
extern "C" int lampa_gdr_chunk_config(int narrow_output) {
  if (narrow_output < 0 || narrow_output > 2) return LAMPA_ERR_INVALID;
  gdr_narrow_output.store(narrow_output);
  return LAMPA_OK;
}

static bool gdr_chunk_supported(int K, int V) {
  return ((K == 64 || K == 128) && (V == 64 || V == 128)) || (K == 32 && V == 32);
}

extern "C" int64_t lampa_gdr_chunk_workspace_bytes(int64_t total_chunks, int64_t n_segments, int HV, int K, int V) {
  if (total_chunks < 0 || n_segments < 0 || HV < 1) return LAMPA_ERR_INVALID;
  if (!gdr_chunk_supported(K, V)) return LAMPA_ERR_UNSUPPORTED;
  return gdr_workspace(total_chunks, n_segments, HV, K, V).bytes;
}

template <typename T, int KT, int VT>
static int gdr_chunk_launch(const void* q, const void* k, const void* v, const float* g, const float* beta, void* o,
                            const float* h0, float* ht, const GdrPlanView pv, int n_seq, int chunks, int segs, int max_nseg,
                            int H, int HV, float scale, int l2norm, unsigned char* ws, hipStream_t s) {
  const GdrWorkspace w = gdr_workspace(chunks, segs, HV, KT, VT);
  unsigned char* tf = ws + w.off_t;
  unsigned char* Mc = ws + w.off_m;
  unsigned char* Nc = ws + w.off_n;
  float* Dc = (float*)(ws + w.off_d);
  float* Si = (float*)(ws + w.off_sinit);
  constexpr int smem_a = GdrSegSmem<KT, VT, false>::BYTES, smem_b = GdrSegSmem<KT, VT, true>::BYTES;
  constexpr int CWN = KT >= 64 ? 16 : 32;  // chain-wave width of the narrow output pass (K = 32 has none)
  constexpr int smem_n = GdrSegSmem<KT, VT, true, false, GdrSegShape<KT, VT, true, CWN>::DOUBLE_Q ? 2 : 1>::BYTES;
  // the dynamic LDS limit is a per-device attribute of a kernel: set once per device and instantiation
  static bool attr_set[64] = {};
  static std::mutex attr_lock;  // (several host threads may call at once)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LAMPA_ERR_LAUNCH;
  std::unique_lock<std::mutex> hold(attr_lock);
  if (!attr_set[dev]) {
    if (hipFuncSetAttribute((const void*)gdr_segment_kernel<T, KT, VT, false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, smem_a) != hipSuccess ||
        hipFuncSetAttribute((const void*)gdr_segment_kernel<T, KT, VT, true>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, smem_b) != hipSuccess ||
        hipFuncSetAttribute((const void*)gdr_segment_kernel<T, KT, VT, true, false, T, CWN>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, smem_n) != hipSuccess)
      return LAMPA_ERR_LAUNCH;
    attr_set[dev] = true;
  }
  hold.unlock();
  LAMPA_PROF(s, "start");
  if (chunks > 0) {
    hipLaunchKernelGGL((gdr_local_kernel<T, T, KT>), dim3(gdr_local_grid(chunks, HV)), dim3(64), 0, s, (const T*)k, g, beta,
                       pv.chunk_tok0, pv.chunk_len, tf, chunks, H, HV, l2norm);
    LAMPA_PROF(s, "gdr_local_kernel");
    if (segs > n_seq) {
      hipLaunchKernelGGL((gdr_segment_kernel<T, KT, VT, false>), dim3(segs * HV), dim3(64 * GdrSegShape<KT, VT, false>::WAVES), smem_a, s,
                         (const T*)q, (const T*)k, (const T*)v, g, beta, pv, pv.chunk_tok0, pv.chunk_len, tf, (const float*)nullptr, Mc, Nc, Dc,
                         (T*)nullptr, (float*)nullptr, H, HV, scale, l2norm, (const unsigned char*)nullptr,
                         (const unsigned char*)nullptr, (const float*)nullptr, (const float*)nullptr, 0);
      LAMPA_PROF(s, "gdr_segment_kernel<composite>");
    }
  }
  const int gmax = (max_nseg + GDR_SCAN_GROUP - 1) / GDR_SCAN_GROUP;
  unsigned char* Gm = ws + w.off_gm;
  unsigned char* Gn = ws + w.off_gn;
  float* Gd = (float*)(ws + w.off_gd);
  // The output pass can walk the composites before its segment itself (K = 64: its chain waves hold whole columns
  // of the state in few enough registers); otherwise a leaf pass writes every segment's initial state.
  const bool two_level = max_nseg >= 3 * GDR_SCAN_GROUP && (int64_t)n_seq * gmax <= w.max_groups;
  const bool walk_in_output = two_level && KT == 64;
  if (two_level) {
    // long sequences: group composites, then every group's scan (which walks the earlier groups' composites first)
    const dim3 block(64 * (KT / 32));
    hipLaunchKernelGGL((gdr_scan2_kernel<T, KT, VT, 4, SCAN_GROUP>), dim3((KT + VT) / 32 * gmax, n_seq, HV), block, 0, s, pv, Mc,
                       Nc, Dc, (const float*)nullptr, (float*)nullptr, Gm, Gn, Gd, HV, 0, gmax);
    LAMPA_PROF(s, "gdr_scan2_kernel<group>");
    if (!walk_in_output) {
      hipLaunchKernelGGL((gdr_scan2_kernel<T, KT, VT, 4, SCAN_LEAF>), dim3(VT / 32 * gmax, n_seq, HV), block, 0, s, pv, Mc, Nc,
                         Dc, h0, Si, Gm, Gn, Gd, HV, segs, gmax);
      LAMPA_PROF(s, "gdr_scan2_kernel<leaf>");
    }
  } else {
    hipLaunchKernelGGL((gdr_scan_kernel<T, KT, VT, 4>), dim3(n_seq, HV, VT / 32), dim3(64 * (KT / 32)), 0, s,
                       pv, Mc, Nc, Dc, h0, Si, HV, segs);
    LAMPA_PROF(s, "gdr_scan_kernel");
  }
  const int narrow = gdr_narrow_output.load();
  if (CWN == 16 && (narrow == 2 || (narrow == 1 && KT + VT > 128)))
    hipLaunchKernelGGL((gdr_segment_kernel<T, KT, VT, true, false, T, CWN>), dim3(segs * HV),
                       dim3(64 * GdrSegShape<KT, VT, true, CWN>::WAVES), smem_n, s, (const T*)q, (const T*)k, (const T*)v, g, beta,
                       pv, pv.chunk_tok0, pv.chunk_len, tf, Si, Mc, Nc, Dc, (T*)o, ht, H, HV, scale, l2norm,
                       (const unsigned char*)Gm, (const unsigned char*)Gn, (const float*)Gd, h0, walk_in_output ? gmax : 0);
  else
  hipLaunchKernelGGL((gdr_segment_kernel<T, KT, VT, true>), dim3(segs * HV), dim3(64 * GdrSegShape<KT, VT, true>::WAVES), smem_b, s, (const T*)q,
                     (const T*)k, (const T*)v, g, beta, pv, pv.chunk_tok0, pv.chunk_len, tf, Si, Mc, Nc, Dc, (T*)o, ht, H, HV, scale,
                     l2norm, (const unsigned char*)Gm, (const unsigned char*)Gn, (const float*)Gd, h0, walk_in_output ? gmax : 0);
  LAMPA_PROF(s, "gdr_segment_kernel<output>");
  return lampa_launch_status();
}

// Chunkwise forward. q, k [total_tokens, H, K]; v, o [total_tokens, HV, V] (dtype 0 bf16 / 1 fp16); g, beta fp32
// [total_tokens, HV]; h0, ht fp32 [n_seq, HV, K, V] (nullable). plan_host / plan_dev: the same plan
// (lampa_gdr_plan_fill) in host and in device memory. workspace: lampa_gdr_chunk_workspace_bytes bytes.
extern "C" int lampa_gdr_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                   void* o, const float* h0, float* ht, const int32_t* plan_host,
                                   const int32_t* plan_dev, int H, int HV, int K, int V, int dtype, float scale,
                                   int l2norm, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!q || !k || !v || !g || !beta || !o || !plan_host || !plan_dev) return LAMPA_ERR_INVALID;
  if (H < 1 || HV < H || HV % H != 0 || l2norm < 0 || l2norm > 2) return LAMPA_ERR_INVALID;
  if (!gdr_chunk_supported(K, V) || (dtype != GDR_BF16 && dtype != GDR_FP16)) return LAMPA_ERR_UNSUPPORTED;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & 15) return LAMPA_ERR_INVALID;
  const int n_seq = plan_host[PLAN_N_SEQ], chunks = plan_host[PLAN_TOTAL_CHUNKS], segs = plan_host[PLAN_N_SEGMENTS];
  if (n_seq < 1 || segs < n_seq) return LAMPA_ERR_INVALID;
  if (!workspace || workspace_bytes < gdr_workspace(chunks, segs, HV, K, V).bytes) return LAMPA_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  unsigned char* ws = (unsigned char*)workspace;
  const GdrPlanView pv = gdr_plan_view(plan_host, plan_dev);
  int max_nseg = 0;
  for (int i = 0; i < n_seq; ++i) max_nseg = plan_host[plan_host[PLAN_OFF_SEQ_NSEG] + i] > max_nseg ? plan_host[plan_host[PLAN_OFF_SEQ_NSEG] + i] : max_nseg;
#define GDR_CASE(TT, KK, VV)                                                                                       \
  return gdr_chunk_launch<TT, KK, VV>(q, k, v, g, beta, o, h0, ht, pv, n_seq, chunks, segs, max_nseg, H, HV, scale, \
                                      l2norm, ws, s)
  if (dtype == GDR_BF16) {
    if (K == 32 && V == 32) GDR_CASE(__bf16, 32, 32);
    if (K == 64 && V == 64) GDR_CASE(__bf16, 64, 64);
    if (K == 64 && V == 128) GDR_CASE(__bf16, 64, 128);
    if (K == 128 && V == 64) GDR_CASE(__bf16, 128, 64);
    if (K == 128 && V == 128) GDR_CASE(__bf16, 128, 128);
  } else {
    if (K == 32 && V == 32) GDR_CASE(_Float16, 32, 32);
    if (K == 64 && V == 64) GDR_CASE(_Float16, 64, 64);
    if (K == 64 && V == 128) GDR_CASE(_Float16, 64, 128);
    if (K == 128 && V == 64) GDR_CASE(_Float16, 128, 64);
    if (K == 128 && V == 128) GDR_CASE(_Float16, 128, 128);
  }
#undef GDR_CASE
  return LAMPA_ERR_UNSUPPORTED;
}

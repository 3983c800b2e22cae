/*
 * lampa_amd.h -- C ABI of liblampa_amd.so: the MI355X (gfx950) implementation of Lampa's data-parallel hot path,
 * E2LSH hashing + stable bucket sort + gather of detector hits, then the chunkwise gated-delta-rule forward.
 *
 * Conventions
 *   - every pointer named *_dev or documented as "device" is HIP device memory on the current device; inputs are
 *     never modified; outputs and workspaces are caller-allocated (query the *_workspace_bytes function first);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); all work is enqueued on it and the
 *     functions return without synchronising;
 *   - return value: 0 on success, negative on error (LAMPA_ERR_*). No C++ exception crosses the boundary;
 *   - state the library keeps between calls: the optional profiling recorder; one helper stream with two events per
 *     (device, caller stream) that lampa_hgdn_chunk_fwd creates on first use and keeps until the process ends (calls
 *     on different streams or host threads never share them); the fixed scratch array of lampa_sort_pairs_static;
 *     per device, how many workgroups of the one-launch LSH kernel the GPU holds (looked up once) and a flag that the
 *     dynamic-LDS limits of the chunk, step, scan and backward kernels have been raised (set on the first call there).
 *     Everything else lives in caller-owned buffers, so calls on different streams do not interfere.
 * The reference (chengjiang123/Lampa) is Python over Triton/ATen, so each entry point names the Python operator or
 * kernel it replaces (file:line in the reference tree).
 */
#ifndef LAMPA_AMD_H
#define LAMPA_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LAMPA_OK 0
#define LAMPA_ERR_INVALID (-1)     /* bad argument */
#define LAMPA_ERR_WORKSPACE (-2)   /* workspace missing or too small */
#define LAMPA_ERR_LAUNCH (-3)      /* HIP reported an error at launch */
#define LAMPA_ERR_UNSUPPORTED (-4) /* shape / dtype outside what the kernels are built for */

/* key kinds of lampa_sort_pairs */
#define LAMPA_KEY_U32 0
#define LAMPA_KEY_I32 1
#define LAMPA_KEY_F32 2 /* torch.sort order: -0.0 == +0.0, NaN last */

/* element types of q, k, v, o */
#define LAMPA_BF16 0
#define LAMPA_FP16 1
#define LAMPA_FP32 2

/* l2 normalisation of q and k inside the kernel */
#define LAMPA_L2_NONE 0
#define LAMPA_L2_CHUNK 1     /* x / sqrt(sum x^2 + 1e-6)      models/hattention/l2norm.py:97-103 */
#define LAMPA_L2_RECURRENT 2 /* x / (sqrt(sum x^2) + 1e-6)    models/hattention/gated_delta_rule_ori.py:436-438 */

/* ------------------------------------------------------------------------------------------------ LSH stage */

/* E2LSH projection. Replaces E2LSH.forward = torch.bmm(vecs, alpha) + permute
 * (models/model_utils/hash_utils.py:368-371; models/baselines/full_mamba2.py:136-141).
 * vecs [n_heads, n_hits, dim] fp32, alpha [n_heads, dim, n_cols] fp32; out element (c, head, n) is written at
 * out[c*stride_c + head*stride_h + n*stride_n] (so both reference layouts are one call).
 * Arithmetic: p = fmaf(x[d], a[d], p) for d = 0..dim-1 starting from 0. */
int lampa_lsh_project_f32(const float* vecs, int n_heads, int64_t n_hits, int dim, const float* alpha, int n_cols,
                          float* out, int64_t stride_c, int64_t stride_h, int64_t stride_n, void* stream);

/* Per-row (min, max) of x [rows, n] -> out [rows, 2]. Replaces the four max/min reductions of lsh_mapping
 * (models/model_utils/hash_utils.py:334-340). */
int lampa_row_minmax_f32(const float* x, int rows, int64_t n, float* out, void* stream);

/* Quantised E2LSH bucket ids and mixed-radix bucket keys of one event.
 * Replaces the hash + range + key-combination steps of the reference's bucketing front end
 * (hash_utils.py:333-371, models/attention/hept.py:79-88) with the textbook id floor((a.x + b) / w).
 * coords [n_hits, dim] fp32 (dim <= 8); alpha [dim, n_tables*n_proj]; beta [n_tables*n_proj]; column
 * c = table*n_proj + projection. Hits n >= n_valid are padding (ids 0, key = total so that they sort last).
 * ids_out [n_tables*n_proj, n_hits] int32 (nullable), keys_out [n_tables, n_hits] int32,
 * meta_out [n_tables, 2*n_proj+3] int32 = lo[n_proj], range[n_proj], total, key_bits, overflow. */
int64_t lampa_lsh_bucket_workspace_bytes(int64_t n_hits, int n_tables, int n_proj);
int lampa_lsh_bucket_keys(const float* coords, int64_t n_hits, int64_t n_valid, int dim, const float* alpha,
                          const float* beta, int n_tables, int n_proj, float w, int32_t* ids_out, int32_t* keys_out,
                          int32_t* meta_out, void* workspace, int64_t workspace_bytes, void* stream);

/* The whole bucketing stage of one event in one call: lampa_lsh_bucket_keys, then lampa_sort_pairs on the packed
 * keys (digit widths from meta, read on the device), then lampa_gather_rows of the hit features when feats != NULL.
 * Replaces the hash -> argsort -> sort_to_buckets sequence of models/attention/hept.py:127-143.
 * perm_out [n_tables, n_hits] int32; feats [n_hits, feat_row_bytes] -> feats_out [n_tables, n_hits, feat_row_bytes].
 * n_passes: 0 (automatic), 3 or 4 sort launches for the 32-bit keys.
 * A call (this one or the batch form) of at most 64 tables whose tiles of 1 024 hits come to at most two workgroups
 * per CU (one or two events of 60 000 hits on 256 CUs), with feature rows made of 16-byte pieces, runs as ONE
 * kernel whose workgroups wait for the other workgroups of their table (flags in the
 * workspace; no host-visible state); any other call runs as separate kernels. The results are the same bits. The waits
 * are bounded: should one run out (two such kernels sharing one GPU at the same time can starve each other), bit 1 of the
 * table's overflow field in meta_out is set, the table's perm_out rows are all -1 and its feats_out rows all zero (every
 * kernel still ends normally): the failure shows in the outputs themselves. Calls of the stage that could overlap on one
 * GPU should therefore be serialised by the caller. */
int64_t lampa_lsh_bucket_sort_workspace_bytes(int64_t n_hits, int n_tables, int n_proj);
int lampa_lsh_bucket_sort(const float* coords, int64_t n_hits, int64_t n_valid, int dim, const float* alpha,
                          const float* beta, int n_tables, int n_proj, float w, int32_t* ids_out, int32_t* keys_out,
                          int32_t* meta_out, int32_t* perm_out, const void* feats, int64_t feat_row_bytes,
                          void* feats_out, int n_passes, void* workspace, int64_t workspace_bytes, void* stream);

/* The same stage for a batch of events in one set of launches (events are independent: own id ranges, own key
 * width; the sort runs over n_events * n_tables segments). This is the data-parallel form of the loop over events
 * around hept.py:127-143. coords [n_events, n_hits, dim]; n_valid_dev: device int32 [n_events] or NULL (all valid);
 * ids_out [E, T*J, N] (nullable), keys_out / perm_out [E, T, N], meta_out [E, T, 2J+3],
 * feats [E, N, feat_row_bytes] -> feats_out [E, T, N, feat_row_bytes]. */
int64_t lampa_lsh_bucket_sort_batch_workspace_bytes(int n_events, int64_t n_hits, int n_tables, int n_proj);
int lampa_lsh_bucket_sort_batch(const float* coords, int n_events, int64_t n_hits, const int32_t* n_valid_dev, int dim,
                                const float* alpha, const float* beta, int n_tables, int n_proj, float w,
                                int32_t* ids_out, int32_t* keys_out, int32_t* meta_out, int32_t* perm_out,
                                const void* feats, int64_t feat_row_bytes, void* feats_out, int n_passes,
                                void* workspace, int64_t workspace_bytes, void* stream);

/* Sort keys of LSHOrdering: key[n] = sum_h 2^h <coords[n], alpha[:, h]>, norm[n] = |coords[n]|.
 * Replaces models/baselines/full_mamba2.py:174-203. coords [n_hits, dim], alpha [dim, n_hashes]. */
int lampa_lsh_ordering_keys(const float* coords, int64_t n_hits, int dim, const float* alpha, int n_hashes,
                            float* key_out, float* norm_out, void* stream);

/* Stable ascending segmented radix sort of (32-bit key, int32 payload) pairs; payload defaults to the position.
 * Replaces argsort / sort(stable=True) (models/attention/hept.py:138-139; full_mamba2.py:203,207,678).
 * keys_in [n_segments, n]; vals_in [n_segments, n] or NULL; vals_out [n_segments, n].
 * key_bits (1..32) or key_bits_dev (device, element s at key_bits_dev[s*key_bits_stride]) bound the significant
 * bits of LAMPA_KEY_U32 keys; n_passes 0 = automatic. */
int64_t lampa_sort_workspace_bytes(int n_segments, int64_t n);
int lampa_sort_pairs(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments, int64_t n,
                     int key_bits, const int32_t* key_bits_dev, int key_bits_stride, int n_passes,
                     int32_t* vals_out, void* workspace, int64_t workspace_bytes, void* stream);

/* lampa_sort_pairs for callers that cannot allocate device memory or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same
 * arguments, same kernels and bit-identical results; the ping-pong buffers and histograms live in a fixed 8 MiB array
 * inside the library image (one copy per GPU, held until the process ends), so the call allocates nothing.
 * lampa_sort_workspace_bytes(n_segments, n) must not exceed lampa_sort_pairs_static_max_bytes() (8 MiB: e.g. 3
 * segments of 140 000 keys), otherwise LAMPA_ERR_WORKSPACE. All calls on one GPU share that array: calls that may
 * overlap on one GPU (different streams or host threads) race and must be serialised by the caller. */
int64_t lampa_sort_pairs_static_max_bytes(void);
int lampa_sort_pairs_static(const void* keys_in, int key_kind, const int32_t* vals_in, int n_segments, int64_t n,
                            int key_bits, const int32_t* key_bits_dev, int key_bits_stride, int n_passes,
                            int32_t* vals_out, void* stream);

/* dst[s, i, :] = src[s % src_segments, idx[s, i], :]. Replaces batched_index_select / sort_to_buckets /
 * unsort_from_buckets and the points.gather of LSHOrdering (hash_utils.py:83-93; hept.py:9-19;
 * full_mamba2.py:213-216,679-682). idx_bytes = 4 (int32) or 8 (int64); rows of row_bytes bytes. A row whose index
 * is outside [0, n_src) is written as zeros (torch.gather would raise; no device-side error exists here). */
int lampa_gather_rows(const void* src, int src_segments, int64_t n_src, const void* idx, int idx_bytes,
                      int n_segments, int64_t n, int64_t row_bytes, void* dst, void* stream);

/* dst[s, idx[s, i], :] = src[s, i, :] (unsort by scatter, the O(n) alternative to full_mamba2.py:678-682). Rows whose
 * index is outside [0, n) are dropped. */
int lampa_scatter_rows(const void* src, const void* idx, int idx_bytes, int n_segments, int64_t n,
                       int64_t row_bytes, void* dst, void* stream);

/* inv[s, perm[s, i]] = i. Replaces invert_permutation (hash_utils.py:46-57). */
int lampa_invert_perm(const void* perm, int idx_bytes, int n_segments, int64_t n, void* inv, void* stream);

/* 1-based quantile region of every hit for each row's number of regions. Replaces quantile_partition
 * (models/model_utils/hash_utils.py:14-26). rank [n] (idx_bytes 4 or 8): position of the hit in the coordinate order
 * (inverse of the argsort); regions [n_rows] device float32 > 0; out [n_rows, n] float32 =
 * floor(rank / ceil(n / regions[r])) + 1. n <= 2^24. */
int lampa_quantile_regions(const void* rank, int idx_bytes, int64_t n, const float* regions, int n_rows, float* out,
                           void* stream);

/* Region shift of the AND-hash. Replaces get_geo_shift (models/attention/hept.py:78-88).
 * out [n_rows, n] = (region_phi * hash_shift[r]) * (ceil(regions_eta[r]) + 1) + region_eta * hash_shift[r]. */
int lampa_geo_shift(const float* region_eta, const float* region_phi, const float* hash_shift,
                    const float* regions_eta, int n_rows, int64_t n, float* out, void* stream);

/* Sort keys of the HEPT bucketing in one pass. Replaces the arithmetic between lsh_mapping and argsort in
 * HEPTAttention.forward (models/attention/hept.py:127-136) without materialising the region indices.
 * hashed, keys [n_rows, n]; rank_eta, rank_phi [n] int32; regions [2, n_rows] (eta row, then phi row);
 * hash_shift [n_rows]; hits at or beyond n_raw get +inf before the shift is added. n <= 2^24. */
int lampa_hept_sort_keys(const float* hashed, const int32_t* rank_eta, const int32_t* rank_phi, const float* regions,
                         const float* hash_shift, int n_rows, int64_t n, int64_t n_raw, float* keys, void* stream);

/* Hash inputs of the HEPT bucketing. Replaces prep_qk and the rearrange + zeroing of the padded rows after it
 * (models/attention/hept.py:54-62,118-128): q_hat = [query | sqrt(2 qw) * coords] with qw[h, r] =
 * sum_k exp(min(sum_d w[h, d, r, k], 50)) and the first appended column reusing qw[h, 0]. query, key [n, H, d];
 * w [H, d, R, Kw]; coords [n, R + 1]; scale_ws: H * (R + 1) floats of device scratch; q_hat, k_hat [n, H, d + R + 1]
 * (heads_first 0) or [H, n, d + R + 1] (heads_first 1); rows at or beyond n_raw are zero. All fp32. */
int lampa_hept_prep_qk(const float* query, const float* key, const float* w, const float* coords, int64_t n, int64_t n_raw,
                       int H, int d, int R, int Kw, int heads_first, float* scale_ws, float* q_hat, float* k_hat,
                       void* stream);

/* ------------------------------------------------------------------------------ operators around the forward */

/* Depthwise causal short convolution with optional bias, SiLU and residual. Replaces causal_conv1d_fwd
 * (models/hattention/short_convolution.py:39-99,262-300). y[t, d] = act(bias[d] + sum_j weight[d, j] *
 * x[t - (W-1) + j, d]) + residual[t, d]; taps before the start of the token's sequence are zero.
 * x, residual, y [n_tokens, D] of dtype (LAMPA_BF16/FP16/FP32) with row strides in elements; weight fp32 [D, W],
 * bias fp32 [D] or NULL; cu_seqlens device int64 [n_seq+1] or NULL (then n_tokens / t_len sequences of t_len tokens);
 * activation 0 none, 1 SiLU. D and the strides multiples of 8, pointers 16-byte aligned, W <= 8.
 * y_split in (0, D): output columns [i*y_split, (i+1)*y_split) go to the i-th of D / y_split tensors
 * [n_tokens, y_split] that lie y_split_stride elements apart (one launch over the q|k|v columns of a fused projection
 * writing q, k and v); y_split <= 0: one [n_tokens, D] output. */
int lampa_causal_conv1d_fwd(const void* x, int64_t x_stride, int64_t n_tokens, int D, int W, const float* weight,
                            const float* bias, const void* residual, int64_t res_stride, const int64_t* cu_seqlens,
                            int n_seq, int64_t t_len, int activation, int dtype, void* y, int64_t y_stride, int y_split,
                            int64_t y_split_stride, void* stream);

/* Fused input projections + short convolution + SiLU of a gated-delta layer (bf16, hidden size K = 128). Replaces
 * the bias-free nn.Linear projections and the ShortConvolution calls after them
 * (models/hattention/modeling_gated_deltaproduct.py:505-547; models/hattention/short_convolution.py:39-99) without
 * writing the projection output to memory. x [n_tokens, K] bf16 (row stride x_stride), n_tokens / t_len dense sequences;
 * W [n_cols, K] bf16 = the projection weights one after the other. The first n_conv columns: y = silu(conv_b +
 * sum_j conv_w[n, j] * pre[t - 3 + j, n]) (4 taps, zero before a sequence start; the projection output rounded to bf16
 * first, as a bf16 linear layer's is), written as n_conv / conv_split tensors [n_tokens, conv_split] one after the
 * other at conv_out; the next plain_cols columns go to plain_out [n_tokens, plain_cols] as they are, the last
 * tail_cols (< 256, a multiple of 8) to tail_out [n_tokens, tail_cols]. n_conv, conv_split, plain_cols multiples of
 * 256. tokens_per_wg: tokens per workgroup run (0 = default). */
int lampa_proj_conv_fwd(const void* x, int64_t x_stride, int64_t n_tokens, int64_t t_len, int K, const void* W, int n_cols,
                        const float* conv_w, const float* conv_b, int n_conv, int conv_split, void* conv_out,
                        int plain_cols, void* plain_out, int tail_cols, void* tail_out, int tokens_per_wg, void* stream);

/* Gated RMS norm of every head fused with the output projection (bf16; 8 heads of 64 channels -> 128 columns).
 * Replaces FusedRMSNormSwishGate followed by o_proj (models/hattention/fused_norm.py:40-111 with the swish gate;
 * models/hattention/modeling_gated_deltaproduct.py:612-623): y[t] = W * vec(rmsnorm(o[t, h]) * norm_w * g[t, h] *
 * sigmoid(g[t, h])), the normalised tensor rounded to bf16 as the unfused pair would store it but never written.
 * o [n_tokens, heads, head_dim] contiguous; g the same shape with token stride g_stride elements; norm_w fp32
 * [head_dim] or NULL; W [n_out, heads * head_dim] row-major; y [n_tokens, n_out].
 * With residual [n_tokens, n_out] (bf16) the residual add and the next layer's pre-norm (RMSNorm with residual,
 * models/hattention/fused_norm.py:2307-2354, as GatedDeltaProductBlock.forward uses it) are applied too:
 * res_out = residual + projection, y = rmsnorm(res_out) * next_w (fp32 [n_out] or NULL) with next_eps. */
int lampa_norm_proj_fwd(const void* o, const void* g, int64_t g_stride, const float* norm_w, const void* W, int64_t n_tokens,
                        int heads, int head_dim, int n_out, float eps, void* y, const void* residual, const float* next_w,
                        float next_eps, void* res_out, int tokens_per_wg, void* stream);

/* RMS norm over the last dimension with optional residual add, weight, bias and output gate. Replaces
 * layer_norm_gated_fwd / layer_norm_fwd with is_rms_norm (models/hattention/fused_norm.py:40-111,456-531,1436-1506).
 * s = x + residual; residual_out = s; y = s / sqrt(mean(s^2) + eps) * weight + bias; with g: y *= g * sigmoid(g)
 * (activation 1) or sigmoid(g) (activation 2). x, g, y [rows, D] of dtype; residual, residual_out of res_dtype;
 * weight, bias fp32 [D]; rstd_out fp32 [rows]; every pointer but x and y may be NULL. D % 8 == 0, D <= 2048.
 * g_group > 0: g is a slice of a wider tensor with g_group rows of D channels per token and g_group_stride elements
 * between tokens (the g_proj columns of a fused projection output); g_group <= 0: g is [rows, D] contiguous. */
int lampa_rms_norm_fwd(const void* x, const void* g, const float* weight, const float* bias, const void* residual,
                       void* residual_out, void* y, float* rstd_out, int64_t rows, int D, float eps, int activation,
                       int dtype, int res_dtype, int g_group, int64_t g_group_stride, void* stream);

/* Decay and write gates of a gated-delta layer. Replaces the elementwise tail of GatedDeltaProduct.forward
 * (models/hattention/modeling_gated_deltaproduct.py:541-547,568-570): g = -exp(A_log) * softplus(a + dt_bias),
 * beta = sigmoid(b) * beta_scale (2 with allow_neg_eigval). a, b [n_tokens, H] of dtype, row strides in elements;
 * A_log, dt_bias fp32 [H]; g, beta fp32 [n_tokens, H]. */
int lampa_gdr_gates_fwd(const void* a, int64_t a_stride, const void* b, int64_t b_stride, const float* A_log,
                        const float* dt_bias, int64_t n_tokens, int H, float beta_scale, int dtype, float* g, float* beta,
                        void* stream);

/* ---------------------------------------------------------------------------------------- gated-delta forward */

/* Token-serial forward with an fp32 state. Replaces fused_recurrent_gated_delta_rule_fwd
 * (models/hattention/gated_delta_rule_ori.py:372-520); also the fp32 mode of the chunk operator.
 * q, k [tokens, H, K]; v, o [tokens, HV, V] (dtype LAMPA_BF16/FP16/FP32); g, beta fp32 [tokens, HV];
 * h0, ht fp32 [n_seq, HV, K, V] (nullable). cu_seqlens: device int64 [n_seq+1] or NULL (n_seq blocks of t_len). */
int lampa_gdr_recurrent_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta, void* o,
                            const float* h0, float* ht, const int64_t* cu_seqlens, int n_seq, int64_t t_len, int H,
                            int HV, int K, int V, int dtype, float scale, int l2norm, void* stream);

/* The same operator with one beta per value column: beta fp32 [tokens, HV, V]. Replaces the IS_BETA_HEADWISE branch of
 * fused_recurrent_gated_delta_rule_fwd_kernel (gated_delta_rule_ori.py:415-418,444-448), which its wrapper takes when
 * beta.ndim == v.ndim (gated_delta_rule_ori.py:515). Every other argument as for lampa_gdr_recurrent_fwd. */
int lampa_gdr_recurrent_headwise_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                     void* o, const float* h0, float* ht, const int64_t* cu_seqlens, int n_seq,
                                     int64_t t_len, int H, int HV, int K, int V, int dtype, float scale, int l2norm,
                                     void* stream);

/* The same operator (gated_delta_rule_ori.py:372-520) for a few long sequences, which one or two wavefronts each would
 * leave the GPU idle with: the caller cuts every sequence into segments and they run in parallel -- every segment's
 * affine map of its initial state, a short serial pass over the maps, then every segment again from its true initial
 * state; fp32 throughout, the same results up to fp32 rounding.
 * cu_seg: device int64 [n_seg+1] token offsets of the segments (every sequence boundary among them; an empty sequence
 * keeps one empty segment); seq_seg0: device int32 [n_seq+1], first segment of every sequence; seg_out: device int32
 * [n_seg], the sequence whose last segment this is, else -1. K and V multiples of 4, K <= 128, q and k 16-byte aligned
 * (LAMPA_ERR_UNSUPPORTED otherwise). workspace: lampa_gdr_recurrent_segmented_workspace_bytes(n_seg, HV, K, V). */
int64_t lampa_gdr_recurrent_segmented_workspace_bytes(int n_seg, int HV, int K, int V);
int lampa_gdr_recurrent_segmented_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                                      void* o, const float* h0, float* ht, const int64_t* cu_seg,
                                      const int32_t* seq_seg0, const int32_t* seg_out, int n_seq, int n_seg, int H,
                                      int HV, int K, int V, int dtype, float scale, int l2norm, void* workspace,
                                      int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------- gated-delta backward */

/* Gradients of the gated-delta forward (lampa_gdr_chunk_fwd and lampa_gdr_recurrent_fwd compute the same function)
 * with respect to q, k, v, g, beta and the initial state, given dout = d o and dht = d (final state). Replaces
 * chunk_gated_delta_rule_bwd (models/hattention/gated_delta_rule_ori.py:83-160) together with the l2norm_bwd calls of
 * ChunkGatedDeltaRuleFunction.backward (gated_delta_rule_ori.py:205-233): with l2norm != 0 the gradients are those of
 * the un-normalised q and k. fp32 arithmetic; token-serial inside segments that run in parallel.
 * q, k, dq, dk [total_tokens, H, K]; v, dout, dv [total_tokens, HV, V] (dtype LAMPA_BF16/FP16/FP32); g, beta, dg, dbeta
 * fp32 [total_tokens, HV]; h0, dht, dh0 fp32 [n_seq, HV, K, V], each nullable (zero initial state; no gradient into
 * the final state; d h0 not wanted).
 * The caller cuts every sequence into segments as for lampa_gdr_recurrent_segmented_fwd (cu_seg, seq_seg0) and adds
 * the tables of the pass that runs backwards: seq_seg0_rev device int32 [n_seq+1] = seq_seg0[s] + s, and seg_rev device
 * int32 [n_seg] = seq_seg0_rev[s] + (last segment of s) - p for segment p of sequence s.
 * K <= 128, K and V multiples of 4, q and k 16-byte aligned, at most 64 value heads per q/k head, n_seq <= 65535
 * (LAMPA_ERR_UNSUPPORTED otherwise). workspace: lampa_gdr_bwd_workspace_bytes(total_tokens, n_seq, n_seg, HV, K, V);
 * it grows with the tokens (the state kept at every 8th token) and with the segments: 1.9 GB for one sequence of
 * 60 000 tokens with 8 heads of 64 x 64 cut into 2048 units. */
int64_t lampa_gdr_bwd_workspace_bytes(int64_t total_tokens, int n_seq, int n_seg, int HV, int K, int V);
int lampa_gdr_bwd(const void* q, const void* k, const void* v, const float* g, const float* beta, const float* h0,
                  const void* dout, const float* dht, void* dq, void* dk, void* dv, float* dg, float* dbeta, float* dh0,
                  const int64_t* cu_seg, const int32_t* seq_seg0, const int32_t* seq_seg0_rev, const int32_t* seg_rev,
                  int64_t total_tokens, int n_seq, int n_seg, int H, int HV, int K, int V, int dtype, float scale,
                  int l2norm, void* workspace, int64_t workspace_bytes, void* stream);

/* The same gradients in the chunked (WY) form on the matrix cores, the form of the reference's own backward pass
 * (chunk_gated_delta_rule_bwd, models/hattention/gated_delta_rule_ori.py:83-160: chunk_bwd_dv_local chunk_o.py:372,
 * chunk_gated_delta_rule_bwd_dhu chunk_delta_h.py:209, chunk_bwd_dqkwg chunk_o.py:128, prepare_wy_repr_bwd wy_fast.py:27;
 * l2norm_bwd gated_delta_rule_ori.py:205-233): per chunk of 64 tokens the affine map of the state (forwards) and of its
 * gradient (backwards), a scan over the maps in three levels of groups of 8, then every gradient of a chunk from its tiles
 * and the two states. For K = V = 64, HV = H, dtype LAMPA_BF16 / LAMPA_FP16 (LAMPA_ERR_UNSUPPORTED otherwise: use
 * lampa_gdr_bwd); every intermediate operand is rounded to the input type, as in the forward pass, so all gradients
 * carry the rounding of that type. g <= 0 is assumed (the forward's masking of positive exponents is not differentiated).
 * Shapes as for lampa_gdr_bwd. plan: lampa_gdr_bwd_chunk_plan_fill's tables of the sequence boundaries
 * (cu_seqlens_host: int64 [n_seq+1]), the same int32 array in host and in device memory.
 * workspace: lampa_gdr_bwd_chunk_workspace_bytes(plan_host, HV): about 41 KiB per (chunk, head) -- the chunk's record,
 * its two map parts and the state and state gradient it starts from, all in the 16-bit input type, plus the maps and
 * states of the groups -- 0.33 GB for one sequence of 60 000 tokens with 8 heads (lampa_gdr_bwd: 1.9 GB there). */
int64_t lampa_gdr_bwd_chunk_plan_size(const int64_t* cu_seqlens_host, int n_seq);
int lampa_gdr_bwd_chunk_plan_fill(const int64_t* cu_seqlens_host, int n_seq, int32_t* plan_host);
int64_t lampa_gdr_bwd_chunk_workspace_bytes(const int32_t* plan_host, int HV);
int lampa_gdr_bwd_chunk(const void* q, const void* k, const void* v, const float* g, const float* beta, const float* h0,
                        const void* dout, const float* dht, void* dq, void* dk, void* dv, float* dg, float* dbeta,
                        float* dh0, const int32_t* plan_host, const int32_t* plan_dev, int H, int HV, int K, int V,
                        int dtype, float scale, int l2norm, void* workspace, int64_t workspace_bytes, void* stream);

/* Chunk / segment tables of the chunkwise forward, built on the host from the sequence boundaries.
 * Replaces prepare_chunk_indices / prepare_chunk_offsets (models/hattention/index.py:69-83).
 * cu_seqlens_host: int64 [n_seq+1]; chunks_per_segment: length of a segment of the split-sequence scan in
 * 64-token chunks. plan[1] = number of chunks, plan[2] = number of segments. */
int64_t lampa_gdr_plan_size(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment);
int lampa_gdr_plan_fill(const int64_t* cu_seqlens_host, int n_seq, int chunks_per_segment, int32_t* plan_host);
/* The same tables with total_segments segments over all sequences, dealt out so that the longest segment is as short
 * as possible (a sequence's segments differ by at most one chunk; every sequence owns at least one segment, and no
 * segment is cut below one chunk). For batches whose (segment, head) workgroups take several rounds on the chip: with
 * segments of one fixed length the last round is partly empty. plan[3] (chunks per segment) is 0 in such a plan. */
int64_t lampa_gdr_plan_size_balanced(const int64_t* cu_seqlens_host, int n_seq, int total_segments);
int lampa_gdr_plan_fill_balanced(const int64_t* cu_seqlens_host, int n_seq, int total_segments, int32_t* plan_host);
/* The same tables with the caller's own segment lengths: seg_chunks[n_segments] in 64-token chunks, the segments of
 * sequence 0 first; every sequence's lengths must add up to its chunks (an empty sequence takes one segment of 0). */
int64_t lampa_gdr_plan_size_lengths(const int64_t* cu_seqlens_host, int n_seq, const int32_t* seg_chunks, int n_segments);
int lampa_gdr_plan_fill_lengths(const int64_t* cu_seqlens_host, int n_seq, const int32_t* seg_chunks, int n_segments,
                                int32_t* plan_host);

/* Chunkwise forward (chunk = 64 tokens). Replaces chunk_gated_delta_rule_fwd and the seven Triton kernels it
 * launches (models/hattention/gated_delta_rule_ori.py:29-80). Shapes as above with H <= HV; K, V in {64, 128} or K = V = 32;
 * dtype LAMPA_BF16 or LAMPA_FP16; plan_host / plan_dev: the same plan in host and device memory. */
int64_t lampa_gdr_chunk_workspace_bytes(int64_t total_chunks, int64_t n_segments, int HV, int K, int V);
int lampa_gdr_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta, void* o,
                        const float* h0, float* ht, const int32_t* plan_host, const int32_t* plan_dev, int H, int HV,
                        int K, int V, int dtype, float scale, int l2norm, void* workspace, int64_t workspace_bytes,
                        void* stream);
/* Process-wide choice of the output pass's form (no counterpart in the reference; for A/B measurements). The pass
 * exists with 32 value columns per recurrence wave (32x32x16 MFMA) and, for K >= 64, with 16 ("narrow": 16x16x32 MFMA,
 * twice the waves, each with half the dependent chain of a chunk). narrow_output 0: never the narrow form; 1 (default):
 * where it is the faster one, i.e. for heads wider than 64 x 64; 2: wherever it is built. Results agree to rounding. */
int lampa_gdr_chunk_config(int narrow_output);

/* Hierarchical (level-weighted) chunkwise forward. Replaces chunk_h_gated_delta_rule -> hattention_kernel ->
 * chunkwise_fwd (models/hattention/gated_delta_rule_apis.py:21-91, kernel.py:338-374, chunkwise_hgdn.py:565-791;
 * specification: hattention_recurrent, recurrent.py:169-216, with HType.WEAK, HStruct.GDELTA, base 2).
 * lam: [total_tokens, HV, L] of type lam_dtype (LAMPA_BF16 / LAMPA_FP16 / LAMPA_FP32), the level weights; the kernel
 * uses lam / lam_div rounded to lam's type, which is what gated_delta_rule_apis.py:68-70 does with lam_div = scale
 * (lam_div = 1: as given). Level 0 = the token itself, level l > 0 = sources whose highest differing position bit is
 * l-1 (base.py:41-46).
 * K = 64, V in {64, 128}; l2norm as for the chunk forward (the reference requires the chunk-path l2norm);
 * the plan's chunks_per_segment must be a power of two unless every sequence is one segment; sequence lengths are
 * multiples of 64 (chunkwise_hgdn.py:598-601), at most 4096 chunks each; L >= 7 + number of bits of the largest chunk index. Zero initial state. level_states (nullable): fp32
 * [n_seq, HV, K, V, L] zeroed by the caller, receives HState.states (recurrent.py:33-36) after the last token of every
 * sequence -- what hattention_prefill returns (kernel.py:467-575); needs equal sequence lengths, multiples of 64. */
int64_t lampa_hgdn_chunk_workspace_bytes(int64_t total_chunks, int64_t n_segments, int HV, int K, int V);
int lampa_hgdn_chunk_fwd(const void* q, const void* k, const void* v, const float* g, const float* beta,
                         const void* lam, int lam_dtype, float lam_div, void* o, float* level_states,
                         const int32_t* plan_host, const int32_t* plan_dev, int H, int HV, int K, int V, int L, int dtype,
                         float scale, int l2norm, void* workspace, int64_t workspace_bytes, void* stream);

/* One token of the hierarchical rule on explicit level states. Replaces hattention_step (models/hattention/
 * kernel.py:577-633; step_state / step_output, recurrent.py:134-166; HState.cascade_weak / insert, recurrent.py:44-97).
 * q, k [B, H, K]; v, o [B, HV, V] (dtype LAMPA_BF16/FP16/FP32); g, beta fp32 [B, HV]; lam [B, HV, L] as above;
 * states fp32 [B, HV, K, V, L] (HState.states), updated in place; z: the levels 0 .. z-1 are full and cascade into
 * level z before the token is inserted (0 for an empty state; otherwise 1 + the number of trailing one bits of
 * tokens_seen - 1). L <= 32. */
int lampa_hgdn_step(const void* q, const void* k, const void* v, const float* g, const float* beta, const void* lam,
                    int lam_dtype, float lam_div, float* states, void* o, int B, int H, int HV, int K, int V, int L, int z,
                    int dtype, float scale, int l2norm, void* stream);

/* Process-wide switches of the one-launch form of lampa_lsh_bucket_sort[_batch] (no counterpart in the reference).
 * enabled = 0: every call takes the separate kernels (what a caller retries with after a call came back with bit 1 of
 * an overflow field set); 1: the library chooses (workgroups of 768 threads on tiles of 768 hits when that is at most
 * one workgroup per CU and 48 tiles per table, else workgroups of 512 threads on tiles of 1 024 hits when they fit the
 * GPU at once, else the separate kernels); 100 / 101: the 512- / 768-thread form for every call that fits.
 * wait_limit: polls a workgroup spends in one wait for the other workgroups of its table
 * before it gives up; < 0 = the built-in bound; 0 = give up at once, which lets a test reach the give-up path from the
 * host with every kernel still ending normally. */
int lampa_lsh_one_launch_config(int enabled, int64_t wait_limit);

/* ------------------------------------------------------------------------------------------------- profiling */

/* Time every kernel the library launches between begin and end with HIP events on the launch stream (a
 * benchmarking aid with no counterpart in the reference; one recording at a time, not thread-safe).
 * lampa_profile_end returns the number of entries written: ms[i] and a static name string per kernel launch. */
int lampa_profile_begin(void);
int lampa_profile_end(int max_entries, float* ms, const char** names);

/* Memory-only twin of the chunk pipeline's output pass (a benchmarking aid with no counterpart in the reference):
 * the same loads and stores per (segment, head) workgroup and chunk (k, v, q rows, the T blocks of the 5376-byte record of the chunk
 * and head, the o rows) with no arithmetic, for K = V = 64 and 2-byte elements on one dense sequence of
 * n_chunks * 64 tokens. q, k, v, o [n_chunks * 64, H, 64]; records n_chunks * H * 5376 bytes of any content; o is
 * overwritten. Its duration is what that access pattern costs on the memory system alone. */
int lampa_gdr_traffic_probe(const void* q, const void* k, const void* v, const void* records, void* o, int n_chunks,
                            int H, int chunks_per_segment, void* stream);
/* The same twin with the reads of the walk that the output pass does before its first chunk when the scan runs in two
 * levels (the composites of the groups of 8 segments before the workgroup's group, then of the segments before it inside
 * the group: 8 KiB of M' and 8 KiB of N per step and wave). composites: (segments + ceil(segments / 8)) * H * 24576
 * bytes of any content. */
int lampa_gdr_traffic_probe_walk(const void* q, const void* k, const void* v, const void* records,
                                 const void* composites, void* o, int n_chunks, int H, int chunks_per_segment,
                                 void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LAMPA_AMD_H */

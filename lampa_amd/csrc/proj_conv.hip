// Fused input projection + depthwise causal short convolution + SiLU of a gated-delta layer on gfx950 (bf16, MFMA).
//
// Replaces, for one layer call, the q / k / v / g / b / a projections (nn.Linear, bias-free) and the three
// ShortConvolution calls that follow the first three (reference chengjiang123/Lampa,
// models/hattention/modeling_gated_deltaproduct.py:505-547 and models/hattention/short_convolution.py:39-99):
//   pre[t, n] = sum_k x[t, k] W[n, k]                 (fp32 accumulate on the matrix cores, rounded to bf16 as a
//                                                      bf16 nn.Linear output is)
//   conv columns:  y[t, n] = silu(bias[n] + sum_j cw[n, j] pre[t - 3 + j, n]),  taps before a sequence start are zero
//   plain columns: y[t, n] = pre[t, n]
// The projection output never goes to HBM: x is read once (K = 128 columns), the outputs are written once.
//
// One workgroup = 4 waves = 256 output columns x a run of consecutive tokens. A wave keeps its 64 columns of W in
// registers for the whole run (2 column tiles x K/16 B-operand fragments), walks the run in tiles of 32 tokens
// (A operand = 32 rows of x straight from HBM, next tile prefetched), and turns each accumulator tile into outputs
// through a private LDS tile that also holds the last 3 pre-activation rows of the previous tile, so the convolution
// needs no recomputation except one extra tile at the start of a run that does not begin a sequence.
#include "gdr_common.h"

#define PC_K 128            // contraction length (hidden size) this kernel is built for
#define PC_NKS (PC_K / 16)
#define PC_W 4              // convolution taps
#define PC_COLS_WG 256
#define PC_COLS_WAVE 64
#define PC_ROWS 32
#define PC_ROWS_LANE 4     // consecutive token rows of a tile that one lane turns into outputs (8 columns each)
#define PC_LD (PC_COLS_WAVE + 8)  // LDS row stride in elements: 144 bytes, keeps 16-byte alignment
#define PC_MAX_BLOCKS 16

struct PcBlock {   // one block of 256 consecutive rows of W
  __bf16* out;     // output tensor of the block's columns
  int out_stride;  // its row stride in elements
  int out_col0;    // column of `out` that the block's first column maps to
  int n_valid;     // columns of the block that exist (the last block of W may be short)
  int conv;        // 1: convolution + SiLU, 0: plain projection output
  int conv_col0;   // row of the convolution weights of the block's first column
};
struct PcPlan {
  PcBlock blocks[PC_MAX_BLOCKS];
};

__device__ __forceinline__ float pc_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

__global__ void __launch_bounds__(256) pc_proj_conv_kernel(const __bf16* __restrict__ x, int64_t x_stride, int64_t n_tokens,
                                                          int64_t t_len, const __bf16* __restrict__ W,
                                                          const float* __restrict__ conv_w, const float* __restrict__ conv_b,
                                                          const PcPlan plan, int tokens_per_wg) {
  __shared__ __align__(16) __bf16 s_y[4][(PC_ROWS + PC_W - 1) * PC_LD];
  const PcBlock blk = plan.blocks[blockIdx.y];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  const int wcol = PC_COLS_WAVE * wave;  // first column of this wave inside the block
  if (wcol >= blk.n_valid) return;       // no workgroup-wide barrier below: a wave may leave alone
  const int64_t T0 = (int64_t)blockIdx.x * tokens_per_wg;
  const int64_t T1 = T0 + tokens_per_wg < n_tokens ? T0 + tokens_per_wg : n_tokens;
  __bf16* sy = s_y[wave];

  // this wave's 64 rows of W as B-operand fragments (rows beyond the end of a short block read as zero)
  bf16x8 bfrag[2][PC_NKS];
#pragma unroll
  for (int ct = 0; ct < 2; ++ct) {
    const int c = wcol + 32 * ct + ln;
    const bool ok = c < blk.n_valid;
    const __bf16* wp = W + ((int64_t)blockIdx.y * PC_COLS_WG + (ok ? c : 0)) * PC_K + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < PC_NKS; ++ks) {
      bfrag[ct][ks] = *reinterpret_cast<const bf16x8*>(wp + 16 * ks);
      if (!ok) {
#pragma unroll
        for (int e = 0; e < 8; ++e) bfrag[ct][ks][e] = (__bf16)0.0f;
      }
    }
  }
  // output role of the lane: 8 consecutive columns (cg) of the 4 consecutive token rows 4 tq .. 4 tq + 3 of a tile
  const int cg = lane & 7, tq = lane >> 3;
  float cw[PC_W][8], cb[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int col = wcol + 8 * cg + c;
    const bool ok = blk.conv && col < blk.n_valid;
    cb[c] = (ok && conv_b) ? conv_b[blk.conv_col0 + col] : 0.0f;
#pragma unroll
    for (int j = 0; j < PC_W; ++j)
      cw[j][c] = ok ? conv_w[(int64_t)(blk.conv_col0 + col) * PC_W + j] : 0.0f;
  }

  auto load_a = [&](int64_t t0, bf16x8* a) {
    int64_t row = t0 + ln;
    row = row < 0 ? 0 : (row >= n_tokens ? n_tokens - 1 : row);
    const __bf16* xp = x + row * x_stride + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < PC_NKS; ++ks) a[ks] = *reinterpret_cast<const bf16x8*>(xp + 16 * ks);
  };

  // a run that starts inside a sequence first computes the tile before it, only for its last rows of history
  const bool need_history = blk.conv && (T0 % t_len) != 0;
  int64_t t0 = need_history ? T0 - PC_ROWS : T0;
  if (!need_history) {
    for (int i = lane; i < (PC_W - 1) * PC_LD; i += 64) sy[i] = (__bf16)0.0f;
  }
  // token position inside the sequence, kept per tile in 32 bits (a 64-bit modulo per output row would cost more than
  // the convolution); sequences shorter than two tiles take the general modulo
  const int tl32 = (int)(t_len < INT32_MAX ? t_len : INT32_MAX);
  const bool small_seq = t_len < 2 * PC_ROWS;
  int ts0 = (int)((t0 % t_len + t_len) % t_len);
  bf16x8 afrag[PC_NKS], anext[PC_NKS];
  load_a(t0, afrag);
  for (; t0 < T1; t0 += PC_ROWS, ts0 = small_seq ? (ts0 + PC_ROWS) % tl32 : (ts0 + PC_ROWS >= tl32 ? ts0 + PC_ROWS - tl32 : ts0 + PC_ROWS)) {
    load_a(t0 + PC_ROWS, anext);
    f32x16 acc[2];
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ct][r] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < PC_NKS; ++ks) acc[ct] = mfma32(afrag[ks], bfrag[ct][ks], acc[ct]);
    }
    // pre-activations of the tile, rounded to bf16, below the 3 rows of history
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        sy[(PC_W - 1 + 8 * (r / 4) + 4 * hh + (r % 4)) * PC_LD + 32 * ct + ln] = (__bf16)acc[ct][r];
    lds_fence();
    if (t0 >= T0) {
      const int col = wcol + 8 * cg;
      const bool store_cols = col < blk.n_valid;
      if (blk.conv) {
        // the lane's 4 consecutive tokens share their taps: 7 rows of pre-activations for 4 outputs
        float pre[PC_ROWS_LANE + PC_W - 1][8];
#pragma unroll
        for (int r = 0; r < PC_ROWS_LANE + PC_W - 1; ++r) {
          const bf16x8 row = *reinterpret_cast<const bf16x8*>(&sy[(PC_ROWS_LANE * tq + r) * PC_LD + 8 * cg]);
#pragma unroll
          for (int c = 0; c < 8; ++c) pre[r][c] = (float)row[c];
        }
        // tokens closer than 3 to the start of their sequence lose the taps that reach across it; a tile that holds no
        // such token (all but the first of a long sequence) skips the masks
        const bool interior = ts0 >= PC_W - 1 && ts0 + PC_ROWS <= tl32;
#pragma unroll
        for (int i = 0; i < PC_ROWS_LANE; ++i) {
          const int tr = PC_ROWS_LANE * tq + i;
          float y[8];
#pragma unroll
          for (int c = 0; c < 8; ++c) y[c] = cb[c];
          if (interior) {
#pragma unroll
            for (int j = 0; j < PC_W; ++j)
#pragma unroll
              for (int c = 0; c < 8; ++c) y[c] = __builtin_fmaf(pre[i + j][c], cw[j][c], y[c]);
          } else {
            int ts = ts0 + tr;
            if (ts >= tl32) ts = small_seq ? ts % tl32 : ts - tl32;
#pragma unroll
            for (int j = 0; j < PC_W; ++j) {
              const bool live = ts - (PC_W - 1) + j >= 0;
#pragma unroll
              for (int c = 0; c < 8; ++c) y[c] = __builtin_fmaf(live ? pre[i + j][c] : 0.0f, cw[j][c], y[c]);
            }
          }
          bf16x8 o;
#pragma unroll
          for (int c = 0; c < 8; ++c) o[c] = (__bf16)(y[c] * pc_sigmoid(y[c]));
          const int64_t t = t0 + tr;
          if (t < T1 && store_cols) *reinterpret_cast<bf16x8*>(blk.out + t * blk.out_stride + blk.out_col0 + col) = o;
        }
      } else {
#pragma unroll
        for (int i = 0; i < PC_ROWS_LANE; ++i) {  // the projection output itself
          const int tr = PC_ROWS_LANE * tq + i;
          const bf16x8 o = *reinterpret_cast<const bf16x8*>(&sy[(tr + PC_W - 1) * PC_LD + 8 * cg]);
          const int64_t t = t0 + tr;
          if (t < T1 && store_cols) *reinterpret_cast<bf16x8*>(blk.out + t * blk.out_stride + blk.out_col0 + col) = o;
        }
      }
    }
    lds_fence();
    // the last 3 rows become the history of the next tile
    for (int i = lane; i < (PC_W - 1) * (PC_COLS_WAVE / 8); i += 64) {
      const int r = i / (PC_COLS_WAVE / 8), c8 = i % (PC_COLS_WAVE / 8);
      *reinterpret_cast<bf16x8*>(&sy[r * PC_LD + 8 * c8]) =
          *reinterpret_cast<const bf16x8*>(&sy[(PC_ROWS + r) * PC_LD + 8 * c8]);
    }
    lds_fence();
#pragma unroll
    for (int ks = 0; ks < PC_NKS; ++ks) afrag[ks] = anext[ks];
  }
}

// x [n_tokens, 128] bf16 (row stride x_stride elements), n_tokens / t_len dense sequences of t_len tokens;
// W [n_cols, 128] bf16 row-major (the rows of the projections one after the other); the first n_conv columns go
// through the convolution (conv_w fp32 [n_conv, 4], conv_b fp32 [n_conv] or NULL) and SiLU and are written as
// n_conv / conv_split tensors [n_tokens, conv_split] at conv_out + i * n_tokens * conv_split; the remaining columns
// are written as they are: the next plain_cols to plain_out [n_tokens, plain_cols], whatever is left (< 256 columns)
// to tail_out [n_tokens, tail_cols]. n_conv, conv_split and plain_cols are multiples of 256; tail_cols a multiple of 8.
extern "C" int lampa_proj_conv_fwd(const void* x, int64_t x_stride, int64_t n_tokens, int64_t t_len, int K, const void* W,
                                   int n_cols, const float* conv_w, const float* conv_b, int n_conv, int conv_split,
                                   void* conv_out, int plain_cols, void* plain_out, int tail_cols, void* tail_out,
                                   int tokens_per_wg, void* stream) {
  if (!x || !W || n_tokens < 0 || t_len < 1 || n_cols < 1) return LAMPA_ERR_INVALID;
  if (K != PC_K) return LAMPA_ERR_UNSUPPORTED;
  if (n_conv < 0 || plain_cols < 0 || tail_cols < 0 || n_conv + plain_cols + tail_cols != n_cols) return LAMPA_ERR_INVALID;
  if (n_conv % PC_COLS_WG || plain_cols % PC_COLS_WG || tail_cols >= PC_COLS_WG || tail_cols % 8) return LAMPA_ERR_UNSUPPORTED;
  if (n_conv && (!conv_w || !conv_out || conv_split < PC_COLS_WG || conv_split % PC_COLS_WG || n_conv % conv_split))
    return LAMPA_ERR_INVALID;
  if ((plain_cols && !plain_out) || (tail_cols && !tail_out)) return LAMPA_ERR_INVALID;
  if (x_stride < PC_K || x_stride % 8 || n_tokens % t_len) return LAMPA_ERR_INVALID;
  if (((uintptr_t)x | (uintptr_t)W | (uintptr_t)conv_out | (uintptr_t)plain_out | (uintptr_t)tail_out) % 16)
    return LAMPA_ERR_UNSUPPORTED;
  const int n_blocks = (n_cols + PC_COLS_WG - 1) / PC_COLS_WG;
  if (n_blocks > PC_MAX_BLOCKS) return LAMPA_ERR_UNSUPPORTED;
  if (n_tokens == 0) return LAMPA_OK;
  if (tokens_per_wg <= 0) {
    // as many runs of tokens as fill the chip once with two workgroups per CU (registers allow no more)
    static int slots = 0;
    if (!slots) {
      int dev = 0, cus = 0;
      if (hipGetDevice(&dev) != hipSuccess ||
          hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
        cus = 256;
      slots = 2 * cus;
    }
    const int runs = slots / n_blocks > 0 ? slots / n_blocks : 1;
    tokens_per_wg = (int)((n_tokens + runs - 1) / runs);
    if (tokens_per_wg < 4 * PC_ROWS) tokens_per_wg = 4 * PC_ROWS;
  }
  tokens_per_wg = (tokens_per_wg + PC_ROWS - 1) / PC_ROWS * PC_ROWS;
  PcPlan plan;
  for (int b = 0; b < n_blocks; ++b) {
    PcBlock& k = plan.blocks[b];
    const int c0 = b * PC_COLS_WG;
    if (c0 < n_conv) {
      const int part = c0 / conv_split;
      k.out = (__bf16*)conv_out + (int64_t)part * n_tokens * conv_split;
      k.out_stride = conv_split; k.out_col0 = c0 - part * conv_split; k.n_valid = PC_COLS_WG; k.conv = 1; k.conv_col0 = c0;
    } else if (c0 < n_conv + plain_cols) {
      k.out = (__bf16*)plain_out;
      k.out_stride = plain_cols; k.out_col0 = c0 - n_conv; k.n_valid = PC_COLS_WG; k.conv = 0; k.conv_col0 = 0;
    } else {
      k.out = (__bf16*)tail_out;
      k.out_stride = tail_cols; k.out_col0 = 0; k.n_valid = tail_cols; k.conv = 0; k.conv_col0 = 0;
    }
  }
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((n_tokens + tokens_per_wg - 1) / tokens_per_wg), n_blocks);
  LAMPA_PROF(s, "start");
  hipLaunchKernelGGL(pc_proj_conv_kernel, grid, dim3(256), 0, s, (const __bf16*)x, x_stride, n_tokens, t_len,
                     (const __bf16*)W, conv_w, conv_b, plan, tokens_per_wg);
  LAMPA_PROF(s, "pc_proj_conv_kernel");
  return lampa_launch_status();
}

// ------------------------------------------------------------------------------- gated RMS norm + output projection
// y[t, :] = W_o * vec_h( rmsnorm(o[t, h, :]) * weight * swish(g[t, h, :]) ): the gated norm of every head
// (models/hattention/fused_norm.py:40-111 with IS_RMS_NORM and the swish gate) feeding the bias-free output projection
// (modeling_gated_deltaproduct.py:612-623) without writing the normalised tensor. One workgroup = 4 waves walks a run
// of 32-token tiles: all threads normalise and gate the tile into LDS (bf16, the A operand; 8 lanes share a head's 64
// channels), then every wave multiplies it with its 32 rows of W_o, which it keeps in registers as B-operand fragments.
#define NP_D 64        // channels per head
#define NP_KMAX 512    // heads * channels this kernel is built for (32 contraction steps of 16)
#define NP_OUT 128     // output columns (4 waves x 32)
#define NP_LDA (NP_KMAX + 8)

__global__ void __launch_bounds__(256, 2) pc_norm_proj_kernel(const __bf16* __restrict__ o, const __bf16* __restrict__ g,
                                                          int64_t g_stride, const float* __restrict__ norm_w,
                                                          const __bf16* __restrict__ W, int64_t n_tokens, float eps,
                                                          __bf16* __restrict__ y, const __bf16* __restrict__ residual,
                                                          const float* __restrict__ next_w, float next_eps,
                                                          __bf16* __restrict__ res_out, int tokens_per_wg) {
  constexpr int NKS = NP_KMAX / 16;
  __shared__ __align__(16) __bf16 s_a[2][PC_ROWS * NP_LDA];
  __shared__ __align__(16) __bf16 s_out[4][PC_ROWS * (32 + 8)];
  __shared__ float s_ss[4][PC_ROWS];  // with a residual: every wave's share of the rows' sums of squares
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, hh = lane >> 5, ln = lane & 31;
  const int64_t T0 = (int64_t)blockIdx.x * tokens_per_wg;
  const int64_t T1 = T0 + tokens_per_wg < n_tokens ? T0 + tokens_per_wg : n_tokens;

  bf16x8 bfrag[NKS];  // rows 32 wave + ln of W_o
  {
    const __bf16* wp = W + (int64_t)(32 * wave + ln) * NP_KMAX + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) bfrag[ks] = *reinterpret_cast<const bf16x8*>(wp + 16 * ks);
  }
  // norm role: 8 lanes per (token, head) row, 8 channels each; 32 rows per pass, 8 passes per tile
  const int sub = tid & 7, rrow = tid >> 3;
  float nw[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) nw[c] = norm_w ? norm_w[8 * sub + c] : 1.0f;

  // (the loads of four passes are issued before the first is used: two memory round trips per tile, not one per pass;
  // all eight at once would cost the second workgroup per CU its registers)
  auto stage = [&](int64_t t0, int buf) {
#pragma unroll
    for (int p0 = 0; p0 < 8; p0 += 4) {
      bf16x8 ovs[4], gvs[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int r = 32 * (p0 + u) + rrow;       // (token, head) row of the tile: token r / 8, head r % 8
        const int tok = r >> 3, head = r & 7;
        int64_t t = t0 + tok;
        t = t < n_tokens ? t : n_tokens - 1;
        ovs[u] = *reinterpret_cast<const bf16x8*>(o + t * NP_KMAX + head * NP_D + 8 * sub);
        gvs[u] = *reinterpret_cast<const bf16x8*>(g + t * g_stride + head * NP_D + 8 * sub);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int r = 32 * (p0 + u) + rrow;
        const int tok = r >> 3, head = r & 7;
        const bf16x8 ov = ovs[u], gv = gvs[u];
        float x[8], ss = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c) { x[c] = (float)ov[c]; ss = __builtin_fmaf(x[c], x[c], ss); }
        ss += __shfl_xor(ss, 1);
        ss += __shfl_xor(ss, 2);
        ss += __shfl_xor(ss, 4);
        const float rstd = 1.0f / sqrtf(ss * (1.0f / NP_D) + eps);
        bf16x8 out;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const float gc = (float)gv[c];
          out[c] = (__bf16)(x[c] * rstd * nw[c] * gc * pc_sigmoid(gc));
        }
        *reinterpret_cast<bf16x8*>(&s_a[buf][tok * NP_LDA + head * NP_D + 8 * sub]) = out;
      }
    }
  };

  const int cg = lane & 3, tq = lane >> 2;  // output role: row 2 tq + i (i < 2), columns 8 cg .. 8 cg + 7 of the wave's 32
  float nxw[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) nxw[c] = (residual && next_w) ? next_w[32 * wave + 8 * cg + c] : 1.0f;
  int buf = 0;
  if (T0 < T1) stage(T0, 0);
  __syncthreads();
  for (int64_t t0 = T0; t0 < T1; t0 += PC_ROWS, buf ^= 1) {
    // the residual rows of this tile are requested first: their latency hides behind the staging and the MFMAs
    bf16x8 rv[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int c = 0; c < 8; ++c) rv[i][c] = (__bf16)0.0f;
      const int64_t t = t0 + 2 * tq + i;
      if (residual && t < T1) rv[i] = *reinterpret_cast<const bf16x8*>(residual + t * NP_OUT + 32 * wave + 8 * cg);
    }
    if (t0 + PC_ROWS < T1) stage(t0 + PC_ROWS, buf ^ 1);   // next tile while this one is multiplied
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    const __bf16* ap = &s_a[buf][ln * NP_LDA + 8 * hh];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) acc = mfma32(*reinterpret_cast<const bf16x8*>(ap + 16 * ks), bfrag[ks], acc);
    __bf16* so = s_out[wave];
#pragma unroll
    for (int r = 0; r < 16; ++r) so[(8 * (r / 4) + 4 * hh + (r % 4)) * 40 + ln] = (__bf16)acc[r];
    lds_fence();
    if (!residual) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int tr = 2 * tq + i;
        const int64_t t = t0 + tr;
        if (t < T1)
          *reinterpret_cast<bf16x8*>(y + t * NP_OUT + 32 * wave + 8 * cg) = *reinterpret_cast<const bf16x8*>(&so[tr * 40 + 8 * cg]);
      }
    } else {
      // residual add and the next layer's RMS norm over the 128 output columns (fused_norm.py:1436-1506 with a
      // residual): res_out = residual + y, y = rmsnorm(res_out) * next_w, the sum of squares taken before rounding
      float sres[2][8];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int tr = 2 * tq + i;
        const bf16x8 yv = *reinterpret_cast<const bf16x8*>(&so[tr * 40 + 8 * cg]);
        float ss = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          sres[i][c] = (float)yv[c] + (float)rv[i][c];
          ss = __builtin_fmaf(sres[i][c], sres[i][c], ss);
        }
        ss += __shfl_xor(ss, 1);
        ss += __shfl_xor(ss, 2);
        if (cg == 0) s_ss[wave][tr] = ss;
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int tr = 2 * tq + i;
        const int64_t t = t0 + tr;
        const float tot = s_ss[0][tr] + s_ss[1][tr] + s_ss[2][tr] + s_ss[3][tr];
        const float rstd = 1.0f / sqrtf(tot * (1.0f / NP_OUT) + next_eps);
        bf16x8 ro, ho;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          ro[c] = (__bf16)sres[i][c];
          ho[c] = (__bf16)(sres[i][c] * rstd * nxw[c]);
        }
        if (t < T1) {
          *reinterpret_cast<bf16x8*>(res_out + t * NP_OUT + 32 * wave + 8 * cg) = ro;
          *reinterpret_cast<bf16x8*>(y + t * NP_OUT + 32 * wave + 8 * cg) = ho;
        }
      }
    }
    __syncthreads();  // the next tile is staged, this tile's A operand and the row sums are free again
  }
}

// o [n_tokens, 8, 64] bf16 contiguous; g the same shape with token stride g_stride elements; norm_w fp32 [64] or NULL;
// W [128, 512] bf16 row-major (the output projection); y [n_tokens, 128] bf16.
// With residual [n_tokens, 128] bf16: res_out = residual + projection (bf16) and y = rmsnorm(res_out) * next_w
// (next_w fp32 [128] or NULL, next_eps), i.e. the residual add and the next layer's pre-norm are applied as well.
extern "C" int lampa_norm_proj_fwd(const void* o, const void* g, int64_t g_stride, const float* norm_w, const void* W,
                                   int64_t n_tokens, int heads, int head_dim, int n_out, float eps, void* y,
                                   const void* residual, const float* next_w, float next_eps, void* res_out,
                                   int tokens_per_wg, void* stream) {
  if (!o || !g || !W || !y || n_tokens < 0) return LAMPA_ERR_INVALID;
  if (residual && (!res_out || ((uintptr_t)residual | (uintptr_t)res_out) % 16)) return LAMPA_ERR_INVALID;
  if (heads * head_dim != NP_KMAX || head_dim != NP_D || n_out != NP_OUT) return LAMPA_ERR_UNSUPPORTED;
  if (g_stride < NP_KMAX || g_stride % 8 || ((uintptr_t)o | (uintptr_t)g | (uintptr_t)W | (uintptr_t)y) % 16)
    return LAMPA_ERR_UNSUPPORTED;
  if (n_tokens == 0) return LAMPA_OK;
  if (tokens_per_wg <= 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
      cus = 256;
    tokens_per_wg = (int)((n_tokens + 2 * cus - 1) / (2 * cus));
    if (tokens_per_wg < 2 * PC_ROWS) tokens_per_wg = 2 * PC_ROWS;
  }
  tokens_per_wg = (tokens_per_wg + PC_ROWS - 1) / PC_ROWS * PC_ROWS;
  hipStream_t s = (hipStream_t)stream;
  LAMPA_PROF(s, "start");
  hipLaunchKernelGGL(pc_norm_proj_kernel, dim3((unsigned)((n_tokens + tokens_per_wg - 1) / tokens_per_wg)), dim3(256), 0, s,
                     (const __bf16*)o, (const __bf16*)g, g_stride, norm_w, (const __bf16*)W, n_tokens, eps, (__bf16*)y,
                     (const __bf16*)residual, next_w, next_eps, (__bf16*)res_out, tokens_per_wg);
  LAMPA_PROF(s, "pc_norm_proj_kernel");
  return lampa_launch_status();
}

// Parameters shared by the LoRA GEMM kernels (host fills, kernels read by value).
#pragma once
#include "kh_common.h"

struct LoraGemmParams {
  const bf16_t* x;
  const bf16_t* w;
  const bf16_t* bias;      // may be null
  const bf16_t* a_cat;     // [R,K] (unused when R == 0)
  const bf16_t* b_cat;     // [N,R]
  const float* col_scale;  // [R]
  const bf16_t* t_ext;     // [M, ldt] precomputed, already scaled shrink result (null: compute it in the kernel)
  int ldt;
  int t_nsplit;            // > 0: W rows come in blocks of t_nsplit rows; block j uses T columns [j*R, (j+1)*R)
  // grouped launch: blockIdx.y selects a row {w, bias, b_cat, t_ext, y} of this device table (null: single layer)
  const uint64_t* grp;
  int dbg;  // always 0 unless the library is built with -DKH_TUNING (kernel experiments; not part of the C ABI)
  const bf16_t* res;       // [M,N] residual added in the epilogue, may be null
  bf16_t* y;
  int M, N, K, R;
  int m_tiles, n_tiles, n_chunk, n_chunks;  // n_chunk = N tiles walked by one workgroup
  // tile -> XCD map (xg_n > 0): the 8 XCDs form an xg_m x xg_n grid over the tile matrix, each owning a block of
  // xr_m x xr_n tiles (see launch_pcfg); 0: contiguous ranges of the (m block, n chunk) list per XCD
  int xg_n, xr_m, xr_n;
  // segmented launch (sg_mode != 0): blockIdx.y = segment s of a batch of requests; rows [sg_start[s], sg_start[s+1])
  // of x / y, weights of adapter sg_adapter[s] (negative: the segment is skipped) at w + adapter * sg_wstride.
  // sg_mode 1 (shrink): y = x . W_a^T.  sg_mode 2 (expand): y += sg_scale[a] * (x . W_a^T) over the first
  // sg_rank[a] K columns (x = the shrink result, row stride K).  M = the longest segment.
  const int32_t* sg_start; const int32_t* sg_adapter; const int32_t* sg_rank; const float* sg_scale;
  int sg_mode; long sg_wstride;
  int geglu;                                // 1: W rows are (value,gate) interleaved in 32-column groups, y is [M,N/2]
  // 3x3 convolution as an implicit GEMM (conv_cin > 0): x is an NHWC image [Nb, conv_h, conv_w, conv_cin], row m
  // of the GEMM is output pixel m of [Nb, conv_ho, conv_wo], K = 9 * conv_cin ordered (kh, kw, ci), padding 1
  int conv_cin, conv_h, conv_w, conv_ho, conv_wo, conv_stride;
  // shrink inside the GEMM launch (il_blocks > 0): the first il_blocks workgroups compute t_ext = the shrink of x
  // (a_cat, col_scale) in 64x64 tiles and count themselves into il_cnt[row block]; the GEMM workgroups wait for their
  // row block's count before they read t_ext.  il_cnt: ceil(M / 128) + 1 ints, zero when the launch starts (arrivals
  // per row block, then a time-out flag); the launch leaves the arrivals in them.
  int il_blocks = 0;
  int* il_cnt = nullptr;
  // two-launch / in-launch forms: rank columns >= r_used of t_ext and b_cat are all zero (0: unknown, use R); the
  // 128x128 / 256x128 and 256x320 kernels then skip the MFMA steps that would only add zeros
  int r_used = 0;
};

// Software-pipelined kernel (lora_gemm_pipe.hip); needs K % 32 == 0.  tile_sel: 0 automatic, >= 16 forces a tile.
int lora_gemm_pipe_launch(const LoraGemmParams& p, int tile_sel, hipStream_t stream);
// 3x3 convolution (conv_* fields set, R == 0, K == 9 * conv_cin, conv_cin % 32 == 0).
int lora_gemm_pipe_launch_conv(const LoraGemmParams& p, hipStream_t stream);
// Segmented multi-adapter form (sg_* fields set; plain GEMM per segment, K % 32 == 0).
int lora_gemm_pipe_launch_sgmv(const LoraGemmParams& p, int n_segments, hipStream_t stream);
// Grouped form: grid.y = n_groups, per-group pointers from p.grp; rank columns (p.R > 0) as extra K tiles.
int lora_gemm_pipe_launch_grouped(const LoraGemmParams& p, int n_groups, hipStream_t stream);
// Shrink and GEMM in one launch for shapes whose 128x128 tiles leave CUs idle (p.a_cat / col_scale / b_cat set, p.t_ext =
// scratch for the shrink result, p.il_cnt = counters); KH_ERR_UNSUPPORTED when the shape does not qualify.
bool lora_gemm_pipe_il_ok(const LoraGemmParams& p);
int lora_gemm_pipe_launch_il(const LoraGemmParams& p, hipStream_t stream);
// Narrow-output variant (lora_gemm_ksplit.hip): (32 * row_groups) x 160 tiles, 8 waves as row_groups x k-slices;
// plain or K-extended GEMM with bias / residual, K % 64 == 0.  row_groups 2 or 4.
bool lora_gemm_ksplit_ok(const LoraGemmParams& p);
int lora_gemm_ksplit_launch(const LoraGemmParams& p, int row_groups, hipStream_t stream);
bool lora_gemm_ksplit_conv_ok(const LoraGemmParams& p);
int lora_gemm_ksplit_launch_conv(const LoraGemmParams& p, int row_groups, hipStream_t stream);
// Wide-tile variant (lora_gemm_wide.hip): 256 x 320 tiles, 8 waves; plain or K-extended GEMM with bias / residual /
// GEGLU; M % 256 == 0, N % 320 == 0, K % 64 == 0.
bool lora_gemm_wide_ok(const LoraGemmParams& p);
int lora_gemm_wide_launch(LoraGemmParams p, hipStream_t stream);

extern "C" int kh_lora_shrink_bf16(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M, int64_t K,
                                   int64_t R, void* stream);

// Kernel experiments (timestamps, frozen operands, alternative tile maps) exist only in builds with -DKH_TUNING; the
// shipped library compiles them out and its entry points reject the flag bits that would select them.
#ifdef KH_TUNING
#define KH_DBG(p, bit) (((p).dbg & (bit)) != 0)
#else
#define KH_DBG(p, bit) false
#endif

// Parameters shared by the LoRA GEMM kernels (host fills, kernels read by value).
#pragma once
#include "kh_common.h"
#include <type_traits>

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
  // LayerNorm folded into the GEMM (ln_part != nullptr): x is the input of a LayerNorm over its K columns whose affine
  // weight is already multiplied into w (and a_cat); the epilogue finishes the normalisation per output row,
  //   y[m,n] = rstd_m * (acc[m,n] - mean_m * ln_c1[n]) + ln_c2[n]   (ln_c1 = row sums of w, ln_c2 = bias + w . beta),
  // with mean / rstd from the row's 16 partial (sum, sum of squares) pairs in ln_part.  The shrink of such a layer
  // stores t = ((x . a^T) - mean * ln_ca1 + ln_ca2 / rstd) * col_scale, i.e. the adapter's share divided by rstd.
  const float* ln_part = nullptr;   // [16][M][2]
  const float* ln_c1 = nullptr;     // [N]
  const float* ln_c2 = nullptr;     // [N]
  const float* ln_ca1 = nullptr;    // [ldt] (shrink)
  const float* ln_ca2 = nullptr;    // [ldt]
  float ln_eps = 0.f;
  int ln_lds = 0;                   // byte offset of the workgroup's mean / rstd arrays in dynamic LDS (set by the launcher)
  // Row statistics of the output for a following folded LayerNorm (st_part != nullptr): column tile j writes the
  // (sum, sum of squares) of its columns of every row to st_part[j][row]; tile 0 also zeroes the slots past the last tile.
  float* st_part = nullptr;         // [16][M][2]
  // Weight prefetch (pf != nullptr): the launch also touches every 128-byte line of pf[0 .. 128 * pf_lines), the weights
  // of the NEXT launch of this family, so that they wait in the memory-side cache when that launch asks for them (a
  // step reads 2.5 GB of weights once each: every launch would otherwise meet its weights in HBM, where the XCDs that
  // share a weight block each fetch it again).  Set from kh_set_weight_prefetch by the entry points.
  // Cross-attention in the epilogue (xa_k != nullptr; the 128x128 / 8-wave tiles only): the layer is an attention's to_q
  // and a 128 x 128 output tile holds 128 queries of two 64-wide heads; instead of storing them the workgroup runs
  // softmax(q k^T * scale) v for them against the xa_S <= 96 keys of those heads and stores that to xa_o (rows like y's,
  // head h at columns 64 h).  Rows m belong to batch sample m / xa_T (xa_T % 128 == 0); k / v: [B, S, heads * 64] views.
  const bf16_t* xa_k = nullptr; const bf16_t* xa_v = nullptr; bf16_t* xa_o = nullptr;
  int xa_S = 0, xa_T = 0;
  long xa_ldk = 0, xa_ldv = 0, xa_ldo = 0, xa_bsk = 0, xa_bsv = 0;
  float xa_scale_log2e = 0.f;
  // GroupNorm statistics of a convolution's result as a by-product of its epilogue (gn_part != nullptr; 3x3 convolutions on
  // the 160-column tiles): a tile holds whole groups of gn_cg channels of BM pixels of one image (gn_hw pixels each), and
  // its workgroup writes their (sum, sum of squares) over conv + gn_add[image][c] to gn_part[image][group][row tile of
  // the image][2] -- the layout kh_group_norm_bf16's second pass folds.
  float* gn_part = nullptr; const bf16_t* gn_add = nullptr;
  int gn_cg = 0, gn_hw = 0;
  const void* pf[3] = {nullptr, nullptr, nullptr};   // up to three ranges: weights, A_cat, B_cat of that launch
  uint32_t pf_lines[3] = {0, 0, 0};
};

// bit 24 of the `flags` of kh_lora_linear_split_bf16 / _norm_bf16: do not use the cooperative in-launch shrink (see include/katz_hip.h)
constexpr int KH_FLAG_NO_COOP = 1 << 24;

// The pending weight prefetch of this host thread (kh_set_weight_prefetch), handed to the next launch.
void kh_take_weight_prefetch(LoraGemmParams& p);

constexpr int KH_LN_LDS = 4096;    // bytes of dynamic LDS a launch with a folded LayerNorm adds: mean, 1/std of up to 256 rows, c1, c2 of up to 256 columns
constexpr int KH_LN_SLOTS = 16;     // partial pairs per row: at most 16 column tiles (N <= 2048 with 128-column tiles)

// Touch lines first, first + n_wg * NT, ... of the prefetch range: one dword per line and lane, loaded into 256 bytes of
// LDS that belong to this wave alone and that its own later DMA overwrites (a wave's loads land in order), so no
// register and no wait is spent on data nobody reads.  wg / n_wg: this workgroup's index among those that take part.
__device__ __forceinline__ void kh_prefetch_lines(const void* const (&pf)[3], const uint32_t (&lines)[3], char* wave_lds, int wg, int n_wg,
                                                  int tid, int nt) {
#if __HIP_DEVICE_COMPILE__
  if (pf[0] == nullptr) return;
  // four rounds over the first range (64 MB with 256 workgroups of 512 threads), one over the others (adapter matrices),
  // no loop; the per-lane offset carries the round, because only it is checked against the range: an offset beyond the
  // range reads nothing
  const uint32_t first = ((uint32_t)wg * (uint32_t)nt + (uint32_t)tid) << 7, step = ((uint32_t)n_wg * (uint32_t)nt) << 7;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(pf[k] != nullptr ? pf[k] : pf[0]), 0,
                                                                        pf[k] != nullptr ? (int)(lines[k] << 7) : 0, 0x00020000);
#pragma unroll
    for (uint32_t r = 0; r < (k == 0 ? 4u : 1u); ++r) {
      const uint32_t off = first + r * step;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)wave_lds, 4, off >= first ? off : 0xFFFFFFFFu, 0, 0, 0);
    }
  }
#endif
}

// The same from waves that have nothing else to do (the idle half of an in-launch shrink workgroup): as many rounds as
// the ranges need, up to 16 (the first range) / 4 (the others), in a loop.
__device__ __forceinline__ void kh_prefetch_lines_idle(const void* const (&pf)[3], const uint32_t (&lines)[3], char* wave_lds, int wg, int n_wg,
                                                       int tid, int nt) {
#if __HIP_DEVICE_COMPILE__
  if (pf[0] == nullptr) return;
  const uint32_t first = ((uint32_t)wg * (uint32_t)nt + (uint32_t)tid) << 7, step = ((uint32_t)n_wg * (uint32_t)nt) << 7;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    if (pf[k] == nullptr) continue;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(pf[k]), 0, (int)(lines[k] << 7), 0x00020000);
    const uint32_t bytes = lines[k] << 7;                       // at most 2 GiB
    uint32_t rounds = (bytes + step - 1) / step;
    const uint32_t cap = k == 0 ? 16u : 4u;
    rounds = rounds < cap ? rounds : cap;
    for (uint32_t r = 0; r < rounds; ++r)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)wave_lds, 4, first + r * step, 0, 0, 0);
  }
#endif
}

// a column tile's pair for one output row, and (from tile 0) zeros in the slots no tile writes
__device__ __forceinline__ void kh_ln_store_stats(float* part, int row, int M, int tile, int n_tiles, float s, float q) {
  u32x2* dst = reinterpret_cast<u32x2*>(part) + row;
  dst[(size_t)tile * M] = u32x2{__float_as_uint(s), __float_as_uint(q)};
  if (tile == 0)
    for (int t = n_tiles; t < KH_LN_SLOTS; ++t) dst[(size_t)t * M] = u32x2{0u, 0u};
}

// sum over the 16 lanes of a DPP row (lanes 16k .. 16k+15), the result in every lane: four cross-lane adds in the VALU
__device__ __forceinline__ float kh_row16_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  v += dpp(v, std::integral_constant<int, 0xb1>{});    // quad_perm [1,0,3,2]
  v += dpp(v, std::integral_constant<int, 0x4e>{});    // quad_perm [2,3,0,1]
  v += dpp(v, std::integral_constant<int, 0x141>{});   // row_half_mirror
  v += dpp(v, std::integral_constant<int, 0x140>{});   // row_mirror
  return v;
}

// mean and 1/std (or std, `want_sigma`) of ROWS consecutive rows from m0 into out_mean / out_2 (LDS), by all NT threads
// of the workgroup, in two steps so that the loads fly while the kernel sets up its operands.  A wave takes sixteen rows
// at a time: lane = (slot group g = lane / 16, row = lane % 16) loads the pairs of slots g, 4 + g, 8 + g, 12 + g (every
// load instruction reads four whole 128-byte lines of the slot-major buffer [slot][row][2]), adds them up, and the four
// groups meet by two cross-lane adds: a fixed order, deterministic.  M = rows of the buffer, D = the row's length.
// Same formula as the stand-alone LayerNorm kernel: biased variance, rstd = rsqrt(var + eps).
template <int ROWS, int NT>
struct KhLnTileStats {
  static constexpr int PASSES = (ROWS + (NT / 64) * 16 - 1) / ((NT / 64) * 16);
  static_assert(KH_LN_SLOTS == 16 && ROWS % 16 == 0 && NT % 64 == 0, "four slot groups of four, sixteen rows per wave and pass");
  u32x2 v[PASSES][4];

  __device__ __forceinline__ void load(const float* part, int m0, int M, int tid) {
    const int lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const u32x2* src = reinterpret_cast<const u32x2*>(part) + (size_t)g * M;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int r = ((tid >> 6) + ps * (NT / 64)) * 16 + r16;          // beyond ROWS: a valid address, never stored
      const int row = m0 + r < M ? m0 + r : M - 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[ps][j] = src[(size_t)(4 * j) * M + row];
    }
  }
  __device__ __forceinline__ void finish(int D, float eps, int tid, float* out_mean, float* out_2, bool want_sigma) const {
    const int lane = tid & 63, r16 = lane & 15, g = lane >> 4;
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int r = ((tid >> 6) + ps * (NT / 64)) * 16 + r16;
      float s = 0.f, q = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) { s += __uint_as_float(v[ps][j][0]); q += __uint_as_float(v[ps][j][1]); }
      s += __shfl_xor(s, 16, 64); q += __shfl_xor(q, 16, 64);
      s += __shfl_xor(s, 32, 64); q += __shfl_xor(q, 32, 64);
      if (g == 0 && r < ROWS) {
        const float mean = s / (float)D;
        float var = q / (float)D - mean * mean;
        var = var > 0.f ? var : 0.f;
        out_mean[r] = mean;
        out_2[r] = want_sigma ? sqrtf(var + eps) : rsqrtf(var + eps);
      }
    }
  }
};

// one thread's share of a row's statistics: the (sum, sum of squares) of the eight bf16 values of a 16-byte piece
__device__ __forceinline__ void kh_piece_sums(const u32x4 o, float& s, float& q) {
  s = 0.f; q = 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float a = bf16_lo(o[e]), b = bf16_hi(o[e]);
    s += a; q += a * a;
    s += b; q += b * b;
  }
}

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
// query projection + cross-attention in its epilogue (xa_k set)
bool lora_gemm_pipe_xattn_ok(const LoraGemmParams& p);
int lora_gemm_pipe_launch_xattn(const LoraGemmParams& p, hipStream_t stream);
// Narrow-output variant (lora_gemm_ksplit.hip): (32 * row_groups) x 160 tiles, 8 waves as row_groups x k-slices;
// plain or K-extended GEMM with bias / residual, K % 64 == 0.  row_groups 2 or 4.
bool lora_gemm_ksplit_ok(const LoraGemmParams& p);
int lora_gemm_ksplit_launch(const LoraGemmParams& p, int row_groups, hipStream_t stream);
// Shrink and GEMM in one launch on the 128 x 160 tiles, every workgroup computing a piece of T first (p.a_cat / col_scale /
// b_cat set, p.t_ext = scratch for the shrink result, p.il_cnt = counters, p.r_used <= 96 of R = 128).
bool lora_gemm_ksplit_coop_ok(const LoraGemmParams& p);
int lora_gemm_ksplit_launch_coop(const LoraGemmParams& p, hipStream_t stream);
int lora_gemm_ksplit_coop_timeouts(int* count, int clear);
bool lora_gemm_ksplit_conv_ok(const LoraGemmParams& p);
int lora_gemm_ksplit_launch_conv(const LoraGemmParams& p, int row_groups, hipStream_t stream);
// the convolution that also leaves GroupNorm statistics (gn_cg / gn_hw set): row groups of the 160-column tiles it would run
// on, 0 when the rules give it other tiles or the groups do not fit them
int lora_gemm_conv_gn_row_groups(const LoraGemmParams& p);
// Wide-tile variant (lora_gemm_wide.hip): 256 x 320 tiles, 8 waves; plain or K-extended GEMM with bias / residual /
// GEGLU; M % 256 == 0, N % 320 == 0, K % 64 == 0.
bool lora_gemm_wide_ok(const LoraGemmParams& p);
int lora_gemm_wide_launch(LoraGemmParams p, hipStream_t stream);

// The shrink of a layer, optionally with a folded LayerNorm in front (ln_part != nullptr; lora_shrink.hip).
int lora_shrink_ln_launch(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M, int64_t K, int64_t R,
                          const float* ln_part, const float* ln_ca1, const float* ln_ca2, float ln_eps, hipStream_t stream, int group, int r_used);

extern "C" int kh_lora_shrink_bf16(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M, int64_t K,
                                   int64_t R, void* stream);

// Kernel experiments (timestamps, frozen operands, alternative tile maps) exist only in builds with -DKH_TUNING; the
// shipped library compiles them out and its entry points reject the flag bits that would select them.
#ifdef KH_TUNING
#define KH_DBG(p, bit) (((p).dbg & (bit)) != 0)
#else
#define KH_DBG(p, bit) false
#endif

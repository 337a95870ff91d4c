// LoRA shrink for layers that share an input: t[M,R] = bf16((x[M,K] . A_cat[R,K]^T) * col_scale[R]).
//
// The low-rank "down" projection of the reference's LoRA linear
// (diffusers-hf/src/diffusers/models/lora.py:224-225, down(hidden_states)) for all adapters of one or
// several layers that read the same x at once: to_q / to_k / to_v of a self-attention take the same
// normalised hidden states, so their A matrices are stacked into one A_cat and x is read once.
// The result stays L2-resident (M*R*2 bytes, ~1 MB) and is consumed by kh_lora_linear_pre_bf16, which
// then runs the base GEMM without the per-tile shrink recompute of the fused kernel.
//
// Bound: the vector L1 path (64 B/clk per CU).  2*M*K*R FLOPs are ~1 GFLOP, but M*R is so small that
// filling 256 CUs means 32x32 or 64x64 output tiles, and a tile of a x b outputs pulls (a+b)*K*2
// bytes through its CU's L1.  A workgroup owns TR*32 rows x TC*32 rank columns; its NW waves split K.
// Each wave streams its 64-column chunks (dealt round-robin) through a PRIVATE two-stage LDS ring
// with global_load_lds: 8 rows x 128 contiguous bytes per instruction, i.e. whole cache lines (with
// 64-byte rows every line is fetched by two different steps and has left the 32 KB L1 in between; a
// fragment load straight from global memory has every lane in a row of its own and runs at a quarter
// of the L1 rate).  A private ring needs no barrier: the wave waits for its own loads (vmcnt), reads
// the fragments, and refills the stage it has just read.  Partial sums of the NW waves meet in LDS
// in a fixed order (deterministic).
// Tried and dropped: splitting K across workgroups with a last-arriver reduction (the device-scope
// release is an L2 write-back on a multi-XCD part: 40 us); direct global -> register fragments (L1
// tag rate, 3-4x slower at K = 5120).
#include "lora_shrink_tile.h"

namespace {

// GROUP > 0: the rank columns come in groups of GROUP (one stacked layer each) of which only the first C::TC * 32 are in
// use; blockIdx.y counts groups, and the tile's workgroup zeroes the group's padding columns for its rows.
template <class C, int GROUP = 0>
__global__ __launch_bounds__(C::NW * 64) void lora_shrink_kernel(const ShrinkParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int STEP = GROUP > 0 ? GROUP : C::TC * 32;
  const int m0 = (int)blockIdx.x * C::TR * 32, r0 = (int)blockIdx.y * STEP;
  lora_shrink_tile<C, false, C::NW * 64>(p, m0, r0, smem);
  if constexpr (GROUP > C::TC * 32) {
    constexpr int PIECES = (GROUP - C::TC * 32) / 8;   // 16-byte pieces per row
    for (int i = threadIdx.x; i < C::TR * 32 * PIECES; i += C::NW * 64) {
      const int row = m0 + i / PIECES;
      if (row < p.M) *reinterpret_cast<u32x4*>(p.t + (size_t)row * p.R + r0 + C::TC * 32 + (i % PIECES) * 8) = u32x4{0, 0, 0, 0};
    }
  }
}

template <class C, int GROUP = 0>
int launch_shrink(const ShrinkParams& p, hipStream_t stream) {
  if (hipError_t e = kh_allow_lds<lora_shrink_kernel<C, GROUP>>(C::LDS); e != hipSuccess) return (int)e;
  constexpr int STEP = GROUP > 0 ? GROUP : C::TC * 32;
  dim3 grid((unsigned)((p.M + C::TR * 32 - 1) / (C::TR * 32)), (unsigned)((p.R + STEP - 1) / STEP));
  kh_launch(KH_TAG_LORA_SHRINK, lora_shrink_kernel<C, GROUP>, grid, dim3(C::NW * 64), C::LDS, stream, p);
  KH_RETURN_LAST_ERROR();
}

template <int TR, int TC, int NWA, int NWB>
int launch_shrink_k(const ShrinkParams& p, hipStream_t stream) {
  // prefer a wave count that deals the 64-column chunks out evenly
  const int KC = p.K / 64;
  if (KC % NWA == 0 || KC % NWB != 0) return launch_shrink<SCfg<NWA, TR, TC>>(p, stream);
  return launch_shrink<SCfg<NWB, TR, TC>>(p, stream);
}

}  // namespace

KH_EXPORT int kh_lora_shrink_bf16(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M,
                                  int64_t K, int64_t R, void* stream) {
  return lora_shrink_ln_launch(x, a_cat, col_scale, t, M, K, R, nullptr, nullptr, nullptr, 0.f, (hipStream_t)stream, 0, 0);
}

// The shrink, optionally of a layer with a folded LayerNorm (ln_part != nullptr; see ShrinkParams).
// group / r_used (both 0: nothing known): the R columns are stacked layers of `group` packed rank columns each, of which
// the columns >= r_used are padding (A_cat rows of zeros) that need not be computed.
int lora_shrink_ln_launch(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M, int64_t K, int64_t R,
                          const float* ln_part, const float* ln_ca1, const float* ln_ca2, float ln_eps, hipStream_t s,
                          int group, int r_used) {
  if (!x || !a_cat || !col_scale || !t || M <= 0 || K <= 0 || R <= 0) return KH_ERR_INVALID_ARG;
  if (ln_part != nullptr && (!ln_ca1 || !ln_ca2)) return KH_ERR_INVALID_ARG;
  if (K % 64 != 0 || R % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 65535 * 32 || M > (1 << 24)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || !kh_aligned16(a_cat) || !kh_aligned16(t) || (ln_part && !kh_aligned16(ln_part))) return KH_ERR_ALIGNMENT;
  ShrinkParams p;
  p.x = (const bf16_t*)x; p.a_cat = (const bf16_t*)a_cat; p.col_scale = col_scale; p.t = (bf16_t*)t;
  p.M = (int)M; p.K = (int)K; p.R = (int)R;
  p.ln_part = ln_part; p.ln_ca1 = ln_ca1; p.ln_ca2 = ln_ca2; p.ln_eps = ln_eps;
  // several stacked layers of rank 96 in 128 on many rows (q / k / v of the 64 x 64 level): one-wave workgroups, each a
  // 32-row x 96-column tile of one layer over the whole K, five to a CU.  With K this short a tile is a handful of chunks
  // and its time is load latency, not bytes: more independent workgroups per CU win (16.3 us against 20.8 with the 64 x 64
  // tiles below at M 8192, K 640, three layers; 64 x 96 tiles of four waves 21.4, 128 x 96 tiles of two waves 25.3, although
  // both read fewer bytes).  A single layer (R 128) stays with the 64 x 64 tiles: 8.4 us against 13.2.
  if (group == 128 && r_used > 64 && r_used <= 96 && R % 128 == 0 && R >= 256 && M >= 4096)
    return launch_shrink<SCfg<1, 1, 3>, 128>(p, s);
  // the largest output tile that still gives most CUs a workgroup (a 64x64 tile reads half the bytes per output of a 32x64 one)
  if (R % 64 == 0 && ((M + 63) / 64) * (R / 64) >= 160) return launch_shrink_k<2, 2, 4, 5>(p, s);
  if (R % 64 == 0 && ((M + 31) / 32) * (R / 64) >= 256) return launch_shrink_k<1, 2, 4, 5>(p, s);
  return launch_shrink_k<1, 1, 8, 5>(p, s);
}

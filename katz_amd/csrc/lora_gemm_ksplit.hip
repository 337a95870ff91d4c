// K1, narrow-output variant: y = [x | T] . [W | B_cat]^T (+ bias, + residual) on bf16 MFMA (gfx950) with
// (32*WM) x 160 output tiles, for layers whose 128x128 tiles would leave much of the chip idle.
//
// Same arithmetic as the two-launch form of lora_gemm_pipe.hip (the reference's LoRA linear,
// diffusers-hf/src/diffusers/models/lora.py:224-225 after a separate shrink launch): T = the scaled
// shrink result, so the adapters' rank columns are extra K tiles of the base GEMM.
//
// Why another tile shape: N = 1280 = 2^8 * 5.  At M = 2048 the 128x128 tiling has 160 tiles for 256 CUs;
// 64x160 has exactly 256, 128x160 has 256 at M = 8192 / N = 640.  A factor 5 does not divide over 8
// waves in M or N, so the waves split K instead: a workgroup's 8 waves form WM row groups of 32 rows times
// WK = 8 / WM k-slices; a wave owns a 32 x 160 strip of accumulators (5 MFMA tiles) and multiplies only its
// own 16-column slices of every 64-column stage (1 x fragment + 5 W fragments per 5 MFMAs).  After the K
// loop the k-slices of a row group meet in LDS and are added in a fixed order (deterministic), then the
// epilogue is the usual one (bias in fp32, round, transpose through LDS, residual, 16-byte row stores).
//
// Operand movement as in lora_gemm_pipe.hip: global -> LDS by global_load_lds (8 rows x 128 bytes per
// instruction, XOR-swizzled pieces), a ring of 3 stages, loads two stages ahead, one barrier per stage,
// fragments double-buffered in registers.  (32*WM + 160) / 8 DMA units per stage do not divide by 8 waves:
// waves below N_HI issue one more than the others, and every wait picks its count by a wave-uniform branch.
#include "kh_common.h"
#include "lora_gemm.h"
#include "lora_shrink_tile.h"

// Bounded waits of the cooperative shrink that have run out on this GPU; read (and cleared) by kh_lora_split_timeouts
// together with the count of the in-launch shrink of lora_gemm_pipe.hip.
static __device__ int kh_coop_timeout_count;

namespace {

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef __amdgpu_buffer_rsrc_t rsrc_t;
template <int I> using IC = std::integral_constant<int, I>;

template <int VM, int LGKM>
__device__ __forceinline__ void wait_cnt() {  // gfx9 encoding: vmcnt = [15:14|3:0], expcnt = [6:4], lgkmcnt = [11:8]
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | ((LGKM & 15) << 8) | ((VM >> 4) << 14));
}

template <int WM_, int NST_ = 4>
struct KCfg {
  static constexpr int WM = WM_, WK = 8 / WM_;       // row groups x k-slices = 8 waves
  static constexpr int BM = 32 * WM, BN = 160, BK = 64, NST = NST_, TN = 5;   // NST ring stages: loads run NST - 1 K tiles ahead
  static constexpr int KSW = 4 / WK;                 // 16-column MFMA steps of a stage per wave
  static constexpr int UNITS = (BM + BN) / 8;        // DMA instructions per stage (8 rows x 128 B each)
  static constexpr int LPS_LO = UNITS / 8, N_HI = UNITS % 8, LPS_HI = LPS_LO + (N_HI ? 1 : 0);
  static constexpr int STAGE = (BM + BN) * 128;
  static constexpr int RING = NST * STAGE;
  static constexpr int PART = (WK - 1) * WM * 80 * 64 * 4;   // fp32 partial strips of the k-slices 1 .. WK-1
  static constexpr int LDC = BN + 8;
  static constexpr int SC = BM * LDC * 2;
  static constexpr int LDS = RING > PART + SC ? RING : PART + SC;
  static constexpr int OPC = BM * (BN / 8);          // 16-byte output pieces per tile
  static constexpr int OPT = (OPC + 511) / 512;      // per thread
  static_assert(WM == 2 || WM == 4, "row groups");
  static_assert(LDS <= 160 * 1024, "LDS budget");
};

// 16 bytes of zeros (and more): what a 3x3 convolution's DMA reads for taps that fall into the padding
__device__ __attribute__((aligned(256))) const uint32_t ks_zero_page[64] = {0};

// CONV: x is an NHWC image and row m of the GEMM is output pixel m of a 3x3 convolution with padding 1 (K = 9 * Cin
// ordered (kh, kw, ci), see lora_gemm_pipe.hip): a stage of 64 K columns is 64 channels of one tap, the x rows of tap
// (kh, kw) sit (kh * W + kw) * Cin elements after the row's base (the pixel above-left of its window), and rows
// whose tap falls outside the image read zeros.
// GNF: the epilogue also leaves the GroupNorm statistics of the result (LoraGemmParams::gn_part).
// COOP: the launch computes its own shrink, cooperatively.  These tiles fill every CU, so there is no idle CU for shrink
// workgroups beside the GEMM ones; instead EVERY workgroup first computes one piece of T -- 32 rows x 96 rank columns: the
// n_tiles = 4 x (ldt / 128) workgroups of a row block of 128 rows share that block's 4 row quarters x ldt / 128 column
// groups of T, workgroup n_blk takes quarter n_blk % 4 of group n_blk / 4 --, stores it write-through, zeroes the 32
// padding columns of its group, counts itself into the row block's counter and then runs its GEMM tile; before its first
// request for T (the last K tiles) it waits, bounded, for the row block's count and reads T past the L2.  A workgroup
// never waits before its own piece is out, so the launch makes progress in whatever order its workgroups become
// resident, as long as no OTHER launch whose workgroups wait for each other shares the device with it (the binding does
// not use this form on a second stream).
template <class C, bool CONV, bool GNF = false, bool COOP = false>
__global__ __launch_bounds__(512, COOP ? 1 : 2) void lora_gemm_ksplit_kernel(const LoraGemmParams p) {
#if __HIP_DEVICE_COMPILE__   // the host pass only needs the kernel's symbol (it cannot lower the buffer-resource type)
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int BM = C::BM, BN = C::BN, TN = C::TN, KSW = C::KSW, NST = C::NST, STAGE = C::STAGE;
  constexpr int LPS_LO = C::LPS_LO, LPS_HI = C::LPS_HI, N_HI = C::N_HI;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WK, wk = wave % C::WK;
  const int l32 = lane & 31, lh = lane >> 5;

  // the next launch's weights (a cooperative launch issues this after its shrink piece, whose rings use the same LDS)
  if (!COOP) kh_prefetch_lines(p.pf, p.pf_lines, smem + wave * 1024, blockIdx.x, gridDim.x, tid, 512);
  // tile of this workgroup: XCD b % 8 owns a block of xr_m x xr_n tiles (its W rows stay in its L2)
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int m_blk = (xcd / p.xg_n) * p.xr_m + local / p.xr_n;
  const int n_blk = (xcd % p.xg_n) * p.xr_n + local % p.xr_n;
  if (local / p.xr_n >= p.xr_m || m_blk >= p.m_tiles || n_blk >= p.n_tiles) return;  // padding of the grid
  const int m0 = m_blk * BM, n0 = n_blk * BN;
  const int M = p.M, N = p.N, K = p.K;
  const int KT1 = K / 64;
  const int KT = KT1 + (p.t_ext != nullptr ? p.R / 64 : 0);
  const bool has_hi = wave < N_HI;
  if constexpr (COOP) {
    // this workgroup's piece of T = bf16((x . A_cat^T) * col_scale) (with a folded LayerNorm in front: the form documented at
    // ShrinkParams), then the padding columns, then the arrival
    const int q4 = n_blk & 3, grp = n_blk >> 2;
    ShrinkParams sp;
    sp.x = p.x; sp.a_cat = p.a_cat; sp.col_scale = p.col_scale; sp.t = const_cast<bf16_t*>(p.t_ext);
    sp.M = M; sp.K = K; sp.R = p.ldt;
    sp.ln_part = p.ln_part; sp.ln_ca1 = p.ln_ca1; sp.ln_ca2 = p.ln_ca2; sp.ln_eps = p.ln_eps;
    // (a quarter that starts past the last row has nothing to compute: the tile's addressing assumes m0 < M)
    if (m0 + 32 * q4 < M) lora_shrink_tile<SCfg<4, 1, 3>, true, 512>(sp, m0 + 32 * q4, grp * 128, smem);
    if (tid < 128) {   // columns 96 .. 127 of the group: 32 rows x 4 pieces of 16 bytes
      const int row = m0 + 32 * q4 + (tid >> 2);
      if (row < M) {
        uint32_t* dst = reinterpret_cast<uint32_t*>(const_cast<bf16_t*>(p.t_ext) + (size_t)row * p.ldt + grp * 128 + 96 + (tid & 3) * 8);
#pragma unroll
        for (int e = 0; e < 4; ++e) __hip_atomic_store(dst + e, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __builtin_amdgcn_s_waitcnt(0);                          // this thread's write-through stores have completed
    __syncthreads();
    if (tid == 0) __hip_atomic_fetch_add(p.il_cnt + m_blk, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    kh_prefetch_lines(p.pf, p.pf_lines, smem + wave * 1024, blockIdx.x, gridDim.x, tid, 512);
  }
  // folded LayerNorm: mean and 1/std of this tile's x rows, read in the epilogue (the barriers of the K loop lie between)
  // and the two per-column terms of this column tile; requested here, finished once the bias loads are under way
  float* sMu = reinterpret_cast<float*>(smem + p.ln_lds);
  float* sRs = sMu + 256;
  float* sc1 = sRs + 256;
  float* sc2 = sc1 + 256;
  KhLnTileStats<BM, 512> ln_stats;
  float ln_c1v = 0.f, ln_c2v = 0.f;
  if (p.ln_part != nullptr) {
    ln_stats.load(p.ln_part, m0, M, tid);
    if (tid < BN) {
      ln_c1v = n0 + tid < N ? p.ln_c1[n0 + tid] : 0.f;
      ln_c2v = n0 + tid < N ? p.ln_c2[n0 + tid] : 0.f;
    }
  }


  // DMA of this lane: unit u = wave + 8*q covers stage rows u*8 .. u*8+7 (x rows first, then W rows); LDS slot = lane:
  // row lane/8, physical piece lane%8, which holds logical piece (lane%8) ^ ((row/2)%8).  The loads are buffer loads:
  // a byte offset per lane that never changes (voff: row and piece) plus a scalar byte offset per K tile, so that the
  // loop carries no vector address arithmetic (with per-lane 64-bit pointers the adds and selects of every stage sat in
  // the same issue stream as the MFMAs and the loop ran at the sum of both).  An offset at or beyond the buffer's size
  // reads zeros without touching memory: that is what a 3x3 convolution's taps in the padding do.
  constexpr uint32_t OOB = 0x80000000u;                // every buffer here is shorter than 2 GiB
  uint32_t voff[LPS_HI], voff2[LPS_HI];
  int tapmask[LPS_HI];                                 // CONV, x units: bit t = tap t of this lane's row is inside the image
  constexpr int XQ = BM / 64;                          // units q < XQ are x rows for every wave, the others W rows
#pragma unroll
  for (int q = 0; q < LPS_HI; ++q) {
    int u = wave + 8 * q;
    u = u < C::UNITS ? u : C::UNITS - 1;               // never issued (has_hi), keep the offset valid
    const int r = u * 8 + (lane >> 3);
    const uint32_t pcb = (uint32_t)(((lane & 7) ^ ((r >> 1) & 7)) * 16);
    tapmask[q] = 0;
    if (CONV && r < BM) {
      int row = m0 + r; row = row < M ? row : M - 1;
      const int wo = row % p.conv_wo, t2 = row / p.conv_wo, ho = t2 % p.conv_ho, nb = t2 / p.conv_ho;
      const int hi0 = ho * p.conv_stride - 1, wi0 = wo * p.conv_stride - 1;
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) {
        const int hi = hi0 + tap / 3, wi = wi0 + tap % 3;
        tapmask[q] |= (hi >= 0 && hi < p.conv_h && wi >= 0 && wi < p.conv_w) ? (1 << tap) : 0;
      }
      // relative to one row and one pixel in front of the image (the buffer's base), so that it is never negative
      voff[q] = (uint32_t)(((nb * p.conv_h + hi0 + 1) * p.conv_w + wi0 + 1) * p.conv_cin) * 2u + pcb;
      voff2[q] = voff[q];
    } else if (r < BM) {
      int row = m0 + r; row = row < M ? row : M - 1;
      voff[q] = (uint32_t)row * (uint32_t)K * 2u + pcb;
      voff2[q] = ((uint32_t)row * (uint32_t)p.ldt + (uint32_t)(p.t_nsplit > 0 ? (n0 / p.t_nsplit) * p.R : 0)) * 2u + pcb;
    } else {
      int row = n0 + r - BM; row = row < N ? row : N - 1;
      voff[q] = (uint32_t)row * (uint32_t)K * 2u + pcb;
      voff2[q] = (uint32_t)row * (uint32_t)p.R * 2u + pcb;
    }
  }
  const size_t x_bytes = CONV ? (size_t)(M / (p.conv_ho * p.conv_wo)) * p.conv_h * p.conv_w * p.conv_cin * 2 : (size_t)M * K * 2;
  const size_t x_lead = CONV ? (size_t)(p.conv_w + 1) * p.conv_cin * 2 : 0;
  const rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(reinterpret_cast<const char*>(p.x) - x_lead), 0,
                                                         (int)(x_bytes + x_lead), 0x00020000);
  const rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.w), 0, (int)((size_t)N * K * 2), 0x00020000);
  const rsrc_t rs_t = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.t_ext != nullptr ? p.t_ext : p.x), 0,
                                                         p.t_ext != nullptr ? (int)((size_t)M * p.ldt * 2) : 0, 0x00020000);
  const rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.t_ext != nullptr ? p.b_cat : p.w), 0,
                                                         p.t_ext != nullptr ? (int)((size_t)N * p.R * 2) : 0, 0x00020000);
  // CONV: K tiles are requested in order, so the tap and the channel offset of the next request are running scalars, and
  // the x offsets with the current tap's padding applied change only when the tap does
  int cv_tap = 0, cv_kw = 0, cv_c0 = 0, cv_shift = 0, cv_row = 0;
  uint32_t xvo[XQ];
#pragma unroll
  for (int q = 0; q < XQ; ++q) xvo[q] = (tapmask[q] & 1) ? voff[q] : OOB;
  auto issue = [&](int t, auto stc) {                  // K tile t into ring stage stc
    char* stage = smem + decltype(stc)::value * STAGE;
    if (CONV || t < KT1) {
      const int so = t * 128;
#pragma unroll
      for (int q = 0; q < LPS_HI; ++q) {
        if (q < LPS_LO || has_hi) {
          if (CONV && q < XQ)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lptr_t)(stage + (wave + 8 * q) * 1024), 16, xvo[q], (cv_shift + cv_c0) * 2, 0, 0);
          else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(q < XQ ? rs_x : rs_w, (lptr_t)(stage + (wave + 8 * q) * 1024), 16, voff[q], so, 0, 0);
        }
      }
    } else {
      if (COOP && t == KT1) {
        // first request for T: wait (bounded) until every workgroup of this row block has delivered its piece
        if (lane == 0) {
          int it = 0;
          while (__hip_atomic_load(p.il_cnt + m_blk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < p.n_tiles && ++it < (1 << 20))
            __builtin_amdgcn_s_sleep(8);
          if (it >= (1 << 20)) {
            __hip_atomic_store(p.il_cnt + (p.M + 127) / 128, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_fetch_add(&kh_coop_timeout_count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
      const int so = (t - KT1) * 128;
#pragma unroll
      for (int q = 0; q < LPS_HI; ++q)
        if (q < LPS_LO || has_hi) {
          // (COOP) T was written inside this launch, maybe on another XCD: read past the (non-coherent) L2
          if (COOP && q < XQ) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_t, (lptr_t)(stage + (wave + 8 * q) * 1024), 16, voff2[q], so, 0, 17 /* sc0 sc1 */);
          else __builtin_amdgcn_raw_ptr_buffer_load_lds(q < XQ ? rs_t : rs_b, (lptr_t)(stage + (wave + 8 * q) * 1024), 16, voff2[q], so, 0, 0);
        }
    }
    if (CONV) {
      cv_c0 += 64;
      if (cv_c0 == p.conv_cin) {
        cv_c0 = 0; ++cv_tap; ++cv_kw; cv_shift += p.conv_cin;
        if (cv_kw == 3) { cv_kw = 0; cv_row += p.conv_w * p.conv_cin; cv_shift = cv_row; }
#pragma unroll
        for (int q = 0; q < XQ; ++q) xvo[q] = ((tapmask[q] >> cv_tap) & 1) ? voff[q] : OOB;
      }
    }
  };
  // wait until at most n of this wave's younger K tiles are outstanding (and its LDS reads are done)
  constexpr int PD = NST - 1;                            // prefetch distance in K tiles
  static_assert(NST == 3 || NST == 4, "groups of 6 or 4 written-out steps");
  auto wait_younger = [&](int n) {
    if (n >= PD - 1) { if (has_hi) wait_cnt<LPS_HI * (PD - 1), 0>(); else wait_cnt<LPS_LO * (PD - 1), 0>(); }
    else if (n == 1) { if (has_hi) wait_cnt<LPS_HI, 0>(); else wait_cnt<LPS_LO, 0>(); }
    else wait_cnt<0, 0>();
  };

  // fragment addresses: byte offsets into a stage that never change (the stage is a compile-time constant of every
  // unrolled step and lands in the instruction's offset field; stage 2 lies beyond that field's 64 KB and gets a
  // second set)
  struct Fr { bf16x8 a[KSW]; bf16x8 b[KSW][TN]; };
  const int sw = (l32 >> 1) & 7;
  int fa[KSW], fb[KSW], fa2[KSW], fb2[KSW];
#pragma unroll
  for (int k = 0; k < KSW; ++k) {
    const int po = ((2 * (wk * KSW + k) + lh) ^ sw) * 16;
    fa[k] = (wm * 32 + l32) * 128 + po;
    fb[k] = (BM + l32) * 128 + po;
    fa2[k] = fa[k] + 2 * STAGE;
    fb2[k] = fb[k] + 2 * STAGE;
  }
  auto read_frags = [&](auto stc, Fr& f) {
    constexpr int ST = decltype(stc)::value;
#pragma unroll
    for (int k = 0; k < KSW; ++k) {
      const char* pa = ST >= 2 ? smem + fa2[k] + (ST - 2) * STAGE : smem + fa[k] + ST * STAGE;
      const char* pb = ST >= 2 ? smem + fb2[k] + (ST - 2) * STAGE : smem + fb[k] + ST * STAGE;
      f.a[k] = *reinterpret_cast<const bf16x8*>(pa);
#pragma unroll
      for (int j = 0; j < TN; ++j) f.b[k][j] = *reinterpret_cast<const bf16x8*>(pb + j * 32 * 128);
    }
  };
  f32x16 acc[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
  auto mma = [&](const Fr& f) {
#pragma unroll
    for (int k = 0; k < KSW; ++k)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[k], f.b[k][j], acc[j], 0, 0, 0);
  };

  // bias of this lane's columns, requested before the loop
  float bv[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + j * 32 + l32;
    bv[j] = (p.bias != nullptr && col < N) ? (float)p.bias[col] : 0.f;
  }
  if (p.ln_part != nullptr) {
    ln_stats.finish(K, p.ln_eps, tid, sMu, sRs, false);
    if (tid < BN) { sc1[tid] = ln_c1v; sc2[tid] = ln_c2v; }
  }
  wait_cnt<0, 15>();

  // K loop.  Step t: tile t is in registers (cur); tile t+1 becomes visible at the barrier, after which every wave has
  // read tile t out of its stage, so that stage takes tile t+1+PD.  lcm(NST, 2) steps (ring stages x two register
  // buffers) are written out, so the stage of every access is a constant; the steady group carries no conditions.
  Fr f0, f1;
  issue(0, IC<0>{});
  if (KT > 1) issue(1, IC<1>{});
  if (PD > 2 && KT > 2) issue(2, IC<2>{});
  wait_younger(KT - 1);
  __builtin_amdgcn_s_barrier();
  if (KT > PD) issue(PD, IC<PD>{});
  read_frags(IC<0>{}, f0);
  // st_next: stage of tile t+1; st_fill: stage that tile t+1+PD refills (= stage of tile t)
  auto step = [&](int t, const Fr& cur, Fr& nxt, auto st_next, auto st_fill, auto steady) {
    if constexpr (decltype(steady)::value) {
      wait_younger(PD - 1);
      __builtin_amdgcn_s_barrier();
      issue(t + 1 + PD, st_fill);
      read_frags(st_next, nxt);
    } else if (t + 1 < KT) {
      wait_younger(KT - 2 - t);
      __builtin_amdgcn_s_barrier();
      if (t + 1 + PD < KT) issue(t + 1 + PD, st_fill);
      read_frags(st_next, nxt);
    }
    mma(cur);
  };
  constexpr int U = (NST % 2 == 0) ? NST : 2 * NST;
  using T1 = std::true_type; using T0 = std::false_type;
  int t = 0;
  for (; t + U + PD < KT; t += U) {
    step(t, f0, f1, IC<1 % NST>{}, IC<0>{}, T1{});
    step(t + 1, f1, f0, IC<2 % NST>{}, IC<1 % NST>{}, T1{});
    step(t + 2, f0, f1, IC<3 % NST>{}, IC<2 % NST>{}, T1{});
    step(t + 3, f1, f0, IC<4 % NST>{}, IC<3 % NST>{}, T1{});
    if constexpr (U == 6) {
      step(t + 4, f0, f1, IC<5 % NST>{}, IC<4 % NST>{}, T1{});
      step(t + 5, f1, f0, IC<6 % NST>{}, IC<5 % NST>{}, T1{});
    }
  }
  for (; t < KT; t += U) {
    step(t, f0, f1, IC<1 % NST>{}, IC<0>{}, T0{});
    if (t + 1 < KT) step(t + 1, f1, f0, IC<2 % NST>{}, IC<1 % NST>{}, T0{});
    if (t + 2 < KT) step(t + 2, f0, f1, IC<3 % NST>{}, IC<2 % NST>{}, T0{});
    if (t + 3 < KT) step(t + 3, f1, f0, IC<4 % NST>{}, IC<3 % NST>{}, T0{});
    if constexpr (U == 6) {
      if (t + 4 < KT) step(t + 4, f0, f1, IC<5 % NST>{}, IC<4 % NST>{}, T0{});
      if (t + 5 < KT) step(t + 5, f1, f0, IC<6 % NST>{}, IC<5 % NST>{}, T0{});
    }
  }
  __syncthreads();   // the ring is dead: partial strips and the staging tile reuse it

  // residual pieces of this thread, requested before the reduction
  u32x4 rr[C::OPT];
  if (p.res != nullptr) {
#pragma unroll
    for (int q = 0; q < C::OPT; ++q) {
      const int c = tid + q * 512, srow = c / (BN / 8), ch = c % (BN / 8);
      const int grow = m0 + srow, gcol = n0 + ch * 8;
      rr[q] = (c < C::OPC && grow < M && gcol < N) ? *reinterpret_cast<const u32x4*>(p.res + (size_t)grow * N + gcol)
                                                  : u32x4{0, 0, 0, 0};
    }
  }
  // k-slices 1 .. WK-1 hand their strips to slice 0 of their row group: 20 x 16 bytes per lane, lane-contiguous
  // (writer lane = reader lane, so the layout is free)
  f32x4* part = reinterpret_cast<f32x4*>(smem);
  if (wk > 0) {
    f32x4* dst = part + ((size_t)((wk - 1) * C::WM + wm) * 20) * 64 + lane;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        dst[(j * 4 + g) * 64] = f32x4{acc[j][4 * g], acc[j][4 * g + 1], acc[j][4 * g + 2], acc[j][4 * g + 3]};
  }
  __syncthreads();
  bf16_t* sC = reinterpret_cast<bf16_t*>(smem + C::PART);
  if (wk == 0) {
#pragma unroll
    for (int s = 1; s < C::WK; ++s) {                  // fixed order: deterministic
      const f32x4* srcp = part + ((size_t)((s - 1) * C::WM + wm) * 20) * 64 + lane;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 v = srcp[(j * 4 + g) * 64];
          acc[j][4 * g] += v[0]; acc[j][4 * g + 1] += v[1]; acc[j][4 * g + 2] += v[2]; acc[j][4 * g + 3] += v[3];
        }
    }
    if (p.ln_part != nullptr) {
      // y = rstd_row * (acc - mean_row * c1_col) + c2_col: four consecutive rows per accumulator group
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int trow = wm * 32 + 8 * g + 4 * lh;
        const f32x4 mu = *reinterpret_cast<const f32x4*>(sMu + trow), rs = *reinterpret_cast<const f32x4*>(sRs + trow);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const float c1 = sc1[j * 32 + l32], c2 = sc2[j * 32 + l32];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            sC[(trow + e) * C::LDC + j * 32 + l32] = (bf16_t)(rs[e] * (acc[j][4 * g + e] - mu[e] * c1) + c2);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = j * 32 + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
          sC[row * C::LDC + col] = (bf16_t)(acc[j][v] + bv[j]);
        }
      }
    }
  }
  __syncthreads();
  if constexpr (GNF) {
    // GroupNorm statistics as a by-product: the staged tile is BM pixels of one image times BN / gn_cg whole groups; their
    // (sum, sum of squares) over the bf16-rounded values (residual included) plus the per-(image, channel) term -- what a GroupNorm
    // kernel reading the stored result would take -- go to gn_part[image][group][row tile of the image].  Three short passes,
    // sums in fixed orders (deterministic); the tile itself is stored below as usual.
    constexpr int PCS = BN / 8, RP = 512 / PCS;               // 16-byte pieces per row, row parts (25 of 20 threads)
    float* colp = reinterpret_cast<float*>(smem);             // [RP][BN][2]: the partial strips are dead
    float* cols = colp + RP * BN * 2;                         // [BN][2] column sums
    static_assert((RP * BN * 2 + BN * 2) * 4 <= C::PART, "column sums fit the dead partial strips");
    const int cg = p.gn_cg, ng = BN / cg, G = N / cg;
    const int n_img = m0 / p.gn_hw, split = (m0 % p.gn_hw) / BM, splits = p.gn_hw / BM;
    if (p.res != nullptr) {
      // the statistics are those of the stored result: the residual goes into the staged tile first (the same rounded adds
      // the store loop would make), and the store loop below then writes the tile as it is
#pragma unroll
      for (int q = 0; q < C::OPT; ++q) {
        const int c = tid + q * 512, srow = c / (BN / 8), ch = c % (BN / 8);
        if (c < C::OPC) {
          u32x4 o = *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + ch * 8);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[q][e]), bf16_hi(o[e]) + bf16_hi(rr[q][e]));
          *reinterpret_cast<u32x4*>(sC + srow * C::LDC + ch * 8) = o;
        }
      }
      __syncthreads();
    }
    // the per-(image, channel) term enters through sum(a + t) = sum(a) + n t and sum((a + t)^2) = sum(a^2) + 2 t sum(a) + n t^2:
    // requested now, used after the first pass
    const float ad = (tid < BN && p.gn_add != nullptr) ? (float)p.gn_add[(size_t)n_img * N + n0 + tid] : 0.f;
    if (tid < RP * PCS) {
      const int ch = tid % PCS, part = tid / PCS;
      float cs[8], cq[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) cs[e] = cq[e] = 0.f;
#pragma unroll
      for (int i = 0; i < (BM + RP - 1) / RP; ++i) {
        const int r = part + i * RP;
        if (r < BM) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(sC + r * C::LDC + ch * 8);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float a = bf16_lo(v[e]), b2 = bf16_hi(v[e]);
            cs[2 * e] += a; cq[2 * e] = fmaf(a, a, cq[2 * e]);
            cs[2 * e + 1] += b2; cq[2 * e + 1] = fmaf(b2, b2, cq[2 * e + 1]);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) *reinterpret_cast<f32x2*>(colp + ((part * BN) + ch * 8 + e) * 2) = f32x2{cs[e], cq[e]};
    }
    __syncthreads();
    if (tid < BN) {
      float s = 0.f, q = 0.f;
#pragma unroll
      for (int part = 0; part < RP; ++part) { const f32x2 v = *reinterpret_cast<const f32x2*>(colp + (part * BN + tid) * 2); s += v[0]; q += v[1]; }
      *reinterpret_cast<f32x2*>(cols + tid * 2) = f32x2{s + (float)BM * ad, q + 2.f * ad * s + (float)BM * ad * ad};
    }
    __syncthreads();
    if (tid < ng) {
      float s = 0.f, q = 0.f;
      for (int c = tid * cg; c < (tid + 1) * cg; ++c) { s += cols[2 * c]; q += cols[2 * c + 1]; }
      *reinterpret_cast<f32x2*>(p.gn_part + (((size_t)n_img * G + n0 / cg + tid) * splits + split) * 2) = f32x2{s, q};
    }
  }
  const KhOut yout(p.y, (size_t)M * N * 2);
  if (p.st_part != nullptr) {
    // as below, and every row's (sum, sum of squares) over this tile's columns for a following folded LayerNorm: the 20
    // pieces of a row meet in LDS (the partial strips are dead) and are added in a fixed order
    float* sp = reinterpret_cast<float*>(smem);          // [BM][20][2]
    static_assert(BM * 20 * 8 <= C::PART, "row statistics fit the dead partial strips");
#pragma unroll
    for (int q = 0; q < C::OPT; ++q) {
      const int c = tid + q * 512, srow = c / (BN / 8), ch = c % (BN / 8);
      const int grow = m0 + srow, gcol = n0 + ch * 8;
      const bool ok = c < C::OPC && grow < M && gcol < N;
      u32x4 o = ok ? *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + ch * 8) : u32x4{0, 0, 0, 0};
      if (p.res != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[q][e]), bf16_hi(o[e]) + bf16_hi(rr[q][e]));
      }
      if (ok) yout.store16(((size_t)grow * N + gcol) * 2, o);
      float ps, pq;
      kh_piece_sums(o, ps, pq);
      if (c < C::OPC) *reinterpret_cast<u32x2*>(sp + 2 * c) = u32x2{__float_as_uint(ps), __float_as_uint(pq)};
    }
    __syncthreads();
    if (tid < BM && m0 + tid < M) {
      float s = 0.f, q2 = 0.f;
#pragma unroll
      for (int ch = 0; ch < BN / 8; ++ch) { s += sp[2 * (tid * (BN / 8) + ch)]; q2 += sp[2 * (tid * (BN / 8) + ch) + 1]; }
      kh_ln_store_stats(p.st_part, m0 + tid, M, n_blk, p.n_tiles, s, q2);
    }
    return;
  }
#pragma unroll
  for (int q = 0; q < C::OPT; ++q) {
    const int c = tid + q * 512, srow = c / (BN / 8), ch = c % (BN / 8);
    const int grow = m0 + srow, gcol = n0 + ch * 8;
    if (c < C::OPC && grow < M && gcol < N) {
      u32x4 o = *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + ch * 8);
      if (!GNF && p.res != nullptr) {   // (GNF: already added into the staged tile)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[q][e]), bf16_hi(o[e]) + bf16_hi(rr[q][e]));
      }
      yout.store16(((size_t)grow * N + gcol) * 2, o);
    }
  }
#endif
}

template <class C, bool CONV = false, bool GNF = false, bool COOP = false>
int launch_ksplit(LoraGemmParams p, hipStream_t stream) {
  p.m_tiles = (p.M + C::BM - 1) / C::BM;
  p.n_tiles = (p.N + C::BN - 1) / C::BN;
  static_assert(C::LDS + KH_LN_LDS <= 160 * 1024, "LDS budget with the row statistics");
  static_assert(!COOP || (SCfg<4, 1, 3>::LDS <= C::LDS && C::BM == 128), "the shrink piece's rings fit the GEMM ring; four quarters per row block");
  if (hipError_t e = kh_allow_lds<lora_gemm_ksplit_kernel<C, CONV, GNF, COOP>>(C::LDS + KH_LN_LDS); e != hipSuccess) return (int)e;
  if ((p.ln_part != nullptr || p.st_part != nullptr) && CONV) return KH_ERR_UNSUPPORTED;
  if (p.st_part != nullptr && p.n_tiles > KH_LN_SLOTS) return KH_ERR_UNSUPPORTED;
  p.ln_lds = C::LDS;
  const size_t lds = (size_t)C::LDS + (p.ln_part != nullptr ? KH_LN_LDS : 0);
  // the XCD grid whose per-XCD block touches the fewest operand rows, padding counted as cost
  double best = 0;
  p.xg_n = 0;
  for (int gm = 1; gm <= 8; gm *= 2) {
    const int gn = 8 / gm;
    const int rm = (p.m_tiles + gm - 1) / gm, rn = (p.n_tiles + gn - 1) / gn;
    const double cost = ((double)rm * C::BM + (double)rn * C::BN) * (8.0 * rm * rn) / ((double)p.m_tiles * p.n_tiles);
    if (p.xg_n == 0 || cost < best) { best = cost; p.xg_n = gn; p.xr_m = rm; p.xr_n = rn; }
  }
  const unsigned grid = 8u * (unsigned)p.xr_m * (unsigned)p.xr_n;
  if constexpr (GNF) {
    // whole groups per tile, whole tiles per image
    if (p.st_part != nullptr || p.gn_cg <= 0 || C::BN % p.gn_cg != 0 || p.N % C::BN != 0 || p.gn_hw % C::BM != 0 ||
        p.M % p.gn_hw != 0)
      return KH_ERR_UNSUPPORTED;
  }
  kh_launch(CONV ? KH_TAG_CONV : KH_TAG_LORA_GEMM, lora_gemm_ksplit_kernel<C, CONV, GNF, COOP>, dim3(grid), dim3(512), lds, stream, p);
  KH_RETURN_LAST_ERROR();
}

}  // namespace

// every operand is addressed as a buffer with 32-bit byte offsets: shorter than 2 GiB each
static bool ks_fits_buffers(const LoraGemmParams& p) {
  const size_t lim = (size_t)1 << 31;
  const size_t xb = p.conv_cin > 0 ? ((size_t)(p.M / (p.conv_ho * p.conv_wo)) * p.conv_h + 1) * p.conv_w * p.conv_cin * 2 + 2 * (size_t)p.conv_cin
                                   : (size_t)p.M * p.K * 2;
  return xb < lim && (size_t)p.N * p.K * 2 < lim && (size_t)p.M * (p.ldt > 0 ? p.ldt : 1) * 2 < lim && (size_t)p.N * (p.R > 0 ? p.R : 1) * 2 < lim;
}

bool lora_gemm_ksplit_ok(const LoraGemmParams& p) {
  const bool plain = p.R == 0 || p.t_ext != nullptr;
  return plain && ks_fits_buffers(p) && p.grp == nullptr && p.sg_mode == 0 && p.conv_cin == 0 && !p.geglu && p.K % 64 == 0 && p.K >= 64 &&
         (p.t_ext == nullptr || (p.R % 64 == 0 && p.ldt % 8 == 0)) && (p.t_nsplit == 0 || p.t_nsplit % 160 == 0) &&
         p.N % 8 == 0;
}

// The cooperative form (see the kernel): the layers whose 128 x 160 tiles fill the chip -- exactly the shapes the rule in
// lora_gemm_pipe_launch gives these tiles --, T of one or several stacked layers with 128 packed rank columns each of which
// at most 96 are in use, four column tiles per 128 rank columns of T.
bool lora_gemm_ksplit_coop_ok(const LoraGemmParams& p) {
  if (!(p.t_ext != nullptr && p.a_cat != nullptr && p.col_scale != nullptr && p.il_cnt != nullptr)) return false;
  if (!lora_gemm_ksplit_ok(p) || p.N % 160 != 0 || p.R != 128 || p.r_used <= 0 || p.r_used > 96 || p.ldt % 128 != 0) return false;
  const long tiles = (long)((p.M + 127) / 128) * ((p.N + 127) / 128), m128 = (p.M + 127) / 128, n160 = p.N / 160;
  if (!(tiles > 256 && tiles <= 384 && m128 * n160 <= 256)) return false;
  const bool t_ok = p.t_nsplit == 0 ? p.ldt == p.R : (p.N % p.t_nsplit == 0 && p.ldt == (p.N / p.t_nsplit) * p.R);
  return t_ok && n160 == 4 * (p.ldt / 128) && n160 <= KH_LN_SLOTS;
}

// this file's share of kh_lora_split_timeouts (synchronous)
int lora_gemm_ksplit_coop_timeouts(int* count, int clear) {
  int v = 0;
  hipError_t e = hipMemcpyFromSymbol(&v, HIP_SYMBOL(kh_coop_timeout_count), sizeof(int), 0, hipMemcpyDeviceToHost);
  if (e != hipSuccess) return (int)e;
  *count = v;
  if (clear && v != 0) {
    const int zero = 0;
    e = hipMemcpyToSymbol(HIP_SYMBOL(kh_coop_timeout_count), &zero, sizeof(int), 0, hipMemcpyHostToDevice);
    if (e != hipSuccess) return (int)e;
  }
  return KH_OK;
}

int lora_gemm_ksplit_launch_coop(const LoraGemmParams& p, hipStream_t stream) {
  if (!lora_gemm_ksplit_coop_ok(p)) return KH_ERR_UNSUPPORTED;
  return launch_ksplit<KCfg<4>, false, false, true>(p, stream);
}

int lora_gemm_ksplit_launch(const LoraGemmParams& p, int row_groups, hipStream_t stream) {
  if (!lora_gemm_ksplit_ok(p)) return KH_ERR_UNSUPPORTED;
  return row_groups == 4 ? launch_ksplit<KCfg<4>>(p, stream) : launch_ksplit<KCfg<2>>(p, stream);
}

// 3x3 convolution on the same tiles (conv_* fields set, R == 0, K == 9 * conv_cin, conv_cin % 64 == 0).
bool lora_gemm_ksplit_conv_ok(const LoraGemmParams& p) {
  return p.conv_cin > 0 && p.conv_cin % 64 == 0 && p.K == 9 * p.conv_cin && ks_fits_buffers(p) && p.R == 0 && p.t_ext == nullptr && p.grp == nullptr &&
         p.sg_mode == 0 && !p.geglu && p.N % 8 == 0;
}

int lora_gemm_ksplit_launch_conv(const LoraGemmParams& p, int row_groups, hipStream_t stream) {
  if (!lora_gemm_ksplit_conv_ok(p)) return KH_ERR_UNSUPPORTED;
  if (p.gn_part != nullptr) return row_groups == 4 ? launch_ksplit<KCfg<4>, true, true>(p, stream) : launch_ksplit<KCfg<2>, true, true>(p, stream);
  return row_groups == 4 ? launch_ksplit<KCfg<4>, true>(p, stream) : launch_ksplit<KCfg<2>, true>(p, stream);
}

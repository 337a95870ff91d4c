// K1, wide-tile variant: y = [x | T] . [W | B_cat]^T (+ bias, + residual | GEGLU) on bf16 MFMA (gfx950) with
// 256 x 320 output tiles, for the layers with the most output columns (the GEGLU projection of the feed-forward,
// diffusers-hf/src/diffusers/models/activations.py:148-149 over attention.py:283-403's ff.net.0.proj).
//
// Same arithmetic as the two-launch form of lora_gemm_pipe.hip (T = the scaled shrink result, so the adapters'
// rank columns are extra K tiles of the base GEMM).  Why another tile shape: N = 10240 at M = 2048 is 640 tiles of
// 128 x 128, two and a half per CU; 256 x 320 tiles are exactly 256, one per CU, and a tile of that size moves
// 0.45 times the operand bytes per FLOP through the CU's load path, which is what the smaller tile runs into.
// The 80 K accumulators of a tile live in the registers of 8 waves (4 row groups x 2 column groups, 64 x 160 =
// 2 x 5 MFMA tiles = 160 registers per lane); the compiler is held to 256 registers per lane.
//
// The MFMA operands are W first, x second: the accumulators then hold, per lane, one output row and runs of four
// consecutive columns, so the epilogue's transpose through LDS writes 8 bytes per instruction instead of 2.
//
// K loop: 64-column stages (128-byte rows, XOR-swizzled 16-byte pieces), two stages in LDS (144 KB), every wave
// issues 9 global_load_lds per stage.  Fragments are double-buffered per 16-column MFMA step: the reads of step
// s+2 are issued before the MFMAs of step s+1, so ten MFMAs cover every read.  The barrier that publishes the
// next stage sits before the last step of the current one: by then every wave has read all of the current stage,
// so the loads of the stage after next can refill it at once, a full stage of MFMAs ahead of their use.
#include "kh_common.h"
#include "lora_gemm.h"

namespace {

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
typedef __amdgpu_buffer_rsrc_t rsrc_t;

template <int VM, int LGKM>
__device__ __forceinline__ void wait_cnt() {  // gfx9 encoding: vmcnt = [15:14|3:0], expcnt = [6:4], lgkmcnt = [11:8]
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | ((LGKM & 15) << 8) | ((VM >> 4) << 14));
}

// GEGLU: bf16(gelu(gate)) for every bf16 gate with 2^-15 <= |gate| < 32, built by each workgroup with the same
// function the direct evaluation uses (so the two agree bit for bit), looked up in the epilogue: the epilogue of a
// tile this size has tens of thousands of gelu evaluations and nothing to overlap them with
constexpr int WTAB_LO = 0x3800, WTAB_N = 2560;               // magnitudes 0x3800 .. 0x41ff, per sign

// 8 waves = 4 row groups x 2 column groups; a wave owns TM x TN MFMA tiles of 32 x 32: tile (128 TM) x (64 TN).
// Only 256 x 320 (TM 2, TN 5) is instantiated: 128 x 256, 256 x 256 and 128 x 320 were measured on the SDXL shapes
// and never beat the tiles of lora_gemm_pipe.hip there.
template <int TM_, int TN_>
struct WCfg {
  static constexpr int TM = TM_, TN = TN_;
  static constexpr int BM = 128 * TM, BN = 64 * TN;
  static constexpr int WR = 32 * TM, WC = 32 * TN;            // rows / columns of a wave
  static constexpr int STAGE = (BM + BN) * 128;               // one 64-column stage
  static constexpr int TAB_OFF = 2 * STAGE;
  static constexpr int BIAS_OFF = TAB_OFF + 2 * WTAB_N * 2;   // the tile's bias values (bf16)
  static constexpr int LDS = BIAS_OFF + BN * 2;
  static constexpr int LN_LDS = 2 * BM * 4 + 2 * BN * 4;      // folded LayerNorm: mean, 1/std per row; c1, c2 per column (fp32)
  static_assert(LDS % 16 == 0 && LDS + LN_LDS <= 160 * 1024, "LDS budget with the LayerNorm terms");
  static constexpr int XU = 2 * TM, WU = TN, LPS = XU + WU;   // DMA instructions per wave per stage (x rows, W rows)
  // staged row of the epilogue: (BN + pad) / 2 dwords = 4 mod 64 banks
  static constexpr int LDC = BN + ((8 + 128 - BN % 128) % 128);
  static_assert((LDC / 2) % 64 == 4 && LDC >= BN, "staging row stride");
  static_assert(LDS <= 160 * 1024, "LDS budget");
  static_assert(128 * LDC * 2 <= 2 * STAGE, "epilogue staging fits the ring");
  static_assert(BN <= 512 && (128 * (BN / 8)) % 512 == 0 && (128 * (BN / 16)) % 512 == 0, "epilogue split");
};

template <class C>
struct WFrT { bf16x8 a[C::TM]; bf16x8 b[C::TN]; };

template <class C>
__global__ __launch_bounds__(512, 2) void lora_gemm_wide_kernel(const LoraGemmParams p) {
#if __HIP_DEVICE_COMPILE__   // the host pass only needs the kernel's symbol (it cannot lower the buffer-resource type)
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int WBM = C::BM, WBN = C::BN, WTM = C::TM, WTN = C::TN, WSTAGE = C::STAGE, WLDC = C::LDC;
  constexpr int WXU = C::XU, WWU = C::WU, WLPS = C::LPS, WTAB_OFF = C::TAB_OFF, WBIAS_OFF = C::BIAS_OFF;
  constexpr int WR = C::WR, WC = C::WC;
  using WFr = WFrT<C>;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lh = lane >> 5;

  kh_prefetch_lines(p.pf, p.pf_lines, smem + wave * (WBM / 8) * 128, blockIdx.x, gridDim.x, tid, 512);   // the next launch's weights
  // tile of this workgroup: XCD b % 8 owns a block of xr_m x xr_n tiles (its W rows stay in its L2)
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int m_blk = (xcd / p.xg_n) * p.xr_m + local / p.xr_n;
  const int n_blk = (xcd % p.xg_n) * p.xr_n + local % p.xr_n;
  if (local / p.xr_n >= p.xr_m || m_blk >= p.m_tiles || n_blk >= p.n_tiles) return;  // padding of the grid
  const int m0 = m_blk * WBM, n0 = n_blk * WBN;
  const int N = p.N, K = p.K;
  const int KT1 = K / 64;
  // only the first r_used rank columns of T / B_cat can be non-zero: stages beyond them are not visited, and of a
  // last stage that they fill at most half only the first two MFMA steps run
  const int r_used = (p.r_used > 0 && p.r_used < p.R) ? p.r_used : p.R;
  const int KT = KT1 + (p.t_ext != nullptr ? (r_used + 63) / 64 : 0);
  const bool half_last = p.t_ext != nullptr && (r_used & 63) != 0 && (r_used & 63) <= 32;

  // DMA: wave w brings x rows 32w .. 32w+31 (4 instructions of 8 rows) and W rows 40w .. 40w+39 (5) of every stage.
  // Lane -> row lane/8 of its 8 rows, physical piece lane%8, which holds logical piece (lane%8) ^ ((stage row / 2) % 8).
  // (stage row / 2) % 8 of instruction q is that of instruction 0 plus 4q mod 8: the piece flips bit 2 for odd q,
  // so two element offsets (even / odd q) per operand describe all of a lane's sources; M and N are multiples of
  // the tile (no clamping).
  // The loads are buffer loads: per lane two byte offsets per operand that never change (row of instruction 0 with the
  // piece of the even / of the odd instructions), everything that moves (K tile, row group of instruction q) is a scalar
  // offset; fragment reads add the stage as a constant (the two stages are written out).  The loop carries next to no
  // vector address arithmetic: with per-lane 64-bit pointers those adds shared the issue stream with the MFMAs.
  const int r8 = lane >> 3;
  const int rx0 = wave * (WBM / 8) + r8, rx1 = rx0 + 8;               // stage rows of x instructions 0 / 1
  const int pcx0 = ((lane & 7) ^ ((rx0 >> 1) & 7)) * 16, pcx1 = ((lane & 7) ^ ((rx1 >> 1) & 7)) * 16;
  const int rw0 = WBM + wave * (WBN / 8) + r8, rw1 = rw0 + 8;          // stage rows of W instructions 0 / 1
  const int pcw0 = ((lane & 7) ^ ((rw0 >> 1) & 7)) * 16, pcw1 = ((lane & 7) ^ ((rw1 >> 1) & 7)) * 16;
  const int wrow = wave * (WBN / 8) + r8;                              // W row of instruction 0 inside the tile
  const int ldt = p.ldt, R = p.R;
  const uint32_t vx0 = (uint32_t)rx0 * (uint32_t)K * 2u + pcx0, vx1 = (uint32_t)rx0 * (uint32_t)K * 2u + pcx1;
  const uint32_t vw0 = (uint32_t)wrow * (uint32_t)K * 2u + pcw0, vw1 = (uint32_t)wrow * (uint32_t)K * 2u + pcw1;
  auto clamp32 = [](size_t bytes) { return (int)(uint32_t)(bytes < 0xFFFFFFFFull ? bytes : 0xFFFFFFFFull); };
  auto mk = [&](const bf16_t* base, size_t bytes) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(base), 0, clamp32(bytes), 0x00020000); };
  const bool ext = p.t_ext != nullptr;
  const size_t tcol = ext && p.t_nsplit > 0 ? (size_t)(n0 / p.t_nsplit) * p.R : 0;
  const rsrc_t rs_x = mk(p.x + (size_t)m0 * K, (size_t)(p.M - m0) * K * 2);
  const rsrc_t rs_w = mk(p.w + (size_t)n0 * K, (size_t)(N - n0) * K * 2);
  const rsrc_t rs_t = mk(ext ? p.t_ext + (size_t)m0 * ldt + tcol : p.x, ext ? ((size_t)(p.M - m0) * ldt - tcol) * 2 : 0);
  const rsrc_t rs_b = mk(ext ? p.b_cat + (size_t)n0 * R : p.w, ext ? (size_t)(N - n0) * R * 2 : 0);
  auto issue = [&](int t, auto stc) {                           // K tile t into stage stc
    char* stage = smem + decltype(stc)::value * WSTAGE;
    if (t < KT1) {
      const int so = t * 128, rstep = 8 * K * 2;                // bytes: K tile, 8 rows further
#pragma unroll
      for (int q = 0; q < WXU; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lptr_t)(stage + (wave * (WBM / 8) + q * 8) * 128), 16, (q & 1) ? vx1 : vx0, so + q * rstep, 0, 0);
#pragma unroll
      for (int q = 0; q < WWU; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lptr_t)(stage + (WBM + wave * (WBN / 8) + q * 8) * 128), 16, (q & 1) ? vw1 : vw0, so + q * rstep, 0, 0);
    } else {
      // the rank columns: y = [x | T] . [W | B_cat]^T (one or two stages per tile: their offsets are formed here)
      const int so = (t - KT1) * 128;
      const uint32_t tx0 = (uint32_t)rx0 * (uint32_t)ldt * 2u + pcx0, tx1 = (uint32_t)rx0 * (uint32_t)ldt * 2u + pcx1;
      const uint32_t tw0 = (uint32_t)wrow * (uint32_t)R * 2u + pcw0, tw1 = (uint32_t)wrow * (uint32_t)R * 2u + pcw1;
#pragma unroll
      for (int q = 0; q < WXU; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_t, (lptr_t)(stage + (wave * (WBM / 8) + q * 8) * 128), 16, (q & 1) ? tx1 : tx0, so + q * 8 * ldt * 2, 0, 0);
#pragma unroll
      for (int q = 0; q < WWU; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lptr_t)(stage + (WBM + wave * (WBN / 8) + q * 8) * 128), 16, (q & 1) ? tw1 : tw0, so + q * 8 * R * 2, 0, 0);
    }
  };
  const int sw = (l32 >> 1) & 7;
  const int abase = (wm * WR + l32) * 128, bbase = (WBM + wn * WC + l32) * 128;
  int po4[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) po4[ks] = ((2 * ks + lh) ^ sw) * 16;
  auto read_frags = [&](auto stc, int ks, WFr& f) {             // MFMA step ks (16 columns) of stage stc
    const char* s = smem + decltype(stc)::value * WSTAGE;
    const char* pa = s + (abase + po4[ks]);
    const char* pb = s + (bbase + po4[ks]);
#pragma unroll
    for (int i = 0; i < WTM; ++i) f.a[i] = *reinterpret_cast<const bf16x8*>(pa + i * 32 * 128);
#pragma unroll
    for (int j = 0; j < WTN; ++j) f.b[j] = *reinterpret_cast<const bf16x8*>(pb + j * 32 * 128);
  };
  f32x16 acc[WTM][WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  auto mma = [&](const WFr& f) {
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int j = 0; j < WTN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.b[j], f.a[i], acc[i][j], 0, 0, 0);   // D = W . x^T: lane = row of x
  };

  // folded LayerNorm: the rows' statistics and the columns' terms are requested before the first stage (older than its
  // loads: they have arrived when it has) and put into LDS after the table below is built
  KhLnTileStats<WBM, 512> ln_stats;
  float ln_c1v = 0.f, ln_c2v = 0.f;
  if (p.ln_part != nullptr) {
    ln_stats.load(p.ln_part, m0, p.M, tid);
    if (tid < WBN) { ln_c1v = p.ln_c1[n0 + tid]; ln_c2v = p.ln_c2[n0 + tid]; }
  }
  // K loop over stages t (stage t & 1).  Steps 0..3 of a stage alternate between the fragment buffers fa / fb.
  WFr fa, fb;
  using S0 = std::integral_constant<int, 0>; using S1 = std::integral_constant<int, 1>;
  issue(0, S0{});
  if (KT > 1) issue(1, S1{});
  uint16_t* gtab = reinterpret_cast<uint16_t*>(smem + WTAB_OFF);
  uint16_t* sbias = reinterpret_cast<uint16_t*>(smem + WBIAS_OFF);   // like the table: written now, read in the epilogue
  if (tid < WBN) sbias[tid] = p.bias != nullptr ? reinterpret_cast<const uint16_t*>(p.bias)[n0 + tid] : (uint16_t)0;
  float* sMu = reinterpret_cast<float*>(smem + C::LDS);   // folded LayerNorm (launched with LN_LDS more bytes)
  float* sRs = sMu + WBM;
  float* sc1 = sRs + WBM;
  float* sc2 = sc1 + WBN;
  if (p.geglu) {   // published by the barriers of the K loop, read in the epilogue
#pragma unroll
    for (int k = 0; k < 2 * WTAB_N / 512; ++k) {
      const int i = tid + k * 512;
      const uint32_t bits = (uint32_t)(i >= WTAB_N ? 0x8000 + (i - WTAB_N) : i) + WTAB_LO;
      gtab[i] = (uint16_t)pack_bf16x2(kh_gelu_erf(bf16_lo(bits)), 0.f);
    }
  }
  if (p.ln_part != nullptr) {
    ln_stats.finish(K, p.ln_eps, tid, sMu, sRs, false);
    if (tid < WBN) { sc1[tid] = ln_c1v; sc2[tid] = ln_c2v; }
  }
  if (KT > 1) wait_cnt<WLPS, 15>(); else wait_cnt<0, 15>();
  __builtin_amdgcn_s_barrier();
  read_frags(S0{}, 0, fa);
  read_frags(S0{}, 1, fb);
  auto stage_body = [&](int t, auto stc, auto nxc) {   // every stage but the last: stage stc, the next one nxc
    mma(fa);                         // step 0
    read_frags(stc, 2, fa);
    mma(fb);                         // step 1
    read_frags(stc, 3, fb);
    mma(fa);                         // step 2
    // stage t+1 has landed (this wave's share; the barrier collects everyone's); every read of stage t is done
    wait_cnt<0, 0>();
    __builtin_amdgcn_s_barrier();
    if (t + 2 < KT) issue(t + 2, stc);
    read_frags(nxc, 0, fa);
    mma(fb);                         // step 3
    read_frags(nxc, 1, fb);
  };
  auto read_frags_rt = [&](int st, int ks, WFr& f) {    // the same with the stage as a value
    const char* pa = smem + (st * WSTAGE + abase + po4[ks]);
    const char* pb = smem + (st * WSTAGE + bbase + po4[ks]);
#pragma unroll
    for (int i = 0; i < WTM; ++i) f.a[i] = *reinterpret_cast<const bf16x8*>(pa + i * 32 * 128);
#pragma unroll
    for (int j = 0; j < WTN; ++j) f.b[j] = *reinterpret_cast<const bf16x8*>(pb + j * 32 * 128);
  };
  int t = 0;
  for (; t + 2 < KT; t += 2) {
    stage_body(t, S0{}, S1{});
    stage_body(t + 1, S1{}, S0{});
  }
  if (t + 1 < KT) stage_body(t, S0{}, S1{});
  {                                  // the last stage: all four steps, or two when its upper half is zero padding
    const int st = (KT - 1) & 1;
    mma(fa);
    if (!half_last) read_frags_rt(st, 2, fa);
    mma(fb);
    if (!half_last) {
      read_frags_rt(st, 3, fb);
      mma(fa);
      mma(fb);
    }
  }
  __syncthreads();   // the ring is dead: the staging tile reuses it

  // Epilogue: bias in fp32, round to bf16, transpose through LDS so that every global store is a 16-byte piece of
  // a contiguous output row; two passes of 128 rows (the waves' upper / lower 32-row MFMA tiles).
  bf16_t* sC = reinterpret_cast<bf16_t*>(smem);
  const int out_ld = p.geglu ? (N >> 1) : N;
  const KhOut yout(p.y, (size_t)p.M * out_ld * 2);
  constexpr int CPR = WBN / 8, ECH = 128 * CPR / 512;        // plain: pieces per staged row, per thread
  constexpr int OPR = WBN / 16, GCH = 128 * OPR / 512;       // GEGLU: output pieces per staged row, per thread
#pragma unroll
  for (int i = 0; i < WTM; ++i) {
    // the MFMA operands are swapped (W rows first), so a lane holds one output row (l32) and, per group of four
    // accumulator registers, four consecutive columns: 8-byte LDS writes.  With 196-dword rows the 16 rows x 2 halves
    // of one write phase cover all 64 banks.
    if (p.ln_part != nullptr) {
      // y = rstd_row * (acc - mean_row * c1_col) + c2_col; this lane's row is one
      const float mu = sMu[wm * WR + i * 32 + l32], rs = sRs[wm * WR + i * 32 + l32];
#pragma unroll
      for (int j = 0; j < WTN; ++j) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int col = wn * WC + j * 32 + 8 * g4 + 4 * lh;
          const f32x4 c1 = *reinterpret_cast<const f32x4*>(sc1 + col), c2 = *reinterpret_cast<const f32x4*>(sc2 + col);
          u32x2 o;
          o[0] = pack_bf16x2(rs * (acc[i][j][4 * g4] - mu * c1[0]) + c2[0], rs * (acc[i][j][4 * g4 + 1] - mu * c1[1]) + c2[1]);
          o[1] = pack_bf16x2(rs * (acc[i][j][4 * g4 + 2] - mu * c1[2]) + c2[2], rs * (acc[i][j][4 * g4 + 3] - mu * c1[3]) + c2[3]);
          *reinterpret_cast<u32x2*>(sC + (wm * 32 + l32) * WLDC + col) = o;
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < WTN; ++j) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int col = wn * WC + j * 32 + 8 * g4 + 4 * lh;
          const u32x2 bb = *reinterpret_cast<const u32x2*>(sbias + col);
          u32x2 o;
          o[0] = pack_bf16x2(acc[i][j][4 * g4] + bf16_lo(bb[0]), acc[i][j][4 * g4 + 1] + bf16_hi(bb[0]));
          o[1] = pack_bf16x2(acc[i][j][4 * g4 + 2] + bf16_lo(bb[1]), acc[i][j][4 * g4 + 3] + bf16_hi(bb[1]));
          *reinterpret_cast<u32x2*>(sC + (wm * 32 + l32) * WLDC + col) = o;
        }
      }
    }
    __syncthreads();
    if (!p.geglu) {
#pragma unroll
      for (int q = 0; q < ECH; ++q) {
        const int c = tid + q * 512, srow = c / CPR, ch = c % CPR;
        const size_t g = (size_t)(m0 + (srow >> 5) * WR + i * 32 + (srow & 31)) * N + n0 + ch * 8;
        u32x4 o = *reinterpret_cast<const u32x4*>(sC + srow * WLDC + ch * 8);
        if (p.res != nullptr) {
          const u32x4 rr = *reinterpret_cast<const u32x4*>(p.res + g);
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[e]), bf16_hi(o[e]) + bf16_hi(rr[e]));
        }
        yout.store16(g * 2, o);
      }
    } else {
      // staged columns come in groups of 64 = 32 value columns then their 32 gate columns
#pragma unroll
      for (int q = 0; q < GCH; ++q) {
        const int c = tid + q * 512, srow = c / OPR, oc = c % OPR;
        const int grp = oc >> 2, sub = oc & 3;
        const size_t g = (size_t)(m0 + (srow >> 5) * WR + i * 32 + (srow & 31)) * out_ld + (n0 >> 1) + grp * 32 + sub * 8;
        const u32x4 hv = *reinterpret_cast<const u32x4*>(sC + srow * WLDC + grp * 64 + sub * 8);
        const u32x4 gv = *reinterpret_cast<const u32x4*>(sC + srow * WLDC + grp * 64 + 32 + sub * 8);
        u32x4 ar;                                       // gelu(gate) rounded to bf16 before the product
        bool outside = false;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t lo = gv[e] & 0xffffu, hi = gv[e] >> 16;
          const uint32_t olo = (lo & 0x7fffu) - WTAB_LO, ohi = (hi & 0x7fffu) - WTAB_LO;
          outside = outside || olo >= (uint32_t)WTAB_N || ohi >= (uint32_t)WTAB_N;
          const uint32_t ilo = (olo < (uint32_t)WTAB_N ? olo : 0u) + (lo >> 15) * WTAB_N;
          const uint32_t ihi = (ohi < (uint32_t)WTAB_N ? ohi : 0u) + (hi >> 15) * WTAB_N;
          ar[e] = (uint32_t)gtab[ilo] | ((uint32_t)gtab[ihi] << 16);
        }
        if (outside) {                                  // tiny, huge or non-finite gates: evaluate directly
#pragma unroll
          for (int e = 0; e < 4; ++e) ar[e] = pack_bf16x2(kh_gelu_erf(bf16_lo(gv[e])), kh_gelu_erf(bf16_hi(gv[e])));
        }
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(bf16_lo(hv[e]) * bf16_lo(ar[e]), bf16_hi(hv[e]) * bf16_hi(ar[e]));
        yout.store16(g * 2, o);
      }
    }
    __syncthreads();
  }
#endif
}

template <class C>
bool wide_ok(const LoraGemmParams& p) {
  const bool plain = p.R == 0 || p.t_ext != nullptr;
  return plain && p.grp == nullptr && p.sg_mode == 0 && p.conv_cin == 0 && p.st_part == nullptr && p.M % C::BM == 0 && p.N % C::BN == 0 &&
         p.K % 64 == 0 && p.K >= 64 && (p.t_ext == nullptr || (p.R % 64 == 0 && p.ldt % 8 == 0)) &&
         (p.t_nsplit == 0 || p.t_nsplit % C::BN == 0) && (long)C::BM * (p.K > p.ldt ? p.K : p.ldt) < (1L << 31) &&
         (long)C::BN * p.K < (1L << 31);
}

template <class C>
int wide_launch(LoraGemmParams p, hipStream_t stream) {
  if (!wide_ok<C>(p)) return KH_ERR_UNSUPPORTED;
  p.m_tiles = p.M / C::BM;
  p.n_tiles = p.N / C::BN;
  if (hipError_t e = kh_allow_lds<lora_gemm_wide_kernel<C>>(C::LDS + C::LN_LDS); e != hipSuccess) return (int)e;
  const size_t lds = (size_t)C::LDS + (p.ln_part != nullptr ? C::LN_LDS : 0);
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
  kh_launch(KH_TAG_LORA_GEMM, lora_gemm_wide_kernel<C>, dim3(grid), dim3(512), lds, stream, p);
  KH_RETURN_LAST_ERROR();
}

}  // namespace

bool lora_gemm_wide_ok(const LoraGemmParams& p) { return wide_ok<WCfg<2, 5>>(p); }
int lora_gemm_wide_launch(LoraGemmParams p, hipStream_t stream) { return wide_launch<WCfg<2, 5>>(p, stream); }

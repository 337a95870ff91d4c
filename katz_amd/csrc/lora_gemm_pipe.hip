// K1, software-pipelined variant: fused base GEMM + LoRA delta on bf16 MFMA (gfx950), K % 32 == 0.
//
// Same arithmetic as lora_gemm.hip (see there for the formula and the reference citations); what
// differs is how operands reach the MFMAs:
//   * x / W / A_cat tiles go global -> LDS directly (global_load_lds_dwordx4, no VGPR staging) into
//     a ring of NST stages of 32 K-columns each; loads run NST-1 tiles ahead of the MFMAs, each
//     wave waits only for its own oldest loads (s_waitcnt vmcnt(n)) and one barrier per K tile
//     publishes them;
//   * LDS rows are 64 bytes, unpadded; the four 16-byte pieces of a row are XOR-swizzled with
//     (row/4)%4 so that the 16 rows one ds_read_b128 phase touches fall into 16 distinct bank
//     groups (the DMA writes lane i to slot i, so the swizzle is applied to the global address a
//     lane fetches, not to where it lands).
#include "kh_common.h"
#include "lora_gemm.h"
#include "lora_shrink_tile.h"
#include <type_traits>

// How many bounded waits of the in-launch shrink (kh_lora_linear_split_bf16) have ever run out on this GPU.  Unlike the
// flag word at the end of a call's counters it is never cleared by the caller's counter resets; read and cleared by
// kh_lora_split_timeouts.
static __device__ int kh_split_timeout_count;

namespace {

// K columns per stage (BKP) are a template parameter: 32 (64-byte LDS rows) or 64 (128-byte rows).

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int NRT_, int NST_, int BKP_ = 32>
struct PCfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NRT = NRT_, NST = NST_;
  static constexpr int BKP = BKP_;              // K columns per stage
  static constexpr int ROWB = BKP * 2;          // bytes per LDS row
  static constexpr int PPR = BKP / 8;           // 16-byte pieces per row
  static constexpr int UROWS = 64 / PPR;        // rows one DMA instruction (64 lanes x 16 B) covers
  static constexpr int SWR = 256 / ROWB;        // rows per 256 bytes: piece p of row r is stored at p ^ ((r / SWR) % PPR)
  static constexpr int KS = BKP / 16;           // MFMA k-steps per stage
  static_assert(BKP == 32 || BKP == 64, "stage depth");
  static constexpr int NW = WAVES_M * WAVES_N, NT = NW * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int R = NRT * 32;
  static constexpr int SM = (NRT > 0) ? TM / WAVES_N : 0;
  static constexpr int RS = R;                                         // A_cat rows staged per K tile
  static constexpr int UX = BM / UROWS, UW = BN / UROWS, UA = RS / UROWS;  // DMA units per stage
  static constexpr int MU = (UX + UW + UA + NW - 1) / NW;              // most units one wave issues per stage
  static constexpr int SW_OFF = BM * ROWB, SA_OFF = (BM + BN) * ROWB;
  static constexpr int STAGE = (BM + BN + RS) * ROWB;
  static constexpr int LDT = R + 8, LDC = BN + 8;
  static constexpr size_t RING = (size_t)NST * STAGE;
  static constexpr size_t SB = (size_t)BN * LDT * 2;
  static constexpr size_t SC = (size_t)WAVES_M * 32 * LDC * 2;
  static constexpr size_t RING_MAX = RING > SB ? (RING > SC ? RING : SC) : (SB > SC ? SB : SC);
  static constexpr size_t ST = (NRT > 0) ? (size_t)BM * LDT * 2 : 0;
  static constexpr size_t ST_OFF = RING_MAX;
  static constexpr size_t LDS_BYTES = RING_MAX + ST;
  static constexpr int OCC = (LDS_BYTES <= 80 * 1024 && TM * TN <= 4) ? 2 : 1;  // workgroups per CU that LDS and registers allow
  static_assert(BM % (32 * WAVES_M) == 0 && BN % (32 * WAVES_N) == 0, "tile/wave mismatch");
  static_assert(NRT == 0 || (TM % WAVES_N == 0), "shrink tiles must split evenly over the waves of a row");
  static_assert(NST >= 2 && NST <= 4, "ring depth");
  static_assert(UX % NW == 0 && UW % NW == 0 && (RS / 8) % NW == 0 && (NRT == 0 || BKP == 32), "DMA work must split evenly over the waves");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// s_waitcnt with vmcnt = VM and lgkmcnt = LGKM (15 = unconstrained), expcnt unconstrained
// (gfx9 encoding: vmcnt = [15:14|3:0], expcnt = [6:4], lgkmcnt = [11:8]).
template <int VM, int LGKM>
__device__ __forceinline__ void wait_cnt() {
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | ((LGKM & 15) << 8) | ((VM >> 4) << 14));
}

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

__device__ __forceinline__ u32x4 ld16(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ bf16x8 lds_frag(const char* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 lds_fragb(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

// Fragments of one K tile (BKP columns = KS 16-wide MFMA steps) held in registers.
template <class C, bool SHRINK>
struct Frags {
  bf16x8 a[C::KS][C::TM];
  bf16x8 b[C::KS][C::TN];
  bf16x8 r[C::KS][SHRINK ? C::NRT : 1];
};

// DMA work of one wave for one K tile: the same number of global_load_lds instructions for every
// wave (so the vmcnt that isolates "my loads of tile t" is a compile-time constant): XI x-units and
// WI W-units of 16 rows, and R/NW rows of A_cat as AI instructions (the last one half-masked when
// R/NW is 8 mod 16).
template <class C, bool SHRINK>
struct Dma {
  static constexpr int XI = C::UX / C::NW, WI = C::UW / C::NW;
  static constexpr int RA = SHRINK ? C::R / C::NW : 0;       // A_cat rows per wave
  static constexpr int AI = (RA + 15) / 16;
  static constexpr int LPS = XI + WI + AI;                    // loads per stage per wave
  static constexpr int N = LPS > 0 ? LPS : 1;
  // per instruction: element offset of the lane's source row in its matrix (row * K + swizzled piece),
  // the same for the K-extension operand (row * ld2 + piece; T for the x rows, B_cat for the W rows),
  // which matrix it is, and the LDS byte offset inside a stage
  long off[N];
  int off2[N];
  int dst[N];
};

// The K loop.  Three things overlap: DMA loads run NST-1 tiles ahead (global -> LDS ring); the LDS ->
// register fragment reads of tile kt+1 are issued right after the barrier that publishes it; the
// MFMAs of tile kt execute from the other register buffer -- half of them before that barrier, so the
// matrix pipe has work queued while the wave waits for its neighbours, half after it, under the reads.
// SHRINK also accumulates T = x . A_cat^T for the shrink m-tiles of this wave (m-tile wn*SM + s of
// its wave row, selected branch-free from the x fragments it holds).
// 16 bytes of zeros (and more): what a 3x3 convolution's DMA reads for taps that fall into the padding
__device__ __attribute__((aligned(256))) const uint32_t kh_zero_page[64] = {0};

struct ConvGeom { int w, cin; };  // input width and channels (elements)

template <class C, bool SHRINK, int NX, bool CONV, class TailLoads, bool IL = false>
__device__ __forceinline__ void k_loop(char* smem, const Dma<C, SHRINK>& dma, const bf16_t* px, const bf16_t* pw,
                                       const bf16_t* pa, const bf16_t* px2, const bf16_t* pw2, int KT, int KT1,
                                       int lane, int wm, int wn,
                                       int l32, int lh, int sw, f32x16 (&acc)[C::TM][C::TN],
                                       f32x16 (&tacc)[C::SM > 0 ? C::SM : 1][C::NRT > 0 ? C::NRT : 1],
                                       TailLoads tail_loads, ConvGeom cg, bool nodma = false, bool fixk = false,
                                       const int* il_cnt = nullptr, int il_target = 0, int* il_err = nullptr,
                                       bool half_last = false) {   // the upper half of the last K tile is all zeros
  constexpr int TM = C::TM, TN = C::TN, NRT = C::NRT, NST = C::NST;
  constexpr int BKP = C::BKP, ROWB = C::ROWB, KS = C::KS;
  constexpr int PD = NST - 1;  // prefetch distance in K tiles
  using D = Dma<C, SHRINK>;
  // convolution: K tiles are requested in order, so the tap (kh, kw) and channel offset of the next
  // request are running scalars; x rows of tap (kh, kw) sit (kh*W + kw)*Cin elements after the row's
  // base (the pixel above-left), rows whose tap falls outside the image read zeros instead
  int cv_tap = 0, cv_kw = 0, cv_c0 = 0, cv_shift = 0, cv_row = 0;
  auto issue = [&](int t) {
    if (nodma) return;  // tuning only
    char* stage = smem + (t % NST) * C::STAGE;
    if constexpr (CONV) {
#pragma unroll
      for (int q = 0; q < D::XI; ++q) {
        const bool valid = (dma.off2[q] >> cv_tap) & 1;
        const bf16_t* g = valid ? px + dma.off[q] + (cv_shift + cv_c0) : reinterpret_cast<const bf16_t*>(kh_zero_page);
        __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)(stage + dma.dst[q]), 16, 0, 0);
      }
#pragma unroll
      for (int q = D::XI; q < D::LPS; ++q)
        __builtin_amdgcn_global_load_lds((gptr_t)(pw + dma.off[q] + t * BKP), (lptr_t)(stage + dma.dst[q]), 16, 0, 0);
      cv_c0 += BKP;
      if (cv_c0 == cg.cin) {
        cv_c0 = 0; ++cv_tap; ++cv_kw; cv_shift += cg.cin;
        if (cv_kw == 3) { cv_kw = 0; cv_row += cg.w * cg.cin; cv_shift = cv_row; }
      }
      return;
    }
    if (IL && t == KT1) {
      // first request for T: wait (bounded) until the shrink workgroups of this row block have all arrived
      if (lane == 0) {
        int it = 0;
        while (__hip_atomic_load(il_cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < il_target && ++it < (1 << 20))
          __builtin_amdgcn_s_sleep(8);
        if (it >= (1 << 20)) {
          __hip_atomic_store(il_err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_fetch_add(&kh_split_timeout_count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < D::LPS; ++q) {
      const bool partial = SHRINK && (q == D::LPS - 1) && (D::RA % 16 != 0);
      // K tiles >= KT1 come from the extension operands: y = [x | T] . [W | B_cat]^T
      const bf16_t* base = q < D::XI ? px : (q < D::XI + D::WI ? pw : pa);
      const bf16_t* base2 = q < D::XI ? px2 : pw2;
      const bf16_t* g = (SHRINK || t < KT1) ? base + dma.off[q] + (fixk ? 0 : t * BKP) : base2 + dma.off2[q] + (t - KT1) * BKP;
      if (IL && t >= KT1 && q < D::XI) {
        // T was written inside this launch, maybe on another XCD: read past the (non-coherent) L2
        __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)(stage + dma.dst[q]), 16, 0, 17 /* sc0 sc1 */);
      } else if (!partial || lane < 32) {
        __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)(stage + dma.dst[q]), 16, 0, 0);
      }
    }
  };
  auto read_frags = [&](int t, Frags<C, SHRINK>& f) {
    const char* st = smem + (t % NST) * C::STAGE;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int po = ((2 * ks + lh) ^ sw) * 16;
#pragma unroll
      for (int i = 0; i < TM; ++i) f.a[ks][i] = lds_frag(st + (wm * C::WTM + i * 32 + l32) * ROWB + po);
#pragma unroll
      for (int j = 0; j < TN; ++j) f.b[ks][j] = lds_frag(st + C::SW_OFF + (wn * C::WTN + j * 32 + l32) * ROWB + po);
      if constexpr (SHRINK) {
#pragma unroll
        for (int r = 0; r < NRT; ++r) f.r[ks][r] = lds_frag(st + C::SA_OFF + (r * 32 + l32) * ROWB + po);
      }
    }
  };
  auto mma1 = [&](const Frags<C, SHRINK>& f, int ks) {
    if constexpr (SHRINK) {
#pragma unroll
      for (int s = 0; s < C::SM; ++s) {
        bf16x8 as = f.a[ks][s];  // wn == 0
#pragma unroll
        for (int q = 1; q < C::WAVES_N; ++q) as = (wn == q) ? f.a[ks][q * C::SM + s] : as;
#pragma unroll
        for (int r = 0; r < NRT; ++r)
          tacc[s][r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as, f.r[ks][r], tacc[s][r], 0, 0, 0);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ks][i], f.b[ks][j], acc[i][j], 0, 0, 0);
  };
  auto mma = [&](const Frags<C, SHRINK>& f, int half) {  // half 0 / 1 of the tile's k-steps
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks) mma1(f, half * (KS / 2) + ks);
  };
  // Publish tile t and fetch its fragments.  Bare s_barrier (no workgroup fence: a fence is
  // s_waitcnt vmcnt(0) and would drain the prefetches).  Before it: this wave's DMA loads of tile t
  // are complete (VM = number of younger loads that may stay outstanding) and so are its LDS reads
  // of tile t-1 (lgkmcnt 0), whose stage the DMA issued after the barrier refills.
  // Steady state: tile kt is in `cur`; tile kt+1 becomes visible, tile kt+1+PD is requested.
  auto step_steady = [&](int kt, const Frags<C, SHRINK>& cur, Frags<C, SHRINK>& nxt) {
    mma(cur, 0);
    wait_cnt<D::LPS*(PD - 1), 0>();
    __builtin_amdgcn_s_barrier();
    issue(kt + 1 + PD);
    read_frags(kt + 1, nxt);
    mma(cur, 1);
  };

  wait_cnt<0, 15>();  // stores of the previous tile's epilogue are out of the way of the counting below
  Frags<C, SHRINK> f0, f1;
  if (KT > PD) {
#pragma unroll
    for (int t = 0; t < PD; ++t) issue(t);
    wait_cnt<D::LPS*(PD - 1), 15>();
    __builtin_amdgcn_s_barrier();
    issue(PD);
    read_frags(0, f0);
    int kt = 0;
    for (; kt + 2 + PD < KT; kt += 2) {
      step_steady(kt, f0, f1);
      step_steady(kt + 1, f1, f0);
    }
    if (kt + 1 + PD < KT) {  // odd number of steady steps: one more, then rename f1 -> f0
      step_steady(kt, f0, f1);
      f0 = f1;
      ++kt;
    }
    // Tail: kt == KT-PD-1, tile kt in f0, tiles kt+1 .. KT-1 in flight, nothing left to request.
    // `tail_loads` may start NX extra global loads per wave (operands of the expand phase): they are
    // younger than every DMA load, so the waits below leave them outstanding.
    tail_loads();
#pragma unroll
    for (int j = 0; j < PD; ++j) {
      Frags<C, SHRINK>& cur = (j & 1) ? f1 : f0;
      Frags<C, SHRINK>& nxt = (j & 1) ? f0 : f1;
      mma(cur, 0);
      switch (j) {  // compile-time after unrolling: PD-1-j DMA tiles younger than tile kt+1+j
        case 0: wait_cnt<D::LPS*(PD - 1) + NX, 0>(); break;
        case 1: wait_cnt<D::LPS*(PD > 2 ? PD - 2 : 0) + NX, 0>(); break;
        case 2: wait_cnt<D::LPS*(PD > 3 ? PD - 3 : 0) + NX, 0>(); break;
        default: wait_cnt<NX, 0>(); break;
      }
      __builtin_amdgcn_s_barrier();
      read_frags(kt + 1 + j, nxt);
      mma(cur, 1);
    }
    const Frags<C, SHRINK>& last = (PD & 1) ? f1 : f0;
    mma(last, 0);
    if (!half_last) mma(last, 1);
  } else {
    // fewer K tiles than ring stages (tiny K): request everything, wait for everything
    for (int t = 0; t < KT; ++t) issue(t);
    tail_loads();
    wait_cnt<NX, 15>();
    __builtin_amdgcn_s_barrier();
    for (int t = 0; t < KT; ++t) {
      read_frags(t, f0);
      mma(f0, 0);
      if (!(half_last && t == KT - 1)) mma(f0, 1);
    }
  }
}

// The K loop of every instantiation that does not accumulate the shrink itself.  What differs from k_loop above is
// how addresses are formed.  Loads are buffer loads: a byte offset per lane that never changes (row and swizzled piece
// inside the tile) plus a scalar byte offset per K tile; fragment reads use per-lane offsets that never change plus the
// stage as an instruction offset, because the ring's stages are written out as constants (lcm(NST, 2) steps per group:
// ring position x register buffer).  The loop then carries no vector address arithmetic: with per-lane 64-bit pointers
// the adds and selects of every stage shared the issue stream with the MFMAs, and a stage cost the sum of both.
// An offset at or beyond the buffer's size reads zeros without touching memory: the convolution's taps in the padding.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
template <int I> using IC = std::integral_constant<int, I>;

template <class C>
struct Dma2 {
  static constexpr int XI = C::UX / C::NW, WI = C::UW / C::NW, LPS = XI + WI;
  uint32_t voff[LPS];    // x units first, then W units: byte offset of this lane's 16 bytes at K column 0
  uint32_t voff2[LPS];   // the same in the K-extension operands (T for the x rows, B_cat for the W rows)
  int tapmask[XI];       // CONV: bit t = tap t of this lane's pixel is inside the image
};

struct Rsrc4 { rsrc_t x, w, t, b; };

template <class C, bool CONV, bool IL>
__device__ __forceinline__ void k_loop2(char* smem, const Dma2<C>& dma, const Rsrc4& rs, int KT, int KT1, int lane, int wave,
                                        int wm, int wn, int l32, int lh, int sw, f32x16 (&acc)[C::TM][C::TN], ConvGeom cg,
                                        const int* il_cnt, int il_target, int* il_err, bool half_last) {
#if __HIP_DEVICE_COMPILE__
  constexpr int TM = C::TM, TN = C::TN, NST = C::NST, BKP = C::BKP, ROWB = C::ROWB, KS = C::KS, STAGE = C::STAGE;
  constexpr int PD = NST - 1;                           // prefetch distance in K tiles
  constexpr int U = (NST % 2 == 0) ? NST : 2 * NST;     // steps per written-out group
  static_assert(NST == 3 || NST == 4, "groups of 6 or 4 steps");
  using D = Dma2<C>;
  using F = Frags<C, false>;
  constexpr uint32_t OOB = 0x80000000u;                 // a convolution's image is shorter than 2 GiB
  int cv_tap = 0, cv_kw = 0, cv_c0 = 0, cv_shift = 0, cv_row = 0;
  uint32_t xvo[D::XI];                                  // CONV: the x offsets with the current tap's padding applied
#pragma unroll
  for (int q = 0; q < D::XI; ++q) xvo[q] = (!CONV || (dma.tapmask[q] & 1)) ? dma.voff[q] : OOB;

  auto issue = [&](int t, auto stc) {
    char* stage = smem + decltype(stc)::value * STAGE;
    if (CONV || t < KT1) {
      const int so = t * (BKP * 2);
#pragma unroll
      for (int q = 0; q < D::XI; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs.x, (lptr_t)(stage + (wave * D::XI + q) * 1024), 16, CONV ? xvo[q] : dma.voff[q],
                                                 CONV ? (cv_shift + cv_c0) * 2 : so, 0, 0);
#pragma unroll
      for (int q = 0; q < D::WI; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs.w, (lptr_t)(stage + C::SW_OFF + (wave * D::WI + q) * 1024), 16, dma.voff[D::XI + q], so, 0, 0);
      if (CONV) {
        cv_c0 += BKP;
        if (cv_c0 == cg.cin) {
          cv_c0 = 0; ++cv_tap; ++cv_kw; cv_shift += cg.cin;
          if (cv_kw == 3) { cv_kw = 0; cv_row += cg.w * cg.cin; cv_shift = cv_row; }
#pragma unroll
          for (int q = 0; q < D::XI; ++q) xvo[q] = ((dma.tapmask[q] >> cv_tap) & 1) ? dma.voff[q] : OOB;
        }
      }
    } else {
      // K tiles >= KT1 come from the extension operands: y = [x | T] . [W | B_cat]^T
      if (IL && t == KT1) {
        // first request for T: wait (bounded) until the shrink workgroups of this row block have all arrived
        if (lane == 0) {
          int it = 0;
          while (__hip_atomic_load(il_cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < il_target && ++it < (1 << 20))
            __builtin_amdgcn_s_sleep(8);
          if (it >= (1 << 20)) {
            __hip_atomic_store(il_err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_fetch_add(&kh_split_timeout_count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
      const int so = (t - KT1) * (BKP * 2);
#pragma unroll
      for (int q = 0; q < D::XI; ++q) {
        // (IL) T was written inside this launch, maybe on another XCD: read past the (non-coherent) L2
        if (IL) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs.t, (lptr_t)(stage + (wave * D::XI + q) * 1024), 16, dma.voff2[q], so, 0, 17 /* sc0 sc1 */);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(rs.t, (lptr_t)(stage + (wave * D::XI + q) * 1024), 16, dma.voff2[q], so, 0, 0);
      }
#pragma unroll
      for (int q = 0; q < D::WI; ++q)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs.b, (lptr_t)(stage + C::SW_OFF + (wave * D::WI + q) * 1024), 16, dma.voff2[D::XI + q], so, 0, 0);
    }
  };
  // fragment offsets inside a stage; stages 2 and 3 lie beyond the 64 KB an instruction offset reaches: second set
  int fa[KS], fb[KS], fa2[KS], fb2[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int po = ((2 * ks + lh) ^ sw) * 16;
    fa[ks] = (wm * C::WTM + l32) * ROWB + po;
    fb[ks] = C::SW_OFF + (wn * C::WTN + l32) * ROWB + po;
    fa2[ks] = fa[ks] + 2 * STAGE;
    fb2[ks] = fb[ks] + 2 * STAGE;
  }
  auto read_frags = [&](auto stc, F& f) {
    constexpr int ST = decltype(stc)::value;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const char* pa = ST >= 2 ? smem + fa2[ks] + (ST - 2) * STAGE : smem + fa[ks] + ST * STAGE;
      const char* pb = ST >= 2 ? smem + fb2[ks] + (ST - 2) * STAGE : smem + fb[ks] + ST * STAGE;
#pragma unroll
      for (int i = 0; i < TM; ++i) f.a[ks][i] = lds_frag(pa + i * 32 * ROWB);
#pragma unroll
      for (int j = 0; j < TN; ++j) f.b[ks][j] = lds_frag(pb + j * 32 * ROWB);
    }
  };
  auto mma = [&](const F& f, int half) {  // half 0 / 1 of the tile's k-steps
#pragma unroll
    for (int k2 = 0; k2 < KS / 2; ++k2) {
      const int ks = half * (KS / 2) + k2;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ks][i], f.b[ks][j], acc[i][j], 0, 0, 0);
    }
  };
  // wait until at most n of this wave's younger K tiles are outstanding, and its LDS reads are done
  auto wait_younger = [&](int n) {
    if (n >= PD - 1) wait_cnt<D::LPS * (PD - 1), 0>();
    else if (n == 1) wait_cnt<D::LPS, 0>();
    else wait_cnt<0, 0>();
  };
  // Step t: tile t is in `cur`.  Half its MFMAs, then tile t+1 becomes visible (this wave's loads of it are complete,
  // its LDS reads of tile t are complete, bare s_barrier: a fence would drain the prefetches), the stage of tile t takes
  // tile t+1+PD, the fragments of tile t+1 are read, the other half of the MFMAs runs under those reads.
  auto step = [&](int t, const F& cur, F& nxt, auto st_next, auto st_fill, auto steady) {
    mma(cur, 0);
    if constexpr (decltype(steady)::value) {
      wait_cnt<D::LPS * (PD - 1), 0>();
      __builtin_amdgcn_s_barrier();
      issue(t + 1 + PD, st_fill);
      read_frags(st_next, nxt);
      mma(cur, 1);
    } else {
      if (t + 1 < KT) {
        wait_younger(KT - 2 - t);
        __builtin_amdgcn_s_barrier();
        if (t + 1 + PD < KT) issue(t + 1 + PD, st_fill);
        read_frags(st_next, nxt);
      }
      if (!(half_last && t == KT - 1)) mma(cur, 1);
    }
  };

  wait_cnt<0, 15>();  // stores of an earlier phase are out of the way of the counting below
  F f0, f1;
  issue(0, IC<0>{});
  if (KT > 1) issue(1, IC<1>{});
  if (PD > 2 && KT > 2) issue(2, IC<2>{});
  wait_younger(KT - 1);
  __builtin_amdgcn_s_barrier();
  if (KT > PD) issue(PD, IC<PD>{});
  read_frags(IC<0>{}, f0);
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
#endif
}

// Cross-attention of a staged query tile (see LoraGemmParams::xa_k): sQ holds the 128 x 128 bf16 tile (row stride LDQ), i.e.
// 128 queries of heads h0 = n0 / 64 and h0 + 1; wave w takes head w / 4 and queries 32 (w % 4) .. + 31.  The arithmetic is
// kh_attention_bf16's (attention.hip) in one pass over at most 96 keys: S^T = K . Q^T on the MFMA with one query per lane,
// exp2 of the scaled scores against the row maximum, O^T += V^T . P^T with P straight from the score registers, the row
// sums as one more MFMA against ones.  K and V^T (keys in pairs per 32-bit word) sit in LDS behind the tile.
template <int LDQ>
struct XAttnTile {
  static constexpr int XS = 96, LDH = 64 + 8, LDV = XS + 8, NT = 512;
  static constexpr int Q_BYTES = 128 * LDQ * 2, K_BYTES = 2 * XS * LDH * 2, V_BYTES = 2 * 64 * LDV * 2;
  static constexpr int LDS_BYTES = Q_BYTES + K_BYTES + V_BYTES;
  static constexpr int VCHUNKS = 2 * (XS / 2) * 8;   // (head, key pair, 8-column piece)
  u32x4 rk[3], rv[2][2];

  // K: 2 heads x 96 keys x 8 pieces of 16 bytes; V: 2 heads x 48 key pairs x 8 pieces (transposed on the way into LDS).
  // Requested before the query tile is staged; keys beyond S read as zeros and are masked in the scores.
  __device__ __forceinline__ void load(const LoraGemmParams& p, int m0, int n0, int tid) {
    const int S = p.xa_S, b = m0 / p.xa_T;
    const bf16_t* kp = p.xa_k + (size_t)b * p.xa_bsk + n0;
    const bf16_t* vp = p.xa_v + (size_t)b * p.xa_bsv + n0;
    const u32x4 z4 = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const int c = tid + i * NT, hh = c / (XS * 8), key = (c % (XS * 8)) >> 3, pc = c & 7;
      rk[i] = key < S ? *reinterpret_cast<const u32x4*>(kp + (size_t)key * p.xa_ldk + hh * 64 + pc * 8) : z4;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = tid + j * NT, hh = c / (VCHUNKS / 2), rest = c % (VCHUNKS / 2), v_kp = rest % (XS / 2), v_dch = rest / (XS / 2);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int key = 2 * v_kp + i;
        rv[j][i] = (c < VCHUNKS && key < S) ? *reinterpret_cast<const u32x4*>(vp + (size_t)key * p.xa_ldv + hh * 64 + v_dch * 8) : z4;
      }
    }
  }

  // after every wave has written its part of sQ (no barrier needed before: K / V^T go to their own LDS ranges)
  __device__ __forceinline__ void run(char* smem, const LoraGemmParams& p, int m0, int n0, int tid) {
    bf16_t* sQ = reinterpret_cast<bf16_t*>(smem);
    bf16_t* sK = reinterpret_cast<bf16_t*>(smem + Q_BYTES);
    uint32_t* sVt = reinterpret_cast<uint32_t*>(smem + Q_BYTES + K_BYTES);     // [2][64][LDV / 2] words of two keys
    const int lane = tid & 63, wave = tid >> 6, l32 = lane & 31, lh = lane >> 5;
    const int S = p.xa_S;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const int c = tid + i * NT, hh = c / (XS * 8), key = (c % (XS * 8)) >> 3, pc = c & 7;
      *reinterpret_cast<u32x4*>(sK + (hh * XS + key) * LDH + pc * 8) = rk[i];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = tid + j * NT;
      if (c < VCHUNKS) {
        const int hh = c / (VCHUNKS / 2), rest = c % (VCHUNKS / 2), v_kp = rest % (XS / 2), v_dch = rest / (XS / 2);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t a = rv[j][0][w], c2 = rv[j][1][w];
          sVt[(hh * 64 + v_dch * 8 + 2 * w) * (LDV / 2) + v_kp] = (a & 0xffffu) | (c2 << 16);
          sVt[(hh * 64 + v_dch * 8 + 2 * w + 1) * (LDV / 2) + v_kp] = (a >> 16) | (c2 & 0xffff0000u);
        }
      }
    }
    __syncthreads();   // the query tile, K and V^T are in LDS

    const int hh = wave >> 2, qg = wave & 3;
    bf16x8 qf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(sQ + (qg * 32 + l32) * LDQ + hh * 64 + ks * 16 + lh * 8);
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // S^T tiles: st[kt][v]: key = kt*32 + 8*(v/4) + 4*lh + v%4, query = l32
    f32x16 st[3];
#pragma unroll
    for (int kt = 0; kt < 3; ++kt)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + (hh * XS + kt * 32 + l32) * LDH + ks * 16 + lh * 8);
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], ks == 0 ? zero : st[kt], 0, 0, 0);
      }
    float mx = -1.0e30f;
#pragma unroll
    for (int kt = 0; kt < 3; ++kt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = kt * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (key >= S) st[kt][v] = -1.0e30f;
        mx = fmaxf(mx, st[kt][v]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mb = mx * p.xa_scale_log2e;
    bf16x8 pf[3][2];
#pragma unroll
    for (int kt = 0; kt < 3; ++kt)
#pragma unroll
      for (int v = 0; v < 16; v += 2) {
        pf[kt][v >> 3][v & 7] = (bf16_t)__builtin_amdgcn_exp2f(st[kt][v] * p.xa_scale_log2e - mb);
        pf[kt][v >> 3][(v & 7) + 1] = (bf16_t)__builtin_amdgcn_exp2f(st[kt][v + 1] * p.xa_scale_log2e - mb);
      }
    // O^T += V^T . P^T: A fragment row d = dt*32 + l32, element e <-> key kt*32 + 8*(2s + e/4) + 4*lh + e%4
    const bf16_t one = (bf16_t)1.0f;
    const bf16x8 ones = {one, one, one, one, one, one, one, one};
    f32x16 oacc[2] = {zero, zero}, rsum = zero;
    const bf16_t* sV = reinterpret_cast<const bf16_t*>(sVt);
#pragma unroll
    for (int kt = 0; kt < 3; ++kt)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          const bf16_t* base = sV + (hh * 64 + dt * 32 + l32) * LDV + kt * 32 + 16 * s2 + 4 * lh;
          const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(base);
          const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(base + 8);
          bf16x8 vf;
#pragma unroll
          for (int e = 0; e < 4; ++e) { vf[e] = v0[e]; vf[4 + e] = v1[e]; }
          oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kt][s2], oacc[dt], 0, 0, 0);
        }
        rsum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf[kt][s2], rsum, 0, 0, 0);
      }
    const float inv = 1.0f / rsum[0];
    bf16_t* op = p.xa_o + (size_t)(m0 + qg * 32 + l32) * p.xa_ldo + n0 + hh * 64;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 o2;
        o2[0] = pack_bf16x2(oacc[dt][4 * g + 0] * inv, oacc[dt][4 * g + 1] * inv);
        o2[1] = pack_bf16x2(oacc[dt][4 * g + 2] * inv, oacc[dt][4 * g + 3] * inv);
        *reinterpret_cast<u32x2*>(op + dt * 32 + 8 * g + 4 * lh) = o2;
      }
  }
};

using ILTileWide = SCfg<4, 2, 2>;               // in-launch shrink tiles: 64 x 64 ...
using ILTileNarrow = SCfg<4, 2, 1>;             // ... and 64 x 32 (see il_narrow; a ring of three stages measured no faster)
constexpr int IL_SHRINK_LDS = ILTileWide::LDS > ILTileNarrow::LDS ? ILTileWide::LDS : ILTileNarrow::LDS;
constexpr int IL_PF_OFF = IL_SHRINK_LDS;        // in-launch shrink workgroups: LDS offset of their prefetch landing zone (1 KB)

// Weight prefetch of a launch with its own shrink: by the idle waves of the shrink workgroups when the first range is short
__host__ __device__ inline bool il_prefetch_by_idle_waves(const LoraGemmParams& p) { return p.pf_lines[0] <= ((8u << 20) >> 7); }

// In-launch shrink on 64 x 32 tiles: a single layer (T has R = 128 columns) of which at most the first 96 rank columns are
// in use (two adapters of ranks 64 + 32, say), short enough in K that its GEMM tiles would otherwise wait for T, and
// small enough in M that the three tiles per 64 rows fit beside the GEMM tiles.  The GEMM tiles never multiply the
// columns the shrink leaves unwritten (r_used bounds their K loop).
__host__ __device__ inline bool il_narrow(const LoraGemmParams& p) {
  return p.R == 128 && p.ldt == 128 && p.r_used > 0 && p.r_used <= 96 && p.K <= 2560 &&
         (long)((p.M + 127) / 128) * ((p.N + 127) / 128) + (long)((p.M + 63) / 64) * 3 <= 256;
}
__host__ __device__ inline int il_col_tiles(const LoraGemmParams& p) { return il_narrow(p) ? 3 : p.ldt / 64; }

// LNF bit 0: the instantiation can fold a LayerNorm in front of the layer into its epilogue (ln_part); bit 1: it can write
// the row statistics for one behind it (st_part).  The plain one (0) carries none of that code.
// XA: the output tile is an attention's queries and the epilogue runs the cross-attention on it (XAttnTile).
template <class C, bool CONV = false, bool IL = false, int LNF = 0, bool XA = false>
__global__ __launch_bounds__(C::NT, C::OCC) void lora_gemm_pipe_kernel(const LoraGemmParams pin) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  LoraGemmParams p = pin;
  if constexpr (IL) {
    // The first il_blocks workgroups are the shrink: 64x64 tiles of T on 4 of the 8 waves, stored write-through,
    // then one arrival per tile on the counter of the GEMM row block the tile belongs to.  They have the lowest
    // block ids, so they are resident before any workgroup that waits for them.
    if ((int)blockIdx.x < pin.il_blocks) {
      // T has ldt columns (several layers' ranks side by side, R each).  Tiles are 64 rows x 64 columns, or -- for a single
      // layer of which only the first 96 of the 128 rank columns are in use -- 64 x 32: three tiles per 64 rows instead of
      // two, each with 3/4 of the operand bytes of a 64 x 64 one.  The GEMM workgroups wait for T at the end of their K
      // loop, and a short layer's shrink tile is not done by then: what a tile streams through its 160 KB of LDS sets
      // when T arrives, and 96 tiles still find a CU each beside 160 GEMM tiles
      const bool narrow = il_narrow(pin);
      const int gx = (pin.M + 63) / 64, gy = il_col_tiles(pin);
      if ((int)blockIdx.x >= gx * gy) return;               // padding to a multiple of 8 (the XCD map of the rest)
      const int bx = blockIdx.x % gx, by = blockIdx.x / gx;
      ShrinkParams sp;
      sp.x = pin.x; sp.a_cat = pin.a_cat; sp.col_scale = pin.col_scale; sp.t = const_cast<bf16_t*>(pin.t_ext);
      sp.M = pin.M; sp.K = pin.K; sp.R = pin.ldt;
      if (LNF & 1) { sp.ln_part = pin.ln_part; sp.ln_ca1 = pin.ln_ca1; sp.ln_ca2 = pin.ln_ca2; sp.ln_eps = pin.ln_eps; }
      // The tile is the work of waves 0..3.  Waves 4..7 touch the next launch's weights instead (towards the memory-side
      // cache, see LoraGemmParams::pf), so that no GEMM wave's first operands queue behind that duty, and end: a barrier
      // waits for the surviving waves only.  They start when most of the tile's own loads are out (T's arrival is what the
      // GEMM workgroups of a short layer wait for: nothing may queue in front of it), and wait for their own loads (into
      // 256 bytes each behind the tile's rings) before they end, so that this workgroup's LDS is not handed on with loads
      // still landing in it.
      if (threadIdx.x >= 256) {
        if (!il_prefetch_by_idle_waves(pin)) return;
        __builtin_amdgcn_s_sleep(127);   // 8128 clocks: measured against 1, 40, 160 and 254 (23.87 / 24.0 / 24.06 / 24.1 / 25.4 ms per step)
        kh_prefetch_lines_idle(pin.pf, pin.pf_lines, smem + IL_PF_OFF + (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) - 4) * 256,
                               (int)blockIdx.x, gx * gy, (int)threadIdx.x - 256, 256);
        __builtin_amdgcn_s_waitcnt(0);
        return;
      }
      if (narrow) lora_shrink_tile<ILTileNarrow, true, 256>(sp, bx * 64, by * 32, smem);
      else lora_shrink_tile<ILTileWide, true, 256>(sp, bx * 64, by * 64, smem);
      __builtin_amdgcn_s_waitcnt(0);                          // this thread's write-through stores have completed
      __syncthreads();
      if (threadIdx.x == 0)
        __hip_atomic_fetch_add(pin.il_cnt + (bx * 64) / C::BM, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
  }
  const int bid = IL ? (int)blockIdx.x - pin.il_blocks : (int)blockIdx.x;
  // the next launch's weights, towards the memory-side cache (see LoraGemmParams::pf); in a launch that carries its own
  // shrink the idle waves of the shrink workgroups do that (above) unless the range is long: a CU keeps only so many
  // missing lines in flight, and 29 MB of convolution weights from 64 CUs took 25 us.  (Not from the 256x128 tiles that run
  // beside their shrink: with a folded LayerNorm they have no register to spare, and a kernel with scratch loses more.)
  if ((!IL || (C::BM != 256 && !il_prefetch_by_idle_waves(pin))) && blockIdx.y == 0)
    kh_prefetch_lines(pin.pf, pin.pf_lines, smem + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) * (C::UX / C::NW) * 1024, bid,
                      (int)gridDim.x - (IL ? pin.il_blocks : 0), threadIdx.x, C::NT);
  if (pin.grp != nullptr) {  // grouped launch: this workgroup's layer
    const uint64_t* g = pin.grp + (size_t)blockIdx.y * 5;
    p.w = reinterpret_cast<const bf16_t*>(g[0]);
    p.bias = reinterpret_cast<const bf16_t*>(g[1]);
    p.b_cat = reinterpret_cast<const bf16_t*>(g[2]);
    p.t_ext = reinterpret_cast<const bf16_t*>(g[3]);
    p.y = reinterpret_cast<bf16_t*>(g[4]);
  }
  float oscale = 1.f;   // segmented expand: the adapter's scale on the product
  int k_cols = p.K;     // K columns the loop covers (the row stride stays p.K)
  int n_store = p.N;    // output columns that are written (segmented shrink: the adapter's rank, not the padded maximum)
  if (pin.sg_mode != 0) {
    const int sg = blockIdx.y;
    const int r0 = pin.sg_start[sg], r1 = pin.sg_start[sg + 1], ad = pin.sg_adapter[sg];
    if (ad < 0 || r1 <= r0) return;   // a request without an adapter keeps its base projection untouched
    p.M = r1 - r0;
    p.x = pin.x + (size_t)r0 * pin.K;
    p.w = pin.w + (size_t)ad * pin.sg_wstride;
    p.y = pin.y + (size_t)r0 * pin.N;
    if (pin.sg_mode == 2) {
      p.res = p.y;                    // read-modify-write of y: every element is read and written by one thread
      oscale = pin.sg_scale[ad];
      k_cols = pin.sg_rank[ad];
    } else {
      n_store = pin.sg_rank[ad] < p.N ? pin.sg_rank[ad] : p.N;   // the expand reads t[:, 0:rank] only
    }
  }
  constexpr int BM = C::BM, BN = C::BN, TM = C::TM, TN = C::TN, NRT = C::NRT, R = C::R, NST = C::NST;
  constexpr int SMT = C::SM > 0 ? C::SM : 1, NRTT = NRT > 0 ? NRT : 1;
  bf16_t* sB = reinterpret_cast<bf16_t*>(smem);                // aliases the ring (after the K loop)
  bf16_t* sC = reinterpret_cast<bf16_t*>(smem);                // aliases the ring (after the expand)
  bf16_t* sT = reinterpret_cast<bf16_t*>(smem + C::ST_OFF);    // fused mode: lives across N tiles

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const int l32 = lane & 31, lh = lane >> 5;

  int m_blk, chunk;
  if (p.xg_n > 0) {
    // Workgroups go round-robin to the 8 XCDs, each with a 4 MB L2 of its own.  XCD (xm, xn) of the
    // xg_m x xg_n grid owns the block of xr_m x xr_n tiles at (xm*xr_m, xn*xr_n) and walks it row by row, so
    // the W rows of its xr_n tile columns stay in its L2 while the x rows stream through once.  (With contiguous
    // ranges of a row-major tile list every XCD reads all of W, twice over: 8.6x the algorithmic bytes.)
    const int xcd = bid & 7, local = bid >> 3;
    m_blk = (xcd / p.xg_n) * p.xr_m + local / p.xr_n;
    chunk = (xcd % p.xg_n) * p.xr_n + local % p.xr_n;
    if (local / p.xr_n >= p.xr_m || m_blk >= p.m_tiles || chunk >= p.n_chunks) return;  // padding of the grid
  } else {
    const uint32_t total = (uint32_t)p.m_tiles * (uint32_t)p.n_chunks;
    const uint32_t logical = xcd_remap((uint32_t)bid, total);
    m_blk = logical / p.n_chunks; chunk = logical % p.n_chunks;
  }
  const int m0 = m_blk * BM;
  if (m0 >= p.M) return;   // segmented launches size the grid for the longest segment
  const int K = p.K, M = p.M, N = p.N;
  constexpr int BKP = C::BKP, ROWB = C::ROWB;
  // folded LayerNorm: mean and 1/std of this tile's x rows, read in the epilogue (the barriers of the K loop lie between)
  // and the two per-column terms of this (single) column tile
  float* sMu = reinterpret_cast<float*>(smem + p.ln_lds);
  float* sRs = sMu + 256;
  float* sc1 = sRs + 256;
  float* sc2 = sc1 + 256;
  static_assert(C::BM <= 256 && C::BN <= 256 && C::BN <= C::NT, "LayerNorm terms: room in LDS, one column per thread");
  // requested first, finished once the DMA descriptors and the bias loads below are under way
  KhLnTileStats<C::BM, C::NT> ln_stats;
  float ln_c1v = 0.f, ln_c2v = 0.f;
  if ((LNF & 1) && p.ln_part != nullptr) {
    ln_stats.load(p.ln_part, m0, M, tid);
    if (tid < C::BN) {
      const int col = chunk * p.n_chunk * C::BN + tid;
      ln_c1v = col < N ? p.ln_c1[col] : 0.f;
      ln_c2v = col < N ? p.ln_c2[col] : 0.f;
    }
  }

  const int KT1 = k_cols / BKP;                                        // K tiles of x / W
  // + rank tiles of T / B_cat (two-launch form).  Only the first r_used rank columns can be non-zero: tiles beyond
  // them are not visited, and of a last tile that they fill at most half only that half is multiplied.
  const int r_used = (p.r_used > 0 && p.r_used < p.R) ? p.r_used : p.R;
  const int KT = KT1 + (p.t_ext != nullptr ? (r_used + BKP - 1) / BKP : 0);
  const bool half_last = p.t_ext != nullptr && (r_used % BKP) != 0 && (r_used % BKP) <= BKP / 2;

  // DMA geometry of this lane inside a 16-row unit: LDS slot = lane (16 bytes each); it holds row
  // lane/4, physical piece lane%4, which stores logical piece (lane%4) ^ ((row/4)%4).
  const int u_row = lane / C::PPR;
  // fragment read: logical piece (2*ks + lh) of row (.. + l32) sits at physical piece ^ ((l32/SWR) % PPR)
  const int sw = (l32 / C::SWR) % C::PPR;

#ifdef KH_TUNING
  // tuning builds only: dbg & 16 turns `res` into a timestamp buffer (8 x int64 per workgroup), no residual
  long long* ts = (p.dbg & 16) ? reinterpret_cast<long long*>(const_cast<bf16_t*>(p.res)) + (size_t)bid * 8 : nullptr;
  if (p.dbg & 16) p.res = nullptr;
  auto stamp = [&](int i) { if (ts != nullptr && tid == 0) ts[i] = (long long)__builtin_readcyclecounter(); };
#else
  auto stamp = [](int) {};
#endif
  stamp(0);
  // (only the instantiations that keep T in LDS walk several column tiles; the others have exactly one per workgroup: no
  // loop, so nothing of the epilogue's address arithmetic is hoisted above the K loop, where registers are scarcest)
  for (int jt = 0; jt < (NRT == 0 ? 1 : p.n_chunk); ++jt) {
    const int n_tile = chunk * p.n_chunk + jt;
    if (n_tile >= p.n_tiles) break;  // uniform over the workgroup
    const int n0 = n_tile * BN;
    const bool shrink = (NRT > 0) && (jt == 0);

    // this wave's DMA sources / LDS destinations for one stage (K offset 0; the loop adds t*32 columns)
    auto dma_setup = [&](auto& d) {
      using D = typename std::remove_reference<decltype(d)>::type;
      int q = 0;
#pragma unroll
      for (int i = 0; i < D::XI; ++i, ++q) {
        const int r = (wave * D::XI + i) * C::UROWS + u_row;  // row inside the x tile
        const int pc = ((lane % C::PPR) ^ ((r / C::SWR) % C::PPR)) * 8;
        int row = (KH_DBG(p, 32) ? 0 : m0) + r; row = row < M ? row : M - 1;
        if constexpr (CONV) {
          // output pixel -> the input pixel above-left of its 3x3 window, and which taps are inside the image
          const int wo = row % p.conv_wo, t2 = row / p.conv_wo, ho = t2 % p.conv_ho, nb = t2 / p.conv_ho;
          const int hi0 = ho * p.conv_stride - 1, wi0 = wo * p.conv_stride - 1;
          int mask = 0;
#pragma unroll
          for (int tap = 0; tap < 9; ++tap) {
            const int hi = hi0 + tap / 3, wi = wi0 + tap % 3;
            mask |= (hi >= 0 && hi < p.conv_h && wi >= 0 && wi < p.conv_w) ? (1 << tap) : 0;
          }
          d.off[q] = ((long)(nb * p.conv_h + hi0) * p.conv_w + wi0) * p.conv_cin + pc;
          d.off2[q] = mask;
        } else {
          d.off[q] = (long)row * K + pc;
          d.off2[q] = row * p.ldt + pc + (p.t_nsplit > 0 ? (n0 / p.t_nsplit) * p.R : 0);
        }
        d.dst[q] = (wave * D::XI + i) * 1024;
      }
#pragma unroll
      for (int i = 0; i < D::WI; ++i, ++q) {
        const int r = (wave * D::WI + i) * C::UROWS + u_row;
        const int pc = ((lane % C::PPR) ^ ((r / C::SWR) % C::PPR)) * 8;
        int row = (KH_DBG(p, 32) ? 0 : n0) + r; row = row < N ? row : N - 1;
        d.off[q] = (long)row * K + pc;
        d.off2[q] = row * p.R + pc;
        d.dst[q] = C::SW_OFF + (wave * D::WI + i) * 1024;
      }
#pragma unroll
      for (int i = 0; i < D::AI; ++i, ++q) {
        int r = wave * D::RA + i * 16 + u_row;          // rank row; lanes >= 32 of a half instruction are masked off
        r = r < C::R ? r : C::R - 1;
        d.off[q] = (long)r * K + (((lane & 3) ^ ((r >> 2) & 3)) * 8);
        d.off2[q] = 0;
        d.dst[q] = C::SA_OFF + (wave * D::RA + i * 16) * ROWB;
      }
    };
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    f32x16 tacc[SMT][NRTT];
#pragma unroll
    for (int s = 0; s < SMT; ++s)
#pragma unroll
      for (int r = 0; r < NRTT; ++r)
#pragma unroll
        for (int v = 0; v < 16; ++v) tacc[s][r][v] = 0.f;

    // operands of the phases after the K loop, requested early: bias / col_scale before the loop, the
    // B_cat tile when the loop enters its tail
    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn * C::WTN + j * 32 + l32;
      bv[j] = (p.bias != nullptr && col < N) ? (float)p.bias[col] : 0.f;
    }
    float csv[NRTT];
#pragma unroll
    for (int r = 0; r < NRTT; ++r) csv[r] = (shrink && NRT > 0) ? p.col_scale[r * 32 + l32] : 0.f;
    if ((LNF & 1) && p.ln_part != nullptr && jt == 0) {
      ln_stats.finish(K, p.ln_eps, tid, sMu, sRs, false);
      if (tid < C::BN) { sc1[tid] = ln_c1v; sc2[tid] = ln_c2v; }
    }

    constexpr int RCH = R > 0 ? R / 8 : 1;                       // 16-byte pieces per T / B_cat row
    constexpr int BCH = NRT > 0 ? BN * RCH / C::NT : 0;          // pieces of the B_cat tile per thread
    static_assert(NRT == 0 || (BN * RCH) % C::NT == 0, "expand tile split");
    u32x4 breg[BCH > 0 ? BCH : 1];
    auto tail_loads = [&]() {
#pragma unroll
      for (int q = 0; q < BCH; ++q) {
        const int c = tid + q * C::NT, row = c / RCH, ch = c % RCH;
        int gr = n0 + row; gr = gr < N ? gr : N - 1;
        breg[q] = ld16(p.b_cat + (size_t)gr * R + ch * 8);
      }
    };

    stamp(1);
    if (shrink) {
      if constexpr (NRT > 0) {
        Dma<C, true> d;
        dma_setup(d);
        k_loop<C, true, BCH, false>(smem, d, p.x, p.w, p.a_cat, p.t_ext, p.b_cat, KT, KT1, lane, wm, wn, l32, lh, sw, acc, tacc, tail_loads, ConvGeom{0, 0});
      }
    } else if constexpr (NRT > 0) {
      // later column tiles of an instantiation that keeps T in LDS: the B_cat tile rides in that loop's tail
      Dma<C, false> d;
      dma_setup(d);
      k_loop<C, false, BCH, CONV>(smem, d, p.x, p.w, p.a_cat, p.t_ext, p.b_cat, KT, KT1, lane, wm, wn, l32, lh, sw, acc, tacc, tail_loads,
                                  ConvGeom{p.conv_w, p.conv_cin}, false, false, nullptr, 0, nullptr, half_last);
    } else {
#if __HIP_DEVICE_COMPILE__
      // buffer form of the operands: every buffer starts at this tile's first row, so the per-lane offsets stay small
      // whatever the size of the matrix (a convolution's image as a whole: shorter than 2 GiB, checked by the launcher)
      Dma2<C> d;
      using D2 = Dma2<C>;
#pragma unroll
      for (int i = 0; i < D2::XI; ++i) {
        const int r = (wave * D2::XI + i) * C::UROWS + u_row;  // row inside the x tile
        const uint32_t pcb = (uint32_t)(((lane % C::PPR) ^ ((r / C::SWR) % C::PPR)) * 16);
        int row = m0 + r; row = row < M ? row : M - 1;
        if constexpr (CONV) {
          // output pixel -> the input pixel above-left of its 3x3 window, and which taps are inside the image; the
          // offset is relative to one row and one pixel in front of the image (the buffer's base): never negative
          const int wo = row % p.conv_wo, t2 = row / p.conv_wo, ho = t2 % p.conv_ho, nb = t2 / p.conv_ho;
          const int hi0 = ho * p.conv_stride - 1, wi0 = wo * p.conv_stride - 1;
          int mask = 0;
#pragma unroll
          for (int tap = 0; tap < 9; ++tap) {
            const int hi = hi0 + tap / 3, wi = wi0 + tap % 3;
            mask |= (hi >= 0 && hi < p.conv_h && wi >= 0 && wi < p.conv_w) ? (1 << tap) : 0;
          }
          d.voff[i] = (uint32_t)(((nb * p.conv_h + hi0 + 1) * p.conv_w + wi0 + 1) * p.conv_cin) * 2u + pcb;
          d.voff2[i] = d.voff[i];
          d.tapmask[i] = mask;
        } else {
          d.voff[i] = (uint32_t)(row - m0) * (uint32_t)K * 2u + pcb;
          d.voff2[i] = (uint32_t)(row - m0) * (uint32_t)p.ldt * 2u + pcb;
          d.tapmask[i] = 0;
        }
      }
#pragma unroll
      for (int i = 0; i < D2::WI; ++i) {
        const int r = (wave * D2::WI + i) * C::UROWS + u_row;
        const uint32_t pcb = (uint32_t)(((lane % C::PPR) ^ ((r / C::SWR) % C::PPR)) * 16);
        int row = n0 + r; row = row < N ? row : N - 1;
        d.voff[D2::XI + i] = (uint32_t)(row - n0) * (uint32_t)K * 2u + pcb;
        d.voff2[D2::XI + i] = (uint32_t)(row - n0) * (uint32_t)p.R * 2u + pcb;
      }
      auto clamp32 = [](size_t bytes) { return (int)(uint32_t)(bytes < 0xFFFFFFFFull ? bytes : 0xFFFFFFFFull); };
      auto mk = [&](const bf16_t* base, size_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(base), 0, clamp32(bytes), 0x00020000);
      };
      Rsrc4 rs;
      if constexpr (CONV) {
        const size_t lead = (size_t)(p.conv_w + 1) * p.conv_cin;
        rs.x = mk(p.x - lead, ((size_t)(M / (p.conv_ho * p.conv_wo)) * p.conv_h * p.conv_w * p.conv_cin + lead) * 2);
      } else {
        rs.x = mk(p.x + (size_t)m0 * K, (size_t)(M - m0) * K * 2);
      }
      rs.w = mk(p.w + (size_t)n0 * K, (size_t)(N - n0) * K * 2);
      const bool ext = p.t_ext != nullptr;
      const size_t tcol = p.t_nsplit > 0 ? (size_t)(n0 / p.t_nsplit) * p.R : 0;
      rs.t = mk(ext ? p.t_ext + (size_t)m0 * p.ldt + tcol : p.x, ext ? ((size_t)(M - m0) * p.ldt - tcol) * 2 : 0);
      rs.b = mk(ext ? p.b_cat + (size_t)n0 * p.R : p.w, ext ? (size_t)(N - n0) * p.R * 2 : 0);
      if constexpr (IL) {
        constexpr int TPB = BM / 64;                                                   // 64-row shrink tiles per row block
        const int gx = (M + 63) / 64, rt = gx - TPB * m_blk < TPB ? gx - TPB * m_blk : TPB;
        k_loop2<C, CONV, true>(smem, d, rs, KT, KT1, lane, wave, wm, wn, l32, lh, sw, acc, ConvGeom{0, 0},
                               p.il_cnt + m_blk, rt * il_col_tiles(p), p.il_cnt + (p.M + 127) / 128, half_last);
      } else {
        k_loop2<C, CONV, false>(smem, d, rs, KT, KT1, lane, wave, wm, wn, l32, lh, sw, acc, ConvGeom{p.conv_w, p.conv_cin},
                                nullptr, 0, nullptr, half_last);
      }
#endif
    }
    stamp(2);
    __syncthreads();  // every wave is done reading the ring before sB / sC reuse it
    stamp(3);
    if constexpr (NRT > 0) {
      if (shrink) {
#pragma unroll
        for (int r = 0; r < NRT; ++r) {
          const int col = r * 32 + l32;
#pragma unroll
          for (int s = 0; s < C::SM; ++s) {
            const int rbase = wm * C::WTM + (wn * C::SM + s) * 32 + 4 * lh;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int row = rbase + 8 * (v >> 2) + (v & 3);
              sT[row * C::LDT + col] = (bf16_t)(tacc[s][r][v] * csv[r]);
            }
          }
        }
      }
#pragma unroll
      for (int q = 0; q < BCH; ++q) {
        const int c = tid + q * C::NT, row = c / RCH, ch = c % RCH;
        *reinterpret_cast<u32x4*>(sB + row * C::LDT + ch * 8) = breg[q];
      }
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < R / 16; ++ks) {
        bf16x8 a[TM], b[TN];
        const int ko = ks * 16 + lh * 8;
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = lds_fragb(sT + (wm * C::WTM + i * 32 + l32) * C::LDT + ko);
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = lds_fragb(sB + (wn * C::WTN + j * 32 + l32) * C::LDT + ko);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
      }
      __syncthreads();  // sB is dead before sC overwrites it
    }

    // Epilogue: bias in fp32, round to bf16, transpose through LDS so that every global store is a
    // 16-byte piece of a contiguous output row.  Residual pieces are requested before the staging
    // writes so their latency hides behind the transpose.
    stamp(4);
    const int out_ld = p.geglu ? (N >> 1) : N;
    const KhOut yout(p.y, (size_t)M * out_ld * 2);
    constexpr int CPR = BN / 8;                                   // 16-byte pieces per staged row
    constexpr int ECH = C::WAVES_M * 32 * CPR / C::NT;            // pieces per thread per pass
    constexpr int OPR = BN / 16;                                  // GEGLU: output pieces per staged row
    constexpr int GCH = C::WAVES_M * 32 * OPR / C::NT;
    static_assert((C::WAVES_M * 32 * CPR) % C::NT == 0 && (C::WAVES_M * 32 * OPR) % C::NT == 0, "epilogue split");
    // cross-attention epilogue: this tile's keys and values are requested first and arrive while the tile is staged
    // (requesting them before the K loop was measured: no faster, and one instantiation then needs scratch memory)
    XAttnTile<C::LDC> xat;
    if constexpr (XA) {
      static_assert(!XA || (BM == 128 && BN == 128 && C::NT == 512 && NRT == 0 && !CONV), "cross-attention epilogue: 128 x 128 tiles");
      static_assert(!XA || XAttnTile<C::LDC>::LDS_BYTES <= (int)C::LDS_BYTES, "cross-attention epilogue: LDS");
      xat.load(p, m0, n0, tid);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      // rows of the staging tile: one 32-row pass per i, or (XA) the whole tile side by side
      const int srb = XA ? wm * C::WTM + i * 32 : wm * 32;
      u32x4 rr[ECH];
      if (!XA && p.res != nullptr) {
#pragma unroll
        for (int q = 0; q < ECH; ++q) {
          const int c = tid + q * C::NT, srow = c / CPR, ch = c % CPR;
          const int grow = m0 + (srow >> 5) * C::WTM + i * 32 + (srow & 31), gcol = n0 + ch * 8;
          rr[q] = (grow < M && gcol < N) ? ld16(p.res + (size_t)grow * N + gcol) : u32x4{0, 0, 0, 0};
        }
      }
      if ((LNF & 1) && p.ln_part != nullptr) {
        // y = rstd_row * (acc - mean_row * c1_col) + c2_col: four consecutive rows per accumulator group
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int trow = wm * C::WTM + i * 32 + 8 * g + 4 * lh;
          const f32x4 mu = *reinterpret_cast<const f32x4*>(sMu + trow), rs = *reinterpret_cast<const f32x4*>(sRs + trow);
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int col = wn * C::WTN + j * 32 + l32;
            const float c1 = sc1[col], c2 = sc2[col];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              sC[(srb + 8 * g + 4 * lh + e) * C::LDC + col] = (bf16_t)(rs[e] * (acc[i][j][4 * g + e] - mu[e] * c1) + c2);
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int col = wn * C::WTN + j * 32 + l32;
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int row = srb + 8 * (v >> 2) + 4 * lh + (v & 3);
            sC[row * C::LDC + col] = (bf16_t)(acc[i][j][v] * oscale + bv[j]);
          }
        }
      }
      if constexpr (XA) continue;
      __syncthreads();
      if ((LNF & 2) && !p.geglu && p.st_part != nullptr) {
        // as below, and every row's (sum, sum of squares) over this tile's columns for a following folded LayerNorm:
        // the CPR pieces of a row sit in CPR neighbouring lanes
#pragma unroll
        for (int q = 0; q < ECH; ++q) {
          const int c = tid + q * C::NT, srow = c / CPR, ch = c % CPR;
          const int grow = m0 + (srow >> 5) * C::WTM + i * 32 + (srow & 31), gcol = n0 + ch * 8;
          const bool ok = grow < M && gcol < N;
          u32x4 o = ok ? *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + ch * 8) : u32x4{0, 0, 0, 0};
          if (p.res != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[q][e]), bf16_hi(o[e]) + bf16_hi(rr[q][e]));
          }
          if (ok) yout.store16(((size_t)grow * N + gcol) * 2, o);
          float ps, pq;
          kh_piece_sums(o, ps, pq);
          static_assert(CPR == 16 || CPR == 32, "a row's pieces fill one or two DPP rows");
          ps = kh_row16_sum(ps);
          pq = kh_row16_sum(pq);
          if constexpr (CPR == 32) {
            ps += __shfl_xor(ps, 16, 64);
            pq += __shfl_xor(pq, 16, 64);
          }
          if (ch == 0 && grow < M) kh_ln_store_stats(p.st_part, grow, M, n_tile, p.n_tiles, ps, pq);
        }
      } else if (!p.geglu) {
#pragma unroll
        for (int q = 0; q < ECH; ++q) {
          const int c = tid + q * C::NT, srow = c / CPR, ch = c % CPR;
          const int grow = m0 + (srow >> 5) * C::WTM + i * 32 + (srow & 31), gcol = n0 + ch * 8;
          if (grow < M && gcol < n_store) {
            u32x4 o = *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + ch * 8);
            if (p.res != nullptr) {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[q][e]), bf16_hi(o[e]) + bf16_hi(rr[q][e]));
            }
            yout.store16(((size_t)grow * N + gcol) * 2, o);
          }
        }
      } else {
        // staged columns come in groups of 64 = 32 value columns then their 32 gate columns
#pragma unroll
        for (int q = 0; q < GCH; ++q) {
          const int c = tid + q * C::NT, srow = c / OPR, oc = c % OPR;
          const int grp = oc >> 2, sub = oc & 3;
          const int grow = m0 + (srow >> 5) * C::WTM + i * 32 + (srow & 31);
          const int gcol = (n0 >> 1) + grp * 32 + sub * 8;
          if (grow < M && gcol < out_ld) {
            const u32x4 hv = *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + grp * 64 + sub * 8);
            const u32x4 gv = *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + grp * 64 + 32 + sub * 8);
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float g0 = bf16_lo(gv[e]), g1 = bf16_hi(gv[e]);
              const float a0 = kh_gelu_erf(g0);
              const float a1 = kh_gelu_erf(g1);
              const uint32_t ar = pack_bf16x2(a0, a1);  // gelu(gate) rounded to bf16 before the product
              o[e] = pack_bf16x2(bf16_lo(hv[e]) * bf16_lo(ar), bf16_hi(hv[e]) * bf16_hi(ar));
            }
            yout.store16(((size_t)grow * out_ld + gcol) * 2, o);
          }
        }
      }
      __syncthreads();
    }
    if constexpr (XA) xat.run(smem, p, m0, n0, tid);
    stamp(5);
  }
}

template <class C, bool CONV = false>
int launch_pcfg(LoraGemmParams p, hipStream_t stream, int n_groups = 1) {
  p.m_tiles = (p.M + C::BM - 1) / C::BM;
  p.n_tiles = (p.N + C::BN - 1) / C::BN;
  int nc = 1;
  if (C::NRT > 0) {
    // walk several N tiles per workgroup (T reused from LDS) while the grid still covers the chip
    while (nc < p.n_tiles && (long)p.m_tiles * ((p.n_tiles + 2 * nc - 1) / (2 * nc)) >= 256) nc *= 2;
  }
  p.n_chunk = nc;
  p.n_chunks = (p.n_tiles + nc - 1) / nc;
  constexpr bool ln_fits = C::LDS_BYTES + KH_LN_LDS <= 160 * 1024 && C::NRT == 0 && !CONV;
  if ((p.ln_part != nullptr || p.st_part != nullptr) && (!ln_fits || p.sg_mode != 0 || p.grp != nullptr)) return KH_ERR_UNSUPPORTED;
  if (p.st_part != nullptr && (p.geglu || p.n_tiles > KH_LN_SLOTS)) return KH_ERR_UNSUPPORTED;
  p.ln_lds = (int)C::LDS_BYTES;
  unsigned grid = (unsigned)(p.m_tiles * p.n_chunks);
  p.xg_n = p.xr_m = p.xr_n = 0;
  if (C::NRT == 0 && !KH_DBG(p, 8)) {
    // choose the XCD grid whose per-XCD block touches the fewest operand rows, padding counted as cost
    double best = 0;
    for (int gm = 1; gm <= 8; gm *= 2) {
      const int gn = 8 / gm;
      const int rm = (p.m_tiles + gm - 1) / gm, rn = (p.n_tiles + gn - 1) / gn;
      const double cost = ((double)rm * C::BM + (double)rn * C::BN) * (8.0 * rm * rn) / ((double)p.m_tiles * p.n_tiles);
      if (p.xg_n == 0 || cost < best) { best = cost; p.xg_n = gn; p.xr_m = rm; p.xr_n = rn; }
    }
    grid = 8u * (unsigned)p.xr_m * (unsigned)p.xr_n;
  }
  if (p.xa_k != nullptr) {   // cross-attention in the epilogue: the 128x128 / 8-wave tiles only
    if constexpr (std::is_same<C, PCfg<128, 128, 2, 4, 0, 4, 64>>::value && !CONV) {
      if (n_groups != 1 || p.sg_mode != 0 || p.geglu || p.res != nullptr || p.st_part != nullptr || p.M % 128 != 0 || p.N % 128 != 0)
        return KH_ERR_UNSUPPORTED;
      auto go = [&](auto lnf) {
        constexpr int L = decltype(lnf)::value;
        if (hipError_t e = kh_allow_lds<lora_gemm_pipe_kernel<C, false, false, L, true>>((int)C::LDS_BYTES + KH_LN_LDS); e != hipSuccess) return (int)e;
        kh_launch(KH_TAG_LORA_GEMM, lora_gemm_pipe_kernel<C, false, false, L, true>, dim3(grid), dim3(C::NT), C::LDS_BYTES + KH_LN_LDS, stream, p);
        KH_RETURN_LAST_ERROR();
      };
      return p.ln_part != nullptr ? go(std::integral_constant<int, 1>{}) : go(std::integral_constant<int, 0>{});
    } else {
      return KH_ERR_UNSUPPORTED;
    }
  }
  if constexpr (ln_fits) {
    auto go = [&](auto lnf) {
      constexpr int L = decltype(lnf)::value;
      if (hipError_t e = kh_allow_lds<lora_gemm_pipe_kernel<C, false, false, L>>((int)C::LDS_BYTES + KH_LN_LDS); e != hipSuccess) return (int)e;
      kh_launch(KH_TAG_LORA_GEMM, lora_gemm_pipe_kernel<C, false, false, L>, dim3(grid, (unsigned)n_groups), dim3(C::NT),
                C::LDS_BYTES + KH_LN_LDS, stream, p);
      KH_RETURN_LAST_ERROR();
    };
    if (p.ln_part != nullptr && p.st_part != nullptr) return go(std::integral_constant<int, 3>{});
    if (p.ln_part != nullptr) return go(std::integral_constant<int, 1>{});
    if (p.st_part != nullptr) return go(std::integral_constant<int, 2>{});
  }
  if (hipError_t e = kh_allow_lds<lora_gemm_pipe_kernel<C, CONV>>((int)C::LDS_BYTES); e != hipSuccess) return (int)e;
  kh_launch(CONV ? KH_TAG_CONV : KH_TAG_LORA_GEMM, lora_gemm_pipe_kernel<C, CONV>, dim3(grid, (unsigned)n_groups), dim3(C::NT), C::LDS_BYTES, stream, p);
  KH_RETURN_LAST_ERROR();
}

template <int BM, int BN, int WM, int WN, int NST>
int launch_prank(const LoraGemmParams& p, hipStream_t stream) {
  // two-launch form: T is an input, the rank columns ride along as extra K tiles of the plain GEMM
  if (p.t_ext != nullptr) return launch_pcfg<PCfg<BM, BN, WM, WN, 0, NST>>(p, stream);
  switch (p.R / 32) {
    case 0: return launch_pcfg<PCfg<BM, BN, WM, WN, 0, NST>>(p, stream);
    case 1: return launch_pcfg<PCfg<BM, BN, WM, WN, 1, NST>>(p, stream);
    case 2: return launch_pcfg<PCfg<BM, BN, WM, WN, 2, NST>>(p, stream);
    case 3: return launch_pcfg<PCfg<BM, BN, WM, WN, 3, NST>>(p, stream);
    case 4: return launch_pcfg<PCfg<BM, BN, WM, WN, 4, NST>>(p, stream);
    default: return KH_ERR_UNSUPPORTED;
  }
}

// plain GEMM (optionally K-extended by the rank columns) with 64 K columns per stage
bool deep_stage_ok(const LoraGemmParams& p) {
  const bool plain = p.R == 0 || p.t_ext != nullptr;
  return plain && p.K % 64 == 0 && (p.t_ext == nullptr || p.R % 64 == 0);
}

bool plain_ok(const LoraGemmParams& p) { return p.R == 0 || p.t_ext != nullptr; }

}  // namespace

// Shrink inside the launch: the shapes whose 128x128 tiles leave at least a quarter of the CUs idle, so that the 64x64
// shrink tiles find CUs of their own next to the GEMM workgroups.  Measured alone at M 2048 / N 1280 / K 1280: 20 us
// against 17.8 + 4.6 for the two launches (the GEMM workgroups run 2 us slower beside the shrink, whether or not they
// have to wait for it); inside the UNet step, K = 5120: 53 us against 49 + 12 (there the two-launch GEMM would use the
// 64x160 tiles, which fill every CU and leave the shrink no room).
// 0: not suited; 1: 128x128 tiles that leave CUs idle; 2: 256x128 tiles for the stacked q/k/v projection (the shrink
// tiles take a round of CUs first, the GEMM tiles follow as they free up: still shorter than two launches)
static int il_form(const LoraGemmParams& p) {
  const long tiles = (long)((p.M + 127) / 128) * ((p.N + 127) / 128);
  const long shr = (long)((p.M + 63) / 64) * il_col_tiles(p);
  const bool t_ok = p.t_nsplit == 0 ? p.ldt == p.R : (p.N % p.t_nsplit == 0 && p.ldt == (p.N / p.t_nsplit) * p.R && p.t_nsplit % 128 == 0);
  const bool ok = p.R > 0 && p.R % 64 == 0 && p.ldt % 64 == 0 && p.K % 64 == 0 && p.t_ext != nullptr && p.a_cat != nullptr &&
                  p.col_scale != nullptr && p.il_cnt != nullptr && t_ok && p.grp == nullptr && p.sg_mode == 0 && p.conv_cin == 0 &&
                  !p.geglu && p.M >= 1024;
  if (!ok) return 0;
  if (tiles <= 192 && tiles + shr <= 256) return 1;
  if (tiles >= 480 && p.K >= 1024 && (long)((p.M + 255) / 256) * ((p.N + 127) / 128) <= 256 && shr <= 256) return 2;
  return 0;
}

bool lora_gemm_pipe_il_ok(const LoraGemmParams& p) { return il_form(p) != 0; }

// See include/katz_hip.h.  Synchronous (a blocking 4-byte copy on the null stream of the current device).
KH_EXPORT int kh_lora_split_timeouts(int32_t* count, int clear) {
  if (!count) return KH_ERR_INVALID_ARG;
  int v = 0;
  hipError_t e = hipMemcpyFromSymbol(&v, HIP_SYMBOL(kh_split_timeout_count), sizeof(int), 0, hipMemcpyDeviceToHost);
  if (e != hipSuccess) return (int)e;
  if (clear && v != 0) {
    const int zero = 0;
    e = hipMemcpyToSymbol(HIP_SYMBOL(kh_split_timeout_count), &zero, sizeof(int), 0, hipMemcpyHostToDevice);
    if (e != hipSuccess) return (int)e;
  }
  int v2 = 0;   // the cooperative form's waits (lora_gemm_ksplit.hip)
  if (const int rc = lora_gemm_ksplit_coop_timeouts(&v2, clear); rc != KH_OK) return rc;
  *count = v + v2;
  return KH_OK;
}

template <class C>
static int launch_il(const LoraGemmParams& pin, hipStream_t stream) {
  LoraGemmParams p = pin;
  p.m_tiles = (p.M + C::BM - 1) / C::BM;
  p.n_tiles = (p.N + C::BN - 1) / C::BN;
  p.n_chunk = 1;
  p.n_chunks = p.n_tiles;
  // dynamic LDS: the GEMM workgroups' ring and, behind it, their LayerNorm terms (KH_LN_LDS); the shrink workgroups' rings
  // start at 0 as well and carry their own row statistics inside
  constexpr int SL = IL_SHRINK_LDS + 1024;    // the shrink workgroups' rings and, behind them, their prefetch landing zone
  constexpr int LDS = (int)C::LDS_BYTES > SL ? (int)C::LDS_BYTES : SL;
  constexpr int LDS_LN = (int)C::LDS_BYTES + KH_LN_LDS > SL ? (int)C::LDS_BYTES + KH_LN_LDS : SL;
  static_assert(LDS_LN <= 160 * 1024, "LDS of one workgroup");
  p.ln_lds = (int)C::LDS_BYTES;
  double best = 0;
  p.xg_n = 0;
  for (int gm = 1; gm <= 8; gm *= 2) {
    const int gn = 8 / gm;
    const int rm = (p.m_tiles + gm - 1) / gm, rn = (p.n_tiles + gn - 1) / gn;
    const double cost = ((double)rm * C::BM + (double)rn * C::BN) * (8.0 * rm * rn) / ((double)p.m_tiles * p.n_tiles);
    if (p.xg_n == 0 || cost < best) { best = cost; p.xg_n = gn; p.xr_m = rm; p.xr_n = rn; }
  }
  const int shr = ((p.M + 63) / 64) * il_col_tiles(p);
  p.il_blocks = (shr + 7) / 8 * 8;
  const unsigned grid = (unsigned)p.il_blocks + 8u * (unsigned)p.xr_m * (unsigned)p.xr_n;
  if (p.xa_k != nullptr) {
    if constexpr (std::is_same<C, PCfg<128, 128, 2, 4, 0, 4, 64>>::value) {
      if (p.res != nullptr || p.st_part != nullptr || p.M % 128 != 0 || p.N % 128 != 0) return KH_ERR_UNSUPPORTED;
      auto go = [&](auto lnf) {
        constexpr int L = decltype(lnf)::value;
        if (hipError_t e = kh_allow_lds<lora_gemm_pipe_kernel<C, false, true, L, true>>(LDS_LN); e != hipSuccess) return (int)e;
        kh_launch(KH_TAG_LORA_GEMM, lora_gemm_pipe_kernel<C, false, true, L, true>, dim3(grid), dim3(C::NT), (size_t)LDS_LN, stream, p);
        KH_RETURN_LAST_ERROR();
      };
      return p.ln_part != nullptr ? go(std::integral_constant<int, 1>{}) : go(std::integral_constant<int, 0>{});
    } else {
      return KH_ERR_UNSUPPORTED;
    }
  }
  if (p.ln_part != nullptr || p.st_part != nullptr) {
    if (p.st_part != nullptr && p.n_tiles > KH_LN_SLOTS) return KH_ERR_UNSUPPORTED;
    auto go = [&](auto lnf) {
      constexpr int L = decltype(lnf)::value;
      if (hipError_t e = kh_allow_lds<lora_gemm_pipe_kernel<C, false, true, L>>(LDS_LN); e != hipSuccess) return (int)e;
      kh_launch(KH_TAG_LORA_GEMM, lora_gemm_pipe_kernel<C, false, true, L>, dim3(grid), dim3(C::NT), (size_t)LDS_LN, stream, p);
      KH_RETURN_LAST_ERROR();
    };
    if (p.ln_part != nullptr && p.st_part != nullptr) return go(std::integral_constant<int, 3>{});
    if (p.ln_part != nullptr) return go(std::integral_constant<int, 1>{});
    return go(std::integral_constant<int, 2>{});
  }
  if (hipError_t e = kh_allow_lds<lora_gemm_pipe_kernel<C, false, true>>(LDS); e != hipSuccess) return (int)e;
  kh_launch(KH_TAG_LORA_GEMM, lora_gemm_pipe_kernel<C, false, true>, dim3(grid), dim3(C::NT), (size_t)LDS, stream, p);
  KH_RETURN_LAST_ERROR();
}

int lora_gemm_pipe_launch_il(const LoraGemmParams& p, hipStream_t stream) {
  switch (il_form(p)) {
    case 1: return launch_il<PCfg<128, 128, 2, 4, 0, 4, 64>>(p, stream);
    case 2: return launch_il<PCfg<256, 128, 4, 2, 0, 3, 64>>(p, stream);
    default: return KH_ERR_UNSUPPORTED;
  }
}

// A query projection with its cross-attention in the epilogue (LoraGemmParams::xa_k): one round of 128x128 tiles, T either
// made inside the launch (il_cnt given and the shape suits that form) or given (t_ext with a_cat == NULL), or R == 0.
bool lora_gemm_pipe_xattn_ok(const LoraGemmParams& p) {
  const long tiles = (long)(p.M / 128) * (p.N / 128);
  return p.M % 128 == 0 && p.N % 128 == 0 && tiles <= 256 && deep_stage_ok(p) && p.xa_T > 0 && p.xa_T % 128 == 0 &&
         p.M % p.xa_T == 0 && p.xa_S >= 1 && p.xa_S <= 96 && !p.geglu && p.res == nullptr && p.st_part == nullptr;
}

int lora_gemm_pipe_launch_xattn(const LoraGemmParams& p, hipStream_t stream) {
  if (p.xa_k == nullptr || !lora_gemm_pipe_xattn_ok(p)) return KH_ERR_UNSUPPORTED;
  if (p.a_cat != nullptr && p.il_cnt != nullptr && il_form(p) == 1) return launch_il<PCfg<128, 128, 2, 4, 0, 4, 64>>(p, stream);
  return launch_pcfg<PCfg<128, 128, 2, 4, 0, 4, 64>>(p, stream);
}

// The 160-column tiles the rules below give this convolution, when the GroupNorm statistics of its result can be a
// by-product of its epilogue: whole tiles per image, whole groups per tile.
int lora_gemm_conv_gn_row_groups(const LoraGemmParams& p) {
  if (p.N % 160 != 0 || !lora_gemm_ksplit_conv_ok(p) || p.gn_cg <= 0 || 160 % p.gn_cg != 0 || p.gn_hw <= 0 || p.M % p.gn_hw != 0)
    return 0;
  const long tiles = (long)((p.M + 127) / 128) * ((p.N + 127) / 128);
  const long n160 = p.N / 160, m128 = (p.M + 127) / 128, m64 = (p.M + 63) / 64;
  int rg = 0;
  if ((tiles > 256 && tiles <= 384 && m128 * n160 <= 256) || (m128 * n160) % 256 == 0) rg = 4;
  else if (tiles <= 192 && m64 * n160 <= 256 && m64 * n160 > tiles && p.K >= 2560) rg = 2;
  return (rg == 0 || p.gn_hw % (32 * rg) != 0) ? 0 : rg;
}

int lora_gemm_pipe_launch_conv(const LoraGemmParams& p, hipStream_t stream) {
  if (p.gn_part != nullptr) {   // the caller has asked lora_gemm_conv_gn_row_groups
    const int rg = lora_gemm_conv_gn_row_groups(p);
    return rg == 0 ? KH_ERR_UNSUPPORTED : lora_gemm_ksplit_launch_conv(p, rg, stream);
  }
  const long tiles = (long)((p.M + 127) / 128) * ((p.N + 127) / 128);
  // 160-column tiles (lora_gemm_ksplit.hip) by the rules of the linear layers
  if (p.N % 160 == 0 && lora_gemm_ksplit_conv_ok(p)) {
    const long n160 = p.N / 160, m128 = (p.M + 127) / 128, m64 = (p.M + 63) / 64;
    // (whole rounds of 128x160 tiles also where 128-column tiles would divide N: the upsamplers' 1280 -> 1280 at 64x64 took
    // 342 us on the 128x128 tiles and takes 249 us on these, 640 -> 640 at 128x128 290 -> 264 us)
    if ((tiles > 256 && tiles <= 384 && m128 * n160 <= 256) || (m128 * n160) % 256 == 0) return lora_gemm_ksplit_launch_conv(p, 4, stream);
    if (tiles <= 192 && m64 * n160 <= 256 && m64 * n160 > tiles && p.K >= 2560) return lora_gemm_ksplit_launch_conv(p, 2, stream);
  }
  if (tiles <= 256 && p.conv_cin % 64 == 0) return launch_pcfg<PCfg<128, 128, 2, 4, 0, 4, 64>, true>(p, stream);
  return launch_pcfg<PCfg<128, 128, 2, 2, 0, 4>, true>(p, stream);
}

int lora_gemm_pipe_launch_sgmv(const LoraGemmParams& p, int n_segments, hipStream_t stream) {
  // one 128x128 tile column covers all of a shrink's rank columns.  The shrink streams long rows: whole 128-byte
  // lines per stage and 8 waves per workgroup; the expand's K is the rank (a few 32-column tiles).
  // (64-row tiles at two workgroups per CU were measured for the shrink: 15.7 against 12.2 us on 8 x 4096 x 640)
  if (p.sg_mode == 1 && p.K % 64 == 0) return launch_pcfg<PCfg<128, 128, 2, 4, 0, 4, 64>>(p, stream, n_segments);
  return launch_pcfg<PCfg<128, 128, 2, 2, 0, 4>>(p, stream, n_segments);
}

int lora_gemm_pipe_launch_grouped(const LoraGemmParams& p, int n_groups, hipStream_t stream) {
  return launch_pcfg<PCfg<128, 128, 2, 2, 0, 4>>(p, stream, n_groups);
}

int lora_gemm_pipe_launch(const LoraGemmParams& p, int tile_sel, hipStream_t stream) {
  switch (tile_sel) {
    case 16: return launch_prank<128, 128, 2, 2, 4>(p, stream);
    case 20: return deep_stage_ok(p) ? launch_pcfg<PCfg<128, 128, 2, 2, 0, 3, 64>>(p, stream) : KH_ERR_UNSUPPORTED;
    case 27: return plain_ok(p) ? launch_pcfg<PCfg<256, 128, 4, 2, 0, 4>>(p, stream) : KH_ERR_UNSUPPORTED;
    case 28: return plain_ok(p) ? launch_pcfg<PCfg<128, 256, 2, 4, 0, 4>>(p, stream) : KH_ERR_UNSUPPORTED;
    case 29: return deep_stage_ok(p) ? launch_pcfg<PCfg<256, 128, 4, 2, 0, 3, 64>>(p, stream) : KH_ERR_UNSUPPORTED;
    case 32: return deep_stage_ok(p) ? launch_pcfg<PCfg<128, 128, 2, 4, 0, 4, 64>>(p, stream) : KH_ERR_UNSUPPORTED;
    case 33: return deep_stage_ok(p) ? launch_pcfg<PCfg<128, 128, 2, 4, 0, 3, 64>>(p, stream) : KH_ERR_UNSUPPORTED;
    case 40: return lora_gemm_ksplit_launch(p, 2, stream);
    case 41: return lora_gemm_ksplit_launch(p, 4, stream);
    case 42: return lora_gemm_wide_launch(p, stream);
    default: break;
  }
  // Default choice.  The limiter is the vector L1 path (every operand byte enters LDS through it), so
  // FLOPs per loaded byte decide: 256x128 tiles (8 waves) when there are enough tiles to keep the chip
  // busy with them; when the 128x128 tiles do not even fill one round of 256 CUs, one 8-wave workgroup
  // per CU with 64-column stages (full 128-byte lines) beats two 4-wave ones; 128x128 / 4 waves /
  // two workgroups per CU otherwise.
  if (lora_gemm_wide_ok(p)) {
    // 256x320 tiles when they fill at least three quarters of whole rounds of the 256 CUs: fewer operand bytes per
    // FLOP than any smaller tile and no ragged last round
    const long wt = (long)(p.M / 256) * (p.N / 320), rounds = (wt + 255) / 256;
    if (wt * 4 >= rounds * 256 * 3) return lora_gemm_wide_launch(p, stream);
  }
  if (plain_ok(p)) {
    const long tiles = (long)((p.M + 127) / 128) * ((p.N + 127) / 128);
    // N a multiple of 160 and a tile count that leaves 128x128 tiles with a ragged last round: 160-column tiles
    // (8 waves splitting K) give every CU exactly one.  64-row tiles pay for their extra operand traffic only
    // on long K.
    if (p.N % 160 == 0 && lora_gemm_ksplit_ok(p)) {
      const long n160 = p.N / 160;
      if (tiles > 256 && tiles <= 384 && (long)((p.M + 127) / 128) * n160 <= 256) return lora_gemm_ksplit_launch(p, 4, stream);
      if (tiles <= 192 && (long)((p.M + 63) / 64) * n160 <= 256 && (long)((p.M + 63) / 64) * n160 > tiles && p.K >= 2560)
        return lora_gemm_ksplit_launch(p, 2, stream);
    }
    if (tiles >= 480 && p.K >= 1024 && !p.geglu) return deep_stage_ok(p) ? launch_pcfg<PCfg<256, 128, 4, 2, 0, 3, 64>>(p, stream) : launch_pcfg<PCfg<256, 128, 4, 2, 0, 4>>(p, stream);
    if (tiles <= 256 && p.M >= 1024 && deep_stage_ok(p)) return launch_pcfg<PCfg<128, 128, 2, 4, 0, 4, 64>>(p, stream);
  }
  return launch_prank<128, 128, 2, 2, 4>(p, stream);
}

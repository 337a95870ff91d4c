// Device code of the LoRA shrink tile, shared by the stand-alone kernel (lora_shrink.hip) and by the GEMM launch that
// runs its shrink on otherwise idle CUs (lora_gemm_pipe.hip).  See lora_shrink.hip for the design.
#pragma once
#include "kh_common.h"
#include "lora_gemm.h"

namespace {

struct ShrinkParams {
  const bf16_t* x; const bf16_t* a_cat; const float* col_scale; bf16_t* t;
  int M, K, R;
  // x is the input of a LayerNorm folded into the layer (see LoraGemmParams): a_cat already carries the norm's weight, and
  // the tile stores ((x . a^T) - mean * ln_ca1 + std * ln_ca2) * col_scale, the adapter's share divided by 1/std
  const float* ln_part = nullptr; const float* ln_ca1 = nullptr; const float* ln_ca2 = nullptr;
  float ln_eps = 0.f;
};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

template <int VM>
__device__ __forceinline__ void wait_vm() {  // vmcnt = VM, other counters unconstrained (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | (15 << 8) | ((VM >> 4) << 14));
}
__device__ __forceinline__ void wait_lgkm0() { __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (0 << 8) | (3 << 14)); }

template <int NW_, int TR_, int TC_, int NS_ = 2>
struct SCfg {
  static constexpr int NW = NW_, TR = TR_, TC = TC_;
  static constexpr int NS = NS_;                     // stages per wave (2 or 3)
  static constexpr int UNITS = (TR + TC) * 4;        // 8-row DMA units per stage (x rows, then A_cat rows)
  static constexpr int STAGE = UNITS * 1024;         // 64 K-columns: 128-byte rows (whole cache lines), XOR-swizzled
  static constexpr int RING = NW * NS * STAGE;
  static constexpr int LD = TC * 32 + 4;             // padded fp32 row of the partial-sum tile
  static constexpr int PART = NW * TR * 32 * LD * 4;
  static constexpr int LDS = RING > PART ? RING : PART;
  static_assert(LDS <= 160 * 1024 && UNITS * (NS - 1) < 64 && (NS == 2 || NS == 3), "LDS / vmcnt budget");
};

// One output tile of t = bf16((x . A_cat^T) * col_scale): rows m0 .. m0 + TR*32, rank columns r0 .. r0 + TC*32, by the NTB
// threads that call it (all live waves of the block: its barriers are workgroup barriers).  NTB may exceed C::NW waves: the
// extra ones only join the barriers and the final fold.  WT: the results are
// stored write-through at agent scope (for readers on other XCDs inside the same launch).
// Operands are read with buffer loads: a byte offset per lane and unit that never changes (row inside the tile, swizzled
// piece, this wave's first chunk) plus a scalar offset per chunk, so the loop carries no vector address arithmetic.
template <class C, bool WT, int NTB>   // NTB: threads of the block
__device__ __forceinline__ void lora_shrink_tile(const ShrinkParams& p, int m0, int r0, char* smem) {
#if __HIP_DEVICE_COMPILE__
  constexpr int NW = C::NW, TR = C::TR, TC = C::TC, NS = C::NS, UNITS = C::UNITS, STAGE = C::STAGE, LD = C::LD;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const bool active = wave < NW;
  const int K = p.K, KC = K / 64;                    // 64-column chunks, dealt to the waves round-robin
  const int n = active ? (KC - wave + NW - 1) / NW : 0;   // chunks wave, wave + NW, ... of this wave
  char* ring = smem + (active ? wave : 0) * (NS * STAGE);

  // DMA: lane i of a unit lands in LDS slot i = row i/8, physical piece i%8, which holds logical piece
  // (i%8) ^ ((row/2)%8); the swizzle is applied to the address the lane fetches
  auto clamp32 = [](size_t bytes) { return (int)(uint32_t)(bytes < 0xFFFFFFFFull ? bytes : 0xFFFFFFFFull); };
  const __amdgpu_buffer_rsrc_t rsx = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.x + (size_t)m0 * K), 0,
                                                                       clamp32((size_t)(p.M - m0) * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsa = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.a_cat + (size_t)r0 * K), 0,
                                                                       clamp32((size_t)(p.R - r0) * K * 2), 0x00020000);
  uint32_t voff[UNITS];
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    const int ru = u * 8 + (lane >> 3);                // row inside the stacked [x rows | A_cat rows] stage
    const uint32_t pcb = (uint32_t)(((lane & 7) ^ ((ru >> 1) & 7)) * 16);
    int row = u < TR * 4 ? ru : ru - TR * 32;
    const int last = u < TR * 4 ? p.M - 1 - m0 : p.R - 1 - r0;
    row = row < last ? row : last;
    voff[u] = (uint32_t)row * (uint32_t)K * 2u + (uint32_t)wave * 128u + pcb;
  }
  auto issue = [&](int i) {                            // this wave's i-th chunk
    char* st = ring + (i % NS) * STAGE;
    const int so = i * (NW * 128);
#pragma unroll
    for (int u = 0; u < UNITS; ++u)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(u < TR * 4 ? rsx : rsa, (lptr_t)(st + u * 1024), 16, voff[u], so, 0, 0);
  };
  f32x16 acc[TR][TC];
#pragma unroll
  for (int i = 0; i < TR; ++i)
#pragma unroll
    for (int j = 0; j < TC; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  const int sw = (l32 >> 1) & 7;

  // folded LayerNorm: the rows' statistics are requested before the first chunk (older than every DMA load, so they have
  // arrived when the first chunk has) and reduced after the loop
  KhLnTileStats<TR * 32, NTB> ln_stats;
  if (p.ln_part != nullptr) ln_stats.load(p.ln_part, m0, p.M, tid);
  if (n > 0) issue(0);
  if (n > 1) issue(1);
  if (NS > 2 && n > 2) issue(2);

  for (int i = 0; i < n; ++i) {
    // chunk i has landed; the chunks behind it (at most NS - 1) may be in flight
    if (NS > 2 && i + 2 < n) wait_vm<2 * UNITS>(); else if (i + 1 < n) wait_vm<UNITS>(); else wait_vm<0>();
    const char* st = ring + (i % NS) * STAGE;
    bf16x8 a[4][TR], b[4][TC];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int po = ((2 * ks + lh) ^ sw) * 16;
#pragma unroll
      for (int r = 0; r < TR; ++r) a[ks][r] = *reinterpret_cast<const bf16x8*>(st + (r * 32 + l32) * 128 + po);
#pragma unroll
      for (int c = 0; c < TC; ++c) b[ks][c] = *reinterpret_cast<const bf16x8*>(st + ((TR + c) * 32 + l32) * 128 + po);
    }
    wait_lgkm0();                   // fragments are in registers: the stage may be refilled
    if (i + NS < n) issue(i + NS);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int r = 0; r < TR; ++r)
#pragma unroll
        for (int c = 0; c < TC; ++c)
          acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks][r], b[ks][c], acc[r][c], 0, 0, 0);
  }
  __syncthreads();                  // every ring is dead: the partial sums reuse the memory
  float* part = reinterpret_cast<float*>(smem);   // [NW][TR*32][LD]
  float* sMu = reinterpret_cast<float*>(smem + C::PART);   // behind the partial sums
  float* sSg = sMu + TR * 32;
  static_assert(C::PART + 2 * TR * 32 * 4 <= C::LDS, "room for the row statistics");
  if (p.ln_part != nullptr) ln_stats.finish(K, p.ln_eps, tid, sMu, sSg, true);   // mean and std of this tile's rows
  if (active) {
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
      for (int j = 0; j < TC; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          part[(wave * TR * 32 + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3)) * LD + j * 32 + l32] = acc[i][j][v];
  }
  __syncthreads();
  constexpr int COLS = TC * 32, ROWS = TR * 32;
  for (int i = tid; i < ROWS * COLS / 2; i += NTB) {   // two neighbouring columns per thread
    const int rr = (2 * i) / COLS, c = (2 * i) % COLS;
    float s0 = part[rr * LD + c], s1 = part[rr * LD + c + 1];
#pragma unroll
    for (int w = 1; w < NW; ++w) {                                  // fixed order: deterministic
      s0 += part[(w * ROWS + rr) * LD + c];
      s1 += part[(w * ROWS + rr) * LD + c + 1];
    }
    if (m0 + rr < p.M && r0 + c < p.R) {
      if (p.ln_part != nullptr) {
        const float mu = sMu[rr], sg = sSg[rr];
        s0 = s0 - mu * p.ln_ca1[r0 + c] + sg * p.ln_ca2[r0 + c];
        s1 = s1 - mu * p.ln_ca1[r0 + c + 1] + sg * p.ln_ca2[r0 + c + 1];
      }
      const uint32_t v = pack_bf16x2(s0 * p.col_scale[r0 + c], s1 * p.col_scale[r0 + c + 1]);
      uint32_t* dst = reinterpret_cast<uint32_t*>(p.t + (size_t)(m0 + rr) * p.R + r0 + c);
      if (WT) __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else *dst = v;
    }
  }
#endif
}

}  // namespace

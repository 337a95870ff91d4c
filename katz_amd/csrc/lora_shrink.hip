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
#include "kh_common.h"

namespace {

struct ShrinkParams {
  const bf16_t* x; const bf16_t* a_cat; const float* col_scale; bf16_t* t;
  int M, K, R;
};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

template <int VM>
__device__ __forceinline__ void wait_vm() {  // vmcnt = VM, other counters unconstrained (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | (15 << 8) | ((VM >> 4) << 14));
}
__device__ __forceinline__ void wait_lgkm0() { __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (0 << 8) | (3 << 14)); }

template <int NW_, int TR_, int TC_>
struct SCfg {
  static constexpr int NW = NW_, TR = TR_, TC = TC_;
  static constexpr int NS = 2;                       // stages per wave
  static constexpr int UNITS = (TR + TC) * 4;        // 8-row DMA units per stage (x rows, then A_cat rows)
  static constexpr int STAGE = UNITS * 1024;         // 64 K-columns: 128-byte rows (whole cache lines), XOR-swizzled
  static constexpr int RING = NW * NS * STAGE;
  static constexpr int LD = TC * 32 + 4;             // padded fp32 row of the partial-sum tile
  static constexpr int PART = NW * TR * 32 * LD * 4;
  static constexpr int LDS = RING > PART ? RING : PART;
  static_assert(LDS <= 160 * 1024 && UNITS < 64, "LDS / vmcnt budget");
};

template <class C>
__global__ __launch_bounds__(C::NW * 64) void lora_shrink_kernel(const ShrinkParams p) {
  constexpr int NW = C::NW, TR = C::TR, TC = C::TC, NS = C::NS, UNITS = C::UNITS, STAGE = C::STAGE, LD = C::LD;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const int m0 = blockIdx.x * TR * 32, r0 = blockIdx.y * TC * 32;
  const int K = p.K, KC = K / 64;                    // 64-column chunks, dealt to the waves round-robin
  const int n = (KC - wave + NW - 1) / NW;           // chunks wave, wave + NW, ... of this wave
  char* ring = smem + wave * (NS * STAGE);

  // DMA: lane i of a unit lands in LDS slot i = row i/8, physical piece i%8, which holds logical piece
  // (i%8) ^ ((row/2)%8); the swizzle is applied to the address the lane fetches
  const bf16_t* src[UNITS];
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    const int ru = u * 8 + (lane >> 3);                // row inside the stacked [x rows | A_cat rows] stage
    const int pc = ((lane & 7) ^ ((ru >> 1) & 7)) * 8;
    if (u < TR * 4) {
      int row = m0 + ru; row = row < p.M ? row : p.M - 1;
      src[u] = p.x + (size_t)row * K + wave * 64 + pc;
    } else {
      int row = r0 + ru - TR * 32; row = row < p.R ? row : p.R - 1;
      src[u] = p.a_cat + (size_t)row * K + wave * 64 + pc;
    }
  }
  auto issue = [&](int i) {                            // this wave's i-th chunk
    char* st = ring + (i % NS) * STAGE;
#pragma unroll
    for (int u = 0; u < UNITS; ++u)
      __builtin_amdgcn_global_load_lds((gptr_t)(src[u] + (size_t)i * (NW * 64)), (lptr_t)(st + u * 1024), 16, 0, 0);
  };
  f32x16 acc[TR][TC];
#pragma unroll
  for (int i = 0; i < TR; ++i)
#pragma unroll
    for (int j = 0; j < TC; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  const int sw = (l32 >> 1) & 7;

  if (n > 0) issue(0);
  if (n > 1) issue(1);
  for (int i = 0; i < n; ++i) {
    if (i + 1 < n) wait_vm<UNITS>(); else wait_vm<0>();   // chunk i has landed; chunk i+1 may be in flight
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
#pragma unroll
  for (int i = 0; i < TR; ++i)
#pragma unroll
    for (int j = 0; j < TC; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        part[(wave * TR * 32 + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3)) * LD + j * 32 + l32] = acc[i][j][v];
  __syncthreads();
  constexpr int COLS = TC * 32, ROWS = TR * 32;
  for (int i = tid; i < ROWS * COLS; i += NW * 64) {
    const int rr = i / COLS, c = i % COLS;
    float sum = part[rr * LD + c];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += part[(w * ROWS + rr) * LD + c];   // fixed order: deterministic
    if (m0 + rr < p.M && r0 + c < p.R) p.t[(size_t)(m0 + rr) * p.R + r0 + c] = (bf16_t)(sum * p.col_scale[r0 + c]);
  }
}

template <class C>
int launch_shrink(const ShrinkParams& p, hipStream_t stream) {
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void*)lora_shrink_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS);
    if (e != hipSuccess) return (int)e;
    attr_done = true;
  }
  dim3 grid((unsigned)((p.M + C::TR * 32 - 1) / (C::TR * 32)), (unsigned)((p.R + C::TC * 32 - 1) / (C::TC * 32)));
  kh_launch(KH_TAG_LORA_SHRINK, lora_shrink_kernel<C>, grid, dim3(C::NW * 64), C::LDS, stream, p);
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
  if (!x || !a_cat || !col_scale || !t || M <= 0 || K <= 0 || R <= 0) return KH_ERR_INVALID_ARG;
  if (K % 64 != 0 || R % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 65535 * 32 || M > (1 << 24)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || !kh_aligned16(a_cat) || !kh_aligned16(t)) return KH_ERR_ALIGNMENT;
  ShrinkParams p;
  p.x = (const bf16_t*)x; p.a_cat = (const bf16_t*)a_cat; p.col_scale = col_scale; p.t = (bf16_t*)t;
  p.M = (int)M; p.K = (int)K; p.R = (int)R;
  hipStream_t s = (hipStream_t)stream;
  // the largest output tile that still gives most CUs a workgroup (a 64x64 tile reads half the bytes per output of a 32x64 one)
  if (R % 64 == 0 && ((M + 63) / 64) * (R / 64) >= 160) return launch_shrink_k<2, 2, 4, 5>(p, s);
  if (R % 64 == 0 && ((M + 31) / 32) * (R / 64) >= 256) return launch_shrink_k<1, 2, 4, 5>(p, s);
  return launch_shrink_k<1, 1, 8, 5>(p, s);
}

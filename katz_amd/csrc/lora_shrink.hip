// LoRA shrink for layers that share an input: t[M,R] = bf16((x[M,K] . A_cat[R,K]^T) * col_scale[R]).
//
// The low-rank "down" projection of the reference's LoRA linear
// (diffusers-hf/src/diffusers/models/lora.py:224-225, down(hidden_states)) for all adapters of one or
// several layers that read the same x at once: to_q / to_k / to_v of a self-attention take the same
// normalised hidden states, so their A matrices are stacked into one A_cat and x is read once.
// The result stays L2-resident (M*R*2 bytes, ~1 MB) and is consumed by kh_lora_linear_pre_bf16, which
// then runs the base GEMM without the per-tile shrink recompute of the fused kernel.
//
// Bound: HBM/L2 (x is streamed from L2; 2*M*K*R FLOPs are ~1 GFLOP).  Grid (M/32, R/32): a workgroup owns
// 32 rows x 32 rank columns; its 4 waves split K four ways (direct global -> register fragments,
// 64 contiguous bytes per row per step), partial sums meet in LDS in a fixed order (deterministic).
// Tried and dropped: splitting K across workgroups with a last-arriver reduction (the device-scope
// release is an L2 write-back on a multi-XCD part: 40 us) and 8-wave workgroups over 96 rank columns
// (too few workgroups: 18 us).
#include "kh_common.h"

namespace {

constexpr int SR_COLS = 32;          // rank columns per workgroup (one MFMA tile)
constexpr int SR_LD = SR_COLS + 4;   // padded fp32 row of the partial-sum tile
constexpr int PF = 4;                // 32-column steps kept in flight per wave

struct ShrinkParams {
  const bf16_t* x; const bf16_t* a_cat; const float* col_scale; bf16_t* t;
  int M, K, R;
};

__device__ __forceinline__ bf16x8 ldg8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

// There are only (M/32)*(R/32)*4 waves (a few per CU), so latency is hidden inside the wave: PF steps
// of both operands are requested before the first MFMA and every consumed buffer is refilled at once.
__global__ __launch_bounds__(256) void lora_shrink_kernel(const ShrinkParams p) {
  __shared__ __attribute__((aligned(16))) float part[4][32][SR_LD];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lh = lane >> 5;
  const int m0 = blockIdx.x * 32, r0 = blockIdx.y * SR_COLS;
  const int K = p.K, kq = K / 4;  // K % 64 == 0: each wave's quarter is a multiple of 16
  int row = m0 + l32; row = row < p.M ? row : p.M - 1;
  // lane (l32, lh) covers k = kbeg + step*32 + lh*16 + [0,16): two MFMA k-steps per 32-column step; both
  // operands use the same mapping, so the product is unchanged
  const bf16_t* xr = p.x + (size_t)row * K + wave * kq + lh * 16;
  const bf16_t* ar = p.a_cat + (size_t)(r0 + l32) * K + wave * kq + lh * 16;

  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  const int steps = kq / 32;
  bf16x8 xb[PF][2], ab[PF][2];
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    if (i < steps) {
      xb[i][0] = ldg8(xr + i * 32); xb[i][1] = ldg8(xr + i * 32 + 8);
      ab[i][0] = ldg8(ar + i * 32); ab[i][1] = ldg8(ar + i * 32 + 8);
    }
  }
  for (int s = 0; s < steps; s += PF) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      if (s + i < steps) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb[i][0], ab[i][0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xb[i][1], ab[i][1], acc, 0, 0, 0);
        const int n = s + i + PF;
        if (n < steps) {
          xb[i][0] = ldg8(xr + n * 32); xb[i][1] = ldg8(xr + n * 32 + 8);
          ab[i][0] = ldg8(ar + n * 32); ab[i][1] = ldg8(ar + n * 32 + 8);
        }
      }
    }
  }
  if (kq % 32 != 0) {
    // last 16 columns of the quarter: standard mapping k = base + lh*8 + [0,8)
    const int off = steps * 32 + lh * 8 - lh * 16;
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ldg8(xr + off), ldg8(ar + off), acc, 0, 0, 0);
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) part[wave][8 * (v >> 2) + 4 * lh + (v & 3)][l32] = acc[v];
  __syncthreads();
  for (int i = tid; i < 32 * SR_COLS; i += 256) {
    const int rr = i / SR_COLS, c = i % SR_COLS;
    const float sum = ((part[0][rr][c] + part[1][rr][c]) + part[2][rr][c]) + part[3][rr][c];
    if (m0 + rr < p.M) p.t[(size_t)(m0 + rr) * p.R + r0 + c] = (bf16_t)(sum * p.col_scale[r0 + c]);
  }
}

}  // namespace

KH_EXPORT int kh_lora_shrink_bf16(const void* x, const void* a_cat, const float* col_scale, void* t, int64_t M,
                                  int64_t K, int64_t R, void* stream) {
  if (!x || !a_cat || !col_scale || !t || M <= 0 || K <= 0 || R <= 0) return KH_ERR_INVALID_ARG;
  if (K % 64 != 0 || R % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 65535 * SR_COLS || M > (1 << 24)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || !kh_aligned16(a_cat) || !kh_aligned16(t)) return KH_ERR_ALIGNMENT;
  ShrinkParams p;
  p.x = (const bf16_t*)x; p.a_cat = (const bf16_t*)a_cat; p.col_scale = col_scale; p.t = (bf16_t*)t;
  p.M = (int)M; p.K = (int)K; p.R = (int)R;
  dim3 grid((unsigned)((M + 31) / 32), (unsigned)((R + SR_COLS - 1) / SR_COLS));
  kh_launch(KH_TAG_LORA_SHRINK, lora_shrink_kernel, grid, dim3(256), 0, (hipStream_t)stream, p);
  KH_RETURN_LAST_ERROR();
}

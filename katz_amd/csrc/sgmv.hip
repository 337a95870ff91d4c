// K2: segmented multi-adapter shrink / expand (one LoRA per request in a batch) for gfx950.
//
// The batch is a list of row segments; segment s = rows [seg_start[s], seg_start[s+1]) of x uses
// adapter seg_adapter[s] (or none when negative):
//   shrink:  t[rows, 0:r_a]  = x[rows, :] . A_a[0:r_a, :]^T
//   expand:  y[rows, :]     += scale_a * t[rows, 0:r_a] . B_a[:, 0:r_a]^T
// i.e. the per-request form of the reference's LoRA linear
// (diffusers-hf/src/diffusers/models/lora.py:222-232, :451-457) with y already holding the base
// projection.  The reference has no batched heterogeneous-adapter path; this is the per-request
// loop over that formula, executed as two launches.
//
// Both are HBM-bound (shrink streams x once, expand read-modify-writes y once).  When K % 32 == 0 they run as
// the segmented mode of the pipelined GEMM kernel (lora_gemm_pipe.hip: blockIdx.y = segment, operands through LDS
// with coalesced global_load_lds, the adapter's scale and the read-modify-write of y in the epilogue): 2.8 TB/s
// (shrink) and 3.2 TB/s (expand) on 8 requests x 4096 tokens x 640.  The kernels in this file are the general
// fallback (any K % 8 == 0): MFMA fragments straight from global memory, every lane in a row of its own, which
// the vector L1 serves at a quarter of its line rate (1.0 / 2.0 TB/s on the same batch).
//
// Adapters are stacked: A_all [n_adapters, RP, K], B_all [n_adapters, N, RP]; RP = padded maximum
// rank (multiple of 32); adapter_rank[a] = rank of adapter a rounded up to a multiple of 32, rows /
// columns beyond the true rank are zero.  t is [rows_total, RP].
#include "kh_common.h"

// lora_gemm.hip: the same arithmetic on the pipelined GEMM kernel (coalesced DMA through LDS), per segment.
int kh_sgmv_on_gemm(int mode, const void* x, const void* w_all, void* y, const int32_t* seg_start, const int32_t* seg_adapter,
                    const int32_t* adapter_rank, const float* adapter_scale, int64_t n_segments, int64_t max_seg_rows,
                    int64_t N, int64_t K, int64_t w_stride, hipStream_t stream);

namespace {

constexpr int MAX_NRT = 4;  // ranks up to 128

struct SgmvParams {
  const bf16_t* x; const bf16_t* a_all; const bf16_t* b_all; bf16_t* t; bf16_t* y;
  const int* seg_start; const int* seg_adapter; const int* adapter_rank; const float* adapter_scale;
  int K, N, RP;
  int n_tiles;  // expand: 128-column tiles
};

__device__ __forceinline__ bf16x8 ldg_frag(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

__global__ __launch_bounds__(256) void sgmv_shrink_kernel(const SgmvParams p) {
  const int seg = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1];
  const int a = p.seg_adapter[seg];
  const int row_base = r0 + (blockIdx.x * 4 + wave) * 32;
  if (a < 0 || row_base >= r1) return;  // wave-uniform; the kernel has no barriers
  const int nrt = p.adapter_rank[a] >> 5;
  const int K = p.K;
  int row = row_base + l32; row = row < r1 ? row : r1 - 1;
  const bf16_t* xr = p.x + (size_t)row * K + lh * 32;
  const bf16_t* ar = p.a_all + (size_t)a * p.RP * K + (size_t)l32 * K + lh * 32;

  f32x16 acc[MAX_NRT];
#pragma unroll
  for (int r = 0; r < MAX_NRT; ++r)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[r][v] = 0.f;

  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 xa[4], xn[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) xa[ks] = (lh * 32 + ks * 8 < K) ? ldg_frag(xr + ks * 8) : zero;
  for (int k0 = 0; k0 < K; k0 += 64) {
    const int kn = k0 + 64;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) xn[ks] = (kn + lh * 32 + ks * 8 < K) ? ldg_frag(xr + kn + ks * 8) : zero;
#pragma unroll
    for (int r = 0; r < MAX_NRT; ++r) {
      if (r < nrt) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const bf16x8 af = (k0 + lh * 32 + ks * 8 < K) ? ldg_frag(ar + (size_t)r * 32 * K + k0 + ks * 8) : zero;
          acc[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[ks], af, acc[r], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) xa[ks] = xn[ks];
  }
#pragma unroll
  for (int r = 0; r < MAX_NRT; ++r) {
    if (r < nrt) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int orow = row_base + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (orow < r1) p.t[(size_t)orow * p.RP + r * 32 + l32] = (bf16_t)acc[r][v];
      }
    }
  }
}

__global__ __launch_bounds__(256) void sgmv_expand_kernel(const SgmvParams p) {
  __shared__ __attribute__((aligned(16))) float stage[4][32][64 + 4];
  const int seg = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1];
  const int a = p.seg_adapter[seg];
  const int rb = blockIdx.x / p.n_tiles, nt = blockIdx.x % p.n_tiles;
  const int row_base = r0 + (rb * 4 + wave) * 32;
  if (a < 0 || row_base >= r1) return;  // wave-uniform; only wave-private LDS is used, no barriers
  const int rank = p.adapter_rank[a];
  const float scale = p.adapter_scale[a];
  const int N = p.N, RP = p.RP;
  const int n0 = nt * 128;
  int row = row_base + l32; row = row < r1 ? row : r1 - 1;
  const bf16_t* tr = p.t + (size_t)row * RP + lh * 8;
  const bf16_t* bb = p.b_all + (size_t)a * N * RP + lh * 8;

  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  for (int ks = 0; ks < rank / 16; ++ks) {
    const bf16x8 tf = ldg_frag(tr + ks * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int col = n0 + j * 32 + l32; col = col < N ? col : N - 1;
      const bf16x8 bf = ldg_frag(bb + (size_t)col * RP + ks * 16);
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tf, bf, acc[j], 0, 0, 0);
    }
  }
  // y += scale * acc, 64 columns at a time through a wave-private fp32 LDS tile so that the
  // read-modify-write touches y in 16-byte pieces of contiguous rows.
#pragma unroll
  for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
    for (int j2 = 0; j2 < 2; ++j2)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        stage[wave][8 * (v >> 2) + 4 * lh + (v & 3)][j2 * 32 + l32] = acc[2 * jj + j2][v] * scale;
    __builtin_amdgcn_s_waitcnt(0);  // LDS writes of this wave are done (lgkmcnt) before it reads them back
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = lane + 64 * i, srow = c >> 3, c8 = c & 7;
      const int grow = row_base + srow, gcol = n0 + jj * 64 + c8 * 8;
      if (grow < r1 && gcol < N) {
        const f32x4 d0 = *reinterpret_cast<const f32x4*>(&stage[wave][srow][c8 * 8]);
        const f32x4 d1 = *reinterpret_cast<const f32x4*>(&stage[wave][srow][c8 * 8 + 4]);
        bf16_t* yp = p.y + (size_t)grow * N + gcol;
        const u32x4 yv = *reinterpret_cast<const u32x4*>(yp);
        u32x4 o;
        o[0] = pack_bf16x2(bf16_lo(yv[0]) + d0[0], bf16_hi(yv[0]) + d0[1]);
        o[1] = pack_bf16x2(bf16_lo(yv[1]) + d0[2], bf16_hi(yv[1]) + d0[3]);
        o[2] = pack_bf16x2(bf16_lo(yv[2]) + d1[0], bf16_hi(yv[2]) + d1[1]);
        o[3] = pack_bf16x2(bf16_lo(yv[3]) + d1[2], bf16_hi(yv[3]) + d1[3]);
        *reinterpret_cast<u32x4*>(yp) = o;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

int check_common(const void* seg_start, const void* seg_adapter, const void* adapter_rank, int64_t n_segments,
                 int64_t max_seg_rows, int64_t RP) {
  if (!seg_start || !seg_adapter || !adapter_rank || n_segments <= 0 || max_seg_rows <= 0) return KH_ERR_INVALID_ARG;
  if (RP <= 0 || RP % 32 != 0 || RP > 32 * MAX_NRT) return KH_ERR_UNSUPPORTED;
  if (n_segments > 65535) return KH_ERR_TOO_LARGE;
  return KH_OK;
}

}  // namespace

KH_EXPORT int kh_sgmv_shrink_bf16(const void* x, const void* a_all, void* t, const int32_t* seg_start,
                                  const int32_t* seg_adapter, const int32_t* adapter_rank, int64_t n_segments,
                                  int64_t max_seg_rows, int64_t K, int64_t RP, void* stream) {
  if (!x || !a_all || !t || K <= 0) return KH_ERR_INVALID_ARG;
  int rc = check_common(seg_start, seg_adapter, adapter_rank, n_segments, max_seg_rows, RP);
  if (rc != KH_OK) return rc;
  if (K % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(x) || !kh_aligned16(a_all) || !kh_aligned16(t)) return KH_ERR_ALIGNMENT;
  if (K % 32 == 0 && max_seg_rows <= (1 << 24))   // t[rows, 0:RP] = x . A_a^T with A_a zero-padded to RP rows
    return kh_sgmv_on_gemm(1, x, a_all, t, seg_start, seg_adapter, adapter_rank, nullptr, n_segments, max_seg_rows, RP, K,
                           RP * K, (hipStream_t)stream);
  SgmvParams p = {};
  p.x = (const bf16_t*)x; p.a_all = (const bf16_t*)a_all; p.t = (bf16_t*)t;
  p.seg_start = seg_start; p.seg_adapter = seg_adapter; p.adapter_rank = adapter_rank;
  p.K = (int)K; p.RP = (int)RP;
  dim3 grid((unsigned)((max_seg_rows + 127) / 128), (unsigned)n_segments);
  kh_launch(KH_TAG_SGMV_SHRINK, sgmv_shrink_kernel, grid, dim3(256), 0, (hipStream_t)stream, p);
  KH_RETURN_LAST_ERROR();
}

KH_EXPORT int kh_sgmv_expand_bf16(const void* t, const void* b_all, void* y, const int32_t* seg_start,
                                  const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                                  int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t RP, void* stream) {
  if (!t || !b_all || !y || !adapter_scale || N <= 0) return KH_ERR_INVALID_ARG;
  int rc = check_common(seg_start, seg_adapter, adapter_rank, n_segments, max_seg_rows, RP);
  if (rc != KH_OK) return rc;
  if (N % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(t) || !kh_aligned16(b_all) || !kh_aligned16(y)) return KH_ERR_ALIGNMENT;
  if (max_seg_rows <= (1 << 24))   // y += scale_a * t[:, 0:rank_a] . B_a[:, 0:rank_a]^T (row stride RP)
    return kh_sgmv_on_gemm(2, t, b_all, y, seg_start, seg_adapter, adapter_rank, adapter_scale, n_segments, max_seg_rows, N, RP,
                           N * RP, (hipStream_t)stream);
  SgmvParams p = {};
  p.t = (bf16_t*)t; p.b_all = (const bf16_t*)b_all; p.y = (bf16_t*)y;
  p.seg_start = seg_start; p.seg_adapter = seg_adapter; p.adapter_rank = adapter_rank; p.adapter_scale = adapter_scale;
  p.N = (int)N; p.RP = (int)RP;
  p.n_tiles = (int)((N + 127) / 128);
  const long gx = ((max_seg_rows + 127) / 128) * p.n_tiles;
  if (gx > 0x7fffffffL) return KH_ERR_TOO_LARGE;
  dim3 grid((unsigned)gx, (unsigned)n_segments);
  kh_launch(KH_TAG_SGMV_EXPAND, sgmv_expand_kernel, grid, dim3(256), 0, (hipStream_t)stream, p);
  KH_RETURN_LAST_ERROR();
}

// K4: GroupNorm (+SiLU) in NHWC or NCHW, and LayerNorm, for gfx950.  HBM-bound kernels.
//
// GroupNorm replaces torch.ops.fast_kernel.group_norm_fp16 as called from
// diffusers-hf/src/diffusers/models/normalization.py:79-103 (kernel
// diffusers-hf/src/fast_kernel/fast_kernel/csrc/group_norm.cu:224-274): per (sample, group)
// mean / variance in fp32 over (C/G)*H*W elements, y = act((x - mean) * rstd * gamma_c + beta_c).
// A row is up to ~0.5 M elements and there are only N*G rows, so every row is split over many
// workgroups: pass 1 writes partial (sum, sum of squares) per split into a caller-provided
// workspace (no atomics, no zeroing, deterministic), pass 2 folds the partials in fp64 and
// streams x -> y.  Nothing is allocated here, so both passes can be captured in a HIP graph.
//
// LayerNorm (diffusers-hf/src/diffusers/models/attention.py:195,225,253 -> nn.LayerNorm,
// eps 1e-5, affine) keeps one row per wave in registers: one read, one write.
#include "kh_common.h"

namespace {

constexpr int GN_THREADS = 256;
constexpr int GN_MAX_C = 4096;  // per-channel scale/shift table in LDS (32 KB)

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int w = 0; w < (int)(blockDim.x >> 6); ++w) t += red[w];
  return t;
}

// ---------------------------------------------------------------- NHWC
// grid (splits, N); a workgroup owns pixels [p0,p1) of sample n over all channels.
// Thread (tx,ty): 16-byte channel chunks tx, tx+NTX, ... of pixels ty, ty+PL, ...
struct GnGeom {
  int N, C, HW, G, Cg, splits;
  int CP;   // 16-byte chunks per pixel (C/8)
  int NTX;  // chunk-threads
  int CPT;  // chunks per thread
  int PL;   // pixel lanes
};

__global__ __launch_bounds__(GN_THREADS) void gn_stats_nhwc(const bf16_t* __restrict__ x, float* __restrict__ ws,
                                                            const GnGeom g) {
  __shared__ float bins[2 * 512];  // per group (sum, sumsq); G <= 512
  const int n = blockIdx.y, split = blockIdx.x;
  const int tid = threadIdx.x;
  for (int i = tid; i < 2 * g.G; i += GN_THREADS) bins[i] = 0.f;
  __syncthreads();
  const int per = (g.HW + g.splits - 1) / g.splits;
  const int p0 = split * per, p1 = min(g.HW, p0 + per);
  const int tx = tid % g.NTX, ty = tid / g.NTX;
  if (ty < g.PL) {
    for (int k = 0; k < g.CPT; ++k) {
      const int cc = tx + k * g.NTX;
      float s[8], q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = q[e] = 0.f;
      const bf16_t* base = x + ((size_t)n * g.HW) * g.C + cc * 8;
      for (int p = p0 + ty; p < p1; p += g.PL) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(base + (size_t)p * g.C);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float a = bf16_lo(v[e]), b = bf16_hi(v[e]);
          s[2 * e] += a; q[2 * e] = fmaf(a, a, q[2 * e]);
          s[2 * e + 1] += b; q[2 * e + 1] = fmaf(b, b, q[2 * e + 1]);
        }
      }
      // fold the 8 channels into their groups (a chunk may straddle group boundaries)
      int cur = (cc * 8) / g.Cg;
      float cs = 0.f, cq = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int grp = (cc * 8 + e) / g.Cg;
        if (grp != cur) {
          atomicAdd(&bins[2 * cur], cs); atomicAdd(&bins[2 * cur + 1], cq);
          cur = grp; cs = 0.f; cq = 0.f;
        }
        cs += s[e]; cq += q[e];
      }
      atomicAdd(&bins[2 * cur], cs); atomicAdd(&bins[2 * cur + 1], cq);
    }
  }
  __syncthreads();
  for (int i = tid; i < g.G; i += GN_THREADS) {
    float* o = ws + (((size_t)n * g.G + i) * g.splits + split) * 2;
    o[0] = bins[2 * i]; o[1] = bins[2 * i + 1];
  }
}

template <bool SILU>
__global__ __launch_bounds__(GN_THREADS) void gn_apply_nhwc(const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                                                            const bf16_t* __restrict__ gamma,
                                                            const bf16_t* __restrict__ beta,
                                                            const float* __restrict__ ws, const GnGeom g, float eps) {
  __shared__ float s_scale[GN_MAX_C];
  __shared__ float s_shift[GN_MAX_C];
  __shared__ float s_mean[512], s_rstd[512];
  const int n = blockIdx.y, split = blockIdx.x;
  const int tid = threadIdx.x;
  const double cnt = (double)g.Cg * (double)g.HW;
  for (int i = tid; i < g.G; i += GN_THREADS) {
    const float* pw = ws + ((size_t)n * g.G + i) * g.splits * 2;
    double s = 0.0, q = 0.0;
    for (int k = 0; k < g.splits; ++k) { s += (double)pw[2 * k]; q += (double)pw[2 * k + 1]; }
    const double mean = s / cnt;
    double var = q / cnt - mean * mean;
    var = var > 0.0 ? var : 0.0;
    s_mean[i] = (float)mean;
    s_rstd[i] = (float)(1.0 / sqrt(var + (double)eps));
  }
  __syncthreads();
  for (int c = tid; c < g.C; c += GN_THREADS) {
    const int grp = c / g.Cg;
    const float ga = gamma ? (float)gamma[c] : 1.f, be = beta ? (float)beta[c] : 0.f;
    const float sc = ga * s_rstd[grp];
    s_scale[c] = sc;
    s_shift[c] = be - s_mean[grp] * sc;
  }
  __syncthreads();
  const int per = (g.HW + g.splits - 1) / g.splits;
  const int p0 = split * per, p1 = min(g.HW, p0 + per);
  const long chunks = (long)(p1 - p0) * g.CP;
  const bf16_t* xb = x + ((size_t)n * g.HW + p0) * g.C;
  bf16_t* yb = y + ((size_t)n * g.HW + p0) * g.C;
  for (long i = tid; i < chunks; i += GN_THREADS) {
    const int c0 = (int)(i % g.CP) * 8;
    const u32x4 v = *reinterpret_cast<const u32x4*>(xb + i * 8);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float a = fmaf(bf16_lo(v[e]), s_scale[c0 + 2 * e], s_shift[c0 + 2 * e]);
      float b = fmaf(bf16_hi(v[e]), s_scale[c0 + 2 * e + 1], s_shift[c0 + 2 * e + 1]);
      if (SILU) { a = silu_f(a); b = silu_f(b); }
      o[e] = pack_bf16x2(a, b);
    }
    *reinterpret_cast<u32x4*>(yb + i * 8) = o;
  }
}

// ---------------------------------------------------------------- NCHW
// grid (splits, N*G); row (n,g) is Cg*HW contiguous elements.
__global__ __launch_bounds__(GN_THREADS) void gn_stats_nchw(const bf16_t* __restrict__ x, float* __restrict__ ws,
                                                            long row_len, int splits) {
  __shared__ float red[GN_THREADS / 64];
  const long row = blockIdx.y;
  const int split = blockIdx.x;
  const long chunks = row_len / 8;  // row_len % 8 == 0 is checked by the host
  const long per = (chunks + splits - 1) / splits;
  const long c0 = split * per, c1 = min(chunks, c0 + per);
  const bf16_t* xb = x + row * row_len;
  float s = 0.f, q = 0.f;
  for (long i = c0 + threadIdx.x; i < c1; i += GN_THREADS) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(xb + i * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float a = bf16_lo(v[e]), b = bf16_hi(v[e]);
      s += a + b;
      q = fmaf(a, a, q); q = fmaf(b, b, q);
    }
  }
  s = block_sum(s, red);
  q = block_sum(q, red);
  if (threadIdx.x == 0) {
    float* o = ws + ((size_t)row * splits + split) * 2;
    o[0] = s; o[1] = q;
  }
}

template <bool SILU>
__global__ __launch_bounds__(GN_THREADS) void gn_apply_nchw(const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                                                            const bf16_t* __restrict__ gamma,
                                                            const bf16_t* __restrict__ beta,
                                                            const float* __restrict__ ws, long row_len, int splits,
                                                            int G, int Cg, int HW, float eps) {
  __shared__ float s_mr[2];
  const long row = blockIdx.y;
  const int split = blockIdx.x;
  if (threadIdx.x == 0) {
    const float* pw = ws + (size_t)row * splits * 2;
    double s = 0.0, q = 0.0;
    for (int k = 0; k < splits; ++k) { s += (double)pw[2 * k]; q += (double)pw[2 * k + 1]; }
    const double mean = s / (double)row_len;
    double var = q / (double)row_len - mean * mean;
    var = var > 0.0 ? var : 0.0;
    s_mr[0] = (float)mean;
    s_mr[1] = (float)(1.0 / sqrt(var + (double)eps));
  }
  __syncthreads();
  const float mean = s_mr[0], rstd = s_mr[1];
  const int grp = (int)(row % G);
  const long chunks = row_len / 8;
  const long per = (chunks + splits - 1) / splits;
  const long c0 = split * per, c1 = min(chunks, c0 + per);
  const bf16_t* xb = x + row * row_len;
  bf16_t* yb = y + row * row_len;
  for (long i = c0 + threadIdx.x; i < c1; i += GN_THREADS) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(xb + i * 8);
    // HW % 8 == 0 (host-checked): the 8 elements share one channel
    const int c = grp * Cg + (int)((i * 8) / HW);
    const float ga = gamma ? (float)gamma[c] : 1.f, be = beta ? (float)beta[c] : 0.f;
    const float sc = ga * rstd, sh = be - mean * sc;
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float a = fmaf(bf16_lo(v[e]), sc, sh), b = fmaf(bf16_hi(v[e]), sc, sh);
      if (SILU) { a = silu_f(a); b = silu_f(b); }
      o[e] = pack_bf16x2(a, b);
    }
    *reinterpret_cast<u32x4*>(yb + i * 8) = o;
  }
}

int gn_splits_nhwc(long N, long HW) {
  long s = HW / 32;  // at least 32 pixels per workgroup
  if (s < 1) s = 1;
  const long cap = (2048 + N - 1) / N;  // enough workgroups to cover 256 CUs several times
  if (s > cap) s = cap;
  if (s > 256) s = 256;
  return (int)s;
}
int gn_splits_nchw(long rows, long row_len) {
  long s = row_len / 8 / GN_THREADS / 4;  // at least 4 chunks per thread
  if (s < 1) s = 1;
  const long cap = (2048 + rows - 1) / rows;
  if (s > cap) s = cap;
  if (s > 256) s = 256;
  return (int)s;
}

// ---------------------------------------------------------------- LayerNorm
// one wave per row, row kept in registers (D <= 64*8*LN_MAXC elements)
constexpr int LN_MAXC = 4;

__global__ __launch_bounds__(256) void layer_norm_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                                                         const bf16_t* __restrict__ gamma,
                                                         const bf16_t* __restrict__ beta, long M, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int chunks = D / 8;
  const bf16_t* xr = x + row * D;
  u32x4 v[LN_MAXC];
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < LN_MAXC; ++k) {
    const int c = lane + 64 * k;
    if (c < chunks) {
      v[k] = *reinterpret_cast<const u32x4*>(xr + c * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) s += bf16_lo(v[k][e]) + bf16_hi(v[k][e]);
    } else {
      v[k] = u32x4{0, 0, 0, 0};
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  const float mean = s / (float)D;
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < LN_MAXC; ++k) {
    const int c = lane + 64 * k;
    if (c < chunks) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a = bf16_lo(v[k][e]) - mean, b = bf16_hi(v[k][e]) - mean;
        q = fmaf(a, a, q); q = fmaf(b, b, q);
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) q += __shfl_xor(q, o, 64);
  const float rstd = rsqrtf(q / (float)D + eps);
  bf16_t* yr = y + row * D;
#pragma unroll
  for (int k = 0; k < LN_MAXC; ++k) {
    const int c = lane + 64 * k;
    if (c < chunks) {
      u32x4 gw = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};  // bf16 1.0 pairs
      u32x4 bw = u32x4{0, 0, 0, 0};
      if (gamma) gw = *reinterpret_cast<const u32x4*>(gamma + c * 8);
      if (beta) bw = *reinterpret_cast<const u32x4*>(beta + c * 8);
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a = (bf16_lo(v[k][e]) - mean) * rstd * bf16_lo(gw[e]) + bf16_lo(bw[e]);
        const float b = (bf16_hi(v[k][e]) - mean) * rstd * bf16_hi(gw[e]) + bf16_hi(bw[e]);
        o[e] = pack_bf16x2(a, b);
      }
      *reinterpret_cast<u32x4*>(yr + c * 8) = o;
    }
  }
}

}  // namespace

KH_EXPORT int64_t kh_group_norm_workspace_bytes(int64_t N, int64_t C, int64_t HW, int64_t G, int channels_last) {
  if (N <= 0 || C <= 0 || HW <= 0 || G <= 0 || C % G != 0) return KH_ERR_INVALID_ARG;
  const long splits = channels_last ? gn_splits_nhwc(N, HW) : gn_splits_nchw(N * G, (C / G) * HW);
  return (int64_t)N * G * splits * 2 * (int64_t)sizeof(float);
}

KH_EXPORT int kh_group_norm_bf16(const void* x, void* y, const void* gamma, const void* beta, float* workspace,
                                 int64_t N, int64_t C, int64_t HW, int64_t G, float eps, int activation,
                                 int channels_last, void* stream) {
  if (!x || !y || !workspace || N <= 0 || C <= 0 || HW <= 0 || G <= 0 || C % G != 0) return KH_ERR_INVALID_ARG;
  if (activation != 0 && activation != 1) return KH_ERR_INVALID_ARG;  // 0 = none, 1 = silu
  if (!kh_aligned16(x) || !kh_aligned16(y) || (gamma && !kh_aligned16(gamma)) || (beta && !kh_aligned16(beta)))
    return KH_ERR_ALIGNMENT;
  if (N > 65535) return KH_ERR_TOO_LARGE;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* xp = (const bf16_t*)x; bf16_t* yp = (bf16_t*)y;
  const bf16_t* gp = (const bf16_t*)gamma; const bf16_t* bp = (const bf16_t*)beta;
  if (channels_last) {
    if (C % 8 != 0 || C > GN_MAX_C || G > 512) return KH_ERR_UNSUPPORTED;
    GnGeom g;
    g.N = (int)N; g.C = (int)C; g.HW = (int)HW; g.G = (int)G; g.Cg = (int)(C / G);
    g.splits = gn_splits_nhwc(N, HW);
    g.CP = (int)(C / 8);
    // chunk-threads: the largest divisor of CP that is <= 256, so every thread owns whole chunks
    int ntx = g.CP < GN_THREADS ? g.CP : GN_THREADS;
    while (g.CP % ntx != 0) --ntx;
    g.NTX = ntx; g.CPT = g.CP / ntx; g.PL = GN_THREADS / ntx;
    dim3 grid((unsigned)g.splits, (unsigned)N);
    hipLaunchKernelGGL(gn_stats_nhwc, grid, dim3(GN_THREADS), 0, s, xp, workspace, g);
    if (activation == 1)
      hipLaunchKernelGGL(gn_apply_nhwc<true>, grid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, workspace, g, eps);
    else
      hipLaunchKernelGGL(gn_apply_nhwc<false>, grid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, workspace, g, eps);
  } else {
    const long Cg = C / G, row_len = Cg * HW, rows = N * G;
    if (HW % 8 != 0) return KH_ERR_UNSUPPORTED;
    if (rows > 65535) return KH_ERR_TOO_LARGE;
    const int splits = gn_splits_nchw(rows, row_len);
    dim3 grid((unsigned)splits, (unsigned)rows);
    hipLaunchKernelGGL(gn_stats_nchw, grid, dim3(GN_THREADS), 0, s, xp, workspace, row_len, splits);
    if (activation == 1)
      hipLaunchKernelGGL(gn_apply_nchw<true>, grid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, workspace, row_len, splits,
                         (int)G, (int)Cg, (int)HW, eps);
    else
      hipLaunchKernelGGL(gn_apply_nchw<false>, grid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, workspace, row_len,
                         splits, (int)G, (int)Cg, (int)HW, eps);
  }
  KH_RETURN_LAST_ERROR();
}

KH_EXPORT int kh_layer_norm_bf16(const void* x, void* y, const void* gamma, const void* beta, int64_t M, int64_t D,
                                 float eps, void* stream) {
  if (!x || !y || M <= 0 || D <= 0) return KH_ERR_INVALID_ARG;
  if (D % 8 != 0 || D > 64 * 8 * LN_MAXC) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(x) || !kh_aligned16(y) || (gamma && !kh_aligned16(gamma)) || (beta && !kh_aligned16(beta)))
    return KH_ERR_ALIGNMENT;
  const long blocks = (M + 3) / 4;
  if (blocks > 0x7fffffffL) return KH_ERR_TOO_LARGE;
  hipLaunchKernelGGL(layer_norm_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,
                     (bf16_t*)y, (const bf16_t*)gamma, (const bf16_t*)beta, (long)M, (int)D, eps);
  KH_RETURN_LAST_ERROR();
}

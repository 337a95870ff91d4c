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

#include <mutex>

// Partial statistics of kh_group_norm_static_bf16: one array per GPU, held until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
constexpr size_t GN_STATIC_WS_BYTES = 256 * 1024;
static __device__ __align__(256) float scratch[GN_STATIC_WS_BYTES / sizeof(float)];

namespace {

constexpr int GN_THREADS = 256;
constexpr int GN_MAX_C = 4096;

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
// Thread (tx,ty) owns the 16-byte channel chunks tx, tx+NTX, ... (at most GN_MAX_CPT of them) for
// the pixels ty, ty+PL, ...: its channels never change, so per-channel constants live in registers
// and consecutive threads read consecutive 16-byte pieces of a pixel row.
constexpr int GN_MAX_CPT = 2;
constexpr int GN_UNROLL = 4;
constexpr int GN_SUNROLL = 16;  // statistics pass: few, long-lived workgroups keep many loads in flight per thread

struct GnGeom {
  int N, C, HW, G, Cg, splits;   // splits: workgroups per sample of the statistics pass
  int asplits;                   // workgroups per sample of the apply pass (more, smaller ones)
  int CP;   // 16-byte chunks per pixel (C/8)
  int NTX;  // chunk-threads
  int CPT;  // chunks per thread
  int PL;   // pixel lanes
};

__device__ __forceinline__ void unpack8(const u32x4 v, float (&f)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) { f[2 * e] = bf16_lo(v[e]); f[2 * e + 1] = bf16_hi(v[e]); }
}

// add_nc (optional): a per-(sample, channel) term added to x before the statistics and the
// normalisation -- the resnet's time-embedding projection, which the reference adds in a separate
// pass between conv1 and norm2 (diffusers-hf/src/diffusers/models/resnet.py:388-390).
__global__ __launch_bounds__(GN_THREADS) void gn_stats_nhwc(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ add_nc,
                                                            float* __restrict__ ws, const GnGeom g) {
  extern __shared__ float part[];  // [2][PL][C]: per pixel-lane, per channel (sum, sumsq)
  const int n = blockIdx.y, split = blockIdx.x;
  const int tid = threadIdx.x;
  const int per = (g.HW + g.splits - 1) / g.splits;
  const int p0 = split * per, p1 = min(g.HW, p0 + per);
  const int tx = tid % g.NTX, ty = tid / g.NTX;
  float* psum = part;
  float* psq = part + g.PL * g.C;
  if (ty < g.PL) {
    for (int k = 0; k < g.CPT; ++k) {
      const int c0 = (tx + k * g.NTX) * 8;
      float sh[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) sh[e] = 0.f;
      if (add_nc) unpack8(*reinterpret_cast<const u32x4*>(add_nc + (size_t)n * g.C + c0), sh);
      float s[8], q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = q[e] = 0.f;
      const bf16_t* base = x + ((size_t)n * g.HW) * g.C + c0;
      int p = p0 + ty;
      for (; p + (GN_SUNROLL - 1) * g.PL < p1; p += GN_SUNROLL * g.PL) {
        u32x4 v[GN_SUNROLL];
#pragma unroll
        for (int u = 0; u < GN_SUNROLL; ++u)
          v[u] = *reinterpret_cast<const u32x4*>(base + (size_t)(p + u * g.PL) * g.C);
#pragma unroll
        for (int u = 0; u < GN_SUNROLL; ++u) {
          float f[8];
          unpack8(v[u], f);
#pragma unroll
          for (int e = 0; e < 8; ++e) { const float a = f[e] + sh[e]; s[e] += a; q[e] = fmaf(a, a, q[e]); }
        }
      }
      for (; p < p1; p += g.PL) {
        float f[8];
        unpack8(*reinterpret_cast<const u32x4*>(base + (size_t)p * g.C), f);
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float a = f[e] + sh[e]; s[e] += a; q[e] = fmaf(a, a, q[e]); }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) { psum[ty * g.C + c0 + e] = s[e]; psq[ty * g.C + c0 + e] = q[e]; }
    }
  }
  __syncthreads();
  // fixed-order fold per group: deterministic (no atomics)
  for (int grp = tid; grp < g.G; grp += GN_THREADS) {
    float s = 0.f, q = 0.f;
    for (int l = 0; l < g.PL; ++l)
      for (int c = grp * g.Cg; c < (grp + 1) * g.Cg; ++c) { s += psum[l * g.C + c]; q += psq[l * g.C + c]; }
    float* o = ws + (((size_t)n * g.G + grp) * g.splits + split) * 2;
    o[0] = s; o[1] = q;
  }
}

template <bool SILU>
__global__ __launch_bounds__(GN_THREADS) void gn_apply_nhwc(const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                                                            const bf16_t* __restrict__ gamma,
                                                            const bf16_t* __restrict__ beta,
                                                            const bf16_t* __restrict__ add_nc,
                                                            const float* __restrict__ ws, const GnGeom g, float eps) {
  __shared__ float s_mean[512], s_rstd[512];
  __shared__ double s_ps[GN_THREADS], s_pq[GN_THREADS];
  const int n = blockIdx.y, split = blockIdx.x;
  const int tid = threadIdx.x;
  const double cnt = (double)g.Cg * (double)g.HW;
  // What does not depend on the statistics is requested first: this thread's channel constants of its first chunk and
  // its first (at most) GN_UNROLL pixels.  Their latency then runs beside the fold of the partial sums below instead of behind it
  // (a kernel this short is a chain of memory round trips: partial sums, constants, first pixels).
  const int per = (g.HW + g.asplits - 1) / g.asplits;
  const int p0 = split * per, p1 = min(g.HW, p0 + per);
  const int tx = tid % g.NTX, ty = tid / g.NTX;
  const bool active = ty < g.PL;
  const u32x4 z4 = {0, 0, 0, 0};
  u32x4 pre[GN_UNROLL], cg0 = z4, cb0 = z4, ca0 = z4;
  if (active) {
    const int c0 = tx * 8;
    if (gamma) cg0 = *reinterpret_cast<const u32x4*>(gamma + c0);
    if (beta) cb0 = *reinterpret_cast<const u32x4*>(beta + c0);
    if (add_nc) ca0 = *reinterpret_cast<const u32x4*>(add_nc + (size_t)n * g.C + c0);
  }
#pragma unroll
  for (int u = 0; u < GN_UNROLL; ++u)
    pre[u] = (active && p0 + ty + u * g.PL < p1) ? *reinterpret_cast<const u32x4*>(x + ((size_t)n * g.HW + p0 + ty + u * g.PL) * g.C + tx * 8) : z4;
  // Fold the statistics pass's partial sums of every group (a workgroup needs all groups: a pixel has all channels).
  // FT threads share a group, each summing every FT-th partial in fp64; their FT sums are then added in a fixed
  // order, so the result does not depend on scheduling.
  const int FT = g.G >= GN_THREADS ? 1 : GN_THREADS / g.G;
  const int gpp = GN_THREADS / FT;   // groups per pass
  for (int base = 0; base < g.G; base += gpp) {
    const int grp = base + tid / FT, part = tid % FT;
    double s = 0.0, q = 0.0;
    if (grp < g.G) {
      const float2* pw = reinterpret_cast<const float2*>(ws) + ((size_t)n * g.G + grp) * g.splits;
      // four loads in flight per thread (a load per addition would pay the memory latency splits / FT times in a row);
      // the additions keep their order
      int k = part;
      for (; k + 3 * FT < g.splits; k += 4 * FT) {
        const float2 v0 = pw[k], v1 = pw[k + FT], v2 = pw[k + 2 * FT], v3 = pw[k + 3 * FT];
        s += (double)v0.x; q += (double)v0.y;
        s += (double)v1.x; q += (double)v1.y;
        s += (double)v2.x; q += (double)v2.y;
        s += (double)v3.x; q += (double)v3.y;
      }
      for (; k < g.splits; k += FT) { const float2 v = pw[k]; s += (double)v.x; q += (double)v.y; }
    }
    s_ps[tid] = s; s_pq[tid] = q;
    __syncthreads();
    if (part == 0 && grp < g.G) {
      for (int j = 1; j < FT; ++j) { s += s_ps[tid + j]; q += s_pq[tid + j]; }
      const double mean = s / cnt;
      double var = q / cnt - mean * mean;
      var = var > 0.0 ? var : 0.0;
      s_mean[grp] = (float)mean;
      s_rstd[grp] = (float)(1.0 / sqrt(var + (double)eps));
    }
    __syncthreads();
  }
  if (!active) return;
  const KhOut yout(y, (size_t)g.N * g.HW * g.C * 2);
  for (int k = 0; k < g.CPT; ++k) {
    const int c0 = (tx + k * g.NTX) * 8;
    u32x4 cg = cg0, cb = cb0, ca = ca0;
    if (k > 0) {
      cg = gamma ? *reinterpret_cast<const u32x4*>(gamma + c0) : z4;
      cb = beta ? *reinterpret_cast<const u32x4*>(beta + c0) : z4;
      ca = add_nc ? *reinterpret_cast<const u32x4*>(add_nc + (size_t)n * g.C + c0) : z4;
    }
    float gaf[8], bef[8], adf[8], sc[8], sh[8];
    unpack8(cg, gaf); unpack8(cb, bef); unpack8(ca, adf);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int grp = (c0 + e) / g.Cg;
      const float ga = gamma ? gaf[e] : 1.f;
      sc[e] = ga * s_rstd[grp];
      sh[e] = bef[e] + (adf[e] - s_mean[grp]) * sc[e];
    }
    const size_t off = ((size_t)n * g.HW) * g.C + c0;
    const bf16_t* xb = x + off;
    auto emit = [&](const u32x4 v, int p) {
      float f[8];
      unpack8(v, f);
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = fmaf(f[2 * e], sc[2 * e], sh[2 * e]);
        float b = fmaf(f[2 * e + 1], sc[2 * e + 1], sh[2 * e + 1]);
        if (SILU) { a = silu_f(a); b = silu_f(b); }
        o[e] = pack_bf16x2(a, b);
      }
      yout.store16((off + (size_t)p * g.C) * 2, o);
    };
    int p = p0 + ty;
    if (k == 0) {   // the pixels requested at the top
#pragma unroll
      for (int u = 0; u < GN_UNROLL; ++u)
        if (p + u * g.PL < p1) emit(pre[u], p + u * g.PL);
      p += GN_UNROLL * g.PL;
    }
    for (; p + (GN_UNROLL - 1) * g.PL < p1; p += GN_UNROLL * g.PL) {
      u32x4 v[GN_UNROLL];
#pragma unroll
      for (int u = 0; u < GN_UNROLL; ++u) v[u] = *reinterpret_cast<const u32x4*>(xb + (size_t)(p + u * g.PL) * g.C);
#pragma unroll
      for (int u = 0; u < GN_UNROLL; ++u) emit(v[u], p + u * g.PL);
    }
    for (; p < p1; p += g.PL) emit(*reinterpret_cast<const u32x4*>(xb + (size_t)p * g.C), p);
  }
}

// ---------------------------------------------------------------- NCHW
// grid (splits, N*G); row (n,g) is Cg*HW contiguous elements.
__global__ __launch_bounds__(GN_THREADS) void gn_stats_nchw(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ add_nc,
                                                            float* __restrict__ ws, long row_len, int splits, int G,
                                                            int Cg, int HW) {
  __shared__ float red[GN_THREADS / 64];
  const long row = blockIdx.y;
  const int split = blockIdx.x;
  const long chunks = row_len / 8;  // row_len % 8 == 0 is checked by the host
  const long per = (chunks + splits - 1) / splits;
  const long c0 = split * per, c1 = min(chunks, c0 + per);
  const bf16_t* xb = x + row * row_len;
  const long cbase = (row / G) * (long)G * Cg + (row % G) * Cg;  // n*C + g*Cg
  float s = 0.f, q = 0.f;
  for (long i = c0 + threadIdx.x; i < c1; i += GN_THREADS) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(xb + i * 8);
    const float ad = add_nc ? (float)add_nc[cbase + (i * 8) / HW] : 0.f;  // HW % 8 == 0: one channel per chunk
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float a = bf16_lo(v[e]) + ad, b = bf16_hi(v[e]) + ad;
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
                                                            const bf16_t* __restrict__ add_nc,
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
    const float ad = add_nc ? (float)add_nc[(row / G) * (long)G * Cg + c] : 0.f;
    const float sc = ga * rstd, sh = be + (ad - mean) * sc;
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
  // Statistics pass: every workgroup of the apply pass folds all of a sample's partial sums, so there should be
  // few of them: at most 64 workgroups per sample, each with 16 loads per thread in flight (as many bytes in
  // flight as four times the workgroups with four loads each), at least 32 pixels per workgroup.
  long s = HW / 32;
  if (s < 1) s = 1;
  const long cap = (256 + N - 1) / N;  // one workgroup per CU is enough at this depth
  if (s > cap) s = cap;
  if (s > 64) s = 64;
  return (int)s;
}
int gn_apply_splits_nhwc(long N, long HW) {
  // about 1024 workgroups in all (4 per CU: a latency-bound stream fills HBM by having more of itself in flight),
  // but at least 4 pixels each
  long per = (N * HW + 1023) / 1024;
  if (per < 4) per = 4;
  long s = (HW + per - 1) / per;
  if (s < 1) s = 1;
  if (s > 4096) s = 4096;
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

KH_EXPORT int kh_group_norm_bf16(const void* x, void* y, const void* gamma, const void* beta, const void* add_nc,
                                 float* workspace, int64_t N, int64_t C, int64_t HW, int64_t G, float eps, int activation,
                                 int channels_last, void* stream) {
  if (!x || !y || !workspace || N <= 0 || C <= 0 || HW <= 0 || G <= 0 || C % G != 0) return KH_ERR_INVALID_ARG;
  if (activation != 0 && activation != 1) return KH_ERR_INVALID_ARG;  // 0 = none, 1 = silu
  if (!kh_aligned16(x) || !kh_aligned16(y) || (gamma && !kh_aligned16(gamma)) || (beta && !kh_aligned16(beta)))
    return KH_ERR_ALIGNMENT;
  if (N > 65535) return KH_ERR_TOO_LARGE;
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* xp = (const bf16_t*)x; bf16_t* yp = (bf16_t*)y;
  const bf16_t* gp = (const bf16_t*)gamma; const bf16_t* bp = (const bf16_t*)beta;
  const bf16_t* ap = (const bf16_t*)add_nc;
  if (ap && !kh_aligned16(ap)) return KH_ERR_ALIGNMENT;
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
    if (g.CPT > GN_MAX_CPT) return KH_ERR_UNSUPPORTED;
    g.asplits = gn_apply_splits_nhwc(N, HW);
    dim3 grid((unsigned)g.splits, (unsigned)N), agrid((unsigned)g.asplits, (unsigned)N);
    const size_t lds = (size_t)2 * g.PL * g.C * sizeof(float);
    kh_launch(KH_TAG_GN_STATS, gn_stats_nhwc, grid, dim3(GN_THREADS), lds, s, xp, ap, workspace, g);
    if (activation == 1)
      kh_launch(KH_TAG_GN_APPLY, gn_apply_nhwc<true>, agrid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, ap, workspace, g, eps);
    else
      kh_launch(KH_TAG_GN_APPLY, gn_apply_nhwc<false>, agrid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, ap, workspace, g, eps);
  } else {
    const long Cg = C / G, row_len = Cg * HW, rows = N * G;
    if (HW % 8 != 0) return KH_ERR_UNSUPPORTED;
    if (rows > 65535) return KH_ERR_TOO_LARGE;
    const int splits = gn_splits_nchw(rows, row_len);
    dim3 grid((unsigned)splits, (unsigned)rows);
    kh_launch(KH_TAG_GN_STATS, gn_stats_nchw, grid, dim3(GN_THREADS), 0, s, xp, ap, workspace, row_len, splits, (int)G,
                       (int)Cg, (int)HW);
    if (activation == 1)
      kh_launch(KH_TAG_GN_APPLY, gn_apply_nchw<true>, grid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, ap, workspace, row_len,
                         splits, (int)G, (int)Cg, (int)HW, eps);
    else
      kh_launch(KH_TAG_GN_APPLY, gn_apply_nchw<false>, grid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, ap, workspace, row_len,
                         splits, (int)G, (int)Cg, (int)HW, eps);
  }
  KH_RETURN_LAST_ERROR();
}

// Second pass alone, on statistics some other kernel has left (kh_conv3x3_gn_stats_nhwc_bf16); see include/katz_hip.h.
KH_EXPORT int kh_group_norm_apply_bf16(const void* x, void* y, const void* gamma, const void* beta, const void* add_nc,
                                       const float* partials, int64_t splits, int64_t N, int64_t C, int64_t HW, int64_t G,
                                       float eps, int activation, void* stream) {
  if (!x || !y || !partials || splits <= 0 || N <= 0 || C <= 0 || HW <= 0 || G <= 0 || C % G != 0) return KH_ERR_INVALID_ARG;
  if (activation != 0 && activation != 1) return KH_ERR_INVALID_ARG;
  if (!kh_aligned16(x) || !kh_aligned16(y) || (gamma && !kh_aligned16(gamma)) || (beta && !kh_aligned16(beta)) ||
      (add_nc && !kh_aligned16(add_nc)) || ((uintptr_t)partials & 7) != 0)
    return KH_ERR_ALIGNMENT;
  if (N > 65535 || splits > (1 << 20)) return KH_ERR_TOO_LARGE;
  if (C % 8 != 0 || C > GN_MAX_C || G > 512) return KH_ERR_UNSUPPORTED;
  GnGeom g;
  g.N = (int)N; g.C = (int)C; g.HW = (int)HW; g.G = (int)G; g.Cg = (int)(C / G);
  g.splits = (int)splits;
  g.CP = (int)(C / 8);
  int ntx = g.CP < GN_THREADS ? g.CP : GN_THREADS;
  while (g.CP % ntx != 0) --ntx;
  g.NTX = ntx; g.CPT = g.CP / ntx; g.PL = GN_THREADS / ntx;
  if (g.CPT > GN_MAX_CPT) return KH_ERR_UNSUPPORTED;
  g.asplits = gn_apply_splits_nhwc(N, HW);
  const dim3 agrid((unsigned)g.asplits, (unsigned)N);
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* xp = (const bf16_t*)x; bf16_t* yp = (bf16_t*)y;
  const bf16_t* gp = (const bf16_t*)gamma; const bf16_t* bp = (const bf16_t*)beta; const bf16_t* ap = (const bf16_t*)add_nc;
  if (activation == 1)
    kh_launch(KH_TAG_GN_APPLY, gn_apply_nhwc<true>, agrid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, ap, partials, g, eps);
  else
    kh_launch(KH_TAG_GN_APPLY, gn_apply_nhwc<false>, agrid, dim3(GN_THREADS), 0, s, xp, yp, gp, bp, ap, partials, g, eps);
  KH_RETURN_LAST_ERROR();
}


// Device address of `scratch` on the current device, resolved once per device.
static int gn_static_workspace(float** out) {
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static float* ptr[MAX_DEV] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEV) return KH_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lk(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    ptr[dev] = (float*)p;
  }
  *out = ptr[dev];
  return KH_OK;
}

KH_EXPORT int kh_group_norm_static_bf16(const void* x, void* y, const void* gamma, const void* beta, const void* add_nc,
                                        int64_t N, int64_t C, int64_t HW, int64_t G, float eps, int activation,
                                        int channels_last, void* stream) {
  const int64_t need = kh_group_norm_workspace_bytes(N, C, HW, G, channels_last);
  if (need < 0) return (int)need;
  if ((uint64_t)need > GN_STATIC_WS_BYTES) return KH_ERR_TOO_LARGE;
  if (!x || !y) return KH_ERR_INVALID_ARG;   // before the first device call (the rest is checked by kh_group_norm_bf16)
  float* ws = nullptr;
  const int rc = gn_static_workspace(&ws);
  if (rc != KH_OK) return rc;
  // The statistics pass overwrites every partial sum the apply pass reads, so nothing has to start at zero.
  return kh_group_norm_bf16(x, y, gamma, beta, add_nc, ws, N, C, HW, G, eps, activation, channels_last, stream);
}

KH_EXPORT int kh_layer_norm_bf16(const void* x, void* y, const void* gamma, const void* beta, int64_t M, int64_t D,
                                 float eps, void* stream) {
  if (!x || !y || M <= 0 || D <= 0) return KH_ERR_INVALID_ARG;
  if (D % 8 != 0 || D > 64 * 8 * LN_MAXC) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(x) || !kh_aligned16(y) || (gamma && !kh_aligned16(gamma)) || (beta && !kh_aligned16(beta)))
    return KH_ERR_ALIGNMENT;
  const long blocks = (M + 3) / 4;
  if (blocks > 0x7fffffffL) return KH_ERR_TOO_LARGE;
  kh_launch(KH_TAG_LAYER_NORM, layer_norm_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,
                     (bf16_t*)y, (const bf16_t*)gamma, (const bf16_t*)beta, (long)M, (int)D, eps);
  KH_RETURN_LAST_ERROR();
}

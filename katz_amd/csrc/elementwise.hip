// K5 + ControlNet residual injection: HBM-bound elementwise kernels for gfx950, 16 bytes per lane.
//
// * kh_geglu_bf16: out = value * gelu(gate) with [value | gate] = proj(x) split along the last
//   axis (diffusers-hf/src/diffusers/models/activations.py:139-149; erf-exact F.gelu by default).
// * kh_gelu_mul_bf16: out = gelu(x) * m, the two-tensor form of the reference's fused op
//   torch.ops.fast_kernel.fast_gelu_mul_fp16 (diffusers-hf/src/fast_kernel/fast_kernel/csrc/gelu.cuh:29-59,
//   tanh approximation 0.5*x*(1+tanh(0.79788456*(x+0.044715*x^3)))).
// * kh_residual_add_bf16: dst += (sum_k src_k) * inv_k -- the ControlNet residual injection
//   skip_j + r_j / sample + r_mid (diffusers-hf/src/diffusers/models/unets/unet_2d_condition.py:1284-1292)
//   including the multi-ControlNet sum-then-mean (:1418-1439).
// * kh_concat_residual_bf16: out[..., :C1] = h, out[..., C1:] = skip + (sum_k r_k) * inv_k over
//   channels-last rows: the up-block torch.cat([hidden, skip], dim=1) is a copy anyway, so the
//   residual add rides on it for free.
// * kh_cfg_euler_step_bf16: classifier-free guidance + one Euler step + the next step's input scaling in one
//   pass (diffusers-hf/src/diffusers/pipelines/controlnet/pipeline_controlnet_sd_xl_katz.py:1565-1570,
//   :1647-1658; diffusers-hf/src/diffusers/schedulers/scheduling_euler_discrete.py:274-298, :435-545).
#include "kh_common.h"

namespace {

constexpr int EW_THREADS = 256;
constexpr int KH_MAX_SRCS = 8;

__device__ __forceinline__ float gelu_erf_f(float x) { return kh_gelu_erf(x); }
__device__ __forceinline__ float gelu_tanh_f(float x) {
  return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}
// gelu is rounded to bf16 before the product, as the reference's separate gelu and mul ops do
template <bool TANH>
__device__ __forceinline__ uint32_t geglu_pair(uint32_t val, uint32_t gate) {
  const float g0 = bf16_lo(gate), g1 = bf16_hi(gate);
  const float a0 = TANH ? gelu_tanh_f(g0) : gelu_erf_f(g0);
  const float a1 = TANH ? gelu_tanh_f(g1) : gelu_erf_f(g1);
  const uint32_t ar = pack_bf16x2(a0, a1);
  return pack_bf16x2(bf16_lo(val) * bf16_lo(ar), bf16_hi(val) * bf16_hi(ar));
}

template <bool TANH>
__global__ __launch_bounds__(EW_THREADS) void geglu_kernel(const bf16_t* __restrict__ proj, bf16_t* __restrict__ out,
                                                           long M, int D) {
  const int cpr = D / 8;
  const long total = M * cpr;
  for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < total; i += (long)gridDim.x * EW_THREADS) {
    const long row = i / cpr;
    const int c = (int)(i % cpr) * 8;
    const u32x4 hv = *reinterpret_cast<const u32x4*>(proj + row * 2 * D + c);
    const u32x4 gv = *reinterpret_cast<const u32x4*>(proj + row * 2 * D + D + c);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = geglu_pair<TANH>(hv[e], gv[e]);
    *reinterpret_cast<u32x4*>(out + row * D + c) = o;
  }
}

template <bool TANH>
__global__ __launch_bounds__(EW_THREADS) void gelu_mul_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ m,
                                                              bf16_t* __restrict__ out, long n) {
  const long chunks = n / 8;
  for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < chunks; i += (long)gridDim.x * EW_THREADS) {
    const u32x4 xv = *reinterpret_cast<const u32x4*>(x + i * 8);
    const u32x4 mv = *reinterpret_cast<const u32x4*>(m + i * 8);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = geglu_pair<TANH>(mv[e], xv[e]);
    *reinterpret_cast<u32x4*>(out + i * 8) = o;
  }
  // tail (n % 8 elements)
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    for (long j = chunks * 8; j < n; ++j) {
      const float g = (float)x[j];
      const float a = (float)(bf16_t)(TANH ? gelu_tanh_f(g) : gelu_erf_f(g));
      out[j] = (bf16_t)((float)m[j] * a);
    }
  }
}

struct SrcList {
  const bf16_t* p[KH_MAX_SRCS];
  int n;
  float inv;
};

__device__ __forceinline__ void accumulate_srcs(const SrcList& s, long off, float (&acc)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int k = 0; k < s.n; ++k) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(s.p[k] + off);
#pragma unroll
    for (int e = 0; e < 4; ++e) { acc[2 * e] += bf16_lo(v[e]); acc[2 * e + 1] += bf16_hi(v[e]); }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] *= s.inv;
}

__global__ __launch_bounds__(EW_THREADS) void residual_add_kernel(bf16_t* __restrict__ dst, const SrcList s, long n) {
  const long chunks = n / 8;
  for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < chunks; i += (long)gridDim.x * EW_THREADS) {
    float acc[8];
    accumulate_srcs(s, i * 8, acc);
    const u32x4 d = *reinterpret_cast<const u32x4*>(dst + i * 8);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(bf16_lo(d[e]) + acc[2 * e], bf16_hi(d[e]) + acc[2 * e + 1]);
    *reinterpret_cast<u32x4*>(dst + i * 8) = o;
  }
}

// rows = N*HW pixels; out row = [h row (C1) | skip row (C2) + residual]
__global__ __launch_bounds__(EW_THREADS) void concat_residual_kernel(const bf16_t* __restrict__ h,
                                                                     const bf16_t* __restrict__ skip, const SrcList s,
                                                                     bf16_t* __restrict__ out, long rows, int C1,
                                                                     int C2) {
  const int cp1 = C1 / 8, cp = (C1 + C2) / 8;
  const long total = rows * cp;
  const KhOut yout(out, (size_t)rows * (C1 + C2) * 2);
  for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < total; i += (long)gridDim.x * EW_THREADS) {
    const long row = i / cp;
    const int c = (int)(i % cp);
    u32x4 o;
    if (c < cp1) {
      o = *reinterpret_cast<const u32x4*>(h + row * C1 + c * 8);
    } else {
      const long off = row * C2 + (long)(c - cp1) * 8;
      o = *reinterpret_cast<const u32x4*>(skip + off);
      if (s.n > 0) {
        float acc[8];
        accumulate_srcs(s, off, acc);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(bf16_lo(o[e]) + acc[2 * e], bf16_hi(o[e]) + acc[2 * e + 1]);
      }
    }
    yout.store16((size_t)(row * (C1 + C2) + c * 8) * 2, o);
  }
}

// nearest-neighbour 2x upsampling, NHWC: out pixel (h, w) = in pixel (h / 2, w / 2); one 16-byte channel chunk per item
__global__ __launch_bounds__(EW_THREADS) void upsample2x_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ y,
                                                                int N, int H, int W, int C) {
  const int cp = C / 8, W2 = 2 * W, H2 = 2 * H;
  const long total = (long)N * H2 * W2 * cp;
  for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < total; i += (long)gridDim.x * EW_THREADS) {
    const int c = (int)(i % cp);
    long p = i / cp;
    const int w = (int)(p % W2); p /= W2;
    const int h = (int)(p % H2);
    const long n = p / H2;
    const u32x4 v = *reinterpret_cast<const u32x4*>(x + ((n * H + (h >> 1)) * W + (w >> 1)) * C + c * 8);
    *reinterpret_cast<u32x4*>(y + i * 8) = v;
  }
}

unsigned ew_grid(long work_items) {
  long b = (work_items + EW_THREADS - 1) / EW_THREADS;
  const long cap = 256L * 16;  // 16 workgroups per CU, grid-stride beyond that
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return (unsigned)b;
}

int fill_srcs(SrcList& s, const void* const* srcs, int n_srcs, float inv) {
  if (n_srcs < 0 || n_srcs > KH_MAX_SRCS) return KH_ERR_TOO_LARGE;
  s.n = n_srcs; s.inv = inv;
  for (int k = 0; k < KH_MAX_SRCS; ++k) s.p[k] = nullptr;
  for (int k = 0; k < n_srcs; ++k) {
    if (!srcs || !srcs[k]) return KH_ERR_INVALID_ARG;
    if (!kh_aligned16(srcs[k])) return KH_ERR_ALIGNMENT;
    s.p[k] = (const bf16_t*)srcs[k];
  }
  return KH_OK;
}

}  // namespace

namespace {

// One thread: 8 latent elements.  Arithmetic in fp32 in the reference's order (epsilon prediction, no churn):
//   eps = u + g*(t - u); x0 = x - sigma*eps; d = (x - x0)/sigma; x' = x + d*(sigma_next - sigma).
template <bool LAT_F32>
// lat_out may be lat_in (a thread reads its eight elements before it writes them): no __restrict__ on the two.
__global__ __launch_bounds__(EW_THREADS) void cfg_euler_kernel(const bf16_t* __restrict__ noise, const void* lat_in,
                                                               void* lat_out, bf16_t* __restrict__ next_in,
                                                               long n, float g, const float* __restrict__ coef) {
  const float sigma = coef[0], dt = coef[1] - coef[0], den = coef[2];
  const long chunks = n / 8;
  for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < chunks; i += (long)gridDim.x * EW_THREADS) {
    const u32x4 uv = *reinterpret_cast<const u32x4*>(noise + i * 8);
    const u32x4 tv = *reinterpret_cast<const u32x4*>(noise + n + i * 8);
    float x[8];
    if (LAT_F32) {
      const float* p = reinterpret_cast<const float*>(lat_in) + i * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = p[e];
    } else {
      const u32x4 xv = *reinterpret_cast<const u32x4*>(reinterpret_cast<const bf16_t*>(lat_in) + i * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[2 * e] = bf16_lo(xv[e]); x[2 * e + 1] = bf16_hi(xv[e]); }
    }
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float u = (e & 1) ? bf16_hi(uv[e >> 1]) : bf16_lo(uv[e >> 1]);
      const float t = (e & 1) ? bf16_hi(tv[e >> 1]) : bf16_lo(tv[e >> 1]);
      const float eps = __fadd_rn(u, __fmul_rn(g, __fsub_rn(t, u)));
      const float x0 = __fsub_rn(x[e], __fmul_rn(sigma, eps));
      const float d = __fdiv_rn(__fsub_rn(x[e], x0), sigma);
      y[e] = __fadd_rn(x[e], __fmul_rn(d, dt));
    }
    u32x4 yo;
#pragma unroll
    for (int e = 0; e < 4; ++e) yo[e] = pack_bf16x2(y[2 * e], y[2 * e + 1]);
    if (LAT_F32) {
      float* p = reinterpret_cast<float*>(lat_out) + i * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) p[e] = y[e];
    } else {
      *reinterpret_cast<u32x4*>(reinterpret_cast<bf16_t*>(lat_out) + i * 8) = yo;
#pragma unroll
      for (int e = 0; e < 4; ++e) { y[2 * e] = bf16_lo(yo[e]); y[2 * e + 1] = bf16_hi(yo[e]); }  // the stored, rounded latents
    }
    if (next_in != nullptr) {
      u32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(__fdiv_rn(y[2 * e], den), __fdiv_rn(y[2 * e + 1], den));
      *reinterpret_cast<u32x4*>(next_in + i * 8) = o;
      *reinterpret_cast<u32x4*>(next_in + n + i * 8) = o;
    }
  }
}

}  // namespace

KH_EXPORT int kh_cfg_euler_step_bf16(const void* noise_pred, const void* latents, void* latents_out, void* model_input_next,
                                     int64_t n, float guidance_scale, const float* coef, int latents_f32, void* stream) {
  if (!noise_pred || !latents || !latents_out || !coef || n <= 0) return KH_ERR_INVALID_ARG;
  if (n % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(noise_pred) || !kh_aligned16(latents) || !kh_aligned16(latents_out) ||
      (model_input_next && !kh_aligned16(model_input_next)) || (n * 2) % 16 != 0)
    return KH_ERR_ALIGNMENT;
  const long chunks = n / 8;
  const unsigned grid = (unsigned)((chunks + EW_THREADS - 1) / EW_THREADS < 4096 ? (chunks + EW_THREADS - 1) / EW_THREADS : 4096);
  if (latents_f32)
    kh_launch(KH_TAG_CFG_EULER, cfg_euler_kernel<true>, dim3(grid), dim3(EW_THREADS), 0, (hipStream_t)stream,
              (const bf16_t*)noise_pred, latents, latents_out, (bf16_t*)model_input_next, (long)n, guidance_scale, coef);
  else
    kh_launch(KH_TAG_CFG_EULER, cfg_euler_kernel<false>, dim3(grid), dim3(EW_THREADS), 0, (hipStream_t)stream,
              (const bf16_t*)noise_pred, latents, latents_out, (bf16_t*)model_input_next, (long)n, guidance_scale, coef);
  KH_RETURN_LAST_ERROR();
}

KH_EXPORT int kh_geglu_bf16(const void* proj, void* out, int64_t M, int64_t D, int approximate_tanh, void* stream) {
  if (!proj || !out || M <= 0 || D <= 0) return KH_ERR_INVALID_ARG;
  if (D % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(proj) || !kh_aligned16(out)) return KH_ERR_ALIGNMENT;
  const unsigned grid = ew_grid(M * (D / 8));
  if (approximate_tanh)
    kh_launch(KH_TAG_GEGLU, geglu_kernel<true>, dim3(grid), dim3(EW_THREADS), 0, (hipStream_t)stream, (const bf16_t*)proj,
                       (bf16_t*)out, (long)M, (int)D);
  else
    kh_launch(KH_TAG_GEGLU, geglu_kernel<false>, dim3(grid), dim3(EW_THREADS), 0, (hipStream_t)stream, (const bf16_t*)proj,
                       (bf16_t*)out, (long)M, (int)D);
  KH_RETURN_LAST_ERROR();
}

KH_EXPORT int kh_gelu_mul_bf16(const void* x, const void* m, void* out, int64_t n, int approximate_tanh, void* stream) {
  if (!x || !m || !out || n <= 0) return KH_ERR_INVALID_ARG;
  if (!kh_aligned16(x) || !kh_aligned16(m) || !kh_aligned16(out)) return KH_ERR_ALIGNMENT;
  const unsigned grid = ew_grid(n / 8 + 1);
  if (approximate_tanh)
    kh_launch(KH_TAG_GEGLU, gelu_mul_kernel<true>, dim3(grid), dim3(EW_THREADS), 0, (hipStream_t)stream, (const bf16_t*)x,
                       (const bf16_t*)m, (bf16_t*)out, (long)n);
  else
    kh_launch(KH_TAG_GEGLU, gelu_mul_kernel<false>, dim3(grid), dim3(EW_THREADS), 0, (hipStream_t)stream, (const bf16_t*)x,
                       (const bf16_t*)m, (bf16_t*)out, (long)n);
  KH_RETURN_LAST_ERROR();
}

KH_EXPORT int kh_residual_add_bf16(void* dst, const void* const* srcs, int n_srcs, float inv_count, int64_t n,
                                   void* stream) {
  if (!dst || n <= 0 || n_srcs <= 0) return KH_ERR_INVALID_ARG;
  if (n % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(dst)) return KH_ERR_ALIGNMENT;
  SrcList s;
  const int rc = fill_srcs(s, srcs, n_srcs, inv_count);
  if (rc != KH_OK) return rc;
  kh_launch(KH_TAG_RESIDUAL_ADD, residual_add_kernel, dim3(ew_grid(n / 8)), dim3(EW_THREADS), 0, (hipStream_t)stream,
                     (bf16_t*)dst, s, (long)n);
  KH_RETURN_LAST_ERROR();
}

KH_EXPORT int kh_concat_residual_bf16(const void* h, const void* skip, const void* const* residuals, int n_residuals,
                                      float inv_count, void* out, int64_t rows, int64_t C1, int64_t C2, void* stream) {
  if (!h || !skip || !out || rows <= 0 || C1 <= 0 || C2 <= 0) return KH_ERR_INVALID_ARG;
  if (C1 % 8 != 0 || C2 % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(h) || !kh_aligned16(skip) || !kh_aligned16(out)) return KH_ERR_ALIGNMENT;
  SrcList s;
  const int rc = fill_srcs(s, residuals, n_residuals, inv_count);
  if (rc != KH_OK) return rc;
  kh_launch(KH_TAG_CONCAT_RESIDUAL, concat_residual_kernel, dim3(ew_grid(rows * ((C1 + C2) / 8))), dim3(EW_THREADS), 0,
                     (hipStream_t)stream, (const bf16_t*)h, (const bf16_t*)skip, s, (bf16_t*)out, (long)rows, (int)C1,
                     (int)C2);
  KH_RETURN_LAST_ERROR();
}

// Upsample2D's interpolation, see include/katz_hip.h.
KH_EXPORT int kh_upsample_nearest2x_nhwc_bf16(const void* x, void* y, int64_t N, int64_t H, int64_t W, int64_t C, void* stream) {
  if (!x || !y || N <= 0 || H <= 0 || W <= 0 || C <= 0) return KH_ERR_INVALID_ARG;
  if (C % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (N > (1 << 20) || H > (1 << 14) || W > (1 << 14) || C > (1 << 20)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || !kh_aligned16(y)) return KH_ERR_ALIGNMENT;
  kh_launch(KH_TAG_UPSAMPLE, upsample2x_kernel, dim3(ew_grid(N * 4 * H * W * (C / 8))), dim3(EW_THREADS), 0, (hipStream_t)stream,
            (const bf16_t*)x, (bf16_t*)y, (int)N, (int)H, (int)W, (int)C);
  KH_RETURN_LAST_ERROR();
}

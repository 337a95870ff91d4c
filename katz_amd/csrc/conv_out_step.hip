// The UNet's last convolution with classifier-free guidance and the Euler step in its epilogue (gfx950).
//
//   noise[b] = conv3x3(x[b], W, bias)                     b = uncond row, text row     (conv_out, diffusers-hf/src/diffusers/
//                                                          models/unets/unet_2d_condition.py:1327-1331, 4 output channels)
//   eps = u + g (t - u)                                    pipeline_controlnet_sd_xl_katz.py:1649-1650
//   x0 = lat - sigma eps; d = (lat - x0) / sigma; lat' = lat + d (sigma_next - sigma)
//                                                          scheduling_euler_discrete.py:505-527 (epsilon prediction, no churn)
//   next_input = [lat'; lat'] / sqrt(sigma_next^2 + 1)     pipeline :1565-1570, scale_model_input :274-298
//
// The reference runs these as a cuDNN convolution, three elementwise kernels and the scheduler's tensor ops.  Here one
// workgroup owns one image row segment of up to 64 pixels for BOTH rows of a guidance pair, so the two convolution
// results of a pixel meet in its LDS and the latent update is the epilogue of the convolution:
//   * 4 waves = 2 batch rows x 2 segments of 32 pixels; implicit GEMM on the 32x32x16 bf16 MFMA with the 4 output
//     channels in columns 0..3 of the B operand (the other 28 columns multiply zeros: 4 GFLOP of matrix-core time for
//     0.75 GFLOP of arithmetic, cheaper than any vector-ALU formulation);
//   * the input patch (3 image rows x 66 pixels, halo included) is staged through LDS in phases of up to 80 input
//     channels with 16-byte coalesced loads, so every input element is read from memory by 3 workgroups, not 9 taps;
//   * noise is rounded to bf16 as the model's output dtype before the guidance, then the fp32 arithmetic of
//     kh_cfg_euler_step_bf16 in the same order (identical results given identical noise).
#include "kh_common.h"

namespace {

constexpr int CO_THREADS = 256;
constexpr int CO_SEG = 64;                  // pixels per workgroup (2 waves x 32 per batch row)
constexpr int CO_PW = CO_SEG + 2;           // patch width with the halo
constexpr int CO_MAXPH = 80;                // input channels per phase
constexpr int CO_NOUT = 4;                  // latent channels

struct ConvOutParams {
  const bf16_t* x;        // [2*Bl, H, W, Cin] NHWC
  const bf16_t* w;        // [4, 3, 3, Cin]
  const bf16_t* bias;     // [4] or null
  const void* lat_in; void* lat_out;   // [Bl, H, W, 4] bf16 or fp32
  bf16_t* next_in;        // [2*Bl, H, W, 4] or null
  bf16_t* noise_out;      // [2*Bl, H, W, 4] or null
  const float* coef;      // {sigma, sigma_next, next_scale}
  float g;
  int Bl, H, W, Cin, ph;  // ph: channels per phase (multiple of 16, divides Cin)
};

template <int PH, bool LAT_F32>   // PH: input channels per phase
__global__ __launch_bounds__(CO_THREADS) void conv_out_step_kernel(const ConvOutParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int ph = PH, ldp = ph + 8;                     // patch pixel stride (elements): 16-byte aligned, odd multiple of 16 B
  bf16_t* sX = reinterpret_cast<bf16_t*>(smem);            // [2][3][CO_PW][ldp]
  bf16_t* sW = sX + 2 * 3 * CO_PW * ldp;                   // [4][9][ldp]   this phase's weights
  float* sO = reinterpret_cast<float*>(sW + CO_NOUT * 9 * ldp);   // [2][CO_SEG][4] convolution results
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const int wb = wave >> 1, ws = wave & 1;                 // batch row of the pair, 32-pixel segment
  // Workgroups go round-robin to the 8 XCDs; remapped so that every XCD owns a band of consecutive image rows and
  // the halo rows two neighbouring workgroups share are found in that XCD's L2.
  const uint32_t gx = gridDim.x;
  const uint32_t logical = xcd_remap(blockIdx.y * gx + blockIdx.x, gx * gridDim.y);
  const int x0 = (int)(logical % gx) * CO_SEG, y = (int)(logical / gx), z = blockIdx.z;
  const int brow[2] = {z, p.Bl + z};                       // uncond row, text row
  const int H = p.H, W = p.W, Cin = p.Cin;

  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;

  constexpr int cpp = ph / 8;                              // 16-byte pieces per pixel and phase
  constexpr int pieces = 2 * 3 * CO_PW * cpp;
  constexpr int LB = 4;                                    // loads in flight per thread
  for (int c0 = 0; c0 < Cin; c0 += ph) {
    __syncthreads();                                       // the previous phase's fragments have been read
    // stage the patch: rows y-1..y+1, pixels x0-1..x0+64, channels c0..c0+ph of both batch rows; zeros outside the image
    for (int i0 = tid; i0 < pieces; i0 += CO_THREADS * LB) {
      u32x4 v[LB];
      int dst[LB];
#pragma unroll
      for (int u = 0; u < LB; ++u) {
        const int i = i0 + u * CO_THREADS;
        const int pc = i % cpp, px = (i / cpp) % CO_PW, r = (i / (cpp * CO_PW)) % 3, b = i / (cpp * CO_PW * 3);
        const int gy = y + r - 1, gx = x0 + px - 1;
        v[u] = u32x4{0, 0, 0, 0};
        dst[u] = i < pieces ? ((b * 3 + r) * CO_PW + px) * ldp + pc * 8 : -1;
        if (i < pieces && gy >= 0 && gy < H && gx >= 0 && gx < W)
          v[u] = *reinterpret_cast<const u32x4*>(p.x + (((size_t)brow[b] * H + gy) * W + gx) * Cin + c0 + pc * 8);
      }
#pragma unroll
      for (int u = 0; u < LB; ++u)
        if (dst[u] >= 0) *reinterpret_cast<u32x4*>(sX + dst[u]) = v[u];
    }
    for (int i = tid; i < CO_NOUT * 9 * cpp; i += CO_THREADS) {
      const int pc = i % cpp, tap = (i / cpp) % 9, co = i / (cpp * 9);
      *reinterpret_cast<u32x4*>(sW + (co * 9 + tap) * ldp + pc * 8) =
          *reinterpret_cast<const u32x4*>(p.w + ((size_t)co * 9 + tap) * Cin + c0 + pc * 8);
    }
    __syncthreads();
    // implicit GEMM: rows = this wave's 32 pixels, columns 0..3 = output channels, K = 9 taps x ph channels
    for (int tap = 0; tap < 9; ++tap) {
      const int dy = tap / 3, dx = tap % 3;
      const bf16_t* xa = sX + ((wb * 3 + dy) * CO_PW + ws * 32 + l32 + dx) * ldp + lh * 8;
      const bf16_t* wa = sW + ((l32 & 3) * 9 + tap) * ldp + lh * 8;
      for (int k = 0; k < ph; k += 16) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(xa + k);
        bf16x8 b = *reinterpret_cast<const bf16x8*>(wa + k);
        if (l32 >= CO_NOUT) b = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
      }
    }
  }
  // acc[v]: pixel = 8*(v/4) + 4*lh + v%4 of the wave's segment, output channel = l32 (valid below 4)
  if (l32 < CO_NOUT) {
    const float bv = p.bias ? (float)p.bias[l32] : 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int px = ws * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
      sO[(wb * CO_SEG + px) * CO_NOUT + l32] = acc[v] + bv;
    }
  }
  __syncthreads();
  // guidance + Euler for the segment's pixels: one thread per (pixel, channel)
  const float sigma = p.coef[0], dt = p.coef[1] - p.coef[0], den = p.coef[2];
  const size_t n = (size_t)H * W * CO_NOUT;                // elements per latent
  for (int i = tid; i < CO_SEG * CO_NOUT; i += CO_THREADS) {
    const int px = i / CO_NOUT, co = i % CO_NOUT;
    if (x0 + px >= W) continue;
    const size_t e = ((size_t)y * W + x0 + px) * CO_NOUT + co;        // element inside one latent
    const bf16_t ub = (bf16_t)sO[px * CO_NOUT + co], tb = (bf16_t)sO[(CO_SEG + px) * CO_NOUT + co];
    if (p.noise_out) {
      p.noise_out[(size_t)brow[0] * n + e] = ub;
      p.noise_out[(size_t)brow[1] * n + e] = tb;
    }
    const float u = (float)ub, t = (float)tb;
    const float xin = LAT_F32 ? reinterpret_cast<const float*>(p.lat_in)[(size_t)z * n + e]
                              : (float)reinterpret_cast<const bf16_t*>(p.lat_in)[(size_t)z * n + e];
    const float eps = __fadd_rn(u, __fmul_rn(p.g, __fsub_rn(t, u)));
    const float xz = __fsub_rn(xin, __fmul_rn(sigma, eps));
    const float d = __fdiv_rn(__fsub_rn(xin, xz), sigma);
    float yv = __fadd_rn(xin, __fmul_rn(d, dt));
    if (LAT_F32) {
      reinterpret_cast<float*>(p.lat_out)[(size_t)z * n + e] = yv;
    } else {
      const bf16_t yb = (bf16_t)yv;
      reinterpret_cast<bf16_t*>(p.lat_out)[(size_t)z * n + e] = yb;
      yv = (float)yb;                                      // the stored, rounded latents feed the next input
    }
    if (p.next_in) {
      const bf16_t o = (bf16_t)__fdiv_rn(yv, den);
      p.next_in[(size_t)brow[0] * n + e] = o;
      p.next_in[(size_t)brow[1] * n + e] = o;
    }
  }
}

constexpr int co_lds_bytes(int ph) {
  const int ldp = ph + 8;
  return (2 * 3 * CO_PW * ldp + CO_NOUT * 9 * ldp) * 2 + 2 * CO_SEG * CO_NOUT * 4;
}

}  // namespace

// See include/katz_hip.h.
KH_EXPORT int kh_conv_out_cfg_euler_bf16(const void* x, const void* w, const void* bias, const void* latents,
                                         void* latents_out, void* model_input_next, void* noise_pred_out, int64_t Bl,
                                         int64_t H, int64_t W, int64_t Cin, float guidance_scale, const float* coef,
                                         int latents_f32, void* stream) {
  if (!x || !w || !latents || !latents_out || !coef || Bl <= 0 || H <= 0 || W <= 0 || Cin <= 0) return KH_ERR_INVALID_ARG;
  if (Cin % 16 != 0) return KH_ERR_UNSUPPORTED;
  if (Bl > 65535 || H > 65535 || W > (1 << 20) || Cin > (1 << 16)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || !kh_aligned16(w) || !kh_aligned16(latents) || !kh_aligned16(latents_out) ||
      (model_input_next && !kh_aligned16(model_input_next)) || (noise_pred_out && !kh_aligned16(noise_pred_out)))
    return KH_ERR_ALIGNMENT;
  ConvOutParams p;
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = (const bf16_t*)bias;
  p.lat_in = latents; p.lat_out = latents_out; p.next_in = (bf16_t*)model_input_next; p.noise_out = (bf16_t*)noise_pred_out;
  p.coef = coef; p.g = guidance_scale;
  p.Bl = (int)Bl; p.H = (int)H; p.W = (int)W; p.Cin = (int)Cin;
  int ph = 16;   // the largest multiple of 16 up to CO_MAXPH that divides Cin
  for (int c = CO_MAXPH; c >= 16; c -= 16)
    if (Cin % c == 0) { ph = c; break; }
  p.ph = ph;
  dim3 grid((unsigned)((W + CO_SEG - 1) / CO_SEG), (unsigned)H, (unsigned)Bl);
  hipStream_t s = (hipStream_t)stream;
#define KH_CO(PH)                                                                                                      \
  case PH: {                                                                                                           \
    constexpr int lds = co_lds_bytes(PH);                                                                              \
    if (latents_f32) {                                                                                                 \
      if (hipError_t e = kh_allow_lds<conv_out_step_kernel<PH, true>>(lds); e != hipSuccess) return (int)e;            \
      kh_launch(KH_TAG_CONV_OUT_STEP, conv_out_step_kernel<PH, true>, grid, dim3(CO_THREADS), (size_t)lds, s, p);      \
    } else {                                                                                                           \
      if (hipError_t e = kh_allow_lds<conv_out_step_kernel<PH, false>>(lds); e != hipSuccess) return (int)e;           \
      kh_launch(KH_TAG_CONV_OUT_STEP, conv_out_step_kernel<PH, false>, grid, dim3(CO_THREADS), (size_t)lds, s, p);     \
    }                                                                                                                  \
    break;                                                                                                             \
  }
  switch (ph) {
    KH_CO(80) KH_CO(64) KH_CO(48) KH_CO(32) KH_CO(16)
    default: return KH_ERR_UNSUPPORTED;
  }
#undef KH_CO
  KH_RETURN_LAST_ERROR();
}

// K1: fused base GEMM + low-rank (LoRA) delta on bf16 MFMA for gfx950.
//
//   y[M,N] = x[M,K] . W[N,K]^T + bias[N] + ((x . A_cat[R,K]^T) * col_scale[R]) . B_cat[N,R]^T (+ residual[M,N])
//
// A_cat / B_cat are the active adapters concatenated along the rank axis, so a
// sum over adapters is one rank-R product; col_scale carries s_i * alpha_i / r_i
// for every rank column of adapter i.  This is the closed form of the
// reference's LoRA-patched Linear (diffusers-hf/src/diffusers/models/lora.py:222-232
// for the low-rank branch, :451-457 for base + scale * delta).
//
// The rank-R intermediate T = x . A_cat^T is accumulated by extra MFMAs inside
// the base GEMM's K loop (the x tile is already in LDS), scaled, rounded to
// bf16 and parked in LDS; the expand product T . B_cat^T is then accumulated
// into the same fp32 accumulators as the base GEMM before the epilogue.  T
// never goes to HBM.  One workgroup walks several N tiles of the same M block
// so that T is computed once per chunk of N tiles rather than once per tile.
#include "kh_common.h"
#include "lora_gemm.h"

namespace {

constexpr int BK = 64;       // K slab per LDS stage (bf16 elements)
constexpr int LDK = BK + 8;  // padded LDS row: 144 B, so the 16 rows one ds_read_b128 phase touches hit 16 distinct bank groups


template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int NRT_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NRT = NRT_;
  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NT = NW * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int R = NRT * 32;
  static constexpr int SM = (NRT > 0) ? TM / WAVES_N : 0;  // shrink m-tiles per wave
  static constexpr int LDT = R + 8;                        // padded row of the T / B_cat tiles
  static constexpr int LDC = BN + 8;                       // padded row of the epilogue staging tile
  static constexpr int XCH = BM * 8 / NT, WCH = BN * 8 / NT, ACH = R * 8 / NT;
  static constexpr size_t SX = (size_t)BM * LDK * 2, SW = (size_t)BN * LDK * 2, SA = (size_t)R * LDK * 2;
  static constexpr size_t SB = (size_t)BN * LDT * 2;
  static constexpr size_t SC = (size_t)WAVES_M * 32 * LDC * 2;
  static constexpr size_t STAGE = SX + SW + SA;
  static constexpr size_t STAGE_MAX = STAGE > SB ? (STAGE > SC ? STAGE : SC) : (SB > SC ? SB : SC);
  static constexpr size_t ST = (NRT > 0) ? (size_t)BM * LDT * 2 : 0;
  static constexpr size_t LDS_BYTES = STAGE_MAX + ST;
  static_assert(BM % (32 * WAVES_M) == 0 && BN % (32 * WAVES_N) == 0, "tile/wave mismatch");
  static_assert(NRT == 0 || (TM % WAVES_N == 0), "shrink tiles must split evenly over the waves of a row");
  static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0 && (R * 8) % NT == 0, "load split");
};

__device__ __forceinline__ u32x4 ld16(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ bf16x8 lds_frag(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <class C>
__global__ __launch_bounds__(C::NT) void lora_gemm_kernel(const LoraGemmParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int BM = C::BM, BN = C::BN, TM = C::TM, TN = C::TN, NRT = C::NRT, R = C::R;
  constexpr int SMT = C::SM > 0 ? C::SM : 1, NRTT = NRT > 0 ? NRT : 1;
  bf16_t* sX = reinterpret_cast<bf16_t*>(smem);
  bf16_t* sW = reinterpret_cast<bf16_t*>(smem + C::SX);
  bf16_t* sA = reinterpret_cast<bf16_t*>(smem + C::SX + C::SW);
  bf16_t* sB = reinterpret_cast<bf16_t*>(smem);                 // aliases the K-loop stage
  bf16_t* sC = reinterpret_cast<bf16_t*>(smem);                 // aliases the K-loop stage
  bf16_t* sT = reinterpret_cast<bf16_t*>(smem + C::STAGE_MAX);  // lives across N tiles

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / C::WAVES_N, wn = wave % C::WAVES_N;
  const int l32 = lane & 31, lh = lane >> 5;

  const uint32_t total = (uint32_t)p.m_tiles * (uint32_t)p.n_chunks;
  const uint32_t logical = xcd_remap(blockIdx.x, total);
  const int m_blk = logical / p.n_chunks, chunk = logical % p.n_chunks;
  const int m0 = m_blk * BM;
  const int K = p.K, M = p.M, N = p.N;
  const int KT = (K + BK - 1) / BK;

  for (int jt = 0; jt < p.n_chunk; ++jt) {
    const int n_tile = chunk * p.n_chunk + jt;
    if (n_tile >= p.n_tiles) break;  // uniform over the workgroup
    const int n0 = n_tile * BN;
    const bool shrink = (NRT > 0) && (jt == 0);

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

    u32x4 rx[C::XCH], rw[C::WCH], ra[C::ACH > 0 ? C::ACH : 1];

    auto load_tile = [&](int kt) {
      const int k0 = kt * BK;
#pragma unroll
      for (int q = 0; q < C::XCH; ++q) {
        const int c = tid + q * C::NT, row = c >> 3, ch = c & 7;
        const int gk = k0 + ch * 8;
        int gr = m0 + row; gr = gr < M ? gr : M - 1;
        rx[q] = (gk < K) ? ld16(p.x + (size_t)gr * K + gk) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int q = 0; q < C::WCH; ++q) {
        const int c = tid + q * C::NT, row = c >> 3, ch = c & 7;
        const int gk = k0 + ch * 8;
        int gr = n0 + row; gr = gr < N ? gr : N - 1;
        rw[q] = (gk < K) ? ld16(p.w + (size_t)gr * K + gk) : u32x4{0, 0, 0, 0};
      }
      if constexpr (NRT > 0) {
        if (shrink) {
#pragma unroll
          for (int q = 0; q < C::ACH; ++q) {
            const int c = tid + q * C::NT, row = c >> 3, ch = c & 7;
            const int gk = k0 + ch * 8;
            ra[q] = (gk < K) ? ld16(p.a_cat + (size_t)row * K + gk) : u32x4{0, 0, 0, 0};
          }
        }
      }
    };
    auto store_tile = [&]() {
#pragma unroll
      for (int q = 0; q < C::XCH; ++q) {
        const int c = tid + q * C::NT, row = c >> 3, ch = c & 7;
        *reinterpret_cast<u32x4*>(sX + row * LDK + ch * 8) = rx[q];
      }
#pragma unroll
      for (int q = 0; q < C::WCH; ++q) {
        const int c = tid + q * C::NT, row = c >> 3, ch = c & 7;
        *reinterpret_cast<u32x4*>(sW + row * LDK + ch * 8) = rw[q];
      }
      if constexpr (NRT > 0) {
        if (shrink) {
#pragma unroll
          for (int q = 0; q < C::ACH; ++q) {
            const int c = tid + q * C::NT, row = c >> 3, ch = c & 7;
            *reinterpret_cast<u32x4*>(sA + row * LDK + ch * 8) = ra[q];
          }
        }
      }
    };

    load_tile(0);
    store_tile();
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      if (kt + 1 < KT) load_tile(kt + 1);  // global loads stay in flight under the MFMAs below
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        bf16x8 a[TM], b[TN];
        const int ko = ks * 16 + lh * 8;
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = lds_frag(sX + (wm * C::WTM + i * 32 + l32) * LDK + ko);
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = lds_frag(sW + (wn * C::WTN + j * 32 + l32) * LDK + ko);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        if constexpr (NRT > 0) {
          if (shrink) {
            // this wave owns shrink m-tiles wn*SM .. wn*SM+SM-1 of its wave row: their x fragments are in a[]
#pragma unroll
            for (int r = 0; r < NRT; ++r) {
              const bf16x8 ar = lds_frag(sA + (r * 32 + l32) * LDK + ko);
#pragma unroll
              for (int q = 0; q < C::WAVES_N; ++q) {
                if (wn == q) {  // wave-uniform: keeps the index into a[] a compile-time constant
#pragma unroll
                  for (int s = 0; s < C::SM; ++s)
                    tacc[s][r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[q * C::SM + s], ar, tacc[s][r], 0, 0, 0);
                }
              }
            }
          }
        }
      }
      __syncthreads();
      if (kt + 1 < KT) {
        store_tile();
        __syncthreads();
      }
    }

    if constexpr (NRT > 0) {
      if (shrink) {
        // T = (x . A_cat^T) * col_scale -> bf16 -> LDS.  Accumulator element v of lane (l32, lh)
        // is row 8*(v/4) + 4*lh + v%4, column l32 of its 32x32 tile.
#pragma unroll
        for (int r = 0; r < NRT; ++r) {
          const int col = r * 32 + l32;
          const float sc = p.col_scale[col];
#pragma unroll
          for (int s = 0; s < C::SM; ++s) {
            const int rbase = wm * C::WTM + (wn * C::SM + s) * 32 + 4 * lh;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int row = rbase + 8 * (v >> 2) + (v & 3);
              sT[row * C::LDT + col] = (bf16_t)(tacc[s][r][v] * sc);
            }
          }
        }
      }
      // expand: acc += T[BM,R] . B_cat[n0:n0+BN, R]^T
      for (int c = tid; c < BN * (R / 8); c += C::NT) {
        const int row = c / (R / 8), ch = c % (R / 8);
        int gr = n0 + row; gr = gr < N ? gr : N - 1;
        *reinterpret_cast<u32x4*>(sB + row * C::LDT + ch * 8) = ld16(p.b_cat + (size_t)gr * R + ch * 8);
      }
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < R / 16; ++ks) {
        bf16x8 a[TM], b[TN];
        const int ko = ks * 16 + lh * 8;
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = lds_frag(sT + (wm * C::WTM + i * 32 + l32) * C::LDT + ko);
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = lds_frag(sB + (wn * C::WTN + j * 32 + l32) * C::LDT + ko);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
      }
      __syncthreads();  // sB is dead before sC overwrites it
    }

    // Epilogue: bias in fp32, round to bf16, transpose through LDS so that every
    // global store is a 16-byte piece of a contiguous output row.
    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn * C::WTN + j * 32 + l32;
      bv[j] = (p.bias != nullptr && col < N) ? (float)p.bias[col] : 0.f;
    }
    const int out_ld = p.geglu ? (N >> 1) : N;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = wn * C::WTN + j * 32 + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
          sC[row * C::LDC + col] = (bf16_t)(acc[i][j][v] + bv[j]);
        }
      }
      __syncthreads();
      if (!p.geglu) {
        constexpr int CPR = BN / 8;  // 16-byte chunks per staged row
        for (int c = tid; c < C::WAVES_M * 32 * CPR; c += C::NT) {
          const int srow = c / CPR, ch = c % CPR;
          const int grow = m0 + (srow >> 5) * C::WTM + i * 32 + (srow & 31);
          const int gcol = n0 + ch * 8;
          if (grow < M && gcol < N) {
            u32x4 o = *reinterpret_cast<const u32x4*>(sC + srow * C::LDC + ch * 8);
            if (p.res != nullptr) {
              const u32x4 rr = ld16(p.res + (size_t)grow * N + gcol);
#pragma unroll
              for (int e = 0; e < 4; ++e)
                o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(rr[e]), bf16_hi(o[e]) + bf16_hi(rr[e]));
            }
            *reinterpret_cast<u32x4*>(p.y + (size_t)grow * N + gcol) = o;
          }
        }
      } else {
        // GEGLU epilogue: staged columns come in groups of 64 = 32 value columns then their 32 gate
        // columns; out = value * gelu_erf(gate), written to y[M, N/2].
        constexpr int OPR = BN / 16;  // 8-element output chunks per staged row
        for (int c = tid; c < C::WAVES_M * 32 * OPR; c += C::NT) {
          const int srow = c / OPR, oc = c % OPR;          // oc: output chunk, 4 chunks per 64-col group
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
              // the reference rounds gelu(gate) to the activation dtype before the product
              const float r0 = bf16_lo(pack_bf16x2(a0, 0.f)), r1 = bf16_lo(pack_bf16x2(a1, 0.f));
              o[e] = pack_bf16x2(bf16_lo(hv[e]) * r0, bf16_hi(hv[e]) * r1);
            }
            *reinterpret_cast<u32x4*>(p.y + (size_t)grow * out_ld + gcol) = o;
          }
        }
      }
      __syncthreads();
    }
  }
}

template <class C>
int launch_cfg(LoraGemmParams p, hipStream_t stream) {
  p.m_tiles = (p.M + C::BM - 1) / C::BM;
  p.n_tiles = (p.N + C::BN - 1) / C::BN;
  // Walk several N tiles per workgroup (T is reused from LDS) as long as the grid still
  // covers the 256 CUs at least twice over.
  int nc = 1;
  if (C::NRT > 0) {
    while (nc < p.n_tiles && (long)p.m_tiles * ((p.n_tiles + 2 * nc - 1) / (2 * nc)) >= 512) nc *= 2;
  }
  p.n_chunk = nc;
  p.n_chunks = (p.n_tiles + nc - 1) / nc;
  if (hipError_t e = kh_allow_lds<lora_gemm_kernel<C>>((int)C::LDS_BYTES); e != hipSuccess) return (int)e;
  const unsigned grid = (unsigned)(p.m_tiles * p.n_chunks);
  kh_launch(KH_TAG_LORA_GEMM, lora_gemm_kernel<C>, dim3(grid), dim3(C::NT), C::LDS_BYTES, stream, p);
  KH_RETURN_LAST_ERROR();
}

template <int BM, int BN, int WM, int WN>
int launch_rank(const LoraGemmParams& p, hipStream_t stream) {
  switch (p.R / 32) {
    case 0: return launch_cfg<Cfg<BM, BN, WM, WN, 0>>(p, stream);
    case 1: return launch_cfg<Cfg<BM, BN, WM, WN, 1>>(p, stream);
    case 2: return launch_cfg<Cfg<BM, BN, WM, WN, 2>>(p, stream);
    case 3: return launch_cfg<Cfg<BM, BN, WM, WN, 3>>(p, stream);
    case 4: return launch_cfg<Cfg<BM, BN, WM, WN, 4>>(p, stream);
    default: return KH_ERR_UNSUPPORTED;
  }
}

// ---------------------------------------------------------------------------------------------
// fp32 variant (debug / fp32 parity path): plain FMA tiles, same fusion (T kept in LDS).
// ---------------------------------------------------------------------------------------------
constexpr int F_BM = 64, F_BN = 64, F_BK = 16, F_RMAX = 128;

__global__ __launch_bounds__(256) void lora_gemm_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ bias,
                                                            const float* __restrict__ a_cat,
                                                            const float* __restrict__ b_cat,
                                                            const float* __restrict__ col_scale,
                                                            const float* __restrict__ res, float* __restrict__ y,
                                                            int M, int N, int K, int R) {
  __shared__ float sX[F_BK][F_BM + 1];
  __shared__ float sW[F_BK][F_BN + 1];
  __shared__ float sT[F_BM][F_RMAX + 1];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * F_BM, n0 = blockIdx.x * F_BN;
  float acc[4][4] = {};

  // shrink: T[r_local, 0..R) for the 64 rows of this block; thread (ty,tx): rows ty*4.., ranks tx, tx+16, ...
  for (int rb = 0; rb < R; rb += F_BN) {
    float t[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += F_BK) {
      for (int c = tid; c < F_BM * F_BK; c += 256) {
        const int r = c / F_BK, kk = c % F_BK;
        const int gr = min(m0 + r, M - 1), gk = k0 + kk;
        sX[kk][r] = gk < K ? x[(size_t)gr * K + gk] : 0.f;
      }
      for (int c = tid; c < F_BN * F_BK; c += 256) {
        const int r = c / F_BK, kk = c % F_BK;
        const int gr = rb + r, gk = k0 + kk;
        sW[kk][r] = (gr < R && gk < K) ? a_cat[(size_t)gr * K + gk] : 0.f;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < F_BK; ++kk) {
        float xv[4], av[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) xv[i] = sX[kk][ty * 4 + i];
#pragma unroll
        for (int j = 0; j < 4; ++j) av[j] = sW[kk][tx + 16 * j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) t[i][j] = fmaf(xv[i], av[j], t[i][j]);
      }
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int rr = rb + tx + 16 * j;
        if (rr < R) sT[ty * 4 + i][rr] = t[i][j] * col_scale[rr];
      }
  }
  __syncthreads();

  for (int k0 = 0; k0 < K; k0 += F_BK) {
    for (int c = tid; c < F_BM * F_BK; c += 256) {
      const int r = c / F_BK, kk = c % F_BK;
      const int gr = min(m0 + r, M - 1), gk = k0 + kk;
      sX[kk][r] = gk < K ? x[(size_t)gr * K + gk] : 0.f;
    }
    for (int c = tid; c < F_BN * F_BK; c += 256) {
      const int r = c / F_BK, kk = c % F_BK;
      const int gr = min(n0 + r, N - 1), gk = k0 + kk;
      sW[kk][r] = gk < K ? w[(size_t)gr * K + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F_BK; ++kk) {
      float xv[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) xv[i] = sX[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = sW[kk][tx + 16 * j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xv[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
  // expand: acc += T . B_cat^T
  for (int r0 = 0; r0 < R; r0 += F_BK) {
    for (int c = tid; c < F_BN * F_BK; c += 256) {
      const int r = c / F_BK, kk = c % F_BK;
      const int gr = min(n0 + r, N - 1), gk = r0 + kk;
      sW[kk][r] = gk < R ? b_cat[(size_t)gr * R + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F_BK; ++kk) {
      if (r0 + kk < R) {
        float tv[4], bv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) tv[i] = sT[ty * 4 + i][r0 + kk];
#pragma unroll
        for (int j = 0; j < 4; ++j) bv[j] = sW[kk][tx + 16 * j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(tv[i], bv[j], acc[i][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gr = m0 + ty * 4 + i;
    if (gr >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gc = n0 + tx + 16 * j;
      if (gc >= N) continue;
      float v = acc[i][j] + (bias ? bias[gc] : 0.f);
      if (res) v += res[(size_t)gr * N + gc];
      y[(size_t)gr * N + gc] = v;
    }
  }
}

}  // namespace

// See include/katz_hip.h: operands of the launch after the next one of this family, per host thread.
static thread_local const void* g_pf_ptr[3] = {nullptr, nullptr, nullptr};
static thread_local uint32_t g_pf_lines[3] = {0, 0, 0};
static thread_local int g_pf_n = 0;

KH_EXPORT int kh_set_weight_prefetch(const void* weights, int64_t bytes) {
  if (bytes < 0 || (weights == nullptr && bytes != 0)) return KH_ERR_INVALID_ARG;
  const int64_t lines = bytes >> 7;
  if (weights == nullptr || lines == 0) { g_pf_n = 0; return KH_OK; }   // clears what is pending
  if (g_pf_n == 3) return KH_ERR_TOO_LARGE;
  g_pf_ptr[g_pf_n] = weights;
  g_pf_lines[g_pf_n] = (uint32_t)(lines < (1 << 24) ? lines : (1 << 24));   // at most 2 GiB
  ++g_pf_n;
  return KH_OK;
}

void kh_take_weight_prefetch(LoraGemmParams& p) {
  for (int k = 0; k < 3; ++k) {
    p.pf[k] = k < g_pf_n ? g_pf_ptr[k] : nullptr;
    p.pf_lines[k] = k < g_pf_n ? g_pf_lines[k] : 0;
  }
  g_pf_n = 0;
}

namespace {
// Every entry point that can carry the hint holds one of these from its first line: however the call ends -- a refused
// argument included -- nothing stays pending for an unrelated later launch, by when the hinted range may have been freed.
struct PendingPrefetchDropped {
  ~PendingPrefetchDropped() { g_pf_n = 0; }
};
}  // namespace

// See include/katz_hip.h for the contract.
KH_EXPORT int kh_lora_linear_bf16(const void* x, const void* w, const void* bias, const void* a_cat,
                                  const void* b_cat, const float* col_scale, const void* residual, void* y,
                                  int64_t M, int64_t N, int64_t K, int64_t R, int flags, void* stream) {
  const PendingPrefetchDropped drop_pending_hint;
  if (!x || !w || !y || M <= 0 || N <= 0 || K <= 0 || R < 0) return KH_ERR_INVALID_ARG;
  if (R > 0 && (!a_cat || !b_cat || !col_scale)) return KH_ERR_INVALID_ARG;
  if (K % 8 != 0 || N % 8 != 0 || R % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 128) return KH_ERR_TOO_LARGE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_TOO_LARGE;
  const bool geglu = (flags & 1) != 0;
  if (geglu && (N % 64 != 0 || residual != nullptr)) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(x) || !kh_aligned16(w) || !kh_aligned16(y) || (R > 0 && (!kh_aligned16(a_cat) || !kh_aligned16(b_cat))) ||
      (residual && !kh_aligned16(residual)))
    return KH_ERR_ALIGNMENT;
  LoraGemmParams p;
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = (const bf16_t*)bias;
  p.a_cat = (const bf16_t*)a_cat; p.b_cat = (const bf16_t*)b_cat; p.col_scale = col_scale;
  p.res = (const bf16_t*)residual; p.y = (bf16_t*)y;
  p.t_ext = nullptr; p.ldt = 0; p.grp = nullptr; p.dbg = 0; p.t_nsplit = 0;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.R = (int)R;
  p.m_tiles = p.n_tiles = p.n_chunk = p.n_chunks = 0;
  p.geglu = geglu ? 1 : 0;
  p.xg_n = p.xr_m = p.xr_n = 0;
  p.sg_start = p.sg_adapter = p.sg_rank = nullptr; p.sg_scale = nullptr; p.sg_mode = 0; p.sg_wstride = 0;
  p.conv_cin = p.conv_h = p.conv_w = p.conv_ho = p.conv_wo = p.conv_stride = 0;
#ifdef KH_TUNING
  p.dbg = (flags >> 16) & 0xff;
#else
  if ((flags >> 16) != 0) return KH_ERR_INVALID_ARG;   // no meaning on this entry point
#endif
  hipStream_t s = (hipStream_t)stream;
  const int tile_sel = (flags >> 8) & 0xff;  // 0 = automatic
  // K % 32 == 0 (every SDXL layer): the software-pipelined kernel; tile_sel 1/2 force the simple kernel
  kh_take_weight_prefetch(p);
  if (K % 32 == 0 && (tile_sel == 0 || tile_sel >= 16)) return lora_gemm_pipe_launch(p, tile_sel, s);
  if (tile_sel == 2) return R > 96 ? KH_ERR_UNSUPPORTED : launch_rank<256, 128, 2, 2>(p, s);
  if (tile_sel == 1) return launch_rank<128, 128, 2, 2>(p, s);
  return launch_rank<128, 128, 2, 2>(p, s);
}

// Base GEMM + expand with a precomputed shrink result t (kh_lora_shrink_bf16); see include/katz_hip.h.
KH_EXPORT int kh_lora_linear_pre_bf16(const void* x, const void* w, const void* bias, const void* t, int64_t ldt,
                                      int64_t n_split, const void* b_cat, const void* residual, void* y, int64_t M,
                                      int64_t N, int64_t K, int64_t R, int flags, void* stream) {
  const PendingPrefetchDropped drop_pending_hint;
  if (!x || !w || !y || !t || !b_cat || M <= 0 || N <= 0 || K <= 0 || R <= 0 || ldt < R) return KH_ERR_INVALID_ARG;
  if (n_split < 0 || (n_split > 0 && (n_split % 128 != 0 || N % n_split != 0 || ldt < (N / n_split) * R)))
    return KH_ERR_INVALID_ARG;
  if (K % 32 != 0 || N % 8 != 0 || R % 32 != 0 || ldt % 8 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 128) return KH_ERR_TOO_LARGE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_TOO_LARGE;
  const bool geglu = (flags & 1) != 0;
  if (geglu && (N % 64 != 0 || residual != nullptr)) return KH_ERR_UNSUPPORTED;
  if (!kh_aligned16(x) || !kh_aligned16(w) || !kh_aligned16(y) || !kh_aligned16(t) || !kh_aligned16(b_cat) ||
      (residual && !kh_aligned16(residual)))
    return KH_ERR_ALIGNMENT;
  LoraGemmParams p;
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = (const bf16_t*)bias;
  p.a_cat = nullptr; p.b_cat = (const bf16_t*)b_cat; p.col_scale = nullptr;
  p.t_ext = (const bf16_t*)t; p.ldt = (int)ldt; p.grp = nullptr; p.dbg = 0; p.t_nsplit = (int)n_split;
  p.res = (const bf16_t*)residual; p.y = (bf16_t*)y;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.R = (int)R;
  p.m_tiles = p.n_tiles = p.n_chunk = p.n_chunks = 0;
  p.geglu = geglu ? 1 : 0;
  p.xg_n = p.xr_m = p.xr_n = 0;
  p.sg_start = p.sg_adapter = p.sg_rank = nullptr; p.sg_scale = nullptr; p.sg_mode = 0; p.sg_wstride = 0;
  p.conv_cin = p.conv_h = p.conv_w = p.conv_ho = p.conv_wo = p.conv_stride = 0;
  p.r_used = ((flags >> 16) & 0xff) * 16;
  if (p.r_used > p.R) return KH_ERR_INVALID_ARG;
  kh_take_weight_prefetch(p);
  return lora_gemm_pipe_launch(p, (flags >> 8) & 0xff, (hipStream_t)stream);
}

// Shrink + base GEMM + expand from the unshrunk operands; one launch where the GEMM leaves CUs idle, two otherwise.
// See include/katz_hip.h.
static LoraGemmParams split_params(const void* x, const void* w, const void* bias, const void* a_cat, const float* col_scale,
                                   const void* b_cat, void* t_scratch, int32_t* counters, const void* residual, void* y,
                                   int64_t M, int64_t N, int64_t K, int64_t R, int64_t n_split, bool geglu) {
  LoraGemmParams p;
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = (const bf16_t*)bias;
  p.a_cat = (const bf16_t*)a_cat; p.b_cat = (const bf16_t*)b_cat; p.col_scale = col_scale;
  p.t_ext = (const bf16_t*)t_scratch; p.ldt = (int)(n_split > 0 ? (N / n_split) * R : R); p.grp = nullptr; p.dbg = 0;
  p.t_nsplit = (int)n_split;
  p.res = (const bf16_t*)residual; p.y = (bf16_t*)y;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.R = (int)R;
  p.m_tiles = p.n_tiles = p.n_chunk = p.n_chunks = 0;
  p.geglu = geglu ? 1 : 0;
  p.xg_n = p.xr_m = p.xr_n = 0;
  p.sg_start = p.sg_adapter = p.sg_rank = nullptr; p.sg_scale = nullptr; p.sg_mode = 0; p.sg_wstride = 0;
  p.conv_cin = p.conv_h = p.conv_w = p.conv_ho = p.conv_wo = p.conv_stride = 0;
  p.il_cnt = counters;
  return p;
}

KH_EXPORT int kh_lora_linear_split_launches(int64_t M, int64_t N, int64_t K, int64_t R, int64_t n_split, int flags) {
  if (M <= 0 || N <= 0 || K <= 0 || R <= 0 || M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_INVALID_ARG;
  if (n_split < 0 || (n_split > 0 && N % n_split != 0)) return KH_ERR_INVALID_ARG;
  if (((flags >> 8) & 0xff) != 0) return 2;
  static int32_t dummy_counter;                  // the rule only asks whether counters were given
  static const char dummy = 0;
  LoraGemmParams p = split_params(&dummy, &dummy, nullptr, &dummy, reinterpret_cast<const float*>(&dummy), &dummy,
                                  const_cast<char*>(&dummy), &dummy_counter, nullptr, const_cast<char*>(&dummy), M, N, K, R,
                                  n_split, (flags & 1) != 0);
  p.r_used = ((flags >> 16) & 0xff) * 16;
  if ((flags & KH_FLAG_NO_COOP) == 0 && lora_gemm_ksplit_coop_ok(p)) return 1;
  return lora_gemm_pipe_il_ok(p) ? 1 : 2;
}

KH_EXPORT int kh_lora_linear_split_bf16(const void* x, const void* w, const void* bias, const void* a_cat,
                                        const float* col_scale, const void* b_cat, void* t_scratch, int32_t* counters,
                                        const void* residual, void* y, int64_t M, int64_t N, int64_t K, int64_t R,
                                        int64_t n_split, int flags, void* stream) {
  const PendingPrefetchDropped drop_pending_hint;
  if (!x || !w || !y || !a_cat || !col_scale || !b_cat || !t_scratch || M <= 0 || N <= 0 || K <= 0 || R <= 0)
    return KH_ERR_INVALID_ARG;
  if (n_split < 0 || (n_split > 0 && (n_split % 128 != 0 || N % n_split != 0))) return KH_ERR_INVALID_ARG;
  const int64_t RT = n_split > 0 ? (N / n_split) * R : R;   // columns of t_scratch / rows of a_cat
  if (K % 64 != 0 || N % 8 != 0 || R % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 128) return KH_ERR_TOO_LARGE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_TOO_LARGE;
  const bool geglu = (flags & 1) != 0;
  if (geglu && (N % 64 != 0 || residual != nullptr)) return KH_ERR_UNSUPPORTED;
  if (((flags >> 16) & 0xff) * 16 > R) return KH_ERR_INVALID_ARG;
  if (!kh_aligned16(x) || !kh_aligned16(w) || !kh_aligned16(y) || !kh_aligned16(a_cat) || !kh_aligned16(b_cat) ||
      !kh_aligned16(t_scratch) || (residual && !kh_aligned16(residual)))
    return KH_ERR_ALIGNMENT;
  if (counters != nullptr && kh_lora_linear_split_launches(M, N, K, R, n_split, flags) == 1) {
    LoraGemmParams p = split_params(x, w, bias, a_cat, col_scale, b_cat, t_scratch, counters, residual, y, M, N, K, R, n_split, geglu);
    p.r_used = ((flags >> 16) & 0xff) * 16;
    kh_take_weight_prefetch(p);
    if ((flags & KH_FLAG_NO_COOP) == 0 && lora_gemm_ksplit_coop_ok(p)) return lora_gemm_ksplit_launch_coop(p, (hipStream_t)stream);
    return lora_gemm_pipe_launch_il(p, (hipStream_t)stream);
  }
  const int rc = lora_shrink_ln_launch(x, a_cat, col_scale, t_scratch, M, K, RT, nullptr, nullptr, nullptr, 0.f, (hipStream_t)stream,
                                       (int)R, ((flags >> 16) & 0xff) * 16);
  if (rc != KH_OK) return rc;
  return kh_lora_linear_pre_bf16(x, w, bias, t_scratch, RT, n_split, b_cat, residual, y, M, N, K, R, flags & 0xff00ff, stream);
}

// LoRA linear behind a LayerNorm that is folded into the GEMM, and / or in front of one (row statistics out); see
// include/katz_hip.h.
namespace {
struct XAttnArgs {   // the attention behind a query projection (kh_lora_linear_xattn_bf16)
  const void* k; const void* v; void* o;
  int64_t T, S, ldk, ldv, ldo, bsk, bsv;
  float scale;
};
}  // namespace

static int lora_linear_norm_impl(const void* x, const void* w, const void* bias, const void* a_cat,
                                 const float* col_scale, const void* b_cat, void* t_scratch, int32_t* counters,
                                 const void* residual, void* y, const float* ln_part, const float* ln_c1,
                                 const float* ln_c2, const float* ln_ca1, const float* ln_ca2, float ln_eps,
                                 float* stats_out, int64_t M, int64_t N, int64_t K, int64_t R, int64_t n_split,
                                 int flags, void* stream, const XAttnArgs* xa) {
  const PendingPrefetchDropped drop_pending_hint;
  if (!x || !w || (!y && !xa) || M <= 0 || N <= 0 || K <= 0 || R < 0) return KH_ERR_INVALID_ARG;
  if (R > 0 && (!a_cat || !col_scale || !b_cat || !t_scratch)) return KH_ERR_INVALID_ARG;
  if (ln_part != nullptr && (!ln_c1 || !ln_c2 || bias != nullptr || (R > 0 && (!ln_ca1 || !ln_ca2)))) return KH_ERR_INVALID_ARG;
  if (n_split < 0 || (n_split > 0 && (n_split % 128 != 0 || N % n_split != 0))) return KH_ERR_INVALID_ARG;
  const int64_t RT = n_split > 0 ? (N / n_split) * R : R;   // columns of t_scratch / rows of a_cat
  if (K % 64 != 0 || N % 8 != 0 || R % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (R > 128) return KH_ERR_TOO_LARGE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_TOO_LARGE;
  const bool geglu = (flags & 1) != 0;
  if (geglu && (N % 64 != 0 || residual != nullptr || stats_out != nullptr)) return KH_ERR_UNSUPPORTED;
  if (stats_out != nullptr && N > 128 * KH_LN_SLOTS) return KH_ERR_TOO_LARGE;
  if (((flags >> 16) & 0xff) * 16 > R) return KH_ERR_INVALID_ARG;
  if (!kh_aligned16(x) || !kh_aligned16(w) || (y && !kh_aligned16(y)) || (R > 0 && (!kh_aligned16(a_cat) || !kh_aligned16(b_cat) ||
      !kh_aligned16(t_scratch))) || (residual && !kh_aligned16(residual)) || (ln_part && !kh_aligned16(ln_part)) ||
      (stats_out && !kh_aligned16(stats_out)))
    return KH_ERR_ALIGNMENT;
  LoraGemmParams p = split_params(x, w, bias, a_cat, col_scale, b_cat, R > 0 ? t_scratch : nullptr, counters, residual, y, M, N, K,
                                  R, n_split, geglu);
  p.r_used = ((flags >> 16) & 0xff) * 16;
  p.ln_part = ln_part; p.ln_c1 = ln_c1; p.ln_c2 = ln_c2; p.ln_ca1 = ln_ca1; p.ln_ca2 = ln_ca2; p.ln_eps = ln_eps;
  p.st_part = stats_out;
  const int tile_sel = (flags >> 8) & 0xff;
  if (xa != nullptr) {
    // the projection's result never reaches memory: its 128 x 128 tiles are 128 queries of two heads each
    if (!xa->k || !xa->v || !xa->o || xa->T <= 0 || xa->S <= 0 || M % xa->T != 0) return KH_ERR_INVALID_ARG;
    if (residual != nullptr || stats_out != nullptr || geglu || n_split != 0 || (tile_sel != 0 && tile_sel != 1)) return KH_ERR_INVALID_ARG;
    if (xa->S > 96 || xa->T % 128 != 0 || N % 128 != 0 || (R % 64) != 0) return KH_ERR_UNSUPPORTED;
    if ((xa->ldk | xa->ldv | xa->ldo | xa->bsk | xa->bsv) % 8 != 0) return KH_ERR_ALIGNMENT;
    if (xa->ldk < N || xa->ldv < N || xa->ldo < N) return KH_ERR_INVALID_ARG;
    if (!kh_aligned16(xa->k) || !kh_aligned16(xa->v) || !kh_aligned16(xa->o)) return KH_ERR_ALIGNMENT;
    p.xa_k = (const bf16_t*)xa->k; p.xa_v = (const bf16_t*)xa->v; p.xa_o = (bf16_t*)xa->o;
    p.xa_S = (int)xa->S; p.xa_T = (int)xa->T;
    p.xa_ldk = xa->ldk; p.xa_ldv = xa->ldv; p.xa_ldo = xa->ldo; p.xa_bsk = xa->bsk; p.xa_bsv = xa->bsv;
    p.xa_scale_log2e = xa->scale * 1.4426950408889634f;
    if (R == 0) { p.ldt = 0; p.t_nsplit = 0; p.il_cnt = nullptr; }
    if (!lora_gemm_pipe_xattn_ok(p)) return KH_ERR_UNSUPPORTED;
    kh_take_weight_prefetch(p);
    if (R == 0) return lora_gemm_pipe_launch_xattn(p, (hipStream_t)stream);
    if (counters != nullptr && tile_sel == 0 && lora_gemm_pipe_il_ok(p)) return lora_gemm_pipe_launch_xattn(p, (hipStream_t)stream);
    const int rc = lora_shrink_ln_launch(x, a_cat, col_scale, t_scratch, M, K, RT, ln_part, ln_ca1, ln_ca2, ln_eps, (hipStream_t)stream, (int)R, p.r_used);
    if (rc != KH_OK) return rc;
    p.a_cat = nullptr; p.col_scale = nullptr; p.il_cnt = nullptr;
    return lora_gemm_pipe_launch_xattn(p, (hipStream_t)stream);
  }
  kh_take_weight_prefetch(p);
  if (R == 0) {
    p.ldt = 0; p.t_nsplit = 0; p.il_cnt = nullptr;
    return lora_gemm_pipe_launch(p, tile_sel, (hipStream_t)stream);
  }
  if (counters != nullptr && tile_sel == 0 && (flags & KH_FLAG_NO_COOP) == 0 && lora_gemm_ksplit_coop_ok(p))
    return lora_gemm_ksplit_launch_coop(p, (hipStream_t)stream);
  if (counters != nullptr && tile_sel == 0 && lora_gemm_pipe_il_ok(p)) return lora_gemm_pipe_launch_il(p, (hipStream_t)stream);
  const int rc = lora_shrink_ln_launch(x, a_cat, col_scale, t_scratch, M, K, RT, ln_part, ln_ca1, ln_ca2, ln_eps, (hipStream_t)stream, (int)R, p.r_used);
  if (rc != KH_OK) return rc;
  p.a_cat = nullptr; p.col_scale = nullptr; p.il_cnt = nullptr;
  return lora_gemm_pipe_launch(p, tile_sel == 1 ? 0 : tile_sel, (hipStream_t)stream);
}

KH_EXPORT int kh_lora_linear_norm_bf16(const void* x, const void* w, const void* bias, const void* a_cat,
                                       const float* col_scale, const void* b_cat, void* t_scratch, int32_t* counters,
                                       const void* residual, void* y, const float* ln_part, const float* ln_c1,
                                       const float* ln_c2, const float* ln_ca1, const float* ln_ca2, float ln_eps,
                                       float* stats_out, int64_t M, int64_t N, int64_t K, int64_t R, int64_t n_split,
                                       int flags, void* stream) {
  return lora_linear_norm_impl(x, w, bias, a_cat, col_scale, b_cat, t_scratch, counters, residual, y, ln_part, ln_c1, ln_c2, ln_ca1,
                               ln_ca2, ln_eps, stats_out, M, N, K, R, n_split, flags, stream, nullptr);
}

// Query projection (kh_lora_linear_norm_bf16 without residual / statistics) with the cross-attention on its result inside
// the same launch; see include/katz_hip.h.
KH_EXPORT int kh_lora_linear_xattn_bf16(const void* x, const void* w, const void* bias, const void* a_cat,
                                        const float* col_scale, const void* b_cat, void* t_scratch, int32_t* counters,
                                        const float* ln_part, const float* ln_c1, const float* ln_c2, const float* ln_ca1,
                                        const float* ln_ca2, float ln_eps, const void* k, const void* v, void* o, int64_t M,
                                        int64_t N, int64_t K, int64_t R, int64_t T, int64_t S, int64_t ldk, int64_t ldv,
                                        int64_t ldo, int64_t bsk, int64_t bsv, float scale, int flags, void* stream) {
  const XAttnArgs xa = {k, v, o, T, S, ldk, ldv, ldo, bsk, bsv, scale};
  return lora_linear_norm_impl(x, w, bias, a_cat, col_scale, b_cat, t_scratch, counters, nullptr, nullptr, ln_part, ln_c1, ln_c2,
                               ln_ca1, ln_ca2, ln_eps, nullptr, M, N, K, R, 0, flags, stream, &xa);
}

// 1 if kh_lora_linear_xattn_bf16 takes these shapes, else 0 (then: the projection and kh_attention_bf16).
KH_EXPORT int kh_lora_linear_xattn_ok(int64_t M, int64_t N, int64_t K, int64_t R, int64_t T, int64_t S) {
  if (M <= 0 || N <= 0 || K <= 0 || R < 0 || T <= 0 || S <= 0 || M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return 0;
  if (M % 128 != 0 || N % 128 != 0 || K % 64 != 0 || R % 64 != 0 || R > 128 || T % 128 != 0 || M % T != 0 || S > 96) return 0;
  return (M / 128) * (N / 128) <= 256 ? 1 : 0;
}

// 3x3 convolution, padding 1, NHWC, as an implicit GEMM on the pipelined kernel; see include/katz_hip.h.
namespace {
int conv3x3_params(LoraGemmParams& p, const void* x, const void* w, const void* bias, const void* residual, void* y, int64_t Nb,
                   int64_t H, int64_t W, int64_t Cin, int64_t Cout, int64_t stride) {
  if (!x || !w || !y || Nb <= 0 || H <= 0 || W <= 0 || Cin <= 0 || Cout <= 0) return KH_ERR_INVALID_ARG;
  if (stride != 1 && stride != 2) return KH_ERR_UNSUPPORTED;
  if (Cin % 32 != 0 || Cout % 8 != 0) return KH_ERR_UNSUPPORTED;
  const int64_t Ho = (H + 2 - 3) / stride + 1, Wo = (W + 2 - 3) / stride + 1;
  const int64_t M = Nb * Ho * Wo;
  if (M > (1 << 24) || Cout > (1 << 24) || 9 * Cin > (1 << 24) || Nb * H * W * Cin >= ((int64_t)1 << 40)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || !kh_aligned16(w) || !kh_aligned16(y) || (residual && !kh_aligned16(residual)))
    return KH_ERR_ALIGNMENT;
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w; p.bias = (const bf16_t*)bias;
  p.a_cat = nullptr; p.b_cat = nullptr; p.col_scale = nullptr;
  p.t_ext = nullptr; p.ldt = 0; p.grp = nullptr; p.dbg = 0; p.t_nsplit = 0;
  p.res = (const bf16_t*)residual; p.y = (bf16_t*)y;
  p.M = (int)M; p.N = (int)Cout; p.K = (int)(9 * Cin); p.R = 0;
  p.m_tiles = p.n_tiles = p.n_chunk = p.n_chunks = 0;
  p.geglu = 0;
  p.xg_n = p.xr_m = p.xr_n = 0;
  p.sg_start = p.sg_adapter = p.sg_rank = nullptr; p.sg_scale = nullptr; p.sg_mode = 0; p.sg_wstride = 0;
  p.conv_cin = (int)Cin; p.conv_h = (int)H; p.conv_w = (int)W; p.conv_ho = (int)Ho; p.conv_wo = (int)Wo;
  p.conv_stride = (int)stride;
  return KH_OK;
}
}  // namespace

KH_EXPORT int kh_conv3x3_nhwc_bf16(const void* x, const void* w, const void* bias, const void* residual, void* y,
                                   int64_t Nb, int64_t H, int64_t W, int64_t Cin, int64_t Cout, int64_t stride,
                                   void* stream) {
  const PendingPrefetchDropped drop_pending_hint;
  LoraGemmParams p;
  if (const int rc = conv3x3_params(p, x, w, bias, residual, y, Nb, H, W, Cin, Cout, stride); rc != KH_OK) return rc;
  kh_take_weight_prefetch(p);
  return lora_gemm_pipe_launch_conv(p, (hipStream_t)stream);
}

// See include/katz_hip.h: row tiles per image of the statistics the convolution leaves, 0 when the shape is not taken.
KH_EXPORT int64_t kh_conv3x3_gn_splits(int64_t Nb, int64_t H, int64_t W, int64_t Cin, int64_t Cout, int64_t stride, int64_t G) {
  static const char dummy[16] __attribute__((aligned(16))) = {0};
  LoraGemmParams p;
  if (G <= 0 || Cout % G != 0) return 0;
  if (conv3x3_params(p, dummy, dummy, nullptr, nullptr, const_cast<char*>(dummy), Nb, H, W, Cin, Cout, stride) != KH_OK) return 0;
  p.gn_cg = (int)(Cout / G); p.gn_hw = p.conv_ho * p.conv_wo;
  const int rg = lora_gemm_conv_gn_row_groups(p);
  return rg == 0 ? 0 : p.gn_hw / (32 * rg);
}

KH_EXPORT int kh_conv3x3_gn_stats_nhwc_bf16(const void* x, const void* w, const void* bias, const void* residual,
                                            const void* add_nc, void* y, float* partials, int64_t Nb, int64_t H, int64_t W,
                                            int64_t Cin, int64_t Cout, int64_t stride, int64_t G, void* stream) {
  const PendingPrefetchDropped drop_pending_hint;
  if (!partials || G <= 0 || Cout % G != 0) return KH_ERR_INVALID_ARG;
  LoraGemmParams p;
  if (const int rc = conv3x3_params(p, x, w, bias, residual, y, Nb, H, W, Cin, Cout, stride); rc != KH_OK) return rc;
  p.gn_cg = (int)(Cout / G); p.gn_hw = p.conv_ho * p.conv_wo;
  if (lora_gemm_conv_gn_row_groups(p) == 0) return KH_ERR_UNSUPPORTED;
  p.gn_part = partials; p.gn_add = (const bf16_t*)add_nc;
  kh_take_weight_prefetch(p);
  return lora_gemm_pipe_launch_conv(p, (hipStream_t)stream);
}

// The segmented multi-adapter kernels (sgmv.hip) run on the pipelined GEMM when the shapes allow.
int kh_sgmv_on_gemm(int mode, const void* x, const void* w_all, void* y, const int32_t* seg_start, const int32_t* seg_adapter,
                    const int32_t* adapter_rank, const float* adapter_scale, int64_t n_segments, int64_t max_seg_rows,
                    int64_t N, int64_t K, int64_t w_stride, hipStream_t stream) {
  LoraGemmParams p;
  p.x = (const bf16_t*)x; p.w = (const bf16_t*)w_all; p.bias = nullptr;
  p.a_cat = nullptr; p.b_cat = nullptr; p.col_scale = nullptr;
  p.t_ext = nullptr; p.ldt = 0; p.grp = nullptr; p.dbg = 0; p.t_nsplit = 0;
  p.res = nullptr; p.y = (bf16_t*)y;
  p.M = (int)max_seg_rows; p.N = (int)N; p.K = (int)K; p.R = 0;
  p.m_tiles = p.n_tiles = p.n_chunk = p.n_chunks = 0;
  p.geglu = 0;
  p.xg_n = p.xr_m = p.xr_n = 0;
  p.conv_cin = p.conv_h = p.conv_w = p.conv_ho = p.conv_wo = p.conv_stride = 0;
  p.sg_start = seg_start; p.sg_adapter = seg_adapter; p.sg_rank = adapter_rank; p.sg_scale = adapter_scale;
  p.sg_mode = mode; p.sg_wstride = (long)w_stride;
  return lora_gemm_pipe_launch_sgmv(p, (int)n_segments, stream);
}

// Many layers that share one input in one launch; see include/katz_hip.h.
KH_EXPORT int kh_lora_linear_grouped_bf16(const void* x, const uint64_t* table, int64_t n_groups, int64_t ldt,
                                          int64_t M, int64_t N, int64_t K, int64_t R, int flags, void* stream) {
  if (!x || !table || n_groups <= 0 || M <= 0 || N <= 0 || K <= 0 || R < 0) return KH_ERR_INVALID_ARG;
  if (K % 32 != 0 || N % 8 != 0 || R % 32 != 0 || ldt % 8 != 0 || (R > 0 && ldt < R)) return KH_ERR_UNSUPPORTED;
  if (R > 128 || n_groups > 65535) return KH_ERR_TOO_LARGE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_TOO_LARGE;
  if ((flags & 1) != 0) return KH_ERR_UNSUPPORTED;  // no GEGLU epilogue in grouped launches
  if (!kh_aligned16(x) || !kh_aligned16(table)) return KH_ERR_ALIGNMENT;
  LoraGemmParams p;
  p.x = (const bf16_t*)x; p.w = nullptr; p.bias = nullptr; p.a_cat = nullptr; p.b_cat = nullptr; p.col_scale = nullptr;
  p.t_ext = nullptr; p.ldt = (int)ldt; p.grp = table; p.dbg = 0; p.t_nsplit = 0;
  p.res = nullptr; p.y = nullptr;
  p.M = (int)M; p.N = (int)N; p.K = (int)K; p.R = (int)R;
  p.m_tiles = p.n_tiles = p.n_chunk = p.n_chunks = 0;
  p.geglu = 0;
  p.xg_n = p.xr_m = p.xr_n = 0;
  p.sg_start = p.sg_adapter = p.sg_rank = nullptr; p.sg_scale = nullptr; p.sg_mode = 0; p.sg_wstride = 0;
  p.conv_cin = p.conv_h = p.conv_w = p.conv_ho = p.conv_wo = p.conv_stride = 0;
  return lora_gemm_pipe_launch_grouped(p, (int)n_groups, (hipStream_t)stream);
}

KH_EXPORT int kh_lora_linear_f32(const float* x, const float* w, const float* bias, const float* a_cat,
                                 const float* b_cat, const float* col_scale, const float* residual, float* y,
                                 int64_t M, int64_t N, int64_t K, int64_t R, void* stream) {
  if (!x || !w || !y || M <= 0 || N <= 0 || K <= 0 || R < 0) return KH_ERR_INVALID_ARG;
  if (R > 0 && (!a_cat || !b_cat || !col_scale)) return KH_ERR_INVALID_ARG;
  if (R > F_RMAX) return KH_ERR_TOO_LARGE;
  dim3 grid((unsigned)((N + F_BN - 1) / F_BN), (unsigned)((M + F_BM - 1) / F_BM));
  kh_launch(KH_TAG_LORA_GEMM_F32, lora_gemm_f32_kernel, grid, dim3(256), 0, (hipStream_t)stream, x, w, bias, a_cat, b_cat,
                     col_scale, residual, y, (int)M, (int)N, (int)K, (int)R);
  KH_RETURN_LAST_ERROR();
}

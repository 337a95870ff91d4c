// Batched LoRA merge: W_l += scale_l * up_l . down_l for many layers in ONE launch (gfx950).
//
// Katz merges an adapter into the UNet weights before a request that uses it: for each of the 722 matched linears
// `unet_state_dict[key] += cur_up @ cur_down * scale` (patch_on_lora,
// diffusers-hf/src/diffusers/pipelines/controlnet/pipeline_controlnet_sd_xl_katz.py:1730-1747; diffusers' own
// _fuse_lora, diffusers-hf/src/diffusers/models/lora.py:403-433, is the same update in fp32).  That is 722 small
// matmuls, adds and a load_state_dict; here it is one kernel over a table of layers.  The update streams every
// weight once (read + write: HBM-bound), the rank-r product is a handful of MFMA steps per 128x128 tile:
//   * grid = all 128x128 tiles of all layers; a workgroup finds its layer by bisection in the tile prefix;
//   * the up tile [128, r] and the down tile [r, 128] go to LDS (down is read column-wise by the MFMA);
//   * W' = bf16(float(W) + scale * acc): fp32 accumulate, one rounding (the reference rounds the product and the
//     scaled product to half first).
// Adapter operands may be bf16 or fp16 storage (Katz keeps adapters as float16 arrays in shared memory,
// load_lora_shm_multi.py:49-61): fp16 operands use the f16 MFMA, so nothing is converted on the way.
#include "kh_common.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int MG_BM = 128, MG_BN = 128, MG_THREADS = 256;
constexpr int MG_RMAX = 128;                 // largest rank (one pass holds the whole rank axis in LDS)
constexpr int MG_LDD = MG_BN + 4;            // sD row stride (elements): rows 8-byte aligned; the 8 rows a column read spans
                                             // between the two wave halves fall 16 banks apart

struct MergeRow {       // one layer; mirrors the six 64-bit words of the table in include/katz_hip.h
  uint64_t w, up, down; // device addresses: W [N,K] bf16, up [N,r], down [r,K]
  int64_t N, K, r;
};

__host__ __device__ constexpr int mg_lds_bytes(int rp) { return (MG_BM * (rp + 8) + rp * MG_LDD) * 2; }

template <bool F16>
__device__ __forceinline__ f32x16 mfma16(const u32x4 a, const u32x4 b, f32x16 c) {
  if constexpr (F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
}

// rp: the largest rank of the table rounded up to 16 (sizes the LDS rows); a layer's own rank may be smaller.
template <bool F16>
__global__ __launch_bounds__(MG_THREADS) void lora_merge_kernel(const MergeRow* __restrict__ table,
                                                                const int* __restrict__ tile_start, int n_layers,
                                                                const float* __restrict__ layer_scale, float scale, int rp_max) {
  extern __shared__ __align__(16) uint16_t mg_smem[];
  const int ldu = rp_max + 8;                 // sU row stride: rows 16-byte aligned, an odd multiple of 16 bytes
  uint16_t* sU = mg_smem;                     // [128][ldu]   up tile, rank axis contiguous
  uint16_t* sD = mg_smem + MG_BM * ldu;       // [rp][130]    down tile, W columns contiguous
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lh = lane >> 5;
  // layer of this tile: the last l with tile_start[l] <= blockIdx.x (uniform over the workgroup)
  int lo = 0, hi = n_layers - 1;
  const int bid = (int)blockIdx.x;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (tile_start[mid] <= bid) lo = mid; else hi = mid - 1;
  }
  const MergeRow L = table[lo];
  const int N = (int)L.N, K = (int)L.K;
  const int r = (int)L.r < rp_max ? (int)L.r : rp_max;   // the host has checked r <= rp_max; never index past the LDS rows
  const int tn = (K + MG_BN - 1) / MG_BN;
  const int t = bid - tile_start[lo];
  const int m0 = (t / tn) * MG_BM, n0 = (t % tn) * MG_BN;
  if (m0 >= N) return;                        // a tile count larger than the layer's (uniform; before any barrier)
  const float s = scale * (layer_scale != nullptr ? layer_scale[lo] : 1.f);
  const uint16_t* up = reinterpret_cast<const uint16_t*>(L.up);
  const uint16_t* down = reinterpret_cast<const uint16_t*>(L.down);
  bf16_t* W = reinterpret_cast<bf16_t*>(L.w);
  const int rp = (r + 15) & ~15;   // this layer's rank in whole MFMA steps, the excess zero-filled

  // 16-byte pieces where the layer allows it (r % 8 == 0, K % 8 == 0, aligned bases: every linear of the UNet), else
  // element by element
  const bool fast = (L.r & 7) == 0 && (K & 7) == 0 && ((L.up | L.down) & 15) == 0;
  if (fast) {
    const int upr = rp / 8;                                     // pieces per up row
    for (int i = tid; i < MG_BM * upr; i += MG_THREADS) {
      const int row = i / upr, k = (i % upr) * 8;
      u32x4 v = u32x4{0, 0, 0, 0};
      if (m0 + row < N && k < r) v = *reinterpret_cast<const u32x4*>(up + (size_t)(m0 + row) * L.r + k);
      *reinterpret_cast<u32x4*>(sU + row * ldu + k) = v;
    }
    for (int i = tid; i < rp * (MG_BN / 8); i += MG_THREADS) {
      const int k = i / (MG_BN / 8), col = (i % (MG_BN / 8)) * 8;
      u32x4 v = u32x4{0, 0, 0, 0};
      if (k < r && n0 + col < K) v = *reinterpret_cast<const u32x4*>(down + (size_t)k * K + n0 + col);
      u32x2* dst = reinterpret_cast<u32x2*>(sD + k * MG_LDD + col);
      dst[0] = u32x2{v[0], v[1]};
      dst[1] = u32x2{v[2], v[3]};
    }
  } else {
    for (int i = tid; i < MG_BM * rp; i += MG_THREADS) {
      const int row = i / rp, k = i % rp;
      sU[row * ldu + k] = (m0 + row < N && k < r) ? up[(size_t)(m0 + row) * L.r + k] : (uint16_t)0;
    }
    for (int i = tid; i < rp * MG_BN; i += MG_THREADS) {
      const int k = i / MG_BN, col = i % MG_BN;
      sD[k * MG_LDD + col] = (k < r && n0 + col < K) ? down[(size_t)k * K + n0 + col] : (uint16_t)0;
    }
  }
  __syncthreads();

  // acc[j][i] = (down^T . up^T) tile: rows are W COLUMNS n0 + wn*64 + j*32 + .., columns are W ROWS m0 + wm*64 + i*32 + l32,
  // so a lane ends up with runs of four consecutive W columns of one W row (8-byte read-modify-writes)
  f32x16 acc[2][2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;

  for (int k0 = 0; k0 < rp; k0 += 16) {
    u32x4 a[2], b[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {       // W column (n0 + wn*64 + j*32 + l32), rank k0 + lh*8 .. +7: a column of sD
      const uint16_t* src = sD + (k0 + lh * 8) * MG_LDD + wn * 64 + j * 32 + l32;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        a[j][e] = (uint32_t)src[(2 * e) * MG_LDD] | ((uint32_t)src[(2 * e + 1) * MG_LDD] << 16);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)         // W row (m0 + wm*64 + i*32 + l32), the same eight ranks: 16 contiguous bytes of sU
      b[i] = *reinterpret_cast<const u32x4*>(sU + (wm * 64 + i * 32 + l32) * ldu + k0 + lh * 8);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[j][i] = mfma16<F16>(a[j], b[i], acc[j][i]);
  }

  // W' = bf16(W + s * acc): fp32 sum, one rounding
  const bool vec = (K & 3) == 0 && ((uintptr_t)W & 7) == 0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = m0 + wm * 64 + i * 32 + l32;
    if (row >= N) continue;
    bf16_t* wr = W + (size_t)row * K;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = n0 + wn * 64 + j * 32 + 8 * g + 4 * lh;
        if (vec && col + 3 < K) {
          u32x2 old = *reinterpret_cast<const u32x2*>(wr + col), out;
          out[0] = pack_bf16x2(bf16_lo(old[0]) + s * acc[j][i][4 * g], bf16_hi(old[0]) + s * acc[j][i][4 * g + 1]);
          out[1] = pack_bf16x2(bf16_lo(old[1]) + s * acc[j][i][4 * g + 2], bf16_hi(old[1]) + s * acc[j][i][4 * g + 3]);
          *reinterpret_cast<u32x2*>(wr + col) = out;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (col + e < K) wr[col + e] = (bf16_t)((float)wr[col + e] + s * acc[j][i][4 * g + e]);
        }
      }
  }
}

}  // namespace

// See include/katz_hip.h.
KH_EXPORT int kh_lora_merge_grouped_bf16(const uint64_t* table, const int32_t* tile_start, const float* layer_scale,
                                         int64_t n_layers, int64_t total_tiles, int64_t max_rank, float scale,
                                         int operands_fp16, void* stream) {
  if (!table || !tile_start || n_layers <= 0 || total_tiles <= 0 || max_rank <= 0) return KH_ERR_INVALID_ARG;
  if (total_tiles > 0x7fffffffL || n_layers > (1 << 24) || max_rank > MG_RMAX) return KH_ERR_TOO_LARGE;
  static_assert(sizeof(MergeRow) == 6 * sizeof(uint64_t), "table row layout");
  const MergeRow* rows = reinterpret_cast<const MergeRow*>(table);
  const int rp = ((int)max_rank + 15) & ~15;
  const int lds = mg_lds_bytes(rp);
  hipError_t e = operands_fp16 ? kh_allow_lds<lora_merge_kernel<true>>(mg_lds_bytes(MG_RMAX))
                               : kh_allow_lds<lora_merge_kernel<false>>(mg_lds_bytes(MG_RMAX));
  if (e != hipSuccess) return (int)e;
  if (operands_fp16)
    kh_launch(KH_TAG_LORA_MERGE, lora_merge_kernel<true>, dim3((unsigned)total_tiles), dim3(MG_THREADS), (size_t)lds,
              (hipStream_t)stream, rows, (const int*)tile_start, (int)n_layers, layer_scale, scale, rp);
  else
    kh_launch(KH_TAG_LORA_MERGE, lora_merge_kernel<false>, dim3((unsigned)total_tiles), dim3(MG_THREADS), (size_t)lds,
              (hipStream_t)stream, rows, (const int*)tile_start, (int)n_layers, layer_scale, scale, rp);
  KH_RETURN_LAST_ERROR();
}

// K2, one launch: segmented multi-adapter LoRA delta  y[rows, :] += scale_a * bf16(x[rows, :] . A_a^T) . B_a^T  per request
// segment (rows [seg_start[s], seg_start[s+1]) use adapter seg_adapter[s], negative: none) for gfx950.
//
// The per-request form of the reference's LoRA linear (diffusers-hf/src/diffusers/models/lora.py:222-232, :451-457)
// with y already holding the base projection; the reference has no batched heterogeneous-adapter path.  Same arithmetic
// as kh_sgmv_shrink_bf16 followed by kh_sgmv_expand_bf16 (t rounded to bf16 between the two products, the product
// rounded to bf16 before it is added to y), but t never leaves the workgroup: one launch instead of two and no round
// trip of t through memory.  Bound: HBM (x read once, y read and written once; the adapter matrices come from L2).
//
// A workgroup (8 waves) owns 128 rows of one segment.
//   phase 1: T[128, 128] = x_tile . A_a^T over K in 64-column stages (ring of three, buffer-addressed LDS DMA, the
//            operand path of lora_gemm_pipe.hip); T is rounded to bf16 and written to LDS in the stage layout, so that
//   phase 2: for every 128-column tile of y:  acc = T . B_a[tile]^T  (K = the adapter's padded rank, one or two stages of
//            B from L2), times the adapter's scale, rounded, transposed through LDS and added to the y pieces, which were
//            requested together with the B tile while the previous tile was being finished.
// Rows / columns of A_a / B_a beyond the adapter's rank are zero by contract, so the padded rank only saves work.
// Batches with few row blocks deal the column tiles of y to several workgroups (blockIdx.z), each of which repeats
// phase 1 for its rows: x is then read from L2 more than once, which such small batches do not notice.
// Grouped form (kh_sgmv_fused_grouped_bf16): several layers that read the same x with the same segments (the to_k / to_v
// projections of every cross-attention read the one text context) in one launch, blockIdx.z = (layer, column range),
// per-layer A / B / y from a device table: 77-row requests give a single layer's launch a few microseconds of traffic,
// 120 layers fill the chip.
#include "kh_common.h"

namespace {

typedef __attribute__((address_space(3))) void* lptr_t;
typedef __amdgpu_buffer_rsrc_t rsrc_t;

template <int VM, int LGKM>
__device__ __forceinline__ void wait_cnt() {  // gfx9 encoding: vmcnt = [15:14|3:0], expcnt = [6:4], lgkmcnt = [11:8]
  __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | ((LGKM & 15) << 8) | ((VM >> 4) << 14));
}

struct FusedParams {
  const bf16_t* x; const bf16_t* a_all; const bf16_t* b_all; bf16_t* y;
  const int* seg_start; const int* seg_adapter; const int* adapter_rank; const float* adapter_scale;
  int K, N, RP;
  int tiles_per_z;   // 128-column tiles of y per workgroup: blockIdx.z selects the range (T is recomputed per range)
  int z_per_layer;   // column ranges per layer (grid.z = layers x z_per_layer)
  const uint64_t* table;   // grouped form: rows {a_all, b_all, y} of device pointers, one per layer; null: the fields above
};

constexpr int BM = 128, BR = 128;                 // rows of a workgroup, rank columns (RP <= 128)
constexpr int STAGE = (BM + BR) * 128;            // 64 K-columns of x rows and of A rows: 32 KB
constexpr int NST = 3;
constexpr int T_OFF = 0, T_BYTES = 2 * BM * 128;  // phase 2: T as two 64-column stages of 128-byte rows (32 KB)
constexpr int B_OFF = T_BYTES, B_TILE = 2 * 128 * 128;   // two buffers of a B tile (128 y columns x 128 rank columns)
constexpr int C_OFF = B_OFF + 2 * B_TILE;         // staging of 64 output rows x (128 + 8) columns
constexpr int LDC = 128 + 8;
constexpr int LDS_BYTES = C_OFF + 64 * LDC * 2;
static_assert(NST * STAGE <= C_OFF, "phase 2's T and B buffers reuse the ring; the staging tile lies behind it");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");

__global__ __launch_bounds__(512, 2) void sgmv_fused_kernel(const FusedParams p) {
#if __HIP_DEVICE_COMPILE__   // the host pass only needs the kernel's symbol (it cannot lower the buffer-resource type)
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int seg = blockIdx.y;
  const int r0 = p.seg_start[seg], r1 = p.seg_start[seg + 1], ad = p.seg_adapter[seg];
  const int m0 = blockIdx.x * BM;
  if (ad < 0 || m0 >= r1 - r0) return;            // uniform over the workgroup
  const int M = r1 - r0;                          // rows of this segment
  const int rank = p.adapter_rank[ad];            // multiple of 32, <= RP
  const float scale = p.adapter_scale[ad];
  const int K = p.K, N = p.N, RP = p.RP;
  const int layer = (int)blockIdx.z / p.z_per_layer, zz = (int)blockIdx.z % p.z_per_layer;
  const bf16_t* a_all = p.a_all; const bf16_t* b_all = p.b_all; bf16_t* y_all = p.y;
  if (p.table != nullptr) {
    const uint64_t* row = p.table + (size_t)layer * 3;
    a_all = reinterpret_cast<const bf16_t*>(row[0]); b_all = reinterpret_cast<const bf16_t*>(row[1]); y_all = reinterpret_cast<bf16_t*>(row[2]);
  }
  const bf16_t* x = p.x + (size_t)r0 * K;
  bf16_t* y = y_all + (size_t)r0 * N;
  const bf16_t* A = a_all + (size_t)ad * RP * K;
  const bf16_t* B = b_all + (size_t)ad * N * RP;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;        // 2 x 4 waves: a wave owns 64 rows x 32 columns of a 128 x 128 tile
  const int l32 = lane & 31, lh = lane >> 5;
  const int sw = (l32 >> 1) & 7;

  auto clamp32 = [](size_t bytes) { return (int)(uint32_t)(bytes < 0xFFFFFFFFull ? bytes : 0xFFFFFFFFull); };
  auto mk = [&](const bf16_t* base, size_t bytes) { return __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(base), 0, clamp32(bytes), 0x00020000); };

  // ---- phase 1: T = x_tile . A^T ----
  // DMA units of 8 rows x 128 bytes: 16 x units and 16 A units per stage, two of each per wave; a lane's byte offset
  // (row, swizzled piece) never changes, the K tile is a scalar offset
  const rsrc_t rs_x = mk(x + (size_t)m0 * K, (size_t)(M - m0) * K * 2);
  const rsrc_t rs_a = mk(A, (size_t)RP * K * 2);
  uint32_t vx[2], va[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = (wave * 2 + q) * 8 + (lane >> 3);
    const uint32_t pcb = (uint32_t)(((lane & 7) ^ ((r >> 1) & 7)) * 16);
    int row = m0 + r; row = row < M ? row : M - 1;
    vx[q] = (uint32_t)(row - m0) * (uint32_t)K * 2u + pcb;
    va[q] = (uint32_t)(r < RP ? r : RP - 1) * (uint32_t)K * 2u + pcb;   // (rows beyond RP: any valid row; their T columns are never used)
  }
  auto issue1 = [&](int t) {
    char* stage = smem + (t % NST) * STAGE;
    const int so = t * 128;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_x, (lptr_t)(stage + (wave * 2 + q) * 1024), 16, vx[q], so, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lptr_t)(stage + BM * 128 + (wave * 2 + q) * 1024), 16, va[q], so, 0, 0);
    }
  };
  // fragments of a 64-column stage: rows (wm * 64 + i * 32 + l32) of the first operand, (wn * 32 + l32) of the second
  struct Fr { bf16x8 a[4][2]; bf16x8 b[4]; };
  auto read_frags = [&](const char* st_a, const char* st_b, Fr& f) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int po = ((2 * ks + lh) ^ sw) * 16;
#pragma unroll
      for (int i = 0; i < 2; ++i) f.a[ks][i] = *reinterpret_cast<const bf16x8*>(st_a + (wm * 64 + i * 32 + l32) * 128 + po);
      f.b[ks] = *reinterpret_cast<const bf16x8*>(st_b + (wn * 32 + l32) * 128 + po);
    }
  };
  f32x16 acc[2];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  };
  auto mma = [&](const Fr& f, int ks_n) {   // the first ks_n 16-column steps of the stage
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
      if (ks < ks_n) {
#pragma unroll
        for (int i = 0; i < 2; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ks][i], f.b[ks], acc[i], 0, 0, 0);
      }
  };
  const int KT = K / 64;
  zero_acc();
  issue1(0);
  if (KT > 1) issue1(1);
  Fr f;
  for (int t = 0; t < KT; ++t) {
    if (t + 1 < KT) wait_cnt<4, 0>(); else wait_cnt<0, 0>();   // this wave's loads of tile t are complete (4 per tile)
    __builtin_amdgcn_s_barrier();                              // everyone's are, and everyone has read tile t-1
    if (t + 2 < KT) issue1(t + 2);                             // into the stage of tile t-1
    const char* st = smem + (t % NST) * STAGE;
    read_frags(st, st + BM * 128, f);
    mma(f, 4);
  }
  __syncthreads();   // the ring is dead

  // T, rounded to bf16, into the stage layout (row r, logical 16-byte piece c of stage s at physical piece c ^ ((r/2) % 8));
  // a lane holds column wn * 32 + l32 of rows 8 * (v / 4) + 4 * lh + (v % 4) of each of its two 32-row tiles
  {
    const int col = wn * 32 + l32, s = col >> 6, cc = col & 63, piece = cc >> 3, within = (cc & 7) * 2;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = wm * 64 + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        *reinterpret_cast<bf16_t*>(smem + T_OFF + s * (BM * 128) + r * 128 + ((piece ^ ((r >> 1) & 7)) * 16) + within) = (bf16_t)acc[i][v];
      }
  }

  // ---- phase 2: y tile += scale * T . B_tile^T for every 128-column tile ----
  const int j0 = zz * p.tiles_per_z;
  const int n_tiles = (N / 128 - j0) < p.tiles_per_z ? (N / 128 - j0) : p.tiles_per_z;   // tiles j0 .. j0 + n_tiles - 1
  const int ks_total = rank / 16;                 // MFMA steps over the padded rank (2, 4, 6 or 8)
  const int nstage = (rank + 63) / 64;            // B stages per tile (1 or 2)
  // B tile j: rows n0 .. n0+127 of B (row stride RP), 64 rank columns per stage; 16 units per stage, two per wave
  const rsrc_t rs_b = mk(B, (size_t)N * RP * 2);
  uint32_t vb[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = (wave * 2 + q) * 8 + (lane >> 3);
    vb[q] = (uint32_t)r * (uint32_t)RP * 2u + (uint32_t)(((lane & 7) ^ ((r >> 1) & 7)) * 16);
  }
  constexpr int CPR = 16, ECH = 64 * CPR / 512;   // 16-byte pieces per staged row; per thread and 64-row pass: 2
  u32x4 yr[2][ECH];                               // this thread's y pieces of the tile in flight (two passes)
  auto issue2 = [&](int j) {                      // B tile j and the y pieces of tile j
    char* bt = smem + B_OFF + (j & 1) * B_TILE;
    const int so = (j0 + j) * 128 * RP * 2;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        // (a second stage beyond the padded rank is still fetched when RP allows: it multiplies nothing)
        const uint32_t off = (s * 128 < RP * 2) ? vb[q] + s * 128 : 0xFFFFFFFFu;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lptr_t)(bt + s * (128 * 128) + (wave * 2 + q) * 1024), 16, off, so, 0, 0);
      }
#pragma unroll
    for (int ps = 0; ps < 2; ++ps)
#pragma unroll
      for (int q = 0; q < ECH; ++q) {
        const int c = tid + q * 512, srow = c / CPR, ch = c % CPR;
        int grow = m0 + (srow >> 5) * 64 + ps * 32 + (srow & 31);
        grow = grow < M ? grow : M - 1;
        yr[ps][q] = *reinterpret_cast<const u32x4*>(y + (size_t)grow * N + (j0 + j) * 128 + ch * 8);
      }
  };
  const bool full = m0 + BM <= M;
  __syncthreads();   // T is written
  issue2(0);
  bf16_t* sC = reinterpret_cast<bf16_t*>(smem + C_OFF);
  for (int j = 0; j < n_tiles; ++j) {
    // B tile j (this wave's share) and this thread's y pieces are here; the four stores of the tile before (younger: a
    // wave's memory operations complete in order) may still be on their way when every thread of the tile stores
    if (j > 0 && full) wait_cnt<2 * ECH, 0>(); else wait_cnt<0, 0>();
    __builtin_amdgcn_s_barrier();
    u32x4 yc[2][ECH];
#pragma unroll
    for (int ps = 0; ps < 2; ++ps)
#pragma unroll
      for (int q = 0; q < ECH; ++q) yc[ps][q] = yr[ps][q];
    if (j + 1 < n_tiles) issue2(j + 1);           // flies under this tile's MFMAs and epilogue
    const char* bt = smem + B_OFF + (j & 1) * B_TILE;
    zero_acc();
    for (int s = 0; s < nstage; ++s) {
      read_frags(smem + T_OFF + s * (BM * 128), bt + s * (128 * 128), f);
      const int left = ks_total - 4 * s;
      mma(f, left < 4 ? left : 4);
    }
    // epilogue: two passes of 64 rows (the waves' upper / lower 32-row tiles): scale, round, transpose through LDS, add y
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        sC[row * LDC + wn * 32 + l32] = (bf16_t)(acc[i][v] * scale);
      }
      __syncthreads();
#pragma unroll
      for (int q = 0; q < ECH; ++q) {
        const int c = tid + q * 512, srow = c / CPR, ch = c % CPR;
        const int grow = m0 + (srow >> 5) * 64 + i * 32 + (srow & 31);
        if (grow < M) {
          u32x4 o = *reinterpret_cast<const u32x4*>(sC + srow * LDC + ch * 8);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = pack_bf16x2(bf16_lo(o[e]) + bf16_lo(yc[i][q][e]), bf16_hi(o[e]) + bf16_hi(yc[i][q][e]));
          *reinterpret_cast<u32x4*>(y + (size_t)grow * N + (j0 + j) * 128 + ch * 8) = o;
        }
      }
      __syncthreads();
    }
  }
#endif
}

}  // namespace

namespace {

int sgmv_fused_impl(const void* x, const void* a_all, const void* b_all, void* y, const uint64_t* table, int64_t n_layers,
                    const int32_t* seg_start, const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                    int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t K, int64_t RP, void* stream) {
  if (!x || !seg_start || !seg_adapter || !adapter_rank || !adapter_scale) return KH_ERR_INVALID_ARG;
  if (table == nullptr && (!a_all || !b_all || !y)) return KH_ERR_INVALID_ARG;
  if (n_segments <= 0 || max_seg_rows <= 0 || N <= 0 || K <= 0 || RP <= 0 || n_layers <= 0) return KH_ERR_INVALID_ARG;
  if (RP > 128) return KH_ERR_TOO_LARGE;
  if (K % 64 != 0 || N % 128 != 0 || RP % 32 != 0) return KH_ERR_UNSUPPORTED;
  if (n_segments > 65535 || max_seg_rows > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return KH_ERR_TOO_LARGE;
  if (!kh_aligned16(x) || (table == nullptr && (!kh_aligned16(a_all) || !kh_aligned16(b_all) || !kh_aligned16(y))) ||
      (table != nullptr && ((uintptr_t)table & 7) != 0))
    return KH_ERR_ALIGNMENT;
  FusedParams p;
  p.x = (const bf16_t*)x; p.a_all = (const bf16_t*)a_all; p.b_all = (const bf16_t*)b_all; p.y = (bf16_t*)y;
  p.seg_start = seg_start; p.seg_adapter = seg_adapter; p.adapter_rank = adapter_rank; p.adapter_scale = adapter_scale;
  p.K = (int)K; p.N = (int)N; p.RP = (int)RP; p.table = table;
  if (hipError_t e = kh_allow_lds<sgmv_fused_kernel>(LDS_BYTES); e != hipSuccess) return (int)e;
  // few row blocks: the column tiles of y are dealt to several workgroups (each recomputes its rows' T) until the chip is covered
  const int64_t row_wgs = ((max_seg_rows + BM - 1) / BM) * n_segments * n_layers, n_tiles = N / 128;
  int64_t z = row_wgs >= 256 ? 1 : (256 + row_wgs - 1) / row_wgs;
  z = z < n_tiles ? z : n_tiles;
  p.tiles_per_z = (int)((n_tiles + z - 1) / z);
  z = (n_tiles + p.tiles_per_z - 1) / p.tiles_per_z;
  p.z_per_layer = (int)z;
  if (z * n_layers > 65535) return KH_ERR_TOO_LARGE;
  dim3 grid((unsigned)((max_seg_rows + BM - 1) / BM), (unsigned)n_segments, (unsigned)(z * n_layers));
  kh_launch(KH_TAG_SGMV_FUSED, sgmv_fused_kernel, grid, dim3(512), LDS_BYTES, (hipStream_t)stream, p);
  KH_RETURN_LAST_ERROR();
}

}  // namespace

// See include/katz_hip.h.
KH_EXPORT int kh_sgmv_fused_bf16(const void* x, const void* a_all, const void* b_all, void* y, const int32_t* seg_start,
                                 const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                                 int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t K, int64_t RP, void* stream) {
  return sgmv_fused_impl(x, a_all, b_all, y, nullptr, 1, seg_start, seg_adapter, adapter_rank, adapter_scale, n_segments, max_seg_rows,
                         N, K, RP, stream);
}

// See include/katz_hip.h.
KH_EXPORT int kh_sgmv_fused_grouped_bf16(const void* x, const uint64_t* table, int64_t n_layers, const int32_t* seg_start,
                                         const int32_t* seg_adapter, const int32_t* adapter_rank, const float* adapter_scale,
                                         int64_t n_segments, int64_t max_seg_rows, int64_t N, int64_t K, int64_t RP, void* stream) {
  if (!table) return KH_ERR_INVALID_ARG;
  return sgmv_fused_impl(x, nullptr, nullptr, nullptr, table, n_layers, seg_start, seg_adapter, adapter_rank, adapter_scale, n_segments,
                         max_seg_rows, N, K, RP, stream);
}

// K3: flash-style attention forward on bf16 MFMA for gfx950, head_dim 64, no mask, no dropout:
//   o = softmax(q k^T * scale) v
// replacing the F.scaled_dot_product_attention call of the reference's attention processor
// (diffusers-hf/src/diffusers/models/attention_processor.py:1269-1283).  q/k/v/o are addressed in
// the projection layout [B, tokens, heads*64] (head h = columns 64h..64h+63) through explicit
// row / batch strides, so the [B,h,T,64] transposes of the reference (:1269-1272, :1280) are never
// materialised.
//
// One workgroup = 4 (or 2) waves = 128 (64) queries of one (batch, head); each wave owns 32 queries.
// Per 64-key tile (K and V^T staged in LDS, double buffered):
//   S^T = K . Q^T      (A = K fragment from LDS, B = Q fragment held in registers)
//   so every lane holds 32 scores of ONE query (query = lane%32): the row max / row sum are
//   in-lane reductions plus one exchange between the two 32-lane halves.
//   O^T += V^T . P^T   (A = V^T fragment from LDS, B = P straight from the score registers:
//   the MFMA K index is a free permutation as long as both operands agree on it.)
#include "kh_common.h"
#include <type_traits>

namespace {

constexpr int HD = 64;        // head dim
constexpr int KV = 64;        // keys per tile
constexpr int LDH = HD + 8;   // padded LDS rows (144 B)
constexpr int LDV = KV + 8;
constexpr float NEG_BIG = -1.0e30f;
constexpr float RESCALE_LOG2 = 8.0f;   // the running maximum moves only for jumps above 2^8

struct AttnParams {
  const bf16_t* q; const bf16_t* k; const bf16_t* v; bf16_t* o;
  int B, H, T, S;
  long ldq, ldk, ldv, ldo;   // row strides (elements)
  long bsq, bsk, bsv, bso;   // batch strides (elements)
  float scale_log2e;
  int q_blocks;
};

template <int NW>   // waves per workgroup: NW*32 queries
// Two waves per SIMD at least: that caps a wave at 256 registers, which makes the compiler keep MFMA results in
// VGPRs (the softmax reads them every tile; from AGPRs every score and every rescaled output costs extra moves).
__global__ __launch_bounds__(NW * 64, 2) void attention_kernel(const AttnParams p) {
  constexpr int NT = NW * 64, KCH = 512 / NT, VCH = 256 / NT;
  __shared__ __attribute__((aligned(16))) bf16_t sK[2][KV * LDH];
  __shared__ __attribute__((aligned(16))) bf16_t sVt[2][HD * LDV];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lh = lane >> 5;
  const uint32_t total = (uint32_t)p.q_blocks * p.H * p.B;
  const uint32_t logical = xcd_remap(blockIdx.x, total);
  const int qb = logical % p.q_blocks;
  const int bh = logical / p.q_blocks;
  const int h = bh % p.H, b = bh / p.H;

  const bf16_t* qp = p.q + (size_t)b * p.bsq + (size_t)h * HD;
  const bf16_t* kp = p.k + (size_t)b * p.bsk + (size_t)h * HD;
  const bf16_t* vp = p.v + (size_t)b * p.bsv + (size_t)h * HD;
  bf16_t* op = p.o + (size_t)b * p.bso + (size_t)h * HD;

  // Q fragments: query = q0 + l32, d = ks*16 + lh*8 .. +7
  const int qrow = qb * (NW * 32) + wave * 32 + l32;
  const int qrow_c = qrow < p.T ? qrow : p.T - 1;
  bf16x8 qf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
    qf[ks] = *reinterpret_cast<const bf16x8*>(qp + (size_t)qrow_c * p.ldq + ks * 16 + lh * 8);

  f32x16 oacc[2];
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[dt][v] = 0.f;
  float m_run = NEG_BIG, l_run = 0.f;

  const int n_tiles = (p.S + KV - 1) / KV;

  // staging registers: K tile = 64 keys x 8 chunks (2 per thread); V tile = 32 key pairs x 8 chunks (1 pair per thread)
  u32x4 rk[KCH], rv[VCH][2];
  // A full tile is read at (uniform tile base) + (per-thread byte offset fixed for the whole kernel): no per-tile
  // address arithmetic in the vector ALU, which is the unit this kernel is bound by.  Only a last, partial
  // tile clamps its rows.
  uint32_t koff[KCH], voff[VCH][2];
#pragma unroll
  for (int i = 0; i < KCH; ++i) {
    const int c = tid + i * NT, row = c >> 3, ch = c & 7;
    koff[i] = (uint32_t)((row * p.ldk + ch * 8) * 2);
  }
#pragma unroll
  for (int j = 0; j < VCH; ++j) {
    const int c = tid + j * NT, v_kp = c & 31, v_dch = c >> 5;
#pragma unroll
    for (int i = 0; i < 2; ++i) voff[j][i] = (uint32_t)(((2 * v_kp + i) * p.ldv + v_dch * 8) * 2);
  }
  auto load_tile = [&](int t) {
    const int s0 = t * KV;
    if (s0 + KV <= p.S) {
      const char* kb = reinterpret_cast<const char*>(kp + (size_t)s0 * p.ldk);
      const char* vb = reinterpret_cast<const char*>(vp + (size_t)s0 * p.ldv);
#pragma unroll
      for (int i = 0; i < KCH; ++i) rk[i] = *reinterpret_cast<const u32x4*>(kb + koff[i]);
#pragma unroll
      for (int j = 0; j < VCH; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i) rv[j][i] = *reinterpret_cast<const u32x4*>(vb + voff[j][i]);
      return;
    }
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + i * NT, row = c >> 3, ch = c & 7;
      int gr = s0 + row; gr = gr < p.S ? gr : p.S - 1;
      rk[i] = *reinterpret_cast<const u32x4*>(kp + (size_t)gr * p.ldk + ch * 8);
    }
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = tid + j * NT, v_kp = c & 31, v_dch = c >> 5;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        int gr = s0 + 2 * v_kp + i; gr = gr < p.S ? gr : p.S - 1;
        rv[j][i] = *reinterpret_cast<const u32x4*>(vp + (size_t)gr * p.ldv + v_dch * 8);
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      const int c = tid + i * NT, row = c >> 3, ch = c & 7;
      *reinterpret_cast<u32x4*>(&sK[buf][row * LDH + ch * 8]) = rk[i];
    }
    // transpose: element e of the pair (key 2kp, key 2kp+1) -> sVt[d = dch*8+e][2kp .. 2kp+1] as one dword
    uint32_t* dst = reinterpret_cast<uint32_t*>(&sVt[buf][0]);
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = tid + j * NT, v_kp = c & 31, v_dch = c >> 5;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t a = rv[j][0][w], c2 = rv[j][1][w];
        const uint32_t lo = (a & 0xffffu) | (c2 << 16);          // d = dch*8 + 2w
        const uint32_t hi = (a >> 16) | (c2 & 0xffff0000u);      // d = dch*8 + 2w + 1
        dst[((v_dch * 8 + 2 * w) * LDV) / 2 + v_kp] = lo;
        dst[((v_dch * 8 + 2 * w + 1) * LDV) / 2 + v_kp] = hi;
      }
    }
  };

  load_tile(0);
  store_tile(0);
  __syncthreads();

  // One 64-key tile.  MASK: the tile may reach beyond S (only the last one can).
  auto tile_step = [&](int t, auto mask_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const int buf = t & 1;
    if (t + 1 < n_tiles) load_tile(t + 1);

    // S^T tiles: st[kt][v] : key = t*64 + kt*32 + 8*(v/4) + 4*lh + v%4, query = l32
    f32x16 st[2];
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(&sK[buf][(kt * 32 + l32) * LDH + ks * 16 + lh * 8]);
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], ks == 0 ? zero : st[kt], 0, 0, 0);
      }
    }
    if constexpr (MASK) {
      const int s0 = t * KV;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = s0 + kt * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
          if (key >= p.S) st[kt][v] = NEG_BIG;
        }
    }
    float mx = NEG_BIG;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, st[kt][v]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // Lazy running maximum: the reference point of the exponentials only moves when the row maximum has grown by
    // more than 2^RESCALE_LOG2 in the exponent domain; until then p = exp2(s - m) may exceed 1 (by at most that
    // factor, harmless in fp32 / bf16) and numerator and denominator stay consistent.  Moving it rescales
    // the 32 output accumulators, which is then rare -- and skipped for the whole wave when no lane moves.
    const bool move = (mx - m_run) * p.scale_log2e > RESCALE_LOG2;
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float m_new = move ? mx : m_run;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * p.scale_log2e);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
    }
    const float mb = m_run * p.scale_log2e;
    bf16x8 pf[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int v = 0; v < 16; v += 2) {
        const float e0 = __builtin_amdgcn_exp2f(st[kt][v] * p.scale_log2e - mb);
        const float e1 = __builtin_amdgcn_exp2f(st[kt][v + 1] * p.scale_log2e - mb);
        pf[kt][v >> 3][v & 7] = (bf16_t)e0;
        pf[kt][v >> 3][(v & 7) + 1] = (bf16_t)e1;
      }
    // O^T += V^T . P^T : A fragment row d = dt*32 + l32, element e <-> key kt*32 + 8*(2s + e/4) + 4*lh + e%4.
    // Row sums ride along on the matrix pipe, which has cycles to spare here (the vector ALU does not):
    // ones^T . P^T puts sum_k P[k][q] of all 64 keys (both lane halves) into every row of column q, i.e. into every
    // register of the lanes of query q.  The denominator is then the sum of the same rounded P values the numerator
    // uses.  Its MFMAs sit between those of the two output tiles, so nothing waits on their dependency chain.
    const bf16_t one = (bf16_t)1.0f;
    const bf16x8 ones = {one, one, one, one, one, one, one, one};
    f32x16 rsum = zero;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          const bf16_t* base = &sVt[buf][(dt * 32 + l32) * LDV + kt * 32 + 16 * s + 4 * lh];
          const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(base);
          const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(base + 8);
          bf16x8 vf;
#pragma unroll
          for (int e = 0; e < 4; ++e) { vf[e] = v0[e]; vf[4 + e] = v1[e]; }
          oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kt][s], oacc[dt], 0, 0, 0);
        }
        rsum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf[kt][s], rsum, 0, 0, 0);
      }
    l_run += rsum[0];

    if (t + 1 < n_tiles) store_tile(buf ^ 1);
    __syncthreads();
  };
  const int full_tiles = p.S / KV;
  for (int t = 0; t < full_tiles; ++t) tile_step(t, std::false_type{});
  if (full_tiles < n_tiles) tile_step(full_tiles, std::true_type{});

  const float inv = 1.0f / l_run;   // the MFMA row sums already cover the keys of both lane halves
  // A lane holds runs of 4 dims (8 bytes); lanes l and l + 32 hold the two halves of every 16-byte piece of their query's
  // row.  Two pieces at a time, the pair trades halves (v_permlane32_swap: the upper half of the first register against the
  // lower half of the second), after which lane l owns the even piece and lane l + 32 the odd one: 16-byte stores.
#if __HIP_DEVICE_COMPILE__
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int gp = 0; gp < 2; ++gp) {
      const int ge = 2 * gp, go = 2 * gp + 1;
      const uint32_t e0 = pack_bf16x2(oacc[dt][4 * ge + 0] * inv, oacc[dt][4 * ge + 1] * inv);
      const uint32_t e1 = pack_bf16x2(oacc[dt][4 * ge + 2] * inv, oacc[dt][4 * ge + 3] * inv);
      const uint32_t o0 = pack_bf16x2(oacc[dt][4 * go + 0] * inv, oacc[dt][4 * go + 1] * inv);
      const uint32_t o1 = pack_bf16x2(oacc[dt][4 * go + 2] * inv, oacc[dt][4 * go + 3] * inv);
      const auto s0 = __builtin_amdgcn_permlane32_swap(e0, o0, false, false);
      const auto s1 = __builtin_amdgcn_permlane32_swap(e1, o1, false, false);
      const u32x4 piece = {s0[0], s1[0], s0[1], s1[1]};
      if (qrow < p.T) {
        const size_t off = (size_t)qrow * p.ldo + dt * 32 + 8 * (2 * gp + lh);
        *reinterpret_cast<u32x4*>(op + off) = piece;   // (plain: written through the L2, 32 bytes of a row at a time gained nothing)
      }
    }
#endif
}

}  // namespace

KH_EXPORT int kh_attention_bf16(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t T,
                                int64_t S, int64_t head_dim, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo,
                                int64_t bsq, int64_t bsk, int64_t bsv, int64_t bso, float scale, void* stream) {
  if (!q || !k || !v || !o || B <= 0 || H <= 0 || T <= 0 || S <= 0) return KH_ERR_INVALID_ARG;
  if (head_dim != HD) return KH_ERR_UNSUPPORTED;
  if ((ldq | ldk | ldv | ldo | bsq | bsk | bsv | bso) % 8 != 0) return KH_ERR_ALIGNMENT;
  if (ldq < H * HD || ldk < H * HD || ldv < H * HD || ldo < H * HD) return KH_ERR_INVALID_ARG;
  if (!kh_aligned16(q) || !kh_aligned16(k) || !kh_aligned16(v) || !kh_aligned16(o)) return KH_ERR_ALIGNMENT;
  AttnParams p;
  p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.o = (bf16_t*)o;
  p.B = (int)B; p.H = (int)H; p.T = (int)T; p.S = (int)S;
  p.ldq = ldq; p.ldk = ldk; p.ldv = ldv; p.ldo = ldo;
  p.bsq = bsq; p.bsk = bsk; p.bsv = bsv; p.bso = bso;
  p.scale_log2e = scale * 1.4426950408889634f;
  // 128 queries per workgroup; 64 for short key sequences on small grids (cross-attention), for a finer spread
  const bool small = ((T + 127) / 128) * H * B < 512 && S <= 256;
  const int qpw = small ? 64 : 128;
  p.q_blocks = (int)((T + qpw - 1) / qpw);
  const long grid = (long)p.q_blocks * H * B;
  if (grid > 0x7fffffffL) return KH_ERR_TOO_LARGE;
  if (small)
    kh_launch(KH_TAG_ATTENTION, attention_kernel<2>, dim3((unsigned)grid), dim3(128), 0, (hipStream_t)stream, p);
  else
    kh_launch(KH_TAG_ATTENTION, attention_kernel<4>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, p);
  KH_RETURN_LAST_ERROR();
}

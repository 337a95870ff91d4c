// Shared device/host helpers for the katz_hip kernels (gfx950 / CDNA4 only).
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <hip/hip_ext.h>
#include <stdint.h>

#define KH_OK 0
#define KH_ERR_INVALID_ARG (-1)
#define KH_ERR_UNSUPPORTED (-2)
#define KH_ERR_ALIGNMENT (-3)
#define KH_ERR_TOO_LARGE (-4)

#define KH_EXPORT extern "C" __attribute__((visibility("default")))

// Launch-error check: kernels are asynchronous, so only launch-time errors are
// visible here; a positive return value is the hipError_t.
#define KH_RETURN_LAST_ERROR()                      \
  do {                                              \
    hipError_t e__ = hipGetLastError();             \
    return e__ == hipSuccess ? KH_OK : (int)e__;    \
  } while (0)

// hipFuncAttributeMaxDynamicSharedMemorySize is a setting per device: remembered per kernel and device, so a process
// that drives several GPUs sets it on each (devices beyond 63: set on every launch).
template <auto Kernel>
inline hipError_t kh_allow_lds(int bytes) {
  static std::atomic<uint64_t> done{0};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev >= 0 && dev < 64 && ((done.load(std::memory_order_relaxed) >> dev) & 1)) return hipSuccess;
  e = hipFuncSetAttribute((const void*)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && dev >= 0 && dev < 64) done.fetch_or(1ull << dev, std::memory_order_relaxed);
  return e;
}

// ---- optional per-launch timing (host) -----------------------------------------------------------
// While profiling is on (kh_profile_begin .. kh_profile_end) every kernel goes out through
// hipExtLaunchKernelGGL with its own start/stop event pair, which time exactly that dispatch on the
// stream it was launched on.  Off (the default) launches are plain and graph-capturable.
enum KhKernelTag {
  KH_TAG_LORA_GEMM = 1, KH_TAG_LORA_GEMM_F32 = 2, KH_TAG_ATTENTION = 3, KH_TAG_GN_STATS = 4, KH_TAG_GN_APPLY = 5,
  KH_TAG_LAYER_NORM = 6, KH_TAG_GEGLU = 7, KH_TAG_RESIDUAL_ADD = 8, KH_TAG_CONCAT_RESIDUAL = 9,
  KH_TAG_SGMV_SHRINK = 10, KH_TAG_SGMV_EXPAND = 11, KH_TAG_LORA_SHRINK = 12, KH_TAG_CONV = 13, KH_TAG_CFG_EULER = 14,
  KH_TAG_UPSAMPLE = 15, KH_TAG_LORA_MERGE = 16, KH_TAG_CONV_OUT_STEP = 17, KH_TAG_SGMV_FUSED = 18
};
bool kh_prof_enabled();
void kh_prof_events(int tag, hipEvent_t* start, hipEvent_t* stop);

template <typename F, typename... Args>
inline void kh_launch(int tag, F kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, Args... args) {
  // hipGetLastError is per thread and sticky across libraries: drop whatever an earlier, unrelated
  // runtime call left behind so that the check after the launch reports this launch only.
  (void)hipGetLastError();
  if (kh_prof_enabled()) {
    hipEvent_t a, b;
    kh_prof_events(tag, &a, &b);
    hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, a, b, 0, args...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
  }
}

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// A kernel's results, stored THROUGH the L2 at agent scope (`sc1`: the line stays in the L2 and the data moves on to the
// memory side at once).  With plain stores a launch's dirty lines leave the eight L2s when the launch ends, all at the same
// moment and with nothing to overlap them; written through, they leave while other waves still compute.  Only for 16-byte
// pieces that fill whole rows (8-byte pieces that complete a line over several instructions got slower).  The store is the
// compiler's own buffer store with a cache-policy operand, NOT inline assembly: a hand-written `global_store_dwordx4` is
// invisible to the compiler's hazard recogniser, which otherwise keeps the next vector instruction from overwriting the
// data registers of a store wider than 8 bytes during its first two wait states -- such stores wrote garbage now and then.
// Offsets are 32 bits: outputs of 4 GiB and more take plain stores.
#if __HIP_DEVICE_COMPILE__
struct KhOut {
  __amdgpu_buffer_rsrc_t rs;
  char* base;
  bool wt;
  __device__ __forceinline__ KhOut(void* y, size_t bytes)
      : rs(__builtin_amdgcn_make_buffer_rsrc(y, 0, (int)(uint32_t)(bytes < 0xFFFFFFFFull ? bytes : 0), 0x00020000)),
        base(reinterpret_cast<char*>(y)),
#if defined(KH_PLAIN_STORES)   // build-time switch back to plain stores (python -m katz_amd.build with -DKH_PLAIN_STORES in HIPCC_FLAGS)
        wt(false) {}
#else
        wt(bytes < 0xFFFFFFFFull) {}
#endif
  __device__ __forceinline__ void store16(size_t byte_off, const u32x4 v) const {
    if (wt) __builtin_amdgcn_raw_buffer_store_b128(v, rs, (int)(uint32_t)byte_off, 0, 16 /* sc1 */);
    else *reinterpret_cast<u32x4*>(base + byte_off) = v;
  }
};
#else
struct KhOut {   // the host pass only parses the kernels
  char* base;
  __host__ __device__ KhOut(void* y, size_t) : base(reinterpret_cast<char*>(y)) {}
  __host__ __device__ void store16(size_t byte_off, const u32x4 v) const { *reinterpret_cast<u32x4*>(base + byte_off) = v; }
};
#endif

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) {
  return __uint_as_float(lo16 << 16);
}
// Low / high bf16 of a packed 32-bit word, widened to fp32.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Round-to-nearest-even fp32 -> bf16 (the compiler emits v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  bf16x2 v;
  v[0] = (bf16_t)a;
  v[1] = (bf16_t)b;
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float a) {
  bf16_t v = (bf16_t)a;
  return __builtin_bit_cast(uint16_t, v);
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }

static inline bool kh_aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

// gelu(x) = 0.5 x (1 + erf(x / sqrt 2)) with erf from Abramowitz & Stegun 7.1.26 (|abs error| <= 1.5e-7, far inside
// the bf16 rounding the result goes through): a reciprocal, an exp2 and five FMAs instead of the library erff.
__device__ __forceinline__ float kh_gelu_erf(float x) {
  const float z = fabsf(x) * 0.70710678118654752f;
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
  const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
  const float e = poly * __builtin_amdgcn_exp2f(-1.4426950408889634f * z * z);   // 1 - erf(z)
  const float half_x = 0.5f * x;
  return x >= 0.f ? half_x * (2.0f - e) : half_x * e;
}

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2). Map a
// hardware block id to a logical tile id such that every XCD walks one
// contiguous range of logical tiles, so neighbouring tiles share an L2.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t bid, uint32_t total) {
  const uint32_t NX = 8;
  uint32_t xcd = bid % NX, local = bid / NX;
  uint32_t per = total / NX, rem = total % NX;
  return xcd * per + (xcd < rem ? xcd : rem) + local;
}

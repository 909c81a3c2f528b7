// Shared host/device helpers for libshareprefill_hip (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "shareprefill_hip.h"
#include "shareprefill_hip_diag.h"

#define SP_WAVE 64

// ---- host-side error plumbing -------------------------------------------------------------------
void sp_set_error(const char* fmt, ...);

#define SP_REQUIRE(cond, code, ...)  \
  do {                               \
    if (!(cond)) {                   \
      sp_set_error(__VA_ARGS__);     \
      return (code);                 \
    }                                \
  } while (0)

#define SP_HIP(call)                                                                           \
  do {                                                                                         \
    hipError_t e_ = (call);                                                                    \
    if (e_ != hipSuccess) {                                                                    \
      sp_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
      return SP_ERR_HIP;                                                                       \
    }                                                                                          \
  } while (0)

#define SP_LAUNCH_CHECK() SP_HIP(hipGetLastError())

__host__ __device__ static inline int64_t sp_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// 1/sqrt(head_dim) of the selection: from the head_dim named in bits 8..15 of flags (units of 8) when the tensors'
// head_dim axis is zero-padded, else from the tensors' own d
static inline float sp_inv_sqrt_dim(uint32_t flags, int d) {
  const int named = (int)((flags >> 8) & 0xffu) * 8;
  return 1.0f / sqrtf((float)(named ? named : d));
}

// ---- kernels of one source file launched from another ----
// pooled block probabilities of query-aware heads on the matrix core (sp_scores.hip), head_dim 128
int sp_block_probs_mfma_launch(const void* qbar, const void* kbar, const int32_t* decision, int32_t hq, int32_t hkv,
                               int32_t nb, uint32_t flags, float* probs, hipStream_t stream);

// ---- bf16 <-> fp32 -------------------------------------------------------------------------------
typedef uint16_t sp_bf16;

__host__ __device__ static inline float sp_bf16_to_f32(sp_bf16 v) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = ((uint32_t)v) << 16;
  return c.f;
}

// round-to-nearest-even, NaN kept quiet
__host__ __device__ static inline sp_bf16 sp_f32_to_bf16(float f) {
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  uint32_t u = c.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return (sp_bf16)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (sp_bf16)(u >> 16);
}

__host__ __device__ static inline float sp_round_bf16(float f) { return sp_bf16_to_f32(sp_f32_to_bf16(f)); }

__host__ __device__ static inline uint32_t sp_f32_bits(float f) {
  union {
    uint32_t u;
    float f;
  } c;
  c.f = f;
  return c.u;
}

// ---- cumulative-mass fixed point -----------------------------------------------------------------
#define SP_FX_BITS 48
#define SP_FX_SAT (1ull << 62)

// order key: fp32 bit pattern; NaN and anything with the sign bit set -> 0
__host__ __device__ static inline uint32_t sp_sort_key(float f) {
  uint32_t u = sp_f32_bits(f);
  if ((u >> 31) || (u & 0x7fffffffu) > 0x7f800000u) return 0u;
  return u;
}

// floor(f * 2^48) for finite f >= 0, saturating at 2^62; NaN / negative -> 0
__host__ __device__ static inline uint64_t sp_to_fixed(float f) {
  uint32_t u = sp_f32_bits(f);
  if (u >> 31) return 0ull;
  uint32_t e = u >> 23;
  if (e == 0u) return 0ull;                                    // zero / subnormal: below 2^-48
  if (e == 255u) return (u & 0x7fffffu) ? 0ull : SP_FX_SAT;    // NaN -> 0, +inf saturates
  uint64_t m = (uint64_t)((u & 0x7fffffu) | 0x800000u);        // value = m * 2^(e-150)
  int sh = (int)e - 150 + SP_FX_BITS;
  if (sh >= 39) return SP_FX_SAT;                              // >= 2^14
  if (sh >= 0) return m << sh;
  if (sh <= -24) return 0ull;
  return m >> (-sh);
}

// thresholds: largest fixed-point sum S with S*2^-48 <= thr (le) or < thr (lt); host only
static inline int64_t sp_thr_le(float thr) {
  double t = (double)thr * 281474976710656.0;
  if (!(t >= 0.0)) return -1;
  if (t >= 9.0e18) return INT64_MAX;
  return (int64_t)__builtin_floor(t);
}
static inline int64_t sp_thr_lt(float thr) {
  double t = (double)thr * 281474976710656.0;
  if (!(t > 0.0)) return -1;
  if (t >= 9.0e18) return INT64_MAX;
  return (int64_t)__builtin_ceil(t) - 1;
}

// ---- wave / block reductions ------------------------------------------------------------------------
__device__ static inline float sp_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, SP_WAVE);
  return v;
}
__device__ static inline float sp_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, SP_WAVE));
  return v;
}

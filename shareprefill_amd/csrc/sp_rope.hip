// Rotary position embedding applied in place to the projected queries and keys, the step in front of the
// attention function: the reference's patched model computes (cos, sin) per position (model_patch.py:121) and the
// Hugging Face attention layer then evaluates
//     x_embed = (x * cos) + (rotate_half(x) * sin),   rotate_half(x) = cat(-x[d/2:], x[:d/2])
// as five elementwise bf16 kernels per tensor.  This kernel does the same arithmetic in one pass over q and k --
// every product and the sum rounded to bf16 exactly where the elementwise kernels round, so the result is
// bit-identical -- reading and writing each element once.  Bound = HBM: 2 * (Hq + Hkv) * N * D * 2 bytes.
#include "sp_common.h"

#define RP_THREADS 256
#define RP_HEAD_LANES 8  // threads that share one (token, chunk pair) and split the heads between them
#define RP_BATCH 5       // heads a thread has in flight at once (8 x 5 = the 32 + 8 heads of an 8B Llama in one go)

typedef uint32_t rp_u32x4 __attribute__((ext_vector_type(4)));

// bf16 pair (lo, hi) of one 32-bit word -> two floats
__device__ static inline float rp_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ static inline float rp_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// round(round(a * ca) + sign * round(b * sb)) on both halves of a word, every rounding to bf16 (nearest even)
__device__ static inline uint32_t rp_word(uint32_t a, uint32_t ca, uint32_t b, uint32_t sb, float sign) {
  const float p0 = sp_round_bf16(rp_lo(a) * rp_lo(ca)), r0 = sign * sp_round_bf16(rp_lo(b) * rp_lo(sb));
  const float p1 = sp_round_bf16(rp_hi(a) * rp_hi(ca)), r1 = sign * sp_round_bf16(rp_hi(b) * rp_hi(sb));
  return (uint32_t)sp_f32_to_bf16(p0 + r0) | ((uint32_t)sp_f32_to_bf16(p1 + r1) << 16);
}

// A thread owns one chunk pair (8 channels of the first half of the head with their partners in the second half) of
// one token, keeps that position's cos / sin in registers and walks heads hl, hl + 8, ... of q and k alike, a batch
// of loads ahead of the arithmetic.  A wave's 64 lanes cover 8 adjacent heads of one token: whole 128-byte lines.
__global__ __launch_bounds__(RP_THREADS) void sp_rope_kernel(sp_bf16* __restrict__ q, sp_bf16* __restrict__ k,
                                                             const sp_bf16* __restrict__ cos_t,
                                                             const sp_bf16* __restrict__ sin_t, int64_t n, int hq,
                                                             int hkv, int d, int64_t sq_n, int64_t sq_h, int64_t sk_n,
                                                             int64_t sk_h, int64_t scs_n, int tokens_per_wg) {
  const int half = d >> 1;
  const int cpd = d >> 4;  // chunk pairs per head
  const int heads = hq + hkv;
  const int64_t tok0 = (int64_t)blockIdx.x * tokens_per_wg;
  const int items = tokens_per_wg * RP_HEAD_LANES * cpd;
  for (int j = threadIdx.x; j < items; j += RP_THREADS) {
    const int c = j % cpd, hl = (j / cpd) % RP_HEAD_LANES;
    const int64_t tok = tok0 + j / (cpd * RP_HEAD_LANES);
    if (tok >= n) break;
    const sp_bf16* cr = cos_t + tok * scs_n;
    const sp_bf16* sr = sin_t + tok * scs_n;
    const rp_u32x4 c1 = *reinterpret_cast<const rp_u32x4*>(cr + 8 * c);
    const rp_u32x4 c2 = *reinterpret_cast<const rp_u32x4*>(cr + half + 8 * c);
    const rp_u32x4 s1 = *reinterpret_cast<const rp_u32x4*>(sr + 8 * c);
    const rp_u32x4 s2 = *reinterpret_cast<const rp_u32x4*>(sr + half + 8 * c);
    sp_bf16* qrow = q + tok * sq_n + 8 * c;
    sp_bf16* krow = k + tok * sk_n + 8 * c;
    for (int h0 = hl; h0 < heads; h0 += RP_HEAD_LANES * RP_BATCH) {
      rp_u32x4 x1[RP_BATCH], x2[RP_BATCH];
      sp_bf16* xp[RP_BATCH];
#pragma unroll
      for (int u = 0; u < RP_BATCH; ++u) {
        const int hs = h0 + u * RP_HEAD_LANES;
        xp[u] = hs < hq ? qrow + (int64_t)hs * sq_h : krow + (int64_t)(hs - hq) * sk_h;
        if (hs < heads) {
          x1[u] = *reinterpret_cast<const rp_u32x4*>(xp[u]);
          x2[u] = *reinterpret_cast<const rp_u32x4*>(xp[u] + half);
        }
      }
#pragma unroll
      for (int u = 0; u < RP_BATCH; ++u) {
        if (h0 + u * RP_HEAD_LANES < heads) {
          rp_u32x4 o1, o2;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            o1[w] = rp_word(x1[u][w], c1[w], x2[u][w], s1[w], -1.0f);  // first half:  x1 * cos + (-x2) * sin
            o2[w] = rp_word(x2[u][w], c2[w], x1[u][w], s2[w], 1.0f);   // second half: x2 * cos +   x1  * sin
          }
          *reinterpret_cast<rp_u32x4*>(xp[u]) = o1;
          *reinterpret_cast<rp_u32x4*>(xp[u] + half) = o2;
        }
      }
    }
  }
}

extern "C" int sp_rope_inplace_bf16(void* q, void* k, const void* cos_t, const void* sin_t, int64_t n, int32_t hq,
                                    int32_t hkv, int32_t d, int64_t q_stride_n, int64_t q_stride_h,
                                    int64_t k_stride_n, int64_t k_stride_h, int64_t cs_stride_n, sp_stream_t stream) {
  SP_REQUIRE(n >= 0 && hq >= 0 && hkv >= 0 && hq + hkv > 0, SP_ERR_INVALID_ARGUMENT,
             "sp_rope_inplace_bf16: n=%lld hq=%d hkv=%d", (long long)n, hq, hkv);
  SP_REQUIRE(d > 0 && d % 16 == 0 && d <= 512, SP_ERR_UNSUPPORTED,
             "sp_rope_inplace_bf16: head_dim %d (a multiple of 16 up to 512 is required)", d);
  if (n == 0) return SP_OK;
  SP_REQUIRE(cos_t && sin_t && (q || hq == 0) && (k || hkv == 0), SP_ERR_INVALID_ARGUMENT,
             "sp_rope_inplace_bf16: null pointer");
  SP_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)cos_t | (uintptr_t)sin_t) % 16 == 0 &&
                 (q_stride_n | q_stride_h | k_stride_n | k_stride_h | cs_stride_n) % 8 == 0,
             SP_ERR_INVALID_ARGUMENT, "sp_rope_inplace_bf16: pointers and strides must be 16-byte aligned");
  const int per_token = RP_HEAD_LANES * (d / 16);  // threads that work on one token
  const int tokens_per_wg = per_token >= RP_THREADS ? 1 : RP_THREADS / per_token;
  const int64_t blocks = sp_ceil_div(n, tokens_per_wg);
  SP_REQUIRE(blocks <= 0x7fffffffll, SP_ERR_UNSUPPORTED, "sp_rope_inplace_bf16: n=%lld too long", (long long)n);
  hipLaunchKernelGGL(sp_rope_kernel, dim3((unsigned)blocks), dim3(RP_THREADS), 0, (hipStream_t)stream,
                     (sp_bf16*)q, (sp_bf16*)k, (const sp_bf16*)cos_t, (const sp_bf16*)sin_t, n, hq, hkv, d,
                     q_stride_n, q_stride_h, k_stride_n, k_stride_h, cs_stride_n, tokens_per_wg);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// Decode step: one query token per head against the whole KV cache (GQA, no mask), bf16 in / bf16 out, fp32
// softmax.  Replaces the flash_attn_func call of the reference's decode branch (shareprefill_attn.py:146-155).
//
// HBM-bound: K and V are read exactly once (2 * n * hkv * d * 2 bytes); everything else is noise.  The cache of
// one kv head is split into chunks; one workgroup streams a chunk for all query heads of the group (so the
// group's `g` heads share every K / V byte), keeps an online softmax, and leaves an unnormalised partial
// (o, m, l); a second tiny kernel merges the partials in chunk order.  No matrix core: with at most 8 query rows
// the products are a few hundred FMAs per thread and tile.
#include "sp_common.h"

#define DC_THREADS 256
#define DC_TILE 128  // keys per tile
#define DC_D 128
#define DC_GMAX 8    // query heads per kv head

typedef uint32_t dc_u32x4 __attribute__((ext_vector_type(4)));

__device__ static __forceinline__ float dc_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ static __forceinline__ float dc_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// grid (splits, hkv); partial layout: o [hkv][splits][g][128] fp32, ml [hkv][splits][g] float2 (m in log2 units, l)
__global__ __launch_bounds__(DC_THREADS, 2) void sp_decode_partial_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const sp_bf16* __restrict__ v, int64_t n, int g,
    int64_t sq_h, int64_t sk_n, int64_t sk_h, int64_t sv_n, int64_t sv_h, float scale_log2, int64_t keys_per_split,
    float* __restrict__ o_part, float2* __restrict__ ml_part) {
  __shared__ float Qs[DC_GMAX][DC_D];     // the group's queries, fp32
  __shared__ float Ps[DC_GMAX][DC_TILE];  // logits, then probabilities of the current tile
  __shared__ float alpha_s[DC_GMAX];
  __shared__ float red[4][DC_GMAX][DC_D];  // cross-wave reduction of the output partials (16 KiB)
  const int split = blockIdx.x, kvh = blockIdx.y, splits = gridDim.x;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const sp_bf16* kh = k + (int64_t)kvh * sk_h;
  const sp_bf16* vh = v + (int64_t)kvh * sv_h;
  for (int i = t; i < g * DC_D; i += DC_THREADS)
    Qs[i / DC_D][i % DC_D] = sp_bf16_to_f32(q[(int64_t)(kvh * g + i / DC_D) * sq_h + i % DC_D]);
  __syncthreads();

  const int64_t key_begin = (int64_t)split * keys_per_split;
  int64_t key_end = key_begin + keys_per_split;
  if (key_end > n) key_end = n;

  // roles: logits -- thread handles key t/2, channel half t%2;  softmax -- head t/32, keys 4*(t%32)..+3;
  //        output -- thread handles channels 8*(t%16)..+7 for keys t/16, t/16+16, ...
  const int qk_key = t >> 1, qk_half = t & 1;
  const int sm_head = t >> 5, sm_k0 = (t & 31) * 4;
  const int pv_chunk = t & 15, pv_sub = t >> 4;
  float acc[DC_GMAX][8];
#pragma unroll
  for (int h = 0; h < DC_GMAX; ++h)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[h][j] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // of head sm_head (replicated over its 32 threads)

  for (int64_t kb = key_begin; kb < key_end; kb += DC_TILE) {
    // ---- loads of this tile: K half row for the logits, eight V chunks for the output ----
    dc_u32x4 kr[8], vr[8];
    {
      int64_t key = kb + qk_key;
      if (key > n - 1) key = n - 1;
      const dc_u32x4* src = reinterpret_cast<const dc_u32x4*>(kh + key * sk_n + qk_half * 64);
#pragma unroll
      for (int i = 0; i < 8; ++i) kr[i] = src[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int64_t vk = kb + pv_sub + 16 * i;
        if (vk > n - 1) vk = n - 1;
        vr[i] = *reinterpret_cast<const dc_u32x4*>(vh + vk * sv_n + pv_chunk * 8);
      }
    }
    // ---- logits: s[h] = q_h . k over this thread's 64 channels, summed with the partner thread ----
    float s[DC_GMAX];
#pragma unroll
    for (int h = 0; h < DC_GMAX; ++h) s[h] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float kf[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        kf[2 * j] = dc_lo(kr[i][j]);
        kf[2 * j + 1] = dc_hi(kr[i][j]);
      }
#pragma unroll
      for (int h = 0; h < DC_GMAX; ++h) {
        if (h < g) {
          const float4 qa = *reinterpret_cast<const float4*>(&Qs[h][qk_half * 64 + i * 8]);
          const float4 qb = *reinterpret_cast<const float4*>(&Qs[h][qk_half * 64 + i * 8 + 4]);
          s[h] += kf[0] * qa.x + kf[1] * qa.y + kf[2] * qa.z + kf[3] * qa.w + kf[4] * qb.x + kf[5] * qb.y +
                  kf[6] * qb.z + kf[7] * qb.w;
        }
      }
    }
    const bool key_ok = kb + qk_key < key_end;
#pragma unroll
    for (int h = 0; h < DC_GMAX; ++h) {
      if (h < g) {
        const float tot = s[h] + __shfl_xor(s[h], 1, SP_WAVE);
        if (qk_half == 0) Ps[h][qk_key] = key_ok ? tot * scale_log2 : -INFINITY;
      }
    }
    __syncthreads();
    // ---- online softmax per head (32 threads a head, fixed xor tree) ----
    if (sm_head < g) {
      float4 sv = *reinterpret_cast<const float4*>(&Ps[sm_head][sm_k0]);
      float mx = fmaxf(fmaxf(sv.x, sv.y), fmaxf(sv.z, sv.w));
#pragma unroll
      for (int o = 1; o < 32; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, SP_WAVE));
      const float m_new = fmaxf(m_run, mx);  // finite: the tile holds at least one real key
      sv.x = __builtin_amdgcn_exp2f(sv.x - m_new);
      sv.y = __builtin_amdgcn_exp2f(sv.y - m_new);
      sv.z = __builtin_amdgcn_exp2f(sv.z - m_new);
      sv.w = __builtin_amdgcn_exp2f(sv.w - m_new);
      float ls = (sv.x + sv.y) + (sv.z + sv.w);
#pragma unroll
      for (int o = 1; o < 32; o <<= 1) ls += __shfl_xor(ls, o, SP_WAVE);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first tile (m_run = -inf)
      l_run = l_run * alpha + ls;
      m_run = m_new;
      *reinterpret_cast<float4*>(&Ps[sm_head][sm_k0]) = sv;
      if ((t & 31) == 0) alpha_s[sm_head] = alpha;
    }
    __syncthreads();
    // ---- output: acc[h][ch] = acc * alpha_h + sum_keys p[h][key] * v[key][ch] ----
#pragma unroll
    for (int h = 0; h < DC_GMAX; ++h) {
      if (h < g) {
        const float a = alpha_s[h];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[h][j] *= a;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float vf[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        vf[2 * j] = dc_lo(vr[i][j]);
        vf[2 * j + 1] = dc_hi(vr[i][j]);
      }
#pragma unroll
      for (int h = 0; h < DC_GMAX; ++h) {
        if (h < g) {
          const float p = Ps[h][pv_sub + 16 * i];  // 0 for keys past the chunk
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[h][j] += p * vf[j];
        }
      }
    }
    __syncthreads();  // Ps / alpha_s are rewritten by the next tile
  }

  // ---- reduce the 16 key groups: inside the wave (lanes l, l^16, l^32, l^48), then across the four waves ----
#pragma unroll
  for (int h = 0; h < DC_GMAX; ++h) {
    if (h < g) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float x = acc[h][j];
        x += __shfl_xor(x, 16, SP_WAVE);
        x += __shfl_xor(x, 32, SP_WAVE);
        if (lane < 16) red[wave][h][pv_chunk * 8 + j] = x;
      }
    }
  }
  __syncthreads();
  float* op = o_part + (((int64_t)kvh * splits + split) * g) * DC_D;
  for (int i = t; i < g * DC_D; i += DC_THREADS) {
    const int h = i / DC_D, c = i % DC_D;
    op[i] = (red[0][h][c] + red[1][h][c]) + (red[2][h][c] + red[3][h][c]);
  }
  if (sm_head < g && (t & 31) == 0)
    ml_part[((int64_t)kvh * splits + split) * g + sm_head] = make_float2(m_run, l_run);
}

// one workgroup of 128 threads per query head: merges the chunk partials in chunk order
__global__ __launch_bounds__(DC_D) void sp_decode_combine_kernel(const float* __restrict__ o_part,
                                                                 const float2* __restrict__ ml_part, int g, int splits,
                                                                 sp_bf16* __restrict__ out) {
  const int hq_idx = blockIdx.x, kvh = hq_idx / g, h = hq_idx % g, c = threadIdx.x;
  float m = -INFINITY;
  for (int s = 0; s < splits; ++s) m = fmaxf(m, ml_part[((int64_t)kvh * splits + s) * g + h].x);
  float l = 0.f, o = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float2 ml = ml_part[((int64_t)kvh * splits + s) * g + h];
    if (ml.x == -INFINITY) continue;  // empty chunk
    const float w = __builtin_amdgcn_exp2f(ml.x - m);
    l += ml.y * w;
    o += o_part[(((int64_t)kvh * splits + s) * g + h) * DC_D + c] * w;
  }
  out[(int64_t)hq_idx * DC_D + c] = sp_f32_to_bf16(o / l);
}

// ---- host -------------------------------------------------------------------------------------------------
static int dc_splits(int64_t n, int32_t hkv) {
  const int64_t tiles = sp_ceil_div(n, DC_TILE);
  int64_t want = sp_ceil_div(512, hkv);  // about two workgroups per CU
  if (want > tiles) want = tiles;
  if (want < 1) want = 1;
  return (int)want;
}

extern "C" size_t sp_decode_workspace_bytes(int64_t n, int32_t hq, int32_t hkv) {
  if (n <= 0 || hq <= 0 || hkv <= 0) return 0;
  return (size_t)dc_splits(n, hkv) * hq * (DC_D * sizeof(float) + sizeof(float2));
}

extern "C" int sp_decode_attn_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv,
                                   int32_t d, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                                   int64_t v_stride_n, int64_t v_stride_h, float softmax_scale, void* out,
                                   void* workspace, size_t workspace_bytes, sp_stream_t stream) {
  SP_REQUIRE(q && k && v && out && workspace, SP_ERR_INVALID_ARGUMENT, "sp_decode_attn_bf16: null pointer");
  SP_REQUIRE(n > 0 && hq > 0 && hkv > 0 && hq % hkv == 0, SP_ERR_INVALID_ARGUMENT,
             "sp_decode_attn_bf16: bad shape n=%lld hq=%d hkv=%d", (long long)n, hq, hkv);
  SP_REQUIRE(softmax_scale > 0.f, SP_ERR_INVALID_ARGUMENT, "sp_decode_attn_bf16: softmax_scale must be > 0");
  SP_REQUIRE(d == DC_D, SP_ERR_UNSUPPORTED, "sp_decode_attn_bf16: head_dim %d unsupported (only 128)", d);
  SP_REQUIRE(hq / hkv <= DC_GMAX, SP_ERR_UNSUPPORTED, "sp_decode_attn_bf16: more than %d query heads per kv head",
             DC_GMAX);
  SP_REQUIRE(k_stride_n % 8 == 0 && k_stride_h % 8 == 0 && v_stride_n % 8 == 0 && v_stride_h % 8 == 0 &&
                 ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_decode_attn_bf16: k/v must be 16-byte aligned with strides multiple of 8");
  SP_REQUIRE(workspace_bytes >= sp_decode_workspace_bytes(n, hq, hkv) && ((uintptr_t)workspace % 8) == 0,
             SP_ERR_WORKSPACE, "sp_decode_attn_bf16: workspace too small or misaligned");
  const int g = hq / hkv;
  const int splits = dc_splits(n, hkv);
  const int64_t keys_per_split = sp_ceil_div(sp_ceil_div(n, splits), DC_TILE) * DC_TILE;
  float* o_part = (float*)workspace;
  float2* ml_part = (float2*)(o_part + (size_t)splits * hq * DC_D);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(sp_decode_partial_kernel, dim3(splits, hkv), dim3(DC_THREADS), 0, s, (const sp_bf16*)q,
                     (const sp_bf16*)k, (const sp_bf16*)v, n, g, q_stride_h, k_stride_n, k_stride_h, v_stride_n,
                     v_stride_h, softmax_scale * 1.4426950408889634f, keys_per_split, o_part, ml_part);
  SP_LAUNCH_CHECK();
  hipLaunchKernelGGL(sp_decode_combine_kernel, dim3(hq), dim3(DC_D), 0, s, o_part, ml_part, g, splits, (sp_bf16*)out);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// Decode step: one query token per head against the whole KV cache (GQA, no mask), bf16 in / bf16 out, fp32
// softmax.  Replaces the flash_attn_func call of the reference's decode branch (shareprefill_attn.py:146-155).
//
// HBM-bound: K and V are read exactly once (2 * n * hkv * d * 2 bytes); everything else has to stay out of the
// way.  The cache of one kv head is split into chunks; one workgroup streams a chunk for all query heads of the
// group (so the group's `g` heads share every K / V byte), keeps an online softmax, and leaves an unnormalised
// partial (o, m, l); a second tiny kernel merges the partials in chunk order.
//
// Both products run on the matrix core with the group's heads as a (mostly empty) 32-wide operand -- the MFMAs
// are free here, the point is to keep the vector ALU out of the inner loop:
//   S^T[keys x heads] = K . Q^T    A = K rows from LDS, B = the queries in registers (columns >= g are zero)
//   O[heads x d]     += P . V      A = P (bf16, from LDS), B = V read from its row-major LDS tile with the
//                                  transposing LDS load (ds_read_b64_tr_b16), which hands every lane four
//                                  consecutive keys of one channel.
#include "sp_common.h"

#include <mutex>

#define DC_THREADS 256
#define DC_TILE 128   // keys per tile
#define DC_D 128
#define DC_GMAX 32    // query heads per kv head (the 32-wide operand of the MFMAs); kernels are built for <= 8, 16, 32
#define DC_PITCH 136  // bf16 elements per LDS row (272 bytes: conflict-free 128-bit reads)

typedef uint32_t dc_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 dc_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 dc_bf16x4 __attribute__((ext_vector_type(4)));
typedef float dc_floatx16 __attribute__((ext_vector_type(16)));
typedef float dc_floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 dc_bf16x2 __attribute__((ext_vector_type(2)));

__device__ static __forceinline__ uint32_t dc_pack2(float a, float b) {
  dc_floatx2 f;
  f[0] = a;
  f[1] = b;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, dc_bf16x2));
}

// thread t fetches chunk t%16 (16 bytes) of rows t/16, t/16+16, ... of a 128-row tile; rows past the end are clamped.
// d < 128 (a smaller head): the chunks beyond the row's d channels are zeros made here, not read -- the tile in LDS is
// the row zero-padded to 128 channels, which changes no product.
// (FULL: d == 128, nothing to pad -- the plain loads of the kernel's own head size)
template <bool FULL>
__device__ static __forceinline__ void dc_fetch(const sp_bf16* __restrict__ x, int64_t n, int64_t stride_n, int64_t kb,
                                               int t, int d, dc_u32x4 (&r)[8]) {
  const bool real = FULL || (t & 15) * 8 < d;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int64_t key = kb + i * 16 + (t >> 4);
    if (key > n - 1) key = n - 1;
    if (FULL) {
      r[i] = *reinterpret_cast<const dc_u32x4*>(x + key * stride_n + (t & 15) * 8);
    } else {
      r[i] = (dc_u32x4){0, 0, 0, 0};
      if (real) r[i] = *reinterpret_cast<const dc_u32x4*>(x + key * stride_n + (t & 15) * 8);
    }
  }
}

__device__ static __forceinline__ void dc_store(sp_bf16* tile, int t, const dc_u32x4 (&r)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) *reinterpret_cast<dc_u32x4*>(tile + (i * 16 + (t >> 4)) * DC_PITCH + (t & 15) * 8) = r[i];
}

// grid (splits, hkv); partial layout: o [hkv][splits][g][128] fp32, ml [hkv][splits][g] float2 (m in log2 units, l)
// G8 = groups of 8 heads the instance handles (g <= 8 * G8): accumulator rows r < 4 * G8 can belong to real heads
template <int G8, bool FULL>
__global__ __launch_bounds__(DC_THREADS, 2) void sp_decode_partial_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const sp_bf16* __restrict__ v, int64_t n, int g,
    int d, int64_t sq_h, int64_t sk_n, int64_t sk_h, int64_t sv_n, int64_t sv_h, float scale_log2,
    int64_t keys_per_split, float* __restrict__ o_part, float2* __restrict__ ml_part) {
  __shared__ __attribute__((aligned(16))) sp_bf16 Ks[DC_TILE * DC_PITCH];
  __shared__ __attribute__((aligned(16))) sp_bf16 Vs[DC_TILE * DC_PITCH];
  constexpr int GM = 8 * G8;
  __shared__ __attribute__((aligned(16))) sp_bf16 Ps[GM * DC_PITCH];  // probabilities [head][key]
  __shared__ float wmax[4][GM], wsum[4][GM], alpha_s[GM];
  const int split = blockIdx.x, kvh = blockIdx.y, splits = gridDim.x;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int lh = lane & 31, hi = lane >> 5;  // operand column / row inside a 32-wide tile, lane half
  const bool head_ok = lh < g;               // this lane's S^T column is a real head
  const sp_bf16* kh = k + (int64_t)kvh * sk_h;
  const sp_bf16* vh = v + (int64_t)kvh * sv_h;

  // B operand of S^T = K . Q^T: column lh = head, k-step ks covers channels 16ks + 8hi .. +7
  dc_bf16x8 qb[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    dc_u32x4 raw = {0, 0, 0, 0};
    if (head_ok && (FULL || 16 * ks + 8 * hi < d))
      raw = *reinterpret_cast<const dc_u32x4*>(q + (int64_t)(kvh * g + lh) * sq_h + 16 * ks + 8 * hi);
    qb[ks] = __builtin_bit_cast(dc_bf16x8, raw);
  }

  const int64_t key_begin = (int64_t)split * keys_per_split;
  int64_t key_end = key_begin + keys_per_split;
  if (key_end > n) key_end = n;

  dc_floatx16 o = {0};                   // rows = heads 8(r/4) + 4hi + r%4 (only r < 4 G8 can be real), col = channel 32*wave + lh
  float m_run = -INFINITY, l_run = 0.f;  // of head lh (every wave keeps the same copy)
  dc_u32x4 kr[8], vr[8];
  if (key_begin < key_end) {
    dc_fetch<FULL>(kh, n, sk_n, key_begin, t, d, kr);
    dc_fetch<FULL>(vh, n, sv_n, key_begin, t, d, vr);
  }
  for (int64_t kb = key_begin; kb < key_end; kb += DC_TILE) {
    __syncthreads();  // the previous tile's operand reads are done
    dc_store(Ks, t, kr);
    dc_store(Vs, t, vr);
    __syncthreads();
    if (kb + DC_TILE < key_end) {  // next tile on its way while this one is used
      dc_fetch<FULL>(kh, n, sk_n, kb + DC_TILE, t, d, kr);
      dc_fetch<FULL>(vh, n, sv_n, kb + DC_TILE, t, d, vr);
    }
    // ---- S^T for this wave's 32 keys: acc[r] = logit(key 32*wave + 8(r/4) + 4hi + r%4, head lh) ----
    dc_floatx16 acc = {0};
    {
      const sp_bf16* arow = Ks + (32 * wave + lh) * DC_PITCH + 8 * hi;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const dc_u32x4 raw = *reinterpret_cast<const dc_u32x4*>(arow + 16 * ks);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(dc_bf16x8, raw), qb[ks], acc, 0, 0, 0);
      }
    }
    const int valid = (int)((key_end - kb) < DC_TILE ? (key_end - kb) : DC_TILE);
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 32 * wave + 8 * (r >> 2) + 4 * hi + (r & 3);
      acc[r] = key < valid ? acc[r] * scale_log2 : -INFINITY;
      mx = fmaxf(mx, acc[r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, SP_WAVE));
    if (head_ok && hi == 0) wmax[wave][lh] = mx;
    __syncthreads();
    float m_new = m_run, alpha = 1.f;
    if (head_ok) {
      m_new = fmaxf(fmaxf(fmaxf(wmax[0][lh], wmax[1][lh]), fmaxf(wmax[2][lh], wmax[3][lh])), m_run);  // finite
      alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first tile
      float ls = 0.f;
      sp_bf16* prow = Ps + lh * DC_PITCH + 32 * wave + 4 * hi;
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const float p0 = __builtin_amdgcn_exp2f(acc[4 * r4 + 0] - m_new), p1 = __builtin_amdgcn_exp2f(acc[4 * r4 + 1] - m_new);
        const float p2 = __builtin_amdgcn_exp2f(acc[4 * r4 + 2] - m_new), p3 = __builtin_amdgcn_exp2f(acc[4 * r4 + 3] - m_new);
        ls += (p0 + p1) + (p2 + p3);
        *reinterpret_cast<uint2*>(prow + 8 * r4) = make_uint2(dc_pack2(p0, p1), dc_pack2(p2, p3));
      }
      ls += __shfl_xor(ls, 32, SP_WAVE);
      if (hi == 0) {
        wsum[wave][lh] = ls;
        if (wave == 0) alpha_s[lh] = alpha;
      }
    }
    __syncthreads();
    if (head_ok) {
      l_run = l_run * alpha + ((wsum[0][lh] + wsum[1][lh]) + (wsum[2][lh] + wsum[3][lh]));
      m_run = m_new;
    }
    // ---- O += P . V for this wave's 32 channels; only accumulator rows of real heads need the rescale ----
#pragma unroll
    for (int r = 0; r < 4 * G8; ++r) {
      const int h = 8 * (r >> 2) + 4 * hi + (r & 3);
      if (h < g) o[r] *= alpha_s[h];
    }
    {
      const sp_bf16* prow = Ps + lh * DC_PITCH + 8 * hi;
      // transposing read: the 16 lanes of a block address 4 key rows x 16 channels (4 lanes x 8 bytes per row) and
      // each lane receives 4 consecutive keys of its channel
      const sp_bf16* vtr = Vs + (8 * hi + ((lane & 15) >> 2)) * DC_PITCH + 32 * wave + 16 * ((lane >> 4) & 1) +
                           4 * (lane & 3);
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        dc_u32x4 praw = {0, 0, 0, 0};
        if (head_ok) praw = *reinterpret_cast<const dc_u32x4*>(prow + 16 * kk);
        const dc_bf16x4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) dc_bf16x4*)(vtr + (16 * kk) * DC_PITCH));
        const dc_bf16x4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) dc_bf16x4*)(vtr + (16 * kk + 4) * DC_PITCH));
        dc_bf16x8 bv;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          bv[j] = b0[j];
          bv[4 + j] = b1[j];
        }
        o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(dc_bf16x8, praw), bv, o, 0, 0, 0);
      }
    }
  }

  float* op = o_part + (((int64_t)kvh * splits + split) * g) * DC_D;
#pragma unroll
  for (int r = 0; r < 4 * G8; ++r) {
    const int h = 8 * (r >> 2) + 4 * hi + (r & 3);
    if (h < g) op[h * DC_D + 32 * wave + lh] = o[r];
  }
  if (wave == 0 && hi == 0 && head_ok) ml_part[((int64_t)kvh * splits + split) * g + lh] = make_float2(m_run, l_run);
}

// one workgroup of 128 threads per query head: merges the chunk partials (sums in chunk order)
#define DC_MAX_SPLITS 512
__global__ __launch_bounds__(DC_D) void sp_decode_combine_kernel(const float* __restrict__ o_part,
                                                                 const float2* __restrict__ ml_part, int g, int splits,
                                                                 int d, sp_bf16* __restrict__ out) {
  __shared__ float w_s[DC_MAX_SPLITS];  // weight of chunk s: exp2(m_s - m), 0 for an empty chunk
  __shared__ float red[2];
  const int hq_idx = blockIdx.x, kvh = hq_idx / g, h = hq_idx % g, c = threadIdx.x;
  const float2* ml = ml_part + (int64_t)kvh * splits * g + h;
  float m = -INFINITY;
  for (int s = c; s < splits; s += DC_D) m = fmaxf(m, ml[(int64_t)s * g].x);
  m = sp_wave_max(m);
  if ((c & 63) == 0) red[c >> 6] = m;
  __syncthreads();
  m = fmaxf(red[0], red[1]);
  for (int s = c; s < splits; s += DC_D) {
    const float ms = ml[(int64_t)s * g].x;
    w_s[s] = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - m);
  }
  __syncthreads();
  const float* op = o_part + ((int64_t)kvh * splits * g + h) * DC_D + c;
  float l = 0.f, o = 0.f;
#pragma unroll 8
  for (int s = 0; s < splits; ++s) {
    l += ml[(int64_t)s * g].y * w_s[s];
    o += op[(int64_t)s * g * DC_D] * w_s[s];
  }
  if (c < d) out[(int64_t)hq_idx * d + c] = sp_f32_to_bf16(o / l);
}

// ---- host -------------------------------------------------------------------------------------------------
static int dc_splits(int64_t n, int32_t hkv) {
  const int64_t tiles = sp_ceil_div(n, DC_TILE);
  int64_t want = sp_ceil_div(512, hkv);  // about two workgroups per CU
  if (want > tiles) want = tiles;
  if (want < 1) want = 1;
  if (want > DC_MAX_SPLITS) want = DC_MAX_SPLITS;
  return (int)want;
}

extern "C" size_t sp_decode_workspace_bytes(int64_t n, int32_t hq, int32_t hkv) {
  if (n <= 0 || hq <= 0 || hkv <= 0) return 0;
  return (size_t)dc_splits(n, hkv) * hq * (DC_D * sizeof(float) + sizeof(float2));
}

// argument checks shared by the two entry points
static int dc_check(const char* who, const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv,
                    int32_t d, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n,
                    int64_t v_stride_h, float softmax_scale, const void* out) {
  SP_REQUIRE(q && k && v && out, SP_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  SP_REQUIRE(n > 0 && hq > 0 && hkv > 0 && hq % hkv == 0, SP_ERR_INVALID_ARGUMENT, "%s: bad shape n=%lld hq=%d hkv=%d",
             who, (long long)n, hq, hkv);
  SP_REQUIRE(softmax_scale > 0.f, SP_ERR_INVALID_ARGUMENT, "%s: softmax_scale must be > 0", who);
  SP_REQUIRE(d >= 8 && d <= DC_D && d % 8 == 0, SP_ERR_UNSUPPORTED,
             "%s: head_dim %d unsupported (a multiple of 8 up to 128)", who, d);
  SP_REQUIRE(hq / hkv <= DC_GMAX, SP_ERR_UNSUPPORTED, "%s: more than %d query heads per kv head", who, DC_GMAX);
  // q, k and v are read with 16-byte loads
  SP_REQUIRE(q_stride_h % 8 == 0 && ((uintptr_t)q % 16) == 0, SP_ERR_UNSUPPORTED,
             "%s: q must be 16-byte aligned with a head stride multiple of 8", who);
  SP_REQUIRE(k_stride_n % 8 == 0 && k_stride_h % 8 == 0 && v_stride_n % 8 == 0 && v_stride_h % 8 == 0 &&
                 ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0,
             SP_ERR_UNSUPPORTED, "%s: k/v must be 16-byte aligned with strides multiple of 8", who);
  return SP_OK;
}

// both kernels; `partials` holds sp_decode_workspace_bytes(n, hq, hkv) bytes, every one of which the first kernel
// writes before the second reads it (nothing has to be cleared)
static int dc_launch(const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv, int32_t d,
                     int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                     float softmax_scale, void* out, void* partials, hipStream_t s) {
  const int g = hq / hkv;
  const int splits = dc_splits(n, hkv);
  const int64_t keys_per_split = sp_ceil_div(sp_ceil_div(n, splits), DC_TILE) * DC_TILE;
  float* o_part = (float*)partials;
  float2* ml_part = (float2*)(o_part + (size_t)splits * hq * DC_D);
  const float scale_log2 = softmax_scale * 1.4426950408889634f;
#define DC_LAUNCH_PARTIAL_(G8, FULL)                                                                                  \
  hipLaunchKernelGGL((sp_decode_partial_kernel<G8, FULL>), dim3(splits, hkv), dim3(DC_THREADS), 0, s, (const sp_bf16*)q, \
                     (const sp_bf16*)k, (const sp_bf16*)v, n, g, (int)d, q_stride_h, k_stride_n, k_stride_h,          \
                     v_stride_n, v_stride_h, scale_log2, keys_per_split, o_part, ml_part)
#define DC_LAUNCH_PARTIAL(G8)     \
  do {                            \
    if (d == DC_D)                \
      DC_LAUNCH_PARTIAL_(G8, true);  \
    else                          \
      DC_LAUNCH_PARTIAL_(G8, false); \
  } while (0)
  if (g <= 8) {
    DC_LAUNCH_PARTIAL(1);
  } else if (g <= 16) {
    DC_LAUNCH_PARTIAL(2);
  } else {
    DC_LAUNCH_PARTIAL(4);
  }
#undef DC_LAUNCH_PARTIAL
#undef DC_LAUNCH_PARTIAL_
  SP_LAUNCH_CHECK();
  hipLaunchKernelGGL(sp_decode_combine_kernel, dim3(hq), dim3(DC_D), 0, s, o_part, ml_part, g, splits, (int)d,
                     (sp_bf16*)out);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_decode_attn_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv,
                                   int32_t d, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                                   int64_t v_stride_n, int64_t v_stride_h, float softmax_scale, void* out,
                                   void* workspace, size_t workspace_bytes, sp_stream_t stream) {
  int rc = dc_check("sp_decode_attn_bf16", q, k, v, n, hq, hkv, d, q_stride_h, k_stride_n, k_stride_h, v_stride_n,
                    v_stride_h, softmax_scale, out);
  if (rc) return rc;
  SP_REQUIRE(workspace != nullptr, SP_ERR_INVALID_ARGUMENT, "sp_decode_attn_bf16: null workspace");
  SP_REQUIRE(workspace_bytes >= sp_decode_workspace_bytes(n, hq, hkv) && ((uintptr_t)workspace % 8) == 0,
             SP_ERR_WORKSPACE, "sp_decode_attn_bf16: workspace too small or misaligned");
  return dc_launch(q, k, v, n, hq, hkv, d, q_stride_h, k_stride_n, k_stride_h, v_stride_n, v_stride_h, softmax_scale, out,
                   workspace, (hipStream_t)stream);
}

// ---- the same step for callers that cannot allocate ---------------------------------------------------------------
// The chunk partials live in a file-scope device array instead of a caller's workspace.  Every GPU the library runs on
// holds its own copy of the array (at its own address) until the process ends; the array's name is only a host-side
// handle, so the device address is looked up once per device with hipGetSymbolAddress and that pointer is what the
// kernels get.
#define DC_STATIC_BYTES SP_DECODE_STATIC_SCRATCH_BYTES
#define DC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[DC_STATIC_BYTES];
static void* dc_scratch_ptr[DC_MAX_DEVICES];  // device address of `scratch` per device, nullptr = not looked up yet
static std::mutex dc_scratch_mutex;

static int dc_static_scratch(void** ptr) {
  int dev = -1;
  SP_HIP(hipGetDevice(&dev));
  SP_REQUIRE(dev >= 0 && dev < DC_MAX_DEVICES, SP_ERR_UNSUPPORTED, "sp_decode_attn_static_bf16: device index %d", dev);
  std::lock_guard<std::mutex> lock(dc_scratch_mutex);
  if (dc_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    SP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SP_REQUIRE(p != nullptr, SP_ERR_HIP, "sp_decode_attn_static_bf16: no device address for the scratch array");
    dc_scratch_ptr[dev] = p;
  }
  *ptr = dc_scratch_ptr[dev];
  return SP_OK;
}

extern "C" int sp_decode_attn_static_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq,
                                          int32_t hkv, int32_t d, int64_t q_stride_h, int64_t k_stride_n,
                                          int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                                          float softmax_scale, void* out, sp_stream_t stream) {
  int rc = dc_check("sp_decode_attn_static_bf16", q, k, v, n, hq, hkv, d, q_stride_h, k_stride_n, k_stride_h,
                    v_stride_n, v_stride_h, softmax_scale, out);
  if (rc) return rc;
  const size_t need = sp_decode_workspace_bytes(n, hq, hkv);
  SP_REQUIRE(need <= DC_STATIC_BYTES, SP_ERR_WORKSPACE,
             "sp_decode_attn_static_bf16: n=%lld hq=%d hkv=%d needs %zu bytes of partials, the built-in scratch holds "
             "%u; use sp_decode_attn_bf16 with a workspace",
             (long long)n, hq, hkv, need, (unsigned)DC_STATIC_BYTES);
  void* partials = nullptr;
  rc = dc_static_scratch(&partials);
  if (rc) return rc;
  return dc_launch(q, k, v, n, hq, hkv, d, q_stride_h, k_stride_n, k_stride_h, v_stride_n, v_stride_h, softmax_scale, out,
                   partials, (hipStream_t)stream);
}

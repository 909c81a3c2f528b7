// GQA causal block-sparse flash attention for gfx950 (bf16 MFMA, fp32 online softmax in base 2).
// Replaces block_wise_prefill_attention_kernel / triton_block_wise_prefill_attention and the CSR
// builder count_kernel (shareprefill/attn/shareprefill_attn.py:187-620): the kernel walks the set
// bits of the row's mask words instead of a sorted id list with row pointers.
//
// Layout of the computation (one workgroup = one 128-query block of one head, 4 waves x 32 queries):
//   S^T = K . Q^T   : A operand = K tile rows from LDS, B operand = Q held in registers for the whole
//                     row.  In the 32x32 accumulator a lane then owns ONE query (lane % 32) and 16 of
//                     the tile's 32 keys, so the row max / row sum are in-lane reductions plus a single
//                     exchange with lane ^ 32.
//   O^T += V^T . P^T: the P^T operand is the S^T accumulator converted to bf16 in place (no LDS round
//                     trip); the V^T operand comes from a key-major repack of V made once per call, whose
//                     key order inside every group of 16 keys matches the accumulator's row order.
// K and V^T tiles are staged through LDS with a 272-byte row pitch (conflict-free 128-bit reads).
#include "sp_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define AT_BS 128
#define AT_D 128
#define AT_PITCH 136  // bf16 elements per LDS row
#define AT_THREADS 256

// position p (0..15) inside a group of 16 keys of the repacked V^T row holds key offset at_perm(p):
// [0-3, 8-11, 4-7, 12-15], the order in which a lane half owns the rows of a 32x32 accumulator
__host__ __device__ static inline int at_perm(int p) { return 8 * ((p & 7) >> 2) + 4 * (p >> 3) + (p & 3); }

// ---- V repack: v[n][hkv][d] -> vt[hkv][nb][d][128 key slots] ------------------------------------------
__global__ __launch_bounds__(AT_THREADS) void sp_repack_v_kernel(const sp_bf16* __restrict__ v,
                                                                 sp_bf16* __restrict__ vt, int64_t n, int64_t sv_n,
                                                                 int64_t sv_h, int64_t nb) {
  __shared__ sp_bf16 tile[AT_BS * AT_PITCH];
  const int64_t blk = blockIdx.x;
  const int kvh = blockIdx.y;
  const int t = threadIdx.x;
  const int chunk = t & 15;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int row = it * 16 + (t >> 4);
    const int64_t key = blk * AT_BS + row;
    uint4 val = make_uint4(0, 0, 0, 0);
    if (key < n) val = *reinterpret_cast<const uint4*>(v + (int64_t)kvh * sv_h + key * sv_n + chunk * 8);
    *reinterpret_cast<uint4*>(&tile[row * AT_PITCH + chunk * 8]) = val;
  }
  __syncthreads();
  sp_bf16* dst = vt + (((int64_t)kvh * nb + blk) * AT_D) * AT_BS;
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int dd = it * 16 + (t >> 4);  // output row = channel
    const int p0 = chunk * 8;           // 8 consecutive key slots
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int slot = p0 + j;
      const int key = (slot & ~15) + at_perm(slot & 15);
      const uint32_t e = tile[key * AT_PITCH + dd];
      if (j & 1)
        w[j >> 1] |= e << 16;
      else
        w[j >> 1] = e;
    }
    *reinterpret_cast<uint4*>(dst + (int64_t)dd * AT_BS + p0) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// ---- work-item -> (head, query block) mapping -------------------------------------------------------
// Workgroups are handed to the 8 XCDs round-robin by linear id.  Each XCD (its own L2) is given the
// query heads of one KV head at a time, heavy (late) rows first, the group's q heads interleaved, so
// that workgroups running together read the same K / V^T tiles.
__device__ static inline void at_map(int id, int hq, int hkv, int nb, int& h, int& r) {
  const int group = hq / hkv;
  int kvh, s;
  if (hkv % 8 == 0) {
    const int xcd = id & 7;
    const int per = group * nb;  // items per kv head
    s = id >> 3;
    kvh = xcd + 8 * (s / per);
    s = s % per;
    h = kvh * group + (s % group);
    r = nb - 1 - (s / group);
  } else if (8 % hkv == 0 && nb % (8 / hkv) == 0) {
    const int split = 8 / hkv;  // XCDs per kv head, rows dealt round-robin between them
    const int xcd = id & 7;
    s = id >> 3;
    kvh = xcd / split;
    h = kvh * group + (s % group);
    r = nb - 1 - ((s / group) * split + (xcd % split));
  } else {
    h = id / nb;
    r = nb - 1 - (id % nb);
  }
}

__device__ static inline bf16x8 at_pack8(const floatx16& a, int base) {
  floatx8 f;
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = a[base + j];
  return __builtin_convertvector(f, bf16x8);
}

__global__ __launch_bounds__(AT_THREADS, 2) void sp_attn_fwd_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const sp_bf16* __restrict__ vt,
    const uint64_t* __restrict__ mask, const int32_t* __restrict__ decision, sp_bf16* __restrict__ out,
    float* __restrict__ avg_attn, int64_t n, int hq, int hkv, int64_t sq_n, int64_t sq_h, int64_t sk_n,
    int64_t sk_h, int nb, int nbw, float scale_log2) {
  __shared__ sp_bf16 Ks[AT_BS * AT_PITCH];
  __shared__ sp_bf16 Vs[AT_D * AT_PITCH];
  __shared__ float wred[4];

  int h, r;
  at_map(blockIdx.x, hq, hkv, nb, h, r);
  const int kvh = h / (hq / hkv);
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int lq = lane & 31, g = lane >> 5;
  const int ld_row = t >> 4, ld_chunk = t & 15;

  // Q^T operand: this lane's query, 8 k-steps of 8 channels
  bf16x8 qb[8];
  {
    int64_t qrow = (int64_t)r * AT_BS + wave * 32 + lq;
    if (qrow > n - 1) qrow = n - 1;
    const sp_bf16* src = q + (int64_t)h * sq_h + qrow * sq_n + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qb[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 16 * ks));
  }
  const sp_bf16* kh = k + (int64_t)kvh * sk_h;
  const sp_bf16* vth = vt + (int64_t)kvh * nb * AT_D * AT_BS;
  const uint64_t* mrow = mask + ((int64_t)h * nb + r) * nbw;

  floatx16 o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o[dt] = (floatx16){0};
  float m_run = -INFINITY, l_run = 0.f;
  const int q_off = wave * 32 + lq;  // query offset inside the block

  for (int w = 0; w <= (r >> 6); ++w) {
    uint64_t word = mrow[w];
    if (w == (r >> 6) && (r & 63) != 63) word &= (2ull << (r & 63)) - 1ull;  // only columns c <= r
    while (word) {
      const int c = w * 64 + __builtin_ctzll(word);
      word &= word - 1;
      // ---- stage K tile and V^T tile ----
      __syncthreads();
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int row = it * 16 + ld_row;
        int64_t key = (int64_t)c * AT_BS + row;
        if (key > n - 1) key = n - 1;
        const uint4 kv = *reinterpret_cast<const uint4*>(kh + key * sk_n + ld_chunk * 8);
        const uint4 vv = *reinterpret_cast<const uint4*>(vth + ((int64_t)c * AT_D + row) * AT_BS + ld_chunk * 8);
        *reinterpret_cast<uint4*>(&Ks[row * AT_PITCH + ld_chunk * 8]) = kv;
        *reinterpret_cast<uint4*>(&Vs[row * AT_PITCH + ld_chunk * 8]) = vv;
      }
      __syncthreads();
      // ---- S^T = K . Q^T ----
      floatx16 s[4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        floatx16 acc = (floatx16){0};
        const sp_bf16* arow = &Ks[(kt * 32 + lq) * AT_PITCH + 8 * g];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(arow + 16 * ks));
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qb[ks], acc, 0, 0, 0);
        }
        s[kt] = acc;
      }
      // ---- online softmax (base 2) ----
      float mx = m_run;
      if (c == r) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key_off = kt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
            float v = s[kt][i] * scale_log2;
            v = (key_off <= q_off) ? v : -INFINITY;
            s[kt][i] = v;
            mx = fmaxf(mx, v);
          }
      } else {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float v = s[kt][i] * scale_log2;
            s[kt][i] = v;
            mx = fmaxf(mx, v);
          }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32, SP_WAVE));
      const float alpha = __builtin_amdgcn_exp2f(m_run - mx);
      m_run = mx;
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float p = __builtin_amdgcn_exp2f(s[kt][i] - mx);
          s[kt][i] = p;
          psum += p;
        }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
      // ---- O^T += V^T . P^T ----
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const bf16x8 p0 = at_pack8(s[kt], 0);
        const bf16x8 p1 = at_pack8(s[kt], 8);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          const sp_bf16* arow = &Vs[(dt * 32 + lq) * AT_PITCH + kt * 32 + 8 * g];
          const bf16x8 a0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(arow));
          const bf16x8 a1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(arow + 16));
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, p0, o[dt], 0, 0, 0);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, p1, o[dt], 0, 0, 0);
        }
      }
    }
  }
  const float l_tot = l_run + __shfl_xor(l_run, 32, SP_WAVE);

  // ---- pivot heads: block-averaged attention map (second pass over the same blocks) ----
  if (decision != nullptr && decision[h] == SP_DEC_DENSE && avg_attn != nullptr) {
    const int64_t rem = n - (int64_t)r * AT_BS;
    const int valid_q = rem < AT_BS ? (int)rem : AT_BS;
    const bool q_valid = q_off < valid_q;
    const float inv_l = 1.0f / l_tot;
    float* arow_out = avg_attn + ((int64_t)h * nb + r) * nb;
    for (int w = 0; w <= (r >> 6); ++w) {
      uint64_t word = mrow[w];
      if (w == (r >> 6) && (r & 63) != 63) word &= (2ull << (r & 63)) - 1ull;
      while (word) {
        const int c = w * 64 + __builtin_ctzll(word);
        word &= word - 1;
        __syncthreads();
#pragma unroll
        for (int it = 0; it < 8; ++it) {
          const int row = it * 16 + ld_row;
          int64_t key = (int64_t)c * AT_BS + row;
          if (key > n - 1) key = n - 1;
          *reinterpret_cast<uint4*>(&Ks[row * AT_PITCH + ld_chunk * 8]) =
              *reinterpret_cast<const uint4*>(kh + key * sk_n + ld_chunk * 8);
        }
        __syncthreads();
        float part = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
          floatx16 acc = (floatx16){0};
          const sp_bf16* arow = &Ks[(kt * 32 + lq) * AT_PITCH + 8 * g];
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(arow + 16 * ks));
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qb[ks], acc, 0, 0, 0);
          }
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key_off = kt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
            const bool ok = q_valid && (c < r || key_off <= q_off) && ((int64_t)c * AT_BS + key_off < n);
            part += ok ? __builtin_amdgcn_exp2f(acc[i] * scale_log2 - m_run) * inv_l : 0.f;
          }
        }
        part = sp_wave_sum(part);
        if (lane == 0) wred[wave] = part;
        __syncthreads();
        if (t == 0) arow_out[c] = ((wred[0] + wred[1]) + (wred[2] + wred[3])) / (float)valid_q;
      }
    }
  }

  // ---- epilogue: normalise, transpose through LDS, coalesced bf16 store ----
  __syncthreads();
  {
    const float inv_l = 1.0f / l_tot;
    sp_bf16* orow = &Ks[q_off * AT_PITCH];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d0 = dt * 32 + 8 * i4 + 4 * g;
        const uint32_t b0 = sp_f32_to_bf16(o[dt][4 * i4 + 0] * inv_l);
        const uint32_t b1 = sp_f32_to_bf16(o[dt][4 * i4 + 1] * inv_l);
        const uint32_t b2 = sp_f32_to_bf16(o[dt][4 * i4 + 2] * inv_l);
        const uint32_t b3 = sp_f32_to_bf16(o[dt][4 * i4 + 3] * inv_l);
        *reinterpret_cast<uint2*>(orow + d0) = make_uint2(b0 | (b1 << 16), b2 | (b3 << 16));
      }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int row = it * 16 + ld_row;
    const int64_t qrow = (int64_t)r * AT_BS + row;
    if (qrow < n) {
      *reinterpret_cast<uint4*>(out + (qrow * hq + h) * AT_D + ld_chunk * 8) =
          *reinterpret_cast<const uint4*>(&Ks[row * AT_PITCH + ld_chunk * 8]);
    }
  }
}

// ---- host ---------------------------------------------------------------------------------------------
extern "C" size_t sp_attn_workspace_bytes(int64_t n, int32_t hkv, int32_t d, int32_t bs) {
  if (n <= 0 || hkv <= 0 || d <= 0 || bs <= 0) return 0;
  const int64_t nb = sp_ceil_div(n, bs);
  return (size_t)hkv * nb * bs * d * sizeof(sp_bf16);
}

extern "C" int sp_attn_repack_v_bf16(const void* v, int64_t n, int32_t hkv, int32_t d, int64_t v_stride_n,
                                     int64_t v_stride_h, int32_t bs, void* workspace, size_t workspace_bytes,
                                     sp_stream_t stream) {
  SP_REQUIRE(v && workspace, SP_ERR_INVALID_ARGUMENT, "sp_attn_repack_v_bf16: null pointer");
  SP_REQUIRE(n > 0 && hkv > 0, SP_ERR_INVALID_ARGUMENT, "sp_attn_repack_v_bf16: bad shape");
  SP_REQUIRE(bs == AT_BS && d == AT_D, SP_ERR_UNSUPPORTED,
             "sp_attn_repack_v_bf16: block size %d / head_dim %d unsupported (only 128 / 128)", bs, d);
  SP_REQUIRE(v_stride_n % 8 == 0 && v_stride_h % 8 == 0 && ((uintptr_t)v % 16) == 0 &&
                 ((uintptr_t)workspace % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_attn_repack_v_bf16: v must be 16-byte aligned, strides multiple of 8");
  SP_REQUIRE(workspace_bytes >= sp_attn_workspace_bytes(n, hkv, d, bs), SP_ERR_WORKSPACE,
             "sp_attn_repack_v_bf16: workspace too small");
  const int64_t nb = sp_ceil_div(n, bs);
  hipLaunchKernelGGL(sp_repack_v_kernel, dim3((unsigned)nb, hkv), dim3(AT_THREADS), 0, (hipStream_t)stream,
                     (const sp_bf16*)v, (sp_bf16*)workspace, n, v_stride_n, v_stride_h, nb);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_block_sparse_attn_fwd_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq,
                                             int32_t hkv, int32_t d, int64_t q_stride_n, int64_t q_stride_h,
                                             int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n,
                                             int64_t v_stride_h, int32_t bs, float softmax_scale,
                                             const uint64_t* mask, const int32_t* decision, void* out,
                                             float* avg_attn, void* workspace, size_t workspace_bytes,
                                             uint32_t flags, sp_stream_t stream) {
  SP_REQUIRE(q && k && v && mask && out && workspace, SP_ERR_INVALID_ARGUMENT,
             "sp_block_sparse_attn_fwd_bf16: null pointer");
  SP_REQUIRE(n > 0 && hq > 0 && hkv > 0 && hq % hkv == 0, SP_ERR_INVALID_ARGUMENT,
             "sp_block_sparse_attn_fwd_bf16: bad shape n=%lld hq=%d hkv=%d", (long long)n, hq, hkv);
  SP_REQUIRE(bs == AT_BS, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: block size %d unsupported (only 128)",
             bs);
  SP_REQUIRE(d == AT_D, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: head_dim %d unsupported (only 128)", d);
  SP_REQUIRE(q_stride_n % 8 == 0 && q_stride_h % 8 == 0 && k_stride_n % 8 == 0 && k_stride_h % 8 == 0 &&
                 ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)out % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: tensors must be 16-byte aligned, strides multiple of 8");
  SP_REQUIRE(workspace_bytes >= sp_attn_workspace_bytes(n, hkv, d, bs), SP_ERR_WORKSPACE,
             "sp_block_sparse_attn_fwd_bf16: workspace too small");
  const int64_t nb = sp_ceil_div(n, bs);
  SP_REQUIRE(nb * hq < (1ll << 31), SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: grid too large");
  if (!(flags & SP_ATTN_V_REPACKED)) {
    int rc = sp_attn_repack_v_bf16(v, n, hkv, d, v_stride_n, v_stride_h, bs, workspace, workspace_bytes, stream);
    if (rc != SP_OK) return rc;
  }
  const float scale_log2 = softmax_scale * 1.4426950408889634f;
  hipLaunchKernelGGL(sp_attn_fwd_kernel, dim3((unsigned)(nb * hq)), dim3(AT_THREADS), 0, (hipStream_t)stream,
                     (const sp_bf16*)q, (const sp_bf16*)k, (const sp_bf16*)workspace, mask, decision, (sp_bf16*)out,
                     avg_attn, n, hq, hkv, q_stride_n, q_stride_h, k_stride_n, k_stride_h, (int)nb,
                     (int)((nb + 63) / 64), scale_log2);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

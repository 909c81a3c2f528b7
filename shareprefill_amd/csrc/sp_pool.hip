// Block pooling (HBM-bound): x[n][h][d] bf16 -> y[nb][h][d] bf16; averages and sums accumulate in fp32.
// Replaces the reference's bnhd_pool_kernel (shareprefill/attn/utils.py:131-208), all five of its pool types
// (avg 0, max 1, min 2, max of absolute values 3, sum 4); the selection itself only ever asks for the average
// (attention_sharing.py:194-196).
//
// One thread owns one 16-byte channel chunk (8 bf16) of one (block, head) and walks a quarter of the
// block's tokens; a wave therefore reads 1 KiB of contiguous channels per token, and the four waves of
// a workgroup split the block's tokens.  The four partial sums are combined in the fixed order
// ((p0+p1)+(p2+p3)) through LDS, so the result does not depend on scheduling.
#include "sp_common.h"

#define POOL_CHUNKS 64  // 16-byte chunks per workgroup (one wave wide)
#define POOL_SPLIT 4    // token sub-ranges per block (one per wave)

// one element into the running value of pool type TYPE
template <int TYPE>
__device__ __forceinline__ void pool_take(float& acc, float v) {
  if (TYPE == SP_POOL_MAX) acc = fmaxf(acc, v);
  else if (TYPE == SP_POOL_MIN) acc = fminf(acc, v);
  else if (TYPE == SP_POOL_MAXABS) acc = fmaxf(acc, fabsf(v));
  else acc += v;
}
// two partial values of pool type TYPE
template <int TYPE>
__device__ __forceinline__ float pool_join(float a, float b) {
  if (TYPE == SP_POOL_MAX || TYPE == SP_POOL_MAXABS) return fmaxf(a, b);
  if (TYPE == SP_POOL_MIN) return fminf(a, b);
  return a + b;
}

template <int TYPE>
__global__ __launch_bounds__(POOL_CHUNKS* POOL_SPLIT) void sp_pool_kernel(
    const sp_bf16* __restrict__ x, sp_bf16* __restrict__ y, int64_t n, int h, int d, int64_t sx_n, int64_t sx_h,
    int bs, int tail_mode, const int32_t* __restrict__ head_enable, int chunks_per_block, int groups_per_block) {
  __shared__ float part[POOL_SPLIT][POOL_CHUNKS][8];
  const int lane = threadIdx.x % POOL_CHUNKS;
  const int sub = threadIdx.x / POOL_CHUNKS;
  const int64_t blk = blockIdx.x / groups_per_block;
  const int grp = blockIdx.x % groups_per_block;
  const int chunk = grp * POOL_CHUNKS + lane;
  const int dchunks = d / 8;
  const bool active = chunk < chunks_per_block;
  const int head = active ? chunk / dchunks : 0;
  const int d0 = active ? (chunk % dchunks) * 8 : 0;
  const bool enabled = active && (head_enable == nullptr || head_enable[head] != 0);

  const int64_t t_begin = blk * bs;
  const int64_t t_end = (t_begin + bs < n) ? t_begin + bs : n;
  // The reference's kernel loads the tokens of a ragged last block that lie beyond the sequence as zeros
  // (utils.py:168-179, other=0), so there a maximum is at least 0 and a minimum at most 0: the neutral start value
  // is 0 for that block, and for sums everywhere.
  const bool ragged = t_end - t_begin < bs;
  const float start = (TYPE == SP_POOL_MAX && !ragged) ? -INFINITY : (TYPE == SP_POOL_MIN && !ragged) ? INFINITY : 0.f;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = start;

  const int per = bs / POOL_SPLIT;
  if (enabled) {
    const sp_bf16* base = x + (int64_t)head * sx_h + d0;
    int64_t t0 = t_begin + (int64_t)sub * per;
    int64_t t1 = t0 + per < t_end ? t0 + per : t_end;
    int64_t t = t0;
    for (; t + 8 <= t1; t += 8) {
      uint4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const uint4*>(base + (t + u) * sx_n);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          pool_take<TYPE>(acc[2 * j], __uint_as_float(w[j] << 16));
          pool_take<TYPE>(acc[2 * j + 1], __uint_as_float(w[j] & 0xffff0000u));
        }
      }
    }
    for (; t < t1; ++t) {
      uint4 v = *reinterpret_cast<const uint4*>(base + t * sx_n);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pool_take<TYPE>(acc[2 * j], __uint_as_float(w[j] << 16));
        pool_take<TYPE>(acc[2 * j + 1], __uint_as_float(w[j] & 0xffff0000u));
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) part[sub][lane][j] = acc[j];
  __syncthreads();
  if (sub == 0 && enabled) {
    const int cnt = (int)(t_end - t_begin);
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float s = pool_join<TYPE>(pool_join<TYPE>(part[0][lane][j], part[1][lane][j]),
                                pool_join<TYPE>(part[2][lane][j], part[3][lane][j]));
      float m;
      if (TYPE != SP_POOL_AVG) {
        m = s;
      } else if (tail_mode == SP_POOL_TAIL_RESCALE && cnt != bs) {
        m = sp_round_bf16(s / (float)bs);
        m = sp_round_bf16(m * (float)bs);
        m = m / (float)cnt;
      } else {
        m = s / (float)cnt;
      }
      uint32_t b = sp_f32_to_bf16(m);
      if (j & 1)
        o[j / 2] |= b << 16;
      else
        o[j / 2] = b;
    }
    uint4 ov = make_uint4(o[0], o[1], o[2], o[3]);
    *reinterpret_cast<uint4*>(y + (blk * h + head) * (int64_t)d + d0) = ov;
  }
}

static int pool_launch(int pool_type, const void* x, void* y, int64_t n, int32_t h, int32_t d, int64_t x_stride_n,
                       int64_t x_stride_h, int32_t bs, int32_t tail_mode, const int32_t* head_enable,
                       sp_stream_t stream);

extern "C" int sp_pool_avg_bf16(const void* x, void* y, int64_t n, int32_t h, int32_t d, int64_t x_stride_n,
                                int64_t x_stride_h, int32_t bs, int32_t tail_mode, const int32_t* head_enable,
                                sp_stream_t stream) {
  return pool_launch(SP_POOL_AVG, x, y, n, h, d, x_stride_n, x_stride_h, bs, tail_mode, head_enable, stream);
}

extern "C" int sp_pool_bf16(const void* x, void* y, int64_t n, int32_t h, int32_t d, int64_t x_stride_n,
                            int64_t x_stride_h, int32_t bs, int32_t pool_type, sp_stream_t stream) {
  SP_REQUIRE(pool_type >= SP_POOL_AVG && pool_type <= SP_POOL_SUM, SP_ERR_INVALID_ARGUMENT,
             "sp_pool_bf16: unknown pool type %d", pool_type);
  return pool_launch(pool_type, x, y, n, h, d, x_stride_n, x_stride_h, bs, SP_POOL_TAIL_TRUE_LENGTH, nullptr, stream);
}

static int pool_launch(int pool_type, const void* x, void* y, int64_t n, int32_t h, int32_t d, int64_t x_stride_n,
                       int64_t x_stride_h, int32_t bs, int32_t tail_mode, const int32_t* head_enable,
                       sp_stream_t stream) {
  SP_REQUIRE(x && y, SP_ERR_INVALID_ARGUMENT, "sp_pool_avg_bf16 / sp_pool_bf16: null tensor pointer");
  SP_REQUIRE(n > 0 && h > 0 && d > 0, SP_ERR_INVALID_ARGUMENT, "sp_pool_avg_bf16 / sp_pool_bf16: n, h, d must be positive");
  SP_REQUIRE(d % 8 == 0, SP_ERR_UNSUPPORTED, "sp_pool_avg_bf16 / sp_pool_bf16: head_dim %d is not a multiple of 8", d);
  SP_REQUIRE(bs >= POOL_SPLIT && bs % POOL_SPLIT == 0, SP_ERR_UNSUPPORTED,
             "sp_pool_avg_bf16 / sp_pool_bf16: block size %d is not a multiple of %d", bs, POOL_SPLIT);
  SP_REQUIRE(x_stride_n % 8 == 0 && x_stride_h % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_pool_avg_bf16 / sp_pool_bf16: tensors must be 16-byte aligned with strides multiple of 8");
  SP_REQUIRE(tail_mode == SP_POOL_TAIL_TRUE_LENGTH || tail_mode == SP_POOL_TAIL_RESCALE, SP_ERR_INVALID_ARGUMENT,
             "sp_pool_avg_bf16 / sp_pool_bf16: unknown tail_mode %d", tail_mode);
  const int64_t nb = sp_ceil_div(n, bs);
  const int chunks_per_block = h * (d / 8);
  const int groups = (int)sp_ceil_div(chunks_per_block, POOL_CHUNKS);
  SP_REQUIRE(nb * groups < (1ll << 31), SP_ERR_UNSUPPORTED, "sp_pool_avg_bf16 / sp_pool_bf16: grid too large");
  dim3 grid((unsigned)(nb * groups));
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(POOL_CHUNKS * POOL_SPLIT), 0, (hipStream_t)stream, (const sp_bf16*)x,
                       (sp_bf16*)y, n, h, d, x_stride_n, x_stride_h, bs, tail_mode, head_enable, chunks_per_block,
                       groups);
  };
  switch (pool_type) {
    case SP_POOL_MAX: launch(sp_pool_kernel<SP_POOL_MAX>); break;
    case SP_POOL_MIN: launch(sp_pool_kernel<SP_POOL_MIN>); break;
    case SP_POOL_MAXABS: launch(sp_pool_kernel<SP_POOL_MAXABS>); break;
    case SP_POOL_SUM: launch(sp_pool_kernel<SP_POOL_SUM>); break;
    default: launch(sp_pool_kernel<SP_POOL_AVG>); break;
  }
  SP_LAUNCH_CHECK();
  return SP_OK;
}

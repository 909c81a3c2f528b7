// Last-block scores: softmax over all keys of the last 128 queries, reduced to the per-token
// vertical (column mean) and slash (anti-diagonal mean) vectors and their 128-token block sums.
// Replaces shareprefill/attn/attention_sharing.py:127-167, sum_all_diagonal_matrix
// (attn/utils.py:79-86) and torch_bhn_sumpool (attn/utils.py:33-44) without ever writing the
// [Hq,128,N] probability matrix to memory.
//
// Three kernels:
//   stats   : per (head, key chunk) the running row max / row sum of the logits (bf16 MFMA);
//   combine : folds the chunk partials into one (max, 1/sum) per query row, in chunk order;
//   probs   : recomputes the logits tile by tile; the column sums (vertical) start in registers and meet in LDS,
//             the probabilities of one 128x128 tile go to LDS and all four waves sum its anti-diagonals (slash).
//             A slash bin receives its upper part from the previous key tile; that part is carried in registers,
//             and each workgroup recomputes one leading tile so that no cross-workgroup accumulation (and no
//             float atomic) is needed.
// Every sum runs in a fixed order, so results are reproducible run to run.
#include "sp_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define LQ_ROWS 128          // query rows (= block size)
#define LQ_TILE 128          // keys per tile
#define LQ_D 128             // head dim
#define LQ_THREADS 256       // 4 waves, wave w owns query rows 32w..32w+31
#define LQ_MIN_TILES 1       // key tiles per workgroup (probs: output tiles, plus one leading tile): a power of two, at
#define LQ_MAX_TILES 32      // most 32 -- as many as still leave about a thousand workgroups at long sequences (32 at
                             // 128K tokens and Llama head counts), as few as give one round of ~512 at short ones (2 at 4K)
#define LQ_PITCH 136         // LDS row pitch (floats) of the probability tile
// Row maxima are kept in base-2 units (max logit * log2 e), so a probability is one fused multiply-add and one
// hardware exp2.  "No logit seen yet" is a large finite negative number, not -inf: then max, difference and exp2
// need no special case (exp2(-inf - finite) = 0 for masked logits, exp2(0) * 0 for an empty history).
#define LQ_LOG2E 1.4426950408889634f
#define LQ_NO_MAX (-1.0e30f)

// lane's A operand: scaled last-block queries, 8 k-steps x 8 bf16
__device__ static __forceinline__ void lq_load_q(const sp_bf16* __restrict__ q, int64_t n, int64_t sq_n, int wave, int lane,
                                        float inv_sqrt_d, bf16x8 (&qa)[8]) {
  const int row = wave * 32 + (lane & 31);
  const sp_bf16* src = q + (n - LQ_ROWS + row) * sq_n + 8 * (lane >> 5);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    uint4 raw = *reinterpret_cast<const uint4*>(src + 16 * ks);
    uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // last_q = bf16(q * (1/sqrt(d))), attention_sharing.py:127
      uint32_t lo = sp_f32_to_bf16(__uint_as_float(w[j] << 16) * inv_sqrt_d);
      uint32_t hi = sp_f32_to_bf16(__uint_as_float(w[j] & 0xffff0000u) * inv_sqrt_d);
      w[j] = lo | (hi << 16);
    }
    raw = make_uint4(w[0], w[1], w[2], w[3]);
    qa[ks] = __builtin_bit_cast(bf16x8, raw);
  }
}

// ---- K tile staging: 128 keys x 128 channels bf16 through LDS (row pitch 272 bytes), coalesced ---------------
#define LQ_KPITCH 136  // bf16 elements per LDS row of the K tile

typedef uint32_t lq_u32x4 __attribute__((ext_vector_type(4)));
struct LqKRegs {
  lq_u32x4 v[8];
};

// thread t fetches chunk t%16 (16 bytes) of key rows t/16, t/16+16, ...; keys past the end are clamped (masked later)
__device__ static __forceinline__ void lq_fetch_k(const sp_bf16* __restrict__ k, int64_t n, int64_t sk_n, int64_t kb, int t,
                                         LqKRegs& kr) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int64_t key = kb + i * 16 + (t >> 4);
    if (key > n - 1) key = n - 1;
    kr.v[i] = *reinterpret_cast<const lq_u32x4*>(k + key * sk_n + (t & 15) * 8);
  }
}

__device__ static __forceinline__ void lq_store_k(sp_bf16* Ks, int t, const LqKRegs& kr) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    *reinterpret_cast<lq_u32x4*>(Ks + (i * 16 + (t >> 4)) * LQ_KPITCH + (t & 15) * 8) = kr.v[i];
}

// logits of this wave's 32 query rows against the 128 keys of the staged tile:
// acc[nt][r] = S[row 32w + 8(r/4) + 4(lane/32) + r%4][key kb + 32nt + lane%32]
__device__ static __forceinline__ void lq_tile_logits(const sp_bf16* Ks, int lane, const bf16x8 (&qa)[8], floatx16 (&acc)[4]) {
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const sp_bf16* src = Ks + (32 * nt + (lane & 31)) * LQ_KPITCH + 8 * (lane >> 5);
    floatx16 c = {0};
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const uint4 raw = *reinterpret_cast<const uint4*>(src + 16 * ks);
      c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[ks], __builtin_bit_cast(bf16x8, raw), c, 0, 0, 0);
    }
    acc[nt] = c;
  }
}

__device__ static __forceinline__ int lq_row_of(int wave, int lane, int r) {
  return wave * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

typedef float lq_floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 lq_bf16x2 __attribute__((ext_vector_type(2)));

// Rounds the logits to bf16 (the reference's qk tensor is bf16, attention_sharing.py:129-139) with the hardware
// round-to-nearest-even conversion, two at a time, and masks what the last query block must not see.  Only the
// tiles that reach into the last 128 tokens (or past the sequence end) need the mask: MASKED is tile-uniform.
template <bool MASKED>
__device__ static __forceinline__ void lq_finish_logits(floatx16 (&acc)[4], uint32_t flags, int64_t kb, int64_t n, int wave,
                                               int lane) {
  if (flags & SP_FLAG_LOGITS_BF16) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        lq_floatx2 f;
        f[0] = acc[nt][r];
        f[1] = acc[nt][r + 1];
        const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, lq_bf16x2));
        acc[nt][r] = __uint_as_float(pk << 16);
        acc[nt][r + 1] = __uint_as_float(pk & 0xffff0000u);
      }
  }
  if (MASKED) {
    // key <= query position  <=>  c - row <= (n - 128) - kb;  key < n  <=>  c < n - kb   (c, row: offsets in the tile)
    const int64_t d64 = (n - LQ_ROWS) - kb, e64 = n - kb;
    const int dlim = d64 > 1024 ? 1024 : (int)d64, elim = e64 > 1024 ? 1024 : (int)e64;
    int ln = lane;
    asm volatile("" : "+v"(ln));  // keeps this rare path's lane arithmetic out of the tile loop's registers
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = lq_row_of(wave, ln, r);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int c = 32 * nt + (ln & 31);
        if (!(c - row <= dlim && c < elim)) acc[nt][r] = -INFINITY;
      }
    }
  }
}

// ---- kernel 1: chunk partials of the row max / row sum ------------------------------------------
// Built for occupancy: four workgroups per CU (16 waves) hide each other's load and barrier latencies.  That needs
// <= 128 registers per lane and <= 40 KiB of LDS per workgroup, so
//   * the K tile goes from global memory straight into LDS (128-bit direct loads, no staging registers), unpadded,
//     with the 16-byte chunk index XOR-swizzled by the row so that the operand reads stay conflict-free;
//   * the product is taken transposed, S^T = K . Q^T: in the 32x32 accumulators a lane then owns ONE query (column
//     lane % 32) and 16 of the tile's keys per 32-key group, so the running max and sum are two registers, not 32,
//     and the fold at the end is one exchange between the two lane halves.
#define LQ_KSW_BYTES (LQ_TILE * LQ_D * 2)  // 32 KiB: [128 keys][16 chunks of 16 bytes], chunk c of row r at c ^ (r & 15)

typedef __attribute__((address_space(3))) void* lq_lds_ptr;
typedef const __attribute__((address_space(1))) void* lq_gbl_ptr;

// Eight wave-instructions per wave fill the tile: instruction `it` of wave w writes the 1 KiB segment 4 * it + w
// (4 key rows); lane i writes chunk position i of the segment and fetches the global chunk that belongs there.
__device__ static __forceinline__ void lq_issue_k_direct(const sp_bf16* __restrict__ k, int64_t n, int64_t sk_n, int64_t kb,
                                                         char* ks, int wave, int lane) {
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int seg = it * 4 + wave;
    const int row = seg * 4 + (lane >> 4);
    const int cl = (lane & 15) ^ (row & 15);
    int64_t key = kb + row;
    if (key > n - 1) key = n - 1;  // rows past the end are clamped onto the last key (masked later)
    __builtin_amdgcn_global_load_lds((lq_gbl_ptr)(k + key * sk_n + cl * 8), (lq_lds_ptr)(ks + seg * 1024), 16, 0, 0);
  }
}

__global__ __launch_bounds__(LQ_THREADS, 4) void sp_lastq_stats_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, int64_t n, int hkv, int group, int64_t sq_n,
    int64_t sq_h, int64_t sk_n, int64_t sk_h, float inv_sqrt_d, uint32_t flags, int n_chunks, int tiles_per_wg,
    float2* __restrict__ partial /* [hq][n_chunks][128] */) {
  __shared__ __attribute__((aligned(1024))) char Ksw[LQ_KSW_BYTES];
  const int h = blockIdx.y;
  const int chunk = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lq = lane & 31, hi = lane >> 5;
  const sp_bf16* qh = q + (int64_t)h * sq_h;
  const sp_bf16* kh = k + (int64_t)(h / group) * sk_h;
  bf16x8 qa[8];  // the lane's query (row 32 wave + lq of the last block), channels 16 ks + 8 hi .. + 7
  lq_load_q(qh, n, sq_n, wave, lane, inv_sqrt_d, qa);
  float m = LQ_NO_MAX, l = 0.f;
  const int64_t n_tiles = sp_ceil_div(n, LQ_TILE);
  const int64_t tile0 = (int64_t)chunk * tiles_per_wg;
  // byte offset of the lane's operand chunk inside a 32-key group: row lq, logical chunk 2 ks + hi
  const int row_off = lq * 256;
  for (int t = 0; t < tiles_per_wg; ++t) {
    const int64_t tile = tile0 + t;
    if (tile >= n_tiles) break;
    const int64_t kb = tile * LQ_TILE;
    __syncthreads();  // the previous tile's operand reads are done
    lq_issue_k_direct(kh, n, sk_n, kb, Ksw, wave, lane);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct loads have landed
    __syncthreads();
    const bool masked = kb + LQ_TILE > n - LQ_ROWS;  // (tile-uniform) reaches into the last block or past the end
    // key <= query position  <=>  c - row <= (n - 128) - kb;  key < n  <=>  c < n - kb   (c, row: offsets in the tile)
    const int64_t d64 = (n - LQ_ROWS) - kb, e64 = n - kb;
    const int dlim = d64 > 1024 ? 1024 : (int)d64, elim = e64 > 1024 ? 1024 : (int)e64;
    // the tile in two halves of 64 keys: 32 accumulator registers alive at a time
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
      // S^T: acc[j][r] = logit(key kb + 64 half + 32 j + 8 (r / 4) + 4 hi + r % 4, this lane's query)
      floatx16 acc[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const char* src = Ksw + (2 * half + j) * 32 * 256 + row_off;
        floatx16 c = {0};
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const uint4 raw = *reinterpret_cast<const uint4*>(src + (((2 * ks + hi) ^ (lq & 15)) << 4));
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, raw), qa[ks], c, 0, 0, 0);
        }
        acc[j] = c;
      }
      if (flags & SP_FLAG_LOGITS_BF16) {  // the reference's qk tensor is bf16 (attention_sharing.py:129-139)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            lq_floatx2 f;
            f[0] = acc[j][r];
            f[1] = acc[j][r + 1];
            const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, lq_bf16x2));
            acc[j][r] = __uint_as_float(pk << 16);
            acc[j][r + 1] = __uint_as_float(pk & 0xffff0000u);
          }
      }
      if (masked) {
        const int row = wave * 32 + lq;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c = 64 * half + 32 * j + 8 * (r >> 2) + 4 * hi + (r & 3);
            if (!(c - row <= dlim && c < elim)) acc[j][r] = -INFINITY;
          }
      }
      float tmax = acc[0][0];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, acc[j][r]);
      const float mn = fmaxf(m, tmax * LQ_LOG2E);
      float add[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) add[r & 3] += __builtin_amdgcn_exp2f(__builtin_fmaf(acc[j][r], LQ_LOG2E, -mn));
      l = __builtin_fmaf(l, __builtin_amdgcn_exp2f(m - mn), (add[0] + add[1]) + (add[2] + add[3]));
      m = mn;
    }
  }
  // the two lane halves hold disjoint keys of the same query
  {
    const float m2 = __shfl_xor(m, 32, SP_WAVE), l2 = __shfl_xor(l, 32, SP_WAVE);
    const float mn = fmaxf(m, m2);
    // (hi = 0 adds its own part first, then the other half's: one order for both lanes)
    const float a = (hi ? l2 : l) * __builtin_amdgcn_exp2f((hi ? m2 : m) - mn);
    const float b = (hi ? l : l2) * __builtin_amdgcn_exp2f((hi ? m : m2) - mn);
    if (hi == 0) partial[((int64_t)h * n_chunks + chunk) * LQ_ROWS + wave * 32 + lq] = make_float2(mn, a + b);
  }
}

// ---- kernel 2: fold chunk partials ------------------------------------------------------------------
// One workgroup per head: 8 groups of 128 threads; group j folds chunks j, j+8, ... of every row, then the eight
// group results are merged in a fixed order.
#define LQ_COMBINE_GROUPS 8
__global__ __launch_bounds__(LQ_ROWS * LQ_COMBINE_GROUPS) void sp_lastq_combine_kernel(
    const float2* __restrict__ partial, int n_chunks, float2* __restrict__ rowstat /* [hq][128] */) {
  __shared__ float gm[LQ_COMBINE_GROUPS][LQ_ROWS], gl[LQ_COMBINE_GROUPS][LQ_ROWS];
  const int h = blockIdx.x, row = threadIdx.x % LQ_ROWS, grp = threadIdx.x / LQ_ROWS;
  const float2* p = partial + (int64_t)h * n_chunks * LQ_ROWS + row;
  float m = LQ_NO_MAX;
  for (int c = grp; c < n_chunks; c += LQ_COMBINE_GROUPS) m = fmaxf(m, p[(int64_t)c * LQ_ROWS].x);
  gm[grp][row] = m;
  __syncthreads();
  m = gm[0][row];
#pragma unroll
  for (int j = 1; j < LQ_COMBINE_GROUPS; ++j) m = fmaxf(m, gm[j][row]);
  float l = 0.f;
  for (int c = grp; c < n_chunks; c += LQ_COMBINE_GROUPS) {
    const float2 v = p[(int64_t)c * LQ_ROWS];
    l += v.y * __builtin_amdgcn_exp2f(v.x - m);
  }
  gl[grp][row] = l;
  __syncthreads();
  if (grp == 0) {
    l = ((gl[0][row] + gl[1][row]) + (gl[2][row] + gl[3][row])) + ((gl[4][row] + gl[5][row]) + (gl[6][row] + gl[7][row]));
    rowstat[h * LQ_ROWS + row] = make_float2(m, 1.0f / l);
  }
}

// ---- kernel 3: probabilities -> vertical / slash ------------------------------------------------------
__global__ __launch_bounds__(LQ_THREADS, 2) void sp_lastq_probs_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, int64_t n, int hkv, int group, int64_t sq_n,
    int64_t sq_h, int64_t sk_n, int64_t sk_h, float inv_sqrt_d, uint32_t flags, const float2* __restrict__ rowstat,
    float* __restrict__ vert_tok, float* __restrict__ slash_tok, float* __restrict__ vert_blk,
    float* __restrict__ slash_blk, int64_t nb, int tiles_per_wg) {
  extern __shared__ float lds[];
  float* P = lds;                            // [128][LQ_PITCH] probability tile (the K tile is staged here first)
  float* vpart = lds + LQ_ROWS * LQ_PITCH;   // [8][128] column sums per (wave, lane half)
  float* spart = vpart + 8 * LQ_TILE;        // [6][128] lower / upper anti-diagonal and column sums per row half
  const int h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const sp_bf16* qh = q + (int64_t)h * sq_h;
  const sp_bf16* kh = k + (int64_t)(h / group) * sk_h;
  bf16x8 qa[8];
  lq_load_q(qh, n, sq_n, wave, lane, inv_sqrt_d, qa);
  // per row: max + log2(sum), so that a probability is exp2(logit * log2 e - rm): the normalisation rides in the
  // exponent instead of costing a multiplication per element
  float rm[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float2 st = rowstat[h * LQ_ROWS + lq_row_of(wave, lane, r)];
    rm[r] = st.x - __builtin_amdgcn_logf(st.y);  // st.y = 1 / sum; v_log_f32 is log2
  }
  const int64_t n_tiles = sp_ceil_div(n, LQ_TILE);
  const int64_t first = (int64_t)blockIdx.x * tiles_per_wg;
  const float inv_rows = 1.0f / (float)LQ_ROWS;
  float carry[2] = {0.f, 0.f};  // wave 0: upper anti-diagonal parts handed from the previous tile to its two bins

  // the K tile is staged in the same LDS region the probability tile is written to afterwards
  sp_bf16* Ks = reinterpret_cast<sp_bf16*>(lds);
  const int64_t t_begin = first > 0 ? first - 1 : 0;
  const int64_t t_end = first + tiles_per_wg < n_tiles ? first + tiles_per_wg : n_tiles;
  LqKRegs kr;
  if (t_begin < t_end) lq_fetch_k(kh, n, sk_n, t_begin * LQ_TILE, threadIdx.x, kr);
  for (int64_t tile = t_begin; tile < t_end; ++tile) {
    const int64_t kb = tile * LQ_TILE;
    lq_store_k(Ks, threadIdx.x, kr);  // (the previous iteration ended with a barrier)
    __syncthreads();
    if (tile + 1 < t_end) lq_fetch_k(kh, n, sk_n, kb + LQ_TILE, threadIdx.x, kr);
    floatx16 acc[4];
    lq_tile_logits(Ks, lane, qa, acc);
    __syncthreads();  // every wave has its logits: the K tile may be overwritten by P
    if (kb + LQ_TILE <= n - LQ_ROWS)
      lq_finish_logits<false>(acc, flags, kb, n, wave, lane);
    else
      lq_finish_logits<true>(acc, flags, kb, n, wave, lane);
    // probabilities (exp2(-inf) = 0 for the masked entries): the tile goes to LDS for the anti-diagonal sums, the
    // column sums start in registers (a lane holds 16 rows of each of its 4 columns)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[nt][r], LQ_LOG2E, -rm[r]));
        P[lq_row_of(wave, lane, r) * LQ_PITCH + 32 * nt + (lane & 31)] = pv;
        part[r & 3] += pv;
      }
      vpart[(2 * wave + (lane >> 5)) * LQ_TILE + 32 * nt + (lane & 31)] = (part[0] + part[1]) + (part[2] + part[3]);
    }
    __syncthreads();
    {
      // anti-diagonals: element (i, c) belongs to bin kb + c - i + 127.  Thread (u, hv) walks rows 64 hv .. 64 hv + 63
      // of the wrapped diagonal u, P[i][(u + 1 + i) mod 128]; rows i <= 126 - u lie above the tile's main diagonal
      // and belong to bin kb + 128 + u (next tile), the others to bin kb + u.  Which of the two a row feeds is the
      // same for all rows of wave 0 (upper) and wave 3 (lower); four independent partial sums per kind.
      int tid = threadIdx.x;
      asm volatile("" : "+v"(tid));  // recompute the walk's addresses per tile: hoisted out of the loop they spill
      const int u = tid & 127, hv = tid >> 7;
      const float* col = P + (64 * hv) * LQ_PITCH;
      float lo[4] = {0.f, 0.f, 0.f, 0.f}, hi[4] = {0.f, 0.f, 0.f, 0.f};
      if (wave == 0) {
#pragma unroll 8
        for (int j = 0; j < 64; ++j) hi[j & 3] += col[j * LQ_PITCH + ((u + 1 + j) & 127)];
      } else if (wave == 3) {
#pragma unroll 8
        for (int j = 0; j < 64; ++j) lo[j & 3] += col[j * LQ_PITCH + ((u + 1 + 64 + j) & 127)];
      } else {
        const int split = 126 - u - 64 * hv;  // rows j <= split of this half are upper rows
#pragma unroll 8
        for (int j = 0; j < 64; ++j) {
          const float pv = col[j * LQ_PITCH + ((u + 1 + 64 * hv + j) & 127)];
          hi[j & 3] += j <= split ? pv : 0.f;
          lo[j & 3] += j <= split ? 0.f : pv;
        }
      }
      spart[(0 + hv) * LQ_TILE + u] = (lo[0] + lo[1]) + (lo[2] + lo[3]);
      spart[(2 + hv) * LQ_TILE + u] = (hi[0] + hi[1]) + (hi[2] + hi[3]);
      // columns: fold the 8 (wave, lane half) partials, four per thread
      const float* vp = vpart + (4 * hv) * LQ_TILE + u;
      spart[(4 + hv) * LQ_TILE + u] = (vp[0] + vp[LQ_TILE]) + (vp[2 * LQ_TILE] + vp[3 * LQ_TILE]);
    }
    __syncthreads();  // also: every wave is done with the tile, the next K tile may overwrite it
    // Final sums, token stores and block sums: wave 0 the anti-diagonals, wave 2 the columns, two bins per lane
    // (the tile is one 128-token block, so a wave's total is the block sum and needs no further exchange).
    if ((wave & 1) == 0) {
      const bool emit = tile >= first;
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int u0 = 2 * ln;
      float val[2];
      if (wave == 0) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          val[e] = (carry[e] + (spart[u0 + e] + spart[LQ_TILE + u0 + e])) * inv_rows;
          carry[e] = spart[2 * LQ_TILE + u0 + e] + spart[3 * LQ_TILE + u0 + e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 2; ++e) val[e] = (spart[4 * LQ_TILE + u0 + e] + spart[5 * LQ_TILE + u0 + e]) * inv_rows;
      }
      float* tok = (wave == 0 ? slash_tok : vert_tok) + (int64_t)h * n + kb;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if (kb + u0 + e >= n) val[e] = 0.f;
        else if (emit) tok[u0 + e] = val[e];
      }
      const float bsum = sp_wave_sum(val[0] + val[1]);
      if (emit && lane == 0) (wave == 0 ? slash_blk : vert_blk)[(int64_t)h * nb + tile] = bsum;
    }
  }
}

// ---- host -------------------------------------------------------------------------------------------------
static inline int lq_tiles_per_wg(int64_t n, int32_t hq) {
  const int64_t work = sp_ceil_div(n, LQ_TILE) * hq;  // (head, key tile) pairs
  int tiles = 8;
  while (tiles < LQ_MAX_TILES && work / (2 * tiles) >= 1024) tiles *= 2;
  // short sequences: one round of workgroups (two per CU) rather than few long-running ones
  while (tiles > LQ_MIN_TILES && work / tiles < 512) tiles /= 2;
  return tiles;
}
// chunk count of the launch (the workspace is sized for it)
static inline int lq_chunks(int64_t n, int32_t hq) {
  return (int)sp_ceil_div(sp_ceil_div(n, LQ_TILE), lq_tiles_per_wg(n, hq));
}

extern "C" size_t sp_lastq_scores_workspace_bytes(int64_t n, int32_t hq, int32_t bs) {
  (void)bs;
  if (n <= 0 || hq <= 0) return 0;
  size_t partial = (size_t)hq * lq_chunks(n, hq) * LQ_ROWS * sizeof(float2);
  size_t rowstat = (size_t)hq * LQ_ROWS * sizeof(float2);
  return partial + rowstat;
}

extern "C" int sp_lastq_scores_bf16(const void* q, const void* k, int64_t n, int32_t hq, int32_t hkv, int32_t d,
                                    int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                                    int32_t bs, uint32_t flags, void* workspace, size_t workspace_bytes,
                                    float* vert_tok, float* slash_tok, float* vert_blk, float* slash_blk,
                                    sp_stream_t stream) {
  SP_REQUIRE(q && k && vert_tok && slash_tok && vert_blk && slash_blk && workspace, SP_ERR_INVALID_ARGUMENT,
             "sp_lastq_scores_bf16: null pointer");
  SP_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0, SP_ERR_INVALID_ARGUMENT,
             "sp_lastq_scores_bf16: hq=%d must be a positive multiple of hkv=%d", hq, hkv);
  SP_REQUIRE(bs == LQ_ROWS, SP_ERR_UNSUPPORTED, "sp_lastq_scores_bf16: block size %d unsupported (only 128)", bs);
  SP_REQUIRE(d == LQ_D, SP_ERR_UNSUPPORTED, "sp_lastq_scores_bf16: head_dim %d unsupported (only 128)", d);
  SP_REQUIRE(n >= bs, SP_ERR_INVALID_ARGUMENT, "sp_lastq_scores_bf16: seq_len %lld is shorter than one block",
             (long long)n);
  SP_REQUIRE(q_stride_n % 8 == 0 && q_stride_h % 8 == 0 && k_stride_n % 8 == 0 && k_stride_h % 8 == 0 &&
                 ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_lastq_scores_bf16: q/k must be 16-byte aligned with strides multiple of 8");
  SP_REQUIRE(workspace_bytes >= sp_lastq_scores_workspace_bytes(n, hq, bs), SP_ERR_WORKSPACE,
             "sp_lastq_scores_bf16: workspace too small");
  const int tiles_per_wg = lq_tiles_per_wg(n, hq);
  const int n_chunks = (int)sp_ceil_div(sp_ceil_div(n, LQ_TILE), tiles_per_wg);
  const int64_t nb = sp_ceil_div(n, bs);
  float2* partial = (float2*)workspace;
  float2* rowstat = partial + (size_t)hq * lq_chunks(n, hq) * LQ_ROWS;
  const float inv_sqrt_d = 1.0f / sqrtf((float)d);
  const int group = hq / hkv;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(sp_lastq_stats_kernel, dim3(n_chunks, hq), dim3(LQ_THREADS), 0, s, (const sp_bf16*)q,
                     (const sp_bf16*)k, n, hkv, group, q_stride_n, q_stride_h, k_stride_n, k_stride_h, inv_sqrt_d,
                     flags, n_chunks, tiles_per_wg, partial);
  SP_LAUNCH_CHECK();
  hipLaunchKernelGGL(sp_lastq_combine_kernel, dim3(hq), dim3(LQ_ROWS * LQ_COMBINE_GROUPS), 0, s, partial, n_chunks,
                     rowstat);
  SP_LAUNCH_CHECK();
  const size_t lds_bytes = (LQ_ROWS * LQ_PITCH + 14 * LQ_TILE) * sizeof(float);
  static bool attr_set[64] = {false};  // per device, once (idempotent)
  int dev = 0;
  SP_HIP(hipGetDevice(&dev));
  SP_REQUIRE(dev >= 0 && dev < 64, SP_ERR_UNSUPPORTED, "sp_lastq_scores_bf16: device index %d", dev);
  if (!attr_set[dev]) {
    SP_HIP(hipFuncSetAttribute((const void*)sp_lastq_probs_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds_bytes));
    attr_set[dev] = true;
  }
  const int grid_x = (int)sp_ceil_div(nb, tiles_per_wg);
  hipLaunchKernelGGL(sp_lastq_probs_kernel, dim3(grid_x, hq), dim3(LQ_THREADS), lds_bytes, s, (const sp_bf16*)q,
                     (const sp_bf16*)k, n, hkv, group, q_stride_n, q_stride_h, k_stride_n, k_stride_h, inv_sqrt_d,
                     flags, rowstat, vert_tok, slash_tok, vert_blk, slash_blk, nb, tiles_per_wg);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

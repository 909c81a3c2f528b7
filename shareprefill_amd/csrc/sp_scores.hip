// Last-block scores: softmax over all keys of the last 128 queries, reduced to the per-token
// vertical (column mean) and slash (anti-diagonal mean) vectors and their 128-token block sums.
// Replaces shareprefill/attn/attention_sharing.py:127-167, sum_all_diagonal_matrix
// (attn/utils.py:79-86) and torch_bhn_sumpool (attn/utils.py:33-44) without ever writing the
// [Hq,128,N] probability matrix to memory.
//
// Three kernels:
//   stats   : per (head, key chunk) the running row max / row sum of the logits (bf16 MFMA);
//   combine : folds the chunk partials into one (max, 1/sum) per query row, in chunk order;
//   probs   : recomputes the logits tile by tile; the column sums (vertical) and, through a permutation of keys and
//             query rows, the anti-diagonal sums (slash) both start in registers, and only a 32 KiB digest of the
//             128x128 probability tile goes through LDS.  A slash bin receives its upper part from the previous key
//             tile; that part is carried through LDS, and each workgroup recomputes one leading tile so that no
//             cross-workgroup accumulation (and no float atomic) is needed.
// Every sum runs in a fixed order, so results are reproducible run to run.
#include "sp_common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define LQ_ROWS 128          // query rows (= block size)
#define LQ_TILE 128          // keys per tile
#define LQ_D 128             // head dim
#define LQ_THREADS 256       // 4 waves per head, wave w owns 32 query rows of the last block
#define LQ_MIN_TILES 1       // key tiles per workgroup of the statistics kernel: a power of two, at most 32 -- as many as
#define LQ_MAX_TILES 32      // still leave one round of workgroups at long sequences, as few as give one at short ones
// Row maxima are kept in base-2 units (max logit * log2 e), so a probability is one fused multiply-add and one
// hardware exp2.  "No logit seen yet" is a large finite negative number, not -inf: then max, difference and exp2
// need no special case (exp2(-inf - finite) = 0 for masked logits, exp2(0) * 0 for an empty history).
#define LQ_LOG2E 1.4426950408889634f
#define LQ_NO_MAX (-1.0e30f)

// lane's operand: scaled last-block queries, 8 k-steps x 8 bf16; MFMA row m = lane % 32 of wave w is query 32 w + m of
// the last block, or query 127 - (32 w + m) with REVERSED
template <bool REVERSED>
__device__ static __forceinline__ void lq_load_q(const sp_bf16* __restrict__ q, int64_t n, int64_t sq_n, int wave, int lane,
                                        float inv_sqrt_d, bf16x8 (&qa)[8]) {
  const int row = REVERSED ? LQ_ROWS - 1 - (wave * 32 + (lane & 31)) : wave * 32 + (lane & 31);
  // (a prompt shorter than 128 tokens, possible with a block size below 128: the rows in front of its first token
  // read token 0 and are dropped by the probabilities kernel like every row in front of the last block)
  int64_t tok = n - LQ_ROWS + row;
  if (tok < 0) tok = 0;
  const sp_bf16* src = q + tok * sq_n + 8 * (lane >> 5);
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

__device__ static __forceinline__ int lq_row_of(int wave, int lane, int r) {
  return wave * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

typedef float lq_floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 lq_bf16x2 __attribute__((ext_vector_type(2)));

// ---- kernel 1: chunk partials of the row max / row sum ------------------------------------------
// Built for occupancy: sixteen waves per CU (two workgroups of two heads) hide each other's load and barrier
// latencies (fetching the next tile while the current one is used changes nothing on top of that).  That needs
// <= 128 registers per lane and <= 80 KiB of LDS per workgroup, so
//   * the K tile goes from global memory straight into LDS (128-bit direct loads, no staging registers), unpadded,
//     with the 16-byte chunk index XOR-swizzled by the row so that the operand reads stay conflict-free;
//   * the product is taken transposed, S^T = K . Q^T: in the 32x32 accumulators a lane then owns ONE query (column
//     lane % 32) and 16 of the tile's keys per 32-key group, so the running max and sum are two registers, not 32,
//     and the fold at the end is one exchange between the two lane halves.
#define LQ_KSW_BYTES (LQ_TILE * LQ_D * 2)  // 32 KiB: [128 keys][16 chunks of 16 bytes], chunk c of row r at c ^ ((r >> SWZ) & 15)

typedef __attribute__((address_space(3))) void* lq_lds_ptr;
typedef const __attribute__((address_space(1))) void* lq_gbl_ptr;

// Both kernels put TWO query heads of a kv group into one workgroup of eight waves (waves 0-3 the first head, 4-7
// the second, each wave 32 queries of the last block): the K tile is fetched once for both, and it is the L2 -> LDS
// traffic of these fetches that bounds the kernels otherwise (one tile per (query head, key tile): 1 GiB per pass at
// 128K tokens and 32 heads, about 5 TB/s when nothing else is done).  A group with an odd head count leaves the second
// half of its last workgroup without a head: those waves fetch and synchronise, and compute nothing.
#define LQ_WG_HEADS 2
#define LQ_WG_THREADS (LQ_THREADS * LQ_WG_HEADS)
static inline __host__ __device__ int lq_pairs(int group) { return (group + LQ_WG_HEADS - 1) / LQ_WG_HEADS; }

// Four wave-instructions per wave fill the tile: instruction `it` of wave w (0..7) writes the 1 KiB segment 8 * it + w
// (4 key rows); lane i writes chunk position i of the segment and fetches the global chunk that belongs there.
// SWZ = 0 serves operand reads of 16 consecutive rows, SWZ = 2 reads of rows 4 apart.
// The address of a lane's chunk is a tile-uniform base (scalar arithmetic) plus a 32-bit lane offset that does not
// change from tile to tile -- row (4 w + lane / 16) * stride + swizzled chunk, computed once: with SWZ = 0 the
// chunk is the same for all four instructions, with SWZ = 2 it takes two values (it % 2).  Only the one tile that
// reaches past the end of the sequence clamps its rows onto the last key (masked later), lane by lane.
template <int SWZ>
struct LqKLane {
  uint32_t off[SWZ == 0 ? 1 : 2];
};

template <int SWZ>
__device__ static __forceinline__ LqKLane<SWZ> lq_k_lane(int64_t sk_n, int wave8, int lane) {
  LqKLane<SWZ> kl;
  const int row0 = wave8 * 4 + (lane >> 4);  // instruction `it` adds 32 rows
#pragma unroll
  for (int v = 0; v < (SWZ == 0 ? 1 : 2); ++v) {
    const int cl = (lane & 15) ^ (((32 * v + row0) >> SWZ) & 15);
    kl.off[v] = (uint32_t)(row0 * (int)sk_n * 2 + cl * 16);
  }
  return kl;
}

template <int SWZ>
__device__ static __forceinline__ void lq_issue_k_direct(const sp_bf16* __restrict__ k, int64_t n, int64_t sk_n, int64_t kb,
                                                         char* ks, int wave8, int lane, const LqKLane<SWZ>& kl) {
  if (kb + LQ_TILE <= n) {
    const char* base = reinterpret_cast<const char*>(k + kb * sk_n);
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const char* src = base + (int64_t)it * 32 * sk_n * 2;  // uniform
      __builtin_amdgcn_global_load_lds((lq_gbl_ptr)(src + kl.off[SWZ == 0 ? 0 : it & 1]),
                                       (lq_lds_ptr)(ks + (it * 8 + wave8) * 1024), 16, 0, 0);
    }
  } else {
#pragma unroll 1
    for (int it = 0; it < 4; ++it) {
      const int seg = it * 8 + wave8;
      const int row = seg * 4 + (lane >> 4);
      const int cl = (lane & 15) ^ ((row >> SWZ) & 15);
      int64_t key = kb + row;
      if (key > n - 1) key = n - 1;
      __builtin_amdgcn_global_load_lds((lq_gbl_ptr)(k + key * sk_n + cl * 8), (lq_lds_ptr)(ks + seg * 1024), 16, 0, 0);
    }
  }
}

__global__ __launch_bounds__(LQ_WG_THREADS, 4) void sp_lastq_stats_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, int64_t n, int hkv, int group, int64_t sq_n,
    int64_t sq_h, int64_t sk_n, int64_t sk_h, float inv_sqrt_d, uint32_t flags, int n_chunks, int tiles_per_wg,
    float2* __restrict__ partial /* [hq][n_chunks][128] */) {
  __shared__ __attribute__((aligned(1024))) char Ksw[LQ_KSW_BYTES];
  const int pairs = lq_pairs(group);
  const int kvh = blockIdx.y / pairs;
  const int chunk = blockIdx.x;
  const int wave8 = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wave = wave8 & 3;                                        // query band of the wave's head
  const int hg = (blockIdx.y % pairs) * LQ_WG_HEADS + (wave8 >> 2);  // head within the kv group
  const bool has_head = hg < group;                                  // (wave-uniform)
  const int h = kvh * group + (has_head ? hg : 0);
  const int lq = lane & 31, hi = lane >> 5;
  const sp_bf16* qh = q + (int64_t)h * sq_h;
  const sp_bf16* kh = k + (int64_t)kvh * sk_h;
  bf16x8 qa[8];  // the lane's query (row 32 wave + lq of the last block), channels 16 ks + 8 hi .. + 7
  lq_load_q<false>(qh, n, sq_n, wave, lane, inv_sqrt_d, qa);
  float m = LQ_NO_MAX, l = 0.f;
  const int64_t n_tiles = sp_ceil_div(n, LQ_TILE);
  const int64_t tile0 = (int64_t)chunk * tiles_per_wg;
  // byte offset of the lane's operand chunk inside a 32-key group: row lq, logical chunk 2 ks + hi
  const int row_off = lq * 256;
  const LqKLane<0> kl = lq_k_lane<0>(sk_n, wave8, lane);
  for (int t = 0; t < tiles_per_wg; ++t) {
    const int64_t tile = tile0 + t;
    if (tile >= n_tiles) break;
    const int64_t kb = tile * LQ_TILE;
    __syncthreads();  // the previous tile's operand reads are done
    lq_issue_k_direct<0>(kh, n, sk_n, kb, Ksw, wave8, lane, kl);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct loads have landed
    __syncthreads();
    if (!has_head) continue;
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
    if (hi == 0 && has_head) partial[((int64_t)h * n_chunks + chunk) * LQ_ROWS + wave * 32 + lq] = make_float2(mn, a + b);
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

// Cross-lane sums without the LDS round trip of a lane permute (each costs a wave alone on its SIMD ~120 cycles of
// waiting, and the digest reader strings twenty of them together): lanes ^ 16 and ^ 32 through the gfx950 swaps (which
// of the two results is the lane's own does not matter to a sum), the 16 lanes of a row through DPP.
__device__ static __forceinline__ float lq_sum_xor16(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)a[0]) + __builtin_bit_cast(float, (uint32_t)a[1]);
}
__device__ static __forceinline__ float lq_sum_xor32(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)a[0]) + __builtin_bit_cast(float, (uint32_t)a[1]);
}
template <int CTRL>
__device__ static __forceinline__ float lq_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// the sum over all 64 lanes, in every lane; fixed order
__device__ static __forceinline__ float lq_wave_sum(float v) {
  v += lq_dpp<0xB1>(v);   // quad_perm [1, 0, 3, 2]
  v += lq_dpp<0x4E>(v);   // quad_perm [2, 3, 0, 1]
  v += lq_dpp<0x141>(v);  // row_half_mirror
  v += lq_dpp<0x140>(v);  // row_mirror
  return lq_sum_xor32(lq_sum_xor16(v));
}

// ---- kernel 3: probabilities -> vertical / slash ------------------------------------------------------
// S = Q . K^T with the queries as the A operand, so that in the 32x32 accumulators a lane owns key columns and 16
// query rows of each: the column (vertical) sums start in registers.  Two permutations make the anti-diagonal
// (slash) sums start in registers too:
//   * a lane's four accumulator sets take the four CONSECUTIVE keys 4 lq .. 4 lq + 3 (the B operand of key sub-tile
//     nt reads K row 4 lq + nt), and
//   * MFMA row m of wave w is query 127 - (32 w + m) of the last block, i.e. the rows run backwards.
// Element (row i' = 32 w + 8 g + 4 hi + j, key 4 lq + nt) then belongs to slash bin  kb + 4 lq + 4 G + (nt + j)  with
// G = 8 w + 2 g + hi: the sixteen elements of a register group g fall on seven bins of the same lane, nine additions
// without any lane exchange, and every bin offset is a multiple of four plus (nt + j).  The lane writes the seven sums
// as two aligned 16-byte LDS stores (offsets 0..3 to Dm[G], 4..6 to Dh[G], which is Dm shifted by one chunk), 32 KiB
// for the whole 128 x 128 tile, and a thread collects four bins with 16-byte reads:
// an eighth of the LDS traffic of a full probability tile, and no select between this tile's and the next tile's bins.
// Bins 128..254 of a tile belong to the next tile's first 127 tokens: they are carried through LDS, and each
// workgroup recomputes one leading tile so that no cross-workgroup accumulation (and no float atomic) is needed.
// LDS of the workgroup (one per CU, two waves per SIMD): two K tiles (the next one is fetched while the current one is
// used), and per head the diagonal digest, the column partials, the carried bins and the block-sum parts.
#define LQP_D_FLOATS (2 * 32 * LQ_TILE)  // Dm[32][128] | Dh[32][128]
struct LqpHeadLds {
  float D[LQP_D_FLOATS];
  float vpart[8][LQ_TILE];  // column sums per (wave, lane half)
  float carry[2][LQ_TILE];  // bins 128..255 of the previous tile, by tile parity
  float bpart[2][2][4];     // [tile parity][slash, vertical][wave] block-sum parts
  float zero16[4];
};
#define LQP_LDS_BYTES (2 * LQ_KSW_BYTES + LQ_WG_HEADS * sizeof(LqpHeadLds))

__global__ __launch_bounds__(LQ_WG_THREADS, 2) void sp_lastq_probs_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, int64_t n, int hkv, int group, int64_t sq_n,
    int64_t sq_h, int64_t sk_n, int64_t sk_h, float inv_sqrt_d, uint32_t flags, const float2* __restrict__ rowstat,
    float* __restrict__ vert_tok, float* __restrict__ slash_tok, float* __restrict__ vert_blk,
    float* __restrict__ slash_blk, int64_t nb, int tiles_per_wg, int bs) {
  extern __shared__ __attribute__((aligned(1024))) char lqp_lds[];
  char* R2 = lqp_lds;  // [2][LQ_KSW_BYTES]
  const int pairs = lq_pairs(group);
  const int kvh = blockIdx.y / pairs;
  const int wave8 = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wave = wave8 & 3;
  const int hg = (blockIdx.y % pairs) * LQ_WG_HEADS + (wave8 >> 2);
  const bool has_head = hg < group;  // (wave-uniform)
  const int h = kvh * group + (has_head ? hg : 0);
  LqpHeadLds& L = reinterpret_cast<LqpHeadLds*>(lqp_lds + 2 * LQ_KSW_BYTES)[wave8 >> 2];
  const int tid = threadIdx.x & (LQ_THREADS - 1);  // thread within the head's four waves
  const int lq = lane & 31, hi = lane >> 5;
  const sp_bf16* qh = q + (int64_t)h * sq_h;
  const sp_bf16* kh = k + (int64_t)kvh * sk_h;
  bf16x8 qa[8];
  lq_load_q<true>(qh, n, sq_n, wave, lane, inv_sqrt_d, qa);
  // per row: max + log2(sum), so that a probability is exp2(logit * log2 e - rm): the normalisation rides in the
  // exponent instead of costing a multiplication per element
  // A block size below 128 has its last block's queries in the tail of the 128 rows: the rows in front of them get
  // rm = +inf, so that every probability of theirs is exp2(-inf) = 0, and the means divide by bs.
  float rm[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int qi = LQ_ROWS - 1 - lq_row_of(wave, lane, r);  // query index inside the last 128 tokens
    const float2 st = rowstat[h * LQ_ROWS + qi];
    rm[r] = qi >= LQ_ROWS - bs ? st.x - __builtin_amdgcn_logf(st.y) : INFINITY;  // st.y = 1 / sum; v_log_f32 is log2
  }
  const int64_t n_tiles = sp_ceil_div(n, LQ_TILE);
  const int64_t first = (int64_t)blockIdx.x * tiles_per_wg;
  const float inv_rows = 1.0f / (float)bs;
  const bool write_blk = bs == LQ_ROWS;  // the block sums of smaller blocks come from sp_lastq_block_sums_kernel
  const int64_t t_begin = first > 0 ? first - 1 : 0;
  const int64_t t_end = first + tiles_per_wg < n_tiles ? first + tiles_per_wg : n_tiles;
  float* Dm = L.D;
  float* Dh = Dm + 32 * LQ_TILE;
  if (tid < LQ_TILE) L.carry[(t_begin & 1) ^ 1][tid] = 0.f;  // nothing is carried into the first tile
  if (tid < 4) L.zero16[tid] = 0.f;
  // B operand of key sub-tile nt, k-step ks: K row 4 lq + nt, logical 16-byte chunk 2 ks + hi (swizzled by row / 4)
  const int b_off = lq * 1024;
  const int b_swz = lq & 15;

  const LqKLane<2> kl = lq_k_lane<2>(sk_n, wave8, lane);
  lq_issue_k_direct<2>(kh, n, sk_n, t_begin * LQ_TILE, R2 + (t_begin & 1) * LQ_KSW_BYTES, wave8, lane, kl);
  for (int64_t tile = t_begin; tile < t_end; ++tile) {
    const int64_t kb = tile * LQ_TILE;
    const int par = (int)(tile & 1);
    const char* R = R2 + par * LQ_KSW_BYTES;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct loads of this tile have landed
    __syncthreads();  // ... and everyone's; the previous tile's K reads and digest reads are done
    if (tile + 1 < t_end)  // the next K tile, into the buffer the previous tile has left
      lq_issue_k_direct<2>(kh, n, sk_n, kb + LQ_TILE, R2 + (par ^ 1) * LQ_KSW_BYTES, wave8, lane, kl);
    if (tid == 0 && tile > first && has_head && write_blk) {  // the previous tile's block sums: its parts were complete one barrier ago
      const float* bp = &L.bpart[par ^ 1][0][0];
      slash_blk[(int64_t)h * nb + tile - 1] = bp[0] + bp[1];
      vert_blk[(int64_t)h * nb + tile - 1] = (bp[4] + bp[5]) + (bp[6] + bp[7]);
    }
    if (has_head) {
      // acc[nt][r] = S[row i' = 32 w + 8 (r / 4) + 4 hi + r % 4][key kb + 4 lq + nt]
      floatx16 acc[4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const char* src = R + b_off + nt * 256;
        floatx16 c = {0};
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const uint4 raw = *reinterpret_cast<const uint4*>(src + (((2 * ks + hi) ^ b_swz) << 4));
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[ks], __builtin_bit_cast(bf16x8, raw), c, 0, 0, 0);
        }
        acc[nt] = c;
      }
      if (flags & SP_FLAG_LOGITS_BF16) {  // the reference's qk tensor is bf16 (attention_sharing.py:129-139)
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
      if (kb + LQ_TILE > n - LQ_ROWS) {  // (tile-uniform) the tile reaches into the last block or past the end
        // key <= query position  <=>  c - i <= (n - 128) - kb;  key < n  <=>  c < n - kb   (c, i: offsets in the tile)
        const int64_t d64 = (n - LQ_ROWS) - kb, e64 = n - kb;
        const int dlim = d64 > 1024 ? 1024 : (int)d64, elim = e64 > 1024 ? 1024 : (int)e64;
        int ln = lane;
        asm volatile("" : "+v"(ln));  // keeps this rare path's lane arithmetic out of the tile loop's registers
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = LQ_ROWS - 1 - lq_row_of(wave, ln, r);
#pragma unroll
          for (int nt = 0; nt < 4; ++nt) {
            const int c = 4 * (ln & 31) + nt;
            if (!(c - i <= dlim && c < elim)) acc[nt][r] = -INFINITY;
          }
        }
      }
      // probabilities (exp2(-inf) = 0 for the masked entries), column sums and the seven diagonal sums of each group
      float vs[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float x[4][4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            x[nt][j] = __builtin_amdgcn_exp2f(__builtin_fmaf(acc[nt][4 * g + j], LQ_LOG2E, -rm[4 * g + j]));
            vs[nt] += x[nt][j];
          }
        float4 dm, dh;
        dm.x = x[0][0];
        dm.y = x[0][1] + x[1][0];
        dm.z = (x[0][2] + x[1][1]) + x[2][0];
        dm.w = (x[0][3] + x[1][2]) + (x[2][1] + x[3][0]);
        dh.x = (x[1][3] + x[2][2]) + x[3][1];
        dh.y = x[2][3] + x[3][2];
        dh.z = x[3][3];
        dh.w = 0.f;
        const int G = 8 * wave + 2 * g + hi;
        *reinterpret_cast<float4*>(Dm + G * LQ_TILE + 4 * lq) = dm;
        *reinterpret_cast<float4*>(Dh + G * LQ_TILE + 4 * lq) = dh;
      }
      *reinterpret_cast<float4*>(&L.vpart[2 * wave + hi][4 * lq]) = make_float4(vs[0], vs[1], vs[2], vs[3]);
    }
    __syncthreads();
    if (has_head) {
      const bool emit = tile >= first;
      // slash: thread (pg, qd) gathers bins 4 pg .. 4 pg + 3 from the eight groups G = 8 qd .. 8 qd + 7 (Dm[G] holds
      // bins 4 G .. 4 G + 127, Dh[G] bins 4 G + 4 .. 4 G + 131), then the four lane quarters of the wave meet.
      // Every LDS read of the stage -- digest chunks, carried bins, column partials -- is issued before the first
      // use of any: one round trip for the wave instead of a chain of them.
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int pg = 16 * wave + (ln & 15), qd = ln >> 4;
      const int p0 = 4 * pg;  // 64 wave + 4 (lane % 16): waves 0, 1 hold this tile's bins, waves 2, 3 the next tile's
      float4 vm[8], vh[8];
#pragma unroll
      for (int gi = 0; gi < 8; ++gi) {
        const int G = 8 * qd + gi;
        const int cm = pg - G;  // chunk of Dm[G]; Dh[G] is one chunk behind.  Chunks outside a row read 16 zero bytes.
        const float* am = (unsigned)cm < 32u ? Dm + G * LQ_TILE + 4 * cm : L.zero16;
        const float* ah = (unsigned)(cm - 1) < 32u ? Dh + G * LQ_TILE + 4 * (cm - 1) : L.zero16;
        vm[gi] = *reinterpret_cast<const float4*>(am);
        vh[gi] = *reinterpret_cast<const float4*>(ah);
      }
      const float4 cr = *reinterpret_cast<const float4*>(&L.carry[par ^ 1][p0 & (LQ_TILE - 1)]);  // (used by waves 0, 1)
      const int col = 32 * wave + (ln & 31);
      float vp[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) vp[j] = L.vpart[j][col];
      float sv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int gi = 0; gi < 8; ++gi) {
        sv[0] += vm[gi].x, sv[1] += vm[gi].y, sv[2] += vm[gi].z, sv[3] += vm[gi].w;
        sv[0] += vh[gi].x, sv[1] += vh[gi].y, sv[2] += vh[gi].z, sv[3] += vh[gi].w;
      }
#pragma unroll
      for (int d = 0; d < 4; ++d) sv[d] = lq_sum_xor32(lq_sum_xor16(sv[d]));
      if (wave < 2) {
        float tot = 0.f;
        if (ln < 16) {
          float* tok = slash_tok + (int64_t)h * n + kb + p0;
          const float crv[4] = {cr.x, cr.y, cr.z, cr.w};
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            float val = (crv[d] + sv[d]) * inv_rows;
            if (kb + p0 + d >= n) val = 0.f;
            else if (emit) tok[d] = val;
            tot += val;
          }
        }
        tot = lq_wave_sum(tot);
        if (ln == 0) L.bpart[par][0][wave] = tot;
      } else if (ln < 16) {
        *reinterpret_cast<float4*>(&L.carry[par][p0 - LQ_TILE]) = make_float4(sv[0], sv[1], sv[2], sv[3]);
      }
      // vertical: lanes 0..31 of wave w fold the eight partials of columns 32 w .. 32 w + 31
      float val = 0.f;
      if (ln < 32) {
        val = (((vp[0] + vp[1]) + (vp[2] + vp[3])) + ((vp[4] + vp[5]) + (vp[6] + vp[7]))) * inv_rows;
        if (kb + col >= n) val = 0.f;
        else if (emit) vert_tok[(int64_t)h * n + kb + col] = val;
      }
      val = lq_wave_sum(val);
      if (ln == 0) L.bpart[par][1][wave] = val;
    }
  }
  __syncthreads();
  if (tid == 0 && t_end > first && has_head && write_blk) {  // the last tile's block sums
    const float* bp = &L.bpart[(t_end - 1) & 1][0][0];
    slash_blk[(int64_t)h * nb + t_end - 1] = bp[0] + bp[1];
    vert_blk[(int64_t)h * nb + t_end - 1] = (bp[4] + bp[5]) + (bp[6] + bp[7]);
  }
}

// Block sums of the token vectors for block sizes below 128 (torch_bhn_sumpool, utils.py:33-44): one thread per
// (head, block) adds its bs tokens in ascending order; tokens beyond the sequence count as zero.
__global__ __launch_bounds__(256) void sp_lastq_block_sums_kernel(const float* __restrict__ vert_tok,
                                                                  const float* __restrict__ slash_tok, int64_t n,
                                                                  int64_t nb, int bs, int64_t total,
                                                                  float* __restrict__ vert_blk,
                                                                  float* __restrict__ slash_blk) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // h * nb + block
  if (i >= total) return;
  const int64_t h = i / nb, b = i % nb;
  const int64_t t0 = b * bs, t1 = t0 + bs < n ? t0 + bs : n;
  float sv = 0.f, ss = 0.f;
  for (int64_t t = t0; t < t1; ++t) {
    sv += vert_tok[h * n + t];
    ss += slash_tok[h * n + t];
  }
  vert_blk[i] = sv;
  slash_blk[i] = ss;
}

// ---- pooled block probabilities of query-aware heads (attention_sharing.py:350-360) -------------------------------
// probs[h][r][c] = softmax over c <= r of  bf16(qbar[r][h] / sqrt d) . kbar[c][kv head of h],  zero for c > r.
// The same two passes as the last-query scores, over 128-row tiles of the pooled queries against 128-row tiles of
// the pooled keys: pass 1 the row maxima and sums (transposed product, a lane owns one query), pass 2 the logits
// again (a lane owns key columns: coalesced rows of the output), normalised in the exponent.  One workgroup per (row
// tile, head); the K tile goes straight from global memory into LDS, XOR-swizzled; heads that are not query-aware
// leave at once.
#define BPM_THREADS 256

// 32 segments of 1 KiB (4 pooled-key rows each): instruction `it` of wave w (0..3) fills segment 4 it + w
__device__ static __forceinline__ void bpm_issue_k(const sp_bf16* __restrict__ kb_head, int64_t row_stride, int nb,
                                                   int c_tile, char* ks, int wave, int lane) {
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int seg = it * 4 + wave;
    const int row = seg * 4 + (lane >> 4);
    const int cl = (lane & 15) ^ (row & 15);
    int key = c_tile * LQ_TILE + row;
    if (key > nb - 1) key = nb - 1;  // rows past the end are clamped onto the last pooled key (masked later)
    __builtin_amdgcn_global_load_lds((lq_gbl_ptr)(kb_head + (int64_t)key * row_stride + cl * 8),
                                     (lq_lds_ptr)(ks + seg * 1024), 16, 0, 0);
  }
}

// elements r, r + 1 of an accumulator rounded to bf16 (hardware conversion, round to nearest even)
__device__ static __forceinline__ void bpm_round_pair(floatx16& v, int r) {
  lq_floatx2 f;
  f[0] = v[r];
  f[1] = v[r + 1];
  const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, lq_bf16x2));
  v[r] = __uint_as_float(pk << 16);
  v[r + 1] = __uint_as_float(pk & 0xffff0000u);
}

__global__ __launch_bounds__(BPM_THREADS, 2) void sp_block_probs_mfma_kernel(
    const sp_bf16* __restrict__ qbar /* [nb][hq][128] */, const sp_bf16* __restrict__ kbar /* [nb][hkv][128] */,
    const int32_t* __restrict__ decision, int hq, int hkv, int nb, uint32_t flags, float inv_sqrt_d,
    float* __restrict__ probs /* [hq][nb][nb] */) {
  __shared__ __attribute__((aligned(1024))) char Ks[LQ_KSW_BYTES];
  __shared__ float2 rstat[LQ_ROWS];
  const int rt = blockIdx.x, h = blockIdx.y;
  if (decision[h] != SP_DEC_QA) return;
  const int kvh = h / (hq / hkv);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lq = lane & 31, hi = lane >> 5;
  const sp_bf16* kb_head = kbar + (int64_t)kvh * LQ_D;
  const int64_t k_stride = (int64_t)hkv * LQ_D;
  // the lane's operand row: pooled query rt * 128 + 32 wave + lq (clamped), scaled and rounded as the reference's
  // avg_q / sqrt(d) in bf16
  bf16x8 qa[8];
  {
    int row = rt * LQ_ROWS + wave * 32 + lq;
    if (row > nb - 1) row = nb - 1;
    const sp_bf16* src = qbar + ((int64_t)row * hq + h) * LQ_D + 8 * hi;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      uint4 raw = *reinterpret_cast<const uint4*>(src + 16 * ks);
      uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = sp_f32_to_bf16(__uint_as_float(w[j] << 16) * inv_sqrt_d);
        const uint32_t hi16 = sp_f32_to_bf16(__uint_as_float(w[j] & 0xffff0000u) * inv_sqrt_d);
        w[j] = lo | (hi16 << 16);
      }
      raw = make_uint4(w[0], w[1], w[2], w[3]);
      qa[ks] = __builtin_bit_cast(bf16x8, raw);
    }
  }
  const int row_off = lq * 256;

  // ---- pass 1: row maximum (base-2 units) and sum, transposed product: the lane's query is row 32 wave + lq ----
  {
    float m = LQ_NO_MAX, l = 0.f;
    const int my_row = rt * LQ_ROWS + wave * 32 + lq;
    for (int ct = 0; ct <= rt; ++ct) {
      __syncthreads();
      bpm_issue_k(kb_head, k_stride, nb, ct, Ks, wave, lane);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
#pragma unroll 1
      for (int half = 0; half < 2; ++half) {
        floatx16 acc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const char* src = Ks + (2 * half + j) * 32 * 256 + row_off;
          floatx16 c = {0};
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) {
            const uint4 raw = *reinterpret_cast<const uint4*>(src + (((2 * ks + hi) ^ (lq & 15)) << 4));
            c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, raw), qa[ks], c, 0, 0, 0);
          }
          acc[j] = c;
        }
        if (flags & SP_FLAG_LOGITS_BF16) {
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; r += 2) bpm_round_pair(acc[j], r);
        }
        if (ct == rt) {  // the diagonal tile: keys beyond the row's own block (and beyond the last block) are masked
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = ct * LQ_TILE + 64 * half + 32 * j + 8 * (r >> 2) + 4 * hi + (r & 3);
              if (key > my_row || key >= nb) acc[j][r] = -INFINITY;
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
    const float m2 = __shfl_xor(m, 32, SP_WAVE), l2 = __shfl_xor(l, 32, SP_WAVE);
    const float mn = fmaxf(m, m2);
    const float a = (hi ? l2 : l) * __builtin_amdgcn_exp2f((hi ? m2 : m) - mn);
    const float b = (hi ? l : l2) * __builtin_amdgcn_exp2f((hi ? m : m2) - mn);
    // max + log2(sum): a probability is then exp2(logit * log2 e - that)
    if (hi == 0) rstat[wave * 32 + lq] = make_float2(mn + __builtin_amdgcn_logf(a + b), 0.f);
  }
  __syncthreads();
  float rm[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) rm[r] = rstat[lq_row_of(wave, lane, r)].x;

  // ---- pass 2: probabilities; acc[nt][r] = S[row 32 wave + 8 (r / 4) + 4 hi + r % 4][key 32 nt + lq] ----
  for (int ct = 0; ct <= rt; ++ct) {
    __syncthreads();
    bpm_issue_k(kb_head, k_stride, nb, ct, Ks, wave, lane);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#pragma unroll 1
    for (int nt = 0; nt < 4; ++nt) {
      const char* src = Ks + nt * 32 * 256 + row_off;
      floatx16 c = {0};
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src + (((2 * ks + hi) ^ (lq & 15)) << 4));
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[ks], __builtin_bit_cast(bf16x8, raw), c, 0, 0, 0);
      }
      if (flags & SP_FLAG_LOGITS_BF16) {
#pragma unroll
        for (int r = 0; r < 16; r += 2) bpm_round_pair(c, r);
      }
      const int key = ct * LQ_TILE + 32 * nt + lq;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = rt * LQ_ROWS + lq_row_of(wave, lane, r);
        float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(c[r], LQ_LOG2E, -rm[r]));
        if (key > row) pv = 0.f;
        if (row < nb && key < nb) probs[((int64_t)h * nb + row) * nb + key] = pv;
      }
    }
  }
  // the rest of the rows: zero beyond the diagonal tile
  {
    const int c0 = (rt + 1) * LQ_TILE;
    for (int i = 0; i < LQ_ROWS; ++i) {
      const int row = rt * LQ_ROWS + i;
      if (row >= nb) break;
      float* out = probs + ((int64_t)h * nb + row) * nb;
      for (int c = c0 + (int)threadIdx.x; c < nb; c += BPM_THREADS) out[c] = 0.f;
    }
  }
}

// launcher for sp_queryaware_select_bf16 (head_dim 128)
int sp_block_probs_mfma_launch(const void* qbar, const void* kbar, const int32_t* decision, int32_t hq, int32_t hkv,
                               int32_t nb, uint32_t flags, float* probs, hipStream_t stream) {
  hipLaunchKernelGGL(sp_block_probs_mfma_kernel, dim3((unsigned)sp_ceil_div(nb, LQ_ROWS), hq), dim3(BPM_THREADS), 0, stream,
                     (const sp_bf16*)qbar, (const sp_bf16*)kbar, decision, (int)hq, (int)hkv, (int)nb, flags,
                     sp_inv_sqrt_dim(flags, LQ_D), probs);
  SP_LAUNCH_CHECK();
  return SP_OK;
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
// Output tiles per workgroup of the probabilities kernel.  A workgroup of T output tiles computes T + 1 (the leading
// tile), and the launch runs in ceil(workgroups / 256) rounds, one workgroup per CU: take the T that minimises
// rounds x (T + 1).
static inline int lq_probs_tiles_per_wg(int64_t nb, int32_t wg_rows) {
  const int64_t slots = 256;
  int best = 1;
  int64_t best_cost = INT64_MAX;
  for (int t = 1; t <= 64; ++t) {
    const int64_t wgs = sp_ceil_div(nb, t) * wg_rows;
    const int64_t cost = sp_ceil_div(wgs, slots) * (t + (sp_ceil_div(nb, t) > 1 ? 1 : 0));
    if (cost < best_cost) best_cost = cost, best = t;
  }
  return best;
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
  SP_REQUIRE(bs == 128 || bs == 64 || bs == 32 || bs == 16, SP_ERR_UNSUPPORTED,
             "sp_lastq_scores_bf16: block size %d unsupported (16, 32, 64 or 128)", bs);
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
  const int64_t nb = sp_ceil_div(n, bs);          // blocks of the caller's size: the length of vert_blk / slash_blk
  const int64_t nb_tiles = sp_ceil_div(n, LQ_TILE);  // 128-token tiles the kernels walk
  float2* partial = (float2*)workspace;
  float2* rowstat = partial + (size_t)hq * lq_chunks(n, hq) * LQ_ROWS;
  const float inv_sqrt_d = sp_inv_sqrt_dim(flags, d);
  const int group = hq / hkv;
  hipStream_t s = (hipStream_t)stream;
  const int wg_rows = hkv * lq_pairs(group);  // workgroups per key chunk: LQ_WG_HEADS heads of one kv group each
  hipLaunchKernelGGL(sp_lastq_stats_kernel, dim3(n_chunks, wg_rows), dim3(LQ_WG_THREADS), 0, s, (const sp_bf16*)q,
                     (const sp_bf16*)k, n, hkv, group, q_stride_n, q_stride_h, k_stride_n, k_stride_h, inv_sqrt_d,
                     flags, n_chunks, tiles_per_wg, partial);
  SP_LAUNCH_CHECK();
  hipLaunchKernelGGL(sp_lastq_combine_kernel, dim3(hq), dim3(LQ_ROWS * LQ_COMBINE_GROUPS), 0, s, partial, n_chunks,
                     rowstat);
  SP_LAUNCH_CHECK();
  static bool attr_set[64] = {false};  // per device, once (idempotent)
  int dev = 0;
  SP_HIP(hipGetDevice(&dev));
  SP_REQUIRE(dev >= 0 && dev < 64, SP_ERR_UNSUPPORTED, "sp_lastq_scores_bf16: device index %d", dev);
  if (!attr_set[dev]) {
    SP_HIP(hipFuncSetAttribute((const void*)sp_lastq_probs_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)LQP_LDS_BYTES));
    attr_set[dev] = true;
  }
  const int tiles_probs = lq_probs_tiles_per_wg(nb_tiles, wg_rows);
  const int grid_x = (int)sp_ceil_div(nb_tiles, tiles_probs);
  hipLaunchKernelGGL(sp_lastq_probs_kernel, dim3(grid_x, wg_rows), dim3(LQ_WG_THREADS), LQP_LDS_BYTES, s, (const sp_bf16*)q,
                     (const sp_bf16*)k, n, hkv, group, q_stride_n, q_stride_h, k_stride_n, k_stride_h, inv_sqrt_d,
                     flags, rowstat, vert_tok, slash_tok, vert_blk, slash_blk, nb_tiles, tiles_probs, (int)bs);
  SP_LAUNCH_CHECK();
  if (bs != LQ_ROWS) {
    const int64_t total = (int64_t)hq * nb;
    hipLaunchKernelGGL(sp_lastq_block_sums_kernel, dim3((unsigned)sp_ceil_div(total, 256)), dim3(256), 0, s, vert_tok,
                       slash_tok, n, nb, (int)bs, total, vert_blk, slash_blk);
    SP_LAUNCH_CHECK();
  }
  return SP_OK;
}

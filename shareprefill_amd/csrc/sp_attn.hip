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

// ---- work distribution ----------------------------------------------------------------------------------
// The kernel is persistent, 2 workgroups per CU.  Work items are (head, query block) rows, grouped in gangs of
// AT_GANG consecutive query blocks of ONE head.  Gangs are dealt statically to the 8 XCDs (queue x = gang
// position % 8; workgroup b serves queue b % 8 first -- workgroups are placed on XCDs round-robin), so the
// 64 workgroups of an XCD start a gang together at column 0 and sweep the key blocks nearly in lock-step:
// every K / V^T tile one of them pulls into the XCD's L2 is hit by the others.  The head order inside a kv
// group is rotated from chunk to chunk so that every queue sees every head, heavy (late) rows go first, and a
// workgroup whose queue is empty steals from the other queues.  Pulling is by atomic tickets only: nobody
// ever waits for anybody, and every workgroup leaves once all eight queues are exhausted.
#define AT_GANG 64

struct AtGeom {
  int group, nb, n_chunks, n_gangs;
};

__device__ static inline int at_queue_items(const AtGeom& gm, int xq) {
  const int gangs = gm.n_gangs > xq ? (gm.n_gangs - xq + 7) / 8 : 0;
  return gangs * AT_GANG;
}

// ticket of queue xq -> (head, query block); false for the padding slots of the last row chunk
__device__ static inline bool at_item(const AtGeom& gm, int xq, int ticket, int& h, int& r) {
  const int pos = (ticket / AT_GANG) * 8 + xq;  // gang position
  const int slot = ticket % AT_GANG;
  const int i = pos % gm.group;
  const int rest = pos / gm.group;
  const int j = rest % gm.n_chunks;  // row chunk, 0 = the last (heaviest) rows
  const int kvh = rest / gm.n_chunks;
  h = kvh * gm.group + (i + j) % gm.group;
  r = gm.nb - 1 - (j * AT_GANG + slot);
  return r >= 0;
}

// ---- LDS staging -------------------------------------------------------------------------------------------
// A block is processed as two sub-tiles of 64 keys.  One stage holds a K sub-tile [64 keys][16 chunks] and a
// V^T sub-tile [128 channels][8 chunks] (chunk = 16 bytes = 8 bf16), 32 KiB; two stages are double-buffered.
// Tiles are filled by direct global->LDS 128-bit loads: lane i of a wave writes LDS chunk (base + i), fetching
// whichever global chunk belongs there.  Instead of row padding the chunk index is XOR-swizzled with the row,
//   K  : chunk c of row r sits at r*16 + (c ^ (r & 15))
//   V^T: chunk c of row r sits at r*8  + (c ^ ((r >> 1) & 7))
// so the 16 lanes that read the same logical chunk of 16 consecutive rows hit 16 different bank groups.
#define AT_SUB 64
#define AT_KSTAGE_BYTES (AT_SUB * AT_D * 2)      // 16 KiB
#define AT_VSTAGE_BYTES (AT_D * AT_SUB * 2)      // 16 KiB
#define AT_STAGE_BYTES (AT_KSTAGE_BYTES + AT_VSTAGE_BYTES)

typedef __attribute__((address_space(3))) void* at_lds_ptr;
typedef const __attribute__((address_space(1))) void* at_gbl_ptr;

// lane-constant byte offsets of the four K and four V^T chunks a lane fetches per sub-tile
struct AtLoadOffsets {
  uint32_t k[4], v[4];
};

__device__ static inline void at_load_offsets(AtLoadOffsets& lo, int64_t sk_n, int wave, int lane) {
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int seg = it * 4 + wave;  // 1 KiB segment of the tile handled by this wave-instruction
    const int krow = seg * 4 + (lane >> 4);
    lo.k[it] = (uint32_t)(krow * (int)sk_n + (((lane & 15) ^ (krow & 15)) * 8)) * 2u;
    const int vrow = seg * 8 + (lane >> 3);
    lo.v[it] = (uint32_t)(vrow * AT_BS + (((lane & 7) ^ ((vrow >> 1) & 7)) * 8)) * 2u;
  }
}

__device__ static inline void at_issue_sub(const AtLoadOffsets& lo, const sp_bf16* __restrict__ kh,
                                           const sp_bf16* __restrict__ vth, int64_t n, int64_t sk_n, int c, int half,
                                           char* stage, int wave, int lane) {
  const int64_t key0 = (int64_t)c * AT_BS + half * AT_SUB;
  const char* vbase = reinterpret_cast<const char*>(vth + (int64_t)c * AT_D * AT_BS + half * AT_SUB);
  if (key0 + AT_SUB <= n) {  // every key row exists: uniform base + lane-constant offset
    const char* kbase = reinterpret_cast<const char*>(kh + key0 * sk_n);
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int seg = it * 4 + wave;
      __builtin_amdgcn_global_load_lds((at_gbl_ptr)(kbase + lo.k[it]), (at_lds_ptr)(stage + seg * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((at_gbl_ptr)(vbase + lo.v[it]),
                                       (at_lds_ptr)(stage + AT_KSTAGE_BYTES + seg * 1024), 16, 0, 0);
    }
  } else {  // ragged tail of the sequence: rows beyond the last key are clamped onto it
    const int64_t lim64 = n - 1 - key0;
    const int lim = lim64 < 0 ? 0 : (int)lim64;
    const sp_bf16* kbase = kh + (lim64 < 0 ? (n - 1) : key0) * sk_n;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int seg = it * 4 + wave;
      const int row = seg * 4 + (lane >> 4);
      const int cl = (lane & 15) ^ (row & 15);
      const int rowc = row < lim ? row : lim;
      const sp_bf16* g = kbase + (uint32_t)(rowc * (int)sk_n + cl * 8);
      __builtin_amdgcn_global_load_lds((at_gbl_ptr)g, (at_lds_ptr)(stage + seg * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((at_gbl_ptr)(vbase + lo.v[it]),
                                       (at_lds_ptr)(stage + AT_KSTAGE_BYTES + seg * 1024), 16, 0, 0);
    }
  }
}

__device__ static inline bf16x8 at_pack8(const floatx16& a, int base) {
  floatx8 f;
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = a[base + j];
  return __builtin_convertvector(f, bf16x8);
}

__device__ static inline bf16x8 at_lds128(const char* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// iterator over the set bits (columns c <= r) of one mask row; uniform across the workgroup
struct AtBlocks {
  const uint64_t* row;
  int r, w;
  uint64_t word;
  __device__ void init(const uint64_t* row_, int r_) {
    row = row_;
    r = r_;
    w = 0;
    word = fetch(0);
  }
  __device__ uint64_t fetch(int wi) const {
    uint64_t x = row[wi];
    if (wi == (r >> 6) && (r & 63) != 63) x &= (2ull << (r & 63)) - 1ull;
    return x;
  }
  __device__ int next() {
    while (word == 0) {
      if (++w > (r >> 6)) return -1;
      word = fetch(w);
    }
    const int c = w * 64 + __builtin_ctzll(word);
    word &= word - 1;
    return c;
  }
};

#define AT_WAIT_VMCNT0() __builtin_amdgcn_s_waitcnt(0x0F70)  // vmcnt(0) only: the direct-to-LDS loads have landed

__global__ __launch_bounds__(AT_THREADS, 2) void sp_attn_fwd_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const sp_bf16* __restrict__ vt,
    const uint64_t* __restrict__ mask, const int32_t* __restrict__ decision, sp_bf16* __restrict__ out,
    float2* __restrict__ rowstat, int64_t n, int hq, int hkv, int64_t sq_n, int64_t sq_h, int64_t sk_n,
    int64_t sk_h, int nb, int nbw, float scale_log2, int* __restrict__ sched) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // 2 stages x 32 KiB
  __shared__ int s_queue, s_ticket;

  AtGeom gm;
  gm.group = hq / hkv;
  gm.nb = nb;
  gm.n_chunks = (nb + AT_GANG - 1) / AT_GANG;
  gm.n_gangs = hq * gm.n_chunks;
  const int xcd = blockIdx.x & 7;
  int first_try = 0;  // queues before this offset are known to be empty (used by thread 0 only)
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int lq = lane & 31, g = lane >> 5;
  const int q_off = wave * 32 + lq;  // query offset inside the block

  // lane-constant LDS read offsets (bytes) inside a stage
  int koff[8];  // K rows lq (+32 via immediate), logical chunk 2*ks + g
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) koff[ks] = lq * 256 + (((2 * ks + g) ^ (lq & 15)) << 4);
  int voff[4];  // V^T rows lq (+32*dt via immediate), logical chunk 4*kt + 2*s + g, index kt*2+s
#pragma unroll
  for (int j = 0; j < 4; ++j) voff[j] = AT_KSTAGE_BYTES + lq * 128 + (((2 * j + g) ^ ((lq >> 1) & 7)) << 4);
  AtLoadOffsets lo;
  at_load_offsets(lo, sk_n, wave, lane);

  const bf16x8 ones = __builtin_bit_cast(bf16x8, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));

  for (;;) {
    __syncthreads();  // previous item's LDS reads are done
    if (t == 0) {
      int found = -1, tk = 0;
      for (int a = first_try; a < 8; ++a) {
        const int xq = (xcd + a) & 7;
        tk = atomicAdd(&sched[xq * 16], 1);
        if (tk < at_queue_items(gm, xq)) {
          found = xq;
          first_try = a;
          break;
        }
      }
      s_queue = found;
      s_ticket = tk;
    }
    __syncthreads();
    if (s_queue < 0) break;
    int h, r;
    if (!at_item(gm, s_queue, s_ticket, h, r)) continue;
    const int kvh = h / gm.group;
    const sp_bf16* kh = k + (int64_t)kvh * sk_h;
    const sp_bf16* vth = vt + (int64_t)kvh * nb * AT_D * AT_BS;
    const uint64_t* mrow = mask + ((int64_t)h * nb + r) * nbw;

    AtBlocks it;
    it.init(mrow, r);
    int c_cur = it.next();
    int half = 0;
    int buf = 0;
    if (c_cur >= 0) at_issue_sub(lo, kh, vth, n, sk_n, c_cur, 0, lds, wave, lane);

    // Q^T operand: this lane's query, 8 k-steps of 8 channels
    bf16x8 qb[8];
    {
      int64_t qrow = (int64_t)r * AT_BS + q_off;
      if (qrow > n - 1) qrow = n - 1;
      const sp_bf16* src = q + (int64_t)h * sq_h + qrow * sq_n + 8 * g;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks)
        qb[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 16 * ks));
    }

    floatx16 o[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) o[dt] = (floatx16){0};
    float m_run = -INFINITY, l_run = 0.f;

    while (c_cur >= 0) {
      // this sub-tile has landed (own loads), and every wave is past the previous sub-tile's compute
      AT_WAIT_VMCNT0();
      __syncthreads();
      // ---- start fetching the next sub-tile into the other stage ----
      int c_next = c_cur, half_next = 1;
      if (half == 1) {
        c_next = it.next();
        half_next = 0;
      }
      if (c_next >= 0)
        at_issue_sub(lo, kh, vth, n, sk_n, c_next, half_next, lds + (buf ^ 1) * AT_STAGE_BYTES, wave, lane);

      const char* st = lds + buf * AT_STAGE_BYTES;
      // ---- S^T = K . Q^T for 64 keys; LDS operands are fetched two k-steps ahead of their MFMAs ----
      floatx16 s[2];
      s[0] = (floatx16){0};
      s[1] = (floatx16){0};
      {
        bf16x8 xa[3][2];
        xa[0][0] = at_lds128(st + koff[0]);
        xa[0][1] = at_lds128(st + koff[0] + 32 * 256);
        xa[1][0] = at_lds128(st + koff[1]);
        xa[1][1] = at_lds128(st + koff[1] + 32 * 256);
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          if (ks + 2 < 8) {
            xa[(ks + 2) % 3][0] = at_lds128(st + koff[ks + 2]);
            xa[(ks + 2) % 3][1] = at_lds128(st + koff[ks + 2] + 32 * 256);
          }
          s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[ks % 3][0], qb[ks], s[0], 0, 0, 0);
          s[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xa[ks % 3][1], qb[ks], s[1], 0, 0, 0);
        }
        __builtin_amdgcn_s_setprio(0);
      }
      // ---- online softmax (base 2): running max on raw logits, scale folded into the exponent ----
      if (c_cur == r) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key_off = half * AT_SUB + kt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
            s[kt][i] = (key_off <= q_off) ? s[kt][i] : -INFINITY;
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kt][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, SP_WAVE));
      const float m_new = fmaxf(m_run, mx * scale_log2);
      if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0ull) {  // some row's max moved: rescale
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
        m_run = m_new;
      }
      // a row with nothing unmasked so far keeps m_run = -inf; exp2(-inf - (-inf)) must not be evaluated
      const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          s[kt][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][i], scale_log2, -m_use));
      // ---- O^T += V^T . P^T; V^T operands fetched one (kt, dt) step ahead ----
      {
        bf16x8 pb[2][2];
        pb[0][0] = at_pack8(s[0], 0);
        pb[0][1] = at_pack8(s[0], 8);
        pb[1][0] = at_pack8(s[1], 0);
        pb[1][1] = at_pack8(s[1], 8);
        bf16x8 va[2][2];
        va[0][0] = at_lds128(st + voff[0]);
        va[0][1] = at_lds128(st + voff[1]);
        __builtin_amdgcn_s_setprio(1);
        // row sums of the bf16 probabilities on the matrix core: ones(32x16) . P^T puts sum_k P[k][q] of the
        // lane's query into every accumulator row (this replaces 32 dependent vector adds per sub-tile)
        floatx16 rs = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[0][0], (floatx16){0}, 0, 0, 0);
        rs = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[0][1], rs, 0, 0, 0);
#pragma unroll
        for (int step = 0; step < 8; ++step) {  // step = kt*4 + dt
          const int kt = step >> 2, dt = step & 3;
          if (step + 1 < 8) {
            const int kt1 = (step + 1) >> 2, dt1 = (step + 1) & 3;
            va[(step + 1) & 1][0] = at_lds128(st + voff[kt1 * 2 + 0] + dt1 * 32 * 128);
            va[(step + 1) & 1][1] = at_lds128(st + voff[kt1 * 2 + 1] + dt1 * 32 * 128);
          }
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[step & 1][0], pb[kt][0], o[dt], 0, 0, 0);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[step & 1][1], pb[kt][1], o[dt], 0, 0, 0);
          if (step == 3) {
            rs = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[1][0], rs, 0, 0, 0);
            rs = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pb[1][1], rs, 0, 0, 0);
          }
        }
        __builtin_amdgcn_s_setprio(0);
        l_run += rs[0];  // the MFMA contracts over both lane halves: all 64 keys of the sub-tile for this query
      }
      buf ^= 1;
      c_cur = c_next;
      half = half_next;
    }
    const float l_tot = l_run;

    // pivot heads: keep the softmax statistics of every query row for the block-average pass
    if (rowstat != nullptr && decision != nullptr && decision[h] == SP_DEC_DENSE && g == 0) {
      const int64_t qrow = (int64_t)r * AT_BS + q_off;
      if (qrow < n) rowstat[(int64_t)h * n + qrow] = make_float2(m_run, l_tot);
    }

    // ---- epilogue: normalise, transpose through LDS (padded rows), coalesced bf16 store ----
    __syncthreads();
    {
      const float inv_l = 1.0f / l_tot;
      sp_bf16* orow = reinterpret_cast<sp_bf16*>(lds) + q_off * AT_PITCH;
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
    for (int i8 = 0; i8 < 8; ++i8) {
      const int row = i8 * 16 + (t >> 4);
      const int64_t qrow = (int64_t)r * AT_BS + row;
      if (qrow < n) {
        *reinterpret_cast<uint4*>(out + (qrow * hq + h) * AT_D + (t & 15) * 8) =
            *reinterpret_cast<const uint4*>(reinterpret_cast<sp_bf16*>(lds) + row * AT_PITCH + (t & 15) * 8);
      }
    }
  }
}

__global__ void sp_zero_i32_kernel(int* p, int count) {
  for (int i = threadIdx.x; i < count; i += blockDim.x) p[i] = 0;
}

// ---- pivot heads: block-averaged attention map (shareprefill_attn.py:425-457) ---------------------------
// avg[h][r][c] = mean over the valid queries of block r of the softmax mass that falls into key block c,
// recomputed from the row statistics the forward kernel left behind.  One workgroup per (query block, head);
// heads that are not pivots leave at once.
__global__ __launch_bounds__(AT_THREADS) void sp_attn_avg_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const uint64_t* __restrict__ mask,
    const int32_t* __restrict__ decision, const float2* __restrict__ rowstat, float* __restrict__ avg_attn, int64_t n,
    int hq, int hkv, int64_t sq_n, int64_t sq_h, int64_t sk_n, int64_t sk_h, int nb, int nbw, float scale_log2) {
  __shared__ sp_bf16 Ks[AT_BS * AT_PITCH];
  __shared__ float wred[4];
  const int r = nb - 1 - blockIdx.x, h = blockIdx.y;
  if (decision[h] != SP_DEC_DENSE) return;
  const int kvh = h / (hq / hkv);
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int lq = lane & 31, g = lane >> 5;
  const int q_off = wave * 32 + lq;
  const int64_t rem = n - (int64_t)r * AT_BS;
  const int valid_q = rem < AT_BS ? (int)rem : AT_BS;
  const bool q_valid = q_off < valid_q;
  int64_t qrow = (int64_t)r * AT_BS + q_off;
  if (qrow > n - 1) qrow = n - 1;
  bf16x8 qb[8];
  {
    const sp_bf16* src = q + (int64_t)h * sq_h + qrow * sq_n + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qb[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 16 * ks));
  }
  const float2 st = rowstat[(int64_t)h * n + qrow];
  const float m_row = st.x, inv_l = 1.0f / st.y;
  const sp_bf16* kh = k + (int64_t)kvh * sk_h;
  float* arow_out = avg_attn + ((int64_t)h * nb + r) * nb;
  AtBlocks it;
  it.init(mask + ((int64_t)h * nb + r) * nbw, r);
  for (int c = it.next(); c >= 0; c = it.next()) {
    __syncthreads();
#pragma unroll
    for (int i8 = 0; i8 < 8; ++i8) {
      const int row = i8 * 16 + (t >> 4);
      int64_t key = (int64_t)c * AT_BS + row;
      if (key > n - 1) key = n - 1;
      *reinterpret_cast<uint4*>(&Ks[row * AT_PITCH + (t & 15) * 8]) =
          *reinterpret_cast<const uint4*>(kh + key * sk_n + (t & 15) * 8);
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
        part += ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(acc[i], scale_log2, -m_row)) * inv_l : 0.f;
      }
    }
    part = sp_wave_sum(part);
    if (lane == 0) wred[wave] = part;
    __syncthreads();
    if (t == 0) arow_out[c] = ((wred[0] + wred[1]) + (wred[2] + wred[3])) / (float)valid_q;
  }
}

// ---- host ---------------------------------------------------------------------------------------------
// workspace layout: [ repacked V^T : hkv*nb*128*128 bf16 | 8 queue tickets : 1 KiB | row statistics : hq*n float2 ]
static size_t at_vt_bytes(int64_t n, int32_t hkv, int32_t d, int32_t bs) {
  return (size_t)hkv * (size_t)sp_ceil_div(n, bs) * bs * d * sizeof(sp_bf16);
}

extern "C" size_t sp_attn_workspace_bytes(int64_t n, int32_t hq, int32_t hkv, int32_t d, int32_t bs) {
  if (n <= 0 || hq <= 0 || hkv <= 0 || d <= 0 || bs <= 0) return 0;
  return at_vt_bytes(n, hkv, d, bs) + 1024 + (size_t)hq * (size_t)n * sizeof(float2);
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
  SP_REQUIRE(workspace_bytes >= at_vt_bytes(n, hkv, d, bs), SP_ERR_WORKSPACE,
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
  SP_REQUIRE(softmax_scale > 0.f, SP_ERR_INVALID_ARGUMENT, "sp_block_sparse_attn_fwd_bf16: softmax_scale must be > 0");
  SP_REQUIRE(bs == AT_BS, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: block size %d unsupported (only 128)",
             bs);
  SP_REQUIRE(d == AT_D, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: head_dim %d unsupported (only 128)", d);
  SP_REQUIRE(q_stride_n % 8 == 0 && q_stride_h % 8 == 0 && k_stride_n % 8 == 0 && k_stride_h % 8 == 0 &&
                 ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)out % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: tensors must be 16-byte aligned, strides multiple of 8");
  SP_REQUIRE((int64_t)AT_BS * k_stride_n < (1ll << 31), SP_ERR_UNSUPPORTED,
             "sp_block_sparse_attn_fwd_bf16: key token stride %lld too large", (long long)k_stride_n);
  SP_REQUIRE(workspace_bytes >= sp_attn_workspace_bytes(n, hq, hkv, d, bs), SP_ERR_WORKSPACE,
             "sp_block_sparse_attn_fwd_bf16: workspace too small");
  const int64_t nb = sp_ceil_div(n, bs);
  SP_REQUIRE(nb * hq < (1ll << 31), SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: grid too large");
  if (!(flags & SP_ATTN_V_REPACKED)) {
    int rc = sp_attn_repack_v_bf16(v, n, hkv, d, v_stride_n, v_stride_h, bs, workspace, workspace_bytes, stream);
    if (rc != SP_OK) return rc;
  }
  const float scale_log2 = softmax_scale * 1.4426950408889634f;
  char* ws = (char*)workspace;
  int* counter = reinterpret_cast<int*>(ws + at_vt_bytes(n, hkv, d, bs));
  float2* rowstat = reinterpret_cast<float2*>(ws + at_vt_bytes(n, hkv, d, bs) + 1024);
  const bool want_avg = decision != nullptr && avg_attn != nullptr;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(sp_zero_i32_kernel, dim3(1), dim3(128), 0, s, counter, 8 * 16);
  SP_LAUNCH_CHECK();
  const size_t lds_bytes = 2 * AT_STAGE_BYTES;
  static int n_cu = 0;
  if (n_cu == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    SP_HIP(hipGetDevice(&dev));
    SP_HIP(hipGetDeviceProperties(&prop, dev));
    SP_HIP(hipFuncSetAttribute((const void*)sp_attn_fwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds_bytes));
    n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  const int64_t total = nb * hq;
  const int grid = (int)(total < 2ll * n_cu ? ((total + 7) / 8) * 8 : 2ll * n_cu);
  hipLaunchKernelGGL(sp_attn_fwd_kernel, dim3(grid), dim3(AT_THREADS), lds_bytes, s, (const sp_bf16*)q,
                     (const sp_bf16*)k, (const sp_bf16*)workspace, mask, decision, (sp_bf16*)out,
                     want_avg ? rowstat : (float2*)nullptr, n, hq, hkv, q_stride_n, q_stride_h, k_stride_n,
                     k_stride_h, (int)nb, (int)((nb + 63) / 64), scale_log2, counter);
  SP_LAUNCH_CHECK();
  if (want_avg) {
    hipLaunchKernelGGL(sp_attn_avg_kernel, dim3((unsigned)nb, hq), dim3(AT_THREADS), 0, s, (const sp_bf16*)q,
                       (const sp_bf16*)k, mask, decision, rowstat, avg_attn, n, hq, hkv, q_stride_n, q_stride_h,
                       k_stride_n, k_stride_h, (int)nb, (int)((nb + 63) / 64), scale_log2);
    SP_LAUNCH_CHECK();
  }
  return SP_OK;
}

// GQA causal block-sparse flash attention for gfx950 (bf16 MFMA, fp32 online softmax in base 2).
// Replaces block_wise_prefill_attention_kernel / triton_block_wise_prefill_attention and the CSR
// builder count_kernel (shareprefill/attn/shareprefill_attn.py:187-620): the kernel walks the set
// bits of the row's mask words instead of a sorted id list with row pointers.
//
// Layout of the computation (one workgroup = a pair of 128-query blocks of one head, 8 waves x 32 queries; a wave
// works on its 32 queries as two 16-query tiles with 16x16x32 MFMAs):
//   S^T = K . Q^T   : A operand = K tile rows from LDS, B operand = Q held in registers for the whole
//                     row.  In a 16x16 accumulator a lane owns ONE query (lane % 16) and 4 of the tile's 16
//                     keys, so the row max / row sum are in-lane reductions plus exchanges with lanes ^ 16, ^ 32.
//   O^T += V^T . P^T: the P^T operand is the S^T accumulators converted to bf16 in place (no LDS round
//                     trip); the V^T operand comes from a key-major repack of V made once per call, whose
//                     key order inside every group of 32 keys matches the accumulators' row order.
// K and V^T sub-tiles (64 keys) are staged through LDS by direct global->LDS loads, XOR-swizzled; every wave runs a
// software pipeline over 32-key half-tiles in which the softmax of one half-tile is issued between the MFMAs of
// its neighbours (see "the software pipeline of one wave" below).
#include "sp_common.h"

#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define AT_BS 128
#define AT_D 128
#define AT_PITCH 136  // bf16 elements per LDS row
#define AT_THREADS 256

// position p (0..31) inside a group of 32 keys of the repacked V^T row holds key offset at_perm32(p):
// [0-3, 16-19, 4-7, 20-23, 8-11, 24-27, 12-15, 28-31]: lane group g of a wave owns rows 4g .. 4g+3 of both 16x16
// S^T accumulators of a half-tile, and its P^T operand is key slots 8g .. 8g+7
__host__ __device__ static inline int at_perm32(int p) { return 16 * ((p >> 2) & 1) + 4 * (p >> 3) + (p & 3); }

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
      const int key = (slot & ~31) + at_perm32(slot & 31);
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
// The kernel is persistent, one workgroup of 8 waves per CU.  A work item is a PAIR of query blocks that read the
// same K / V: waves 0-3 own one, waves 4-7 the other, and both consume the same K / V^T tiles from LDS (the union
// of the two rows' masks), which halves the L2->LDS traffic wherever the two keep the same columns -- and wherever
// they do not, the row that does not keep a column idles while the other computes.  Two pairings exist, chosen per
// two adjacent heads (2i, 2i+1) of a kv group by sp_attn_pairing_kernel, whichever gives the smaller unions:
//   rows  : item (h, p) = rows 2p and 2p+1 of head h (verticals are shared, slashes shift by one block);
//   heads : item (h, p) = row 2p + (h & 1) of heads 2i and 2i+1 (heads that share a pattern keep the same columns).
// Items are grouped in gangs of AT_GANG consecutive pairs of ONE head (all of a head's pairs when it has fewer: a short
// prompt's queues then hold no padding tickets, each of which would cost a workgroup an atomic and two barriers).  Gangs are dealt statically to the 8 XCDs (queue x = gang position % 8; workgroup b serves queue b % 8
// first -- workgroups are placed on XCDs round-robin), so the 32 workgroups of an XCD start a gang together at
// column 0 and sweep the key blocks nearly in lock-step: every K / V^T tile one of them pulls into the XCD's
// L2 is hit by the others.  The head order inside a kv group is rotated from chunk to chunk so that every
// queue sees every head, heavy (late) rows go first, and a workgroup whose queue is empty steals from the
// other queues.  Pulling is by atomic tickets only: nobody ever waits for anybody, and every workgroup leaves
// once all eight queues are exhausted.
// Up to 32K tokens a launch has few gangs per workgroup, the heaviest of them a large part of a workgroup's whole
// share, and every head's K / V^T fit the memory-side cache together, so the order above (one kv head after the
// other) only makes the last kv head's heavy rows start late: there sp_attn_order_kernel ranks the gangs by the
// number of blocks their items visit and the queues are dealt from that ranking, heaviest first.
#define AT_GANG 32
// The 1 KiB scheduler area (int indices): 0..127 eight queue tickets (one per 64 bytes), 128..191 the pivot slot of
// every head (one byte each, AT_NO_SLOT = its block sums are not kept), 192..195 {shader cycles, 100 MHz ticks} of
// workgroup 0, 196 the number of pivot slots in use, 200..231 the pairing of every two adjacent heads (one byte each,
// see sp_attn_pairing_kernel), 232..239 the queue tickets of the pivot heads' launch (so that both launches of a call
// find their tickets cleared by sp_attn_prep_kernel and nothing has to be cleared in between).
#define AT_SLOT_TABLE 128
#define AT_CLOCK_SLOT 192
#define AT_NPIV_SLOT 196
#define AT_ORDER_SLOT 197  // 1: the gang positions of this call go through the order table (sp_attn_order_kernel)
#define AT_PAIR_TABLE 200
#define AT_PIVOT_TICKETS 232  // 232..239: the eight queue tickets of the pivot heads' own launch
#define AT_NO_SLOT 255
// Behind the 1 KiB of slots: the order table, AT_ORDER_MAX gang positions (uint16), see sp_attn_order_kernel.
#define AT_ORDER_MAX 1024
#define AT_SCHED_BYTES (1024 + AT_ORDER_MAX * 2)
#define AT_MAX_HEADS 256
#define AT_FWD_THREADS 512

struct AtGeom {
  int group, n_pairs, gang, n_chunks, n_gangs;
  const uint16_t* order;  // gang position -> gang (nullptr: identity)
};

__device__ static inline int at_queue_items(const AtGeom& gm, int xq) {
  const int gangs = gm.n_gangs > xq ? (gm.n_gangs - xq + 7) / 8 : 0;
  return gangs * gm.gang;
}

// gang position (before any reordering) -> head and chunk of row pairs, 0 = the last (heaviest) rows
__device__ static inline void at_gang_of(const AtGeom& gm, int pos, int& h, int& j) {
  const int i = pos % gm.group;
  const int rest = pos / gm.group;
  j = rest % gm.n_chunks;
  const int kvh = rest / gm.n_chunks;
  h = kvh * gm.group + (i + j) % gm.group;
}

// ticket of queue xq -> (head, row pair); false for the padding slots of the last chunk
__device__ static inline bool at_item(const AtGeom& gm, int xq, int ticket, int& h, int& pair) {
  int pos = (ticket / gm.gang) * 8 + xq;  // gang position
  const int slot = ticket % gm.gang;
  if (gm.order != nullptr) pos = gm.order[pos];
  int j;
  at_gang_of(gm, pos, h, j);
  pair = gm.n_pairs - 1 - (j * gm.gang + slot);
  return pair >= 0;
}

__device__ static inline void at_geometry(AtGeom& gm, int hq, int hkv, int nb) {
  gm.group = hq / hkv;
  gm.n_pairs = (nb + 1) / 2;
  gm.gang = gm.n_pairs < AT_GANG ? gm.n_pairs : AT_GANG;
  gm.n_chunks = (gm.n_pairs + gm.gang - 1) / gm.gang;
  gm.n_gangs = hq * gm.n_chunks;
  gm.order = nullptr;
}

// ---- LDS staging -------------------------------------------------------------------------------------------
// A block is processed as two sub-tiles of 64 keys.  LDS holds a ring of four K sub-tile buffers
// [64 keys][16 chunks] and a ring of four V^T sub-tile buffers [128 channels][8 chunks] (chunk = 16 bytes =
// 8 bf16), 16 KiB each.  While sub-tile u is computed on (K of u, V^T of u-1: the P.V product trails by one
// sub-tile), K of u+1..u+3 and V^T of u..u+2 are in flight.  Tiles are filled by direct global->LDS 128-bit
// loads: lane i of a wave writes LDS chunk (base + i), fetching whichever global chunk belongs there.  Instead
// of row padding the chunk index is XOR-swizzled with the row,
//   K  : chunk c of row r sits at r*16 + (c ^ (r & 15))
//   V^T: chunk c of row r sits at r*8  + (c ^ ((r >> 1) & 7))
// so the 16 lanes that read the same logical chunk of 16 consecutive rows hit 16 different bank groups.
#define AT_SUB 64
#define AT_RING 4
#define AT_KBUF_BYTES (AT_SUB * AT_D * 2)  // 16 KiB
#define AT_VBUF_BYTES (AT_D * AT_SUB * 2)  // 16 KiB
#define AT_LIST_MAX 4096                      // union blocks of a row pair (nb <= 4096)
#define AT_LIST_BYTES (AT_LIST_MAX * 4)
#define AT_LDS_BYTES (AT_RING * (AT_KBUF_BYTES + AT_VBUF_BYTES) + AT_LIST_BYTES)

typedef __attribute__((address_space(3))) void* at_lds_ptr;
typedef const __attribute__((address_space(1))) void* at_gbl_ptr;

// Lane-constant byte offsets of the first K and V^T chunk a lane fetches per sub-tile.  A wave-instruction fills
// one 1 KiB segment (seg = it*8 + wave, wave = 0..7): 4 K rows or 8 V^T rows.  Row and swizzle of a lane do not
// depend on `it` beyond a uniform step (32 K rows / 64 V^T rows), which goes into the scalar base address.
struct AtLoadOffsets {
  uint32_t k, v;
};

__device__ static inline void at_load_offsets(AtLoadOffsets& lo, int64_t sk_n, int wave, int lane) {
  const int krow = wave * 4 + (lane >> 4);
  lo.k = (uint32_t)(krow * (int)sk_n + (((lane & 15) ^ (krow & 15)) * 8)) * 2u;
  const int vrow = wave * 8 + (lane >> 3);
  lo.v = (uint32_t)(vrow * AT_BS + (((lane & 7) ^ ((vrow >> 1) & 7)) * 8)) * 2u;
}

// two wave-instructions per wave and sub-tile; kbase = address of the sub-tile's first key row
__device__ static inline void at_issue_k(const AtLoadOffsets& lo, const char* kbase, int64_t sk_n, char* kbuf,
                                         int wave) {
#pragma unroll
  for (int it = 0; it < 2; ++it)
    __builtin_amdgcn_global_load_lds((at_gbl_ptr)(kbase + (int64_t)it * 64 * sk_n + lo.k),
                                     (at_lds_ptr)(kbuf + (it * 8 + wave) * 1024), 16, 0, 0);
}

// ragged tail of the sequence (last block only): rows beyond the last key are clamped onto it
__device__ static inline void at_issue_k_tail(const sp_bf16* __restrict__ kh, int64_t n, int64_t sk_n, int64_t key0,
                                              char* kbuf, int wave, int t) {
  const int64_t lim64 = n - 1 - key0;
  const int lim = lim64 < 0 ? 0 : (int)lim64;
  const sp_bf16* kbase = kh + (lim64 < 0 ? (n - 1) : key0) * sk_n;
  int lane = t & 63;
  asm volatile("" : "+v"(lane));  // keeps this rare path's lane arithmetic from being hoisted out of the key loop
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int seg = it * 8 + wave;
    const int row = seg * 4 + (lane >> 4);
    const int cl = (lane & 15) ^ (row & 15);
    const int rowc = row < lim ? row : lim;
    const sp_bf16* g = kbase + (uint32_t)(rowc * (int)sk_n + cl * 8);
    __builtin_amdgcn_global_load_lds((at_gbl_ptr)g, (at_lds_ptr)(kbuf + seg * 1024), 16, 0, 0);
  }
}

// the repacked V^T is zero-filled beyond the last key, so no tail case; vbase = first channel row of the sub-tile
__device__ static inline void at_issue_v(const AtLoadOffsets& lo, const char* vbase, char* vbuf, int wave) {
#pragma unroll
  for (int it = 0; it < 2; ++it)
    __builtin_amdgcn_global_load_lds((at_gbl_ptr)(vbase + it * 64 * AT_BS * 2 + lo.v),
                                     (at_lds_ptr)(vbuf + (it * 8 + wave) * 1024), 16, 0, 0);
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

// causally trimmed 64-column word wi of the mask row of query block r
__device__ static inline uint64_t at_trim(uint64_t x, int wi, int r) {
  if (wi > (r >> 6)) return 0ull;
  if (wi == (r >> 6) && (r & 63) != 63) x &= (2ull << (r & 63)) - 1ull;
  return x;
}

// entry of the per-pair block list: column | row-membership flags
#define AT_IN_A (1u << 30)
#define AT_IN_B (1u << 31)
#define AT_COL_MASK 0x00FFFFFFu

#define AT_WAIT_VMCNT0() __builtin_amdgcn_s_waitcnt(0x0F70)  // vmcnt(0) only: the direct-to-LDS loads have landed
#define AT_PIN() __builtin_amdgcn_sched_barrier(0)            // nothing is scheduled across this point
// lane-derived values from an opaque copy of the thread index (not loop invariant as far as the compiler knows)
#define AT_LANE_VIEW(tv)                         \
  int tv##_o = (tv);                             \
  asm volatile("" : "+v"(tv##_o));               \
  const int lq = tv##_o & 15, g = (tv##_o >> 4) & 3; \
  const int q_off = (tv##_o >> 6) * 32 + lq /* the first of the lane's two queries; the second is 16 further */

// ---- the software pipeline of one wave ------------------------------------------------------------------------
// A wave owns 32 queries as two 16-query tiles (qt = 0, 1) and works with v_mfma_f32_16x16x32_bf16: A 16x32, B 32x16,
// C/D 16x16 (lane l: column l%16, rows 4*(l/16) .. +3).  Against the 32x32x16 form the same flops read and rewrite
// only half as many accumulator registers (K = 32 per instruction), which is what the power-limited chip rewards.
//   S^T[16 keys x 16 q] = K frag[16 keys x 32 ch] . Q^T frag[32 ch x 16 q]      4 channel steps per tile
//   O^T[16 ch x 16 q]  += V^T frag[16 ch x 32 key slots] . P^T[32 key slots x 16 q]
// Every LDS operand (a K or V^T fragment, 1 KiB) feeds the two query tiles.  A lane holds, per query tile, the
// logits of keys 4g .. 4g+3 of both 16-key tiles of a half-tile (g = l/16): exactly the eight key slots 8g .. 8g+7
// of the P^T operand once the V^T repack orders the keys that way (at_perm32), so P is the S accumulator converted
// to bf16 in place.
// Keys are consumed in half-tiles of 32.  For half-tile j the wave issues, in ONE instruction stream,
//     S(j+1) = K(j+1) . Q^T        16 MFMAs  (matrix core)
//     O     += V^T(j-1) . P(j-1)   16 MFMAs  (matrix core), + 2 for the row sums  ones . P(j-1)
//     P(j)   = exp2(S(j)*scale - m), bf16 packing               ~45 vector instructions
// interleaved one LDS operand read : two MFMAs : two or three vector instructions.  A wave issues in order but
// an MFMA executes for 16 cycles after it is issued, so the vector work of half-tile j runs in the shadow of the
// matrix work of its neighbours; scheduling barriers pin that order.  The running max m is lazy (see at_commit):
// it moves only when some probability came out at 2 or more, and then O and the row sums are rescaled and that
// half-tile's probabilities are formed again before they are used.
typedef uint32_t at_u32x4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t at_pack2(float a, float b) {
  floatx2 f;
  f[0] = a;
  f[1] = b;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// compile-time loop: f(std::integral_constant<int, K>) for K = 0 .. N-1
template <int K, int N, typename F>
__device__ __forceinline__ void at_static_for(F&& f) {
  if constexpr (K < N) {
    f(std::integral_constant<int, K>{});
    at_static_for<K + 1, N>(f);
  }
}

// LDS operand fetch the compiler does not track: it returns at once and the register is valid only after an
// explicit AT_WAIT_LGKM(n) (n = younger fetches allowed to be still in flight; LDS reads return in order).
// Reason: while direct-to-LDS tile loads are in flight the compiler waits for ALL outstanding LDS reads before
// every use of any of them, which exposes the full LDS latency in front of each MFMA.
template <int IMM>
__device__ __forceinline__ bf16x8 at_lds128_async(uint32_t addr) {
  at_u32x4 r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(IMM));
  return __builtin_bit_cast(bf16x8, r);
}
#define AT_WAIT_LGKM(n) __builtin_amdgcn_s_waitcnt(0xC07F | ((n) << 8))

__device__ __forceinline__ uint32_t at_lds_addr(const char* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)p;
}

// The MFMAs of the pipeline are written as inline assembly that accumulates IN PLACE.  Through the builtin the
// register allocator is free to give an MFMA's result other registers than its accumulator operand, and it does so
// for this kernel: the accumulators then change registers from step to step and every step ends in ~80 register
// copies where the rare rescale branch joins the main path.  The compiler does not know the result latency of
// these instructions: a vector instruction that reads an MFMA result sits at least three operand slots behind it
// by construction, and where that is not so (at_settle_*) explicit wait states are inserted.
__device__ __forceinline__ void at_mfma_first(floatx4& d, bf16x8 a, bf16x8 b) {  // d = a . b
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
}
__device__ __forceinline__ void at_mfma_acc(floatx4& d, bf16x8 a, bf16x8 b) {  // d += a . b
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
}
// ... and the same with the wait states that let vector instructions read the results of this and every earlier MFMA
// INSIDE the statement.  A separate settling statement tied to the result registers is not enough where the reader
// follows closely: to satisfy the tie the register allocator may first copy a result into other registers -- with a
// vector move that reads the result while the MFMA is still in flight -- and put the wait states behind that copy
// (seen in the generated code of the pivot instantiation: a copy of the row sums five wait states behind their MFMA).
__device__ __forceinline__ void at_mfma_acc_settled(floatx4& d, bf16x8 a, bf16x8 b) {  // d += a . b, then 16 wait states
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\ts_nop 15" : "+v"(d) : "v"(a), "v"(b));
}
__device__ __forceinline__ void at_settle_o(floatx4 (&o)[9][2]) {
  asm volatile("s_nop 15"
               : "+v"(o[0][0]), "+v"(o[0][1]), "+v"(o[1][0]), "+v"(o[1][1]), "+v"(o[2][0]), "+v"(o[2][1]),
                 "+v"(o[3][0]), "+v"(o[3][1]), "+v"(o[4][0]), "+v"(o[4][1]), "+v"(o[5][0]), "+v"(o[5][1]),
                 "+v"(o[6][0]), "+v"(o[6][1]), "+v"(o[7][0]), "+v"(o[7][1]), "+v"(o[8][0]), "+v"(o[8][1]));
}

// LDS addresses of a block's operands, one XOR each, made once per block: K channel step ks of sub-tile 2b at
// ka[ks] (key tile, second half of the sub-tile and sub-tile 2b+1 via immediate offsets), V^T key-slot half h of
// sub-tile 2b-1 at va[0][h] and of sub-tile 2b at va[1][h] (channel tile via immediate offsets).
struct AtAddr {
  uint32_t ka[4];
  uint32_t va[2][2];
};

__device__ __forceinline__ void at_block_addr(AtAddr& ad, const char* kb, const char* vb, const char* vb1, int koff,
                                              int voff) {
  const uint32_t k0 = at_lds_addr(kb) + (uint32_t)koff;  // buffers are 256-byte aligned: the XOR stays inside
  const uint32_t v0 = at_lds_addr(vb) + (uint32_t)voff, v1 = at_lds_addr(vb1) + (uint32_t)voff;
#pragma unroll
  for (int i = 0; i < 4; ++i) ad.ka[i] = k0 ^ (uint32_t)(i << 6);
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
    ad.va[0][hh] = v0 ^ (uint32_t)(hh << 6);
    ad.va[1][hh] = v1 ^ (uint32_t)(hh << 6);
  }
}

// max(a, b, c) / max(a, b) as single instructions: through fmaxf the compiler first quiets every operand it cannot
// prove to be no signalling NaN (v_max x, x), which the MFMA results behind inline assembly all are to it
__device__ __forceinline__ float at_max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float at_max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// the lane's 16 logits of a half-tile in softmax order: query tile idx / 8, then key slots 8g .. 8g+7 of the lane
// (key tile (idx / 4) % 2, row idx % 4); s is indexed [key tile][query tile]
#define AT_SVAL(s, idx) (s)[((idx) >> 2) & 1][(idx) >> 3][(idx) & 3]

// KQ: which 32-key quarter (0..3) of the block's two K buffers S_out is computed from; VB / KT: which V^T buffer
// (0: sub-tile 2b-1, 1: sub-tile 2b) and which half of it P_prev belongs to.
// Slot order: the 8 operand slots of S_out first (channel step outermost, so that the four accumulators take turns),
// then the 8 of O (one channel tile each) and the two row-sum MFMAs; det receives the OR of P_out's packed words.
// The first two operands of a stage that starts with the S product of 32-key quarter KQ, fetched ahead of the stage
// (at the end of the one before it, or right behind the block's barrier): the stage then does not open with an LDS
// round trip in which, the other wave of the SIMD being at the same point, nobody issues anything.
template <int KQ>
__device__ __forceinline__ void at_prefetch_qk(const AtAddr& ad, bf16x8 (&pre)[2]) {
  pre[0] = at_lds128_async<(KQ >> 1) * AT_KBUF_BYTES + ((KQ & 1) * 32) * 256>(ad.ka[0]);
  pre[1] = at_lds128_async<(KQ >> 1) * AT_KBUF_BYTES + ((KQ & 1) * 32 + 16) * 256>(ad.ka[0]);
}

// PRE: operands 0 and 1 of the stage are already in flight in `pre` (at_prefetch_qk<KQ>, and nothing else has been
// read from LDS since).  NEXT >= 0: the stage ends by fetching the first two operands of the next one, quarter NEXT.
// HALF: q, k and v are zero beyond channel 64 (a head_dim of at most 64 padded to the tiles' 128): the S product takes the
// first two of its four channel steps and O the first four of its eight channel tiles -- half the operand slots.
// SETTLE: the stage's last MFMA carries the wait states after which vector instructions may read every MFMA result
// (a run's first stage, whose S the next stage's softmax reads at once; a pivot head's stage in front of the block sums).
template <bool DO_QK, bool DO_PV, int KQ, int VB, int KT, bool PRE, int NEXT, bool HALF, bool SETTLE>
__device__ __forceinline__ void at_fused(const AtAddr& ad, const bf16x8 (&qb)[2][4], floatx4 (&s_out)[2][2],
                                         const floatx4 (&s_in)[2][2], const bf16x8 (&p_prev)[2], bf16x8 (&p_out)[2],
                                         floatx4 (&o)[9][2], float sc, const float (&neg_m)[2], uint32_t (&det)[2],
                                         const bf16x8& ones, bf16x8 (&pre)[2]) {
  static_assert(!PRE || DO_QK, "only stages that start with the S product take prefetched operands");
  constexpr int QS = DO_QK ? (HALF ? 4 : 8) : 0;  // operand slots of the S product: (channel step, key tile) pairs
  constexpr int PS = DO_PV ? (HALF ? 4 : 8) : 0;  // operand slots of the P.V product: channel tiles
  constexpr int NP = QS + PS;                     // each slot holds one MFMA per query tile
  static_assert(NP == 4 || NP == 8 || NP == 16, "a fused stage has 4, 8 or 16 operand slots");
  constexpr int EPS = 16 / NP;  // softmax elements handled per operand slot
  constexpr int AHEAD = 2;      // LDS operands are fetched this many slots before their MFMAs
  bf16x8 opnd[NP];
  float x[16], e[16];
  uint32_t pk[8];
  auto fetch = [&](auto kc) {
    constexpr int k = decltype(kc)::value;
    constexpr bool qk = k < QS;
    constexpr int i = qk ? k : k - QS;
    if constexpr (qk)  // slot i: channel step i / 2, key tile i % 2
      opnd[k] = at_lds128_async<(KQ >> 1) * AT_KBUF_BYTES + ((KQ & 1) * 32 + (i & 1) * 16) * 256>(ad.ka[i >> 1]);
    else  // slot i: channel tile i
      opnd[k] = at_lds128_async<i * 16 * 128>(ad.va[VB][KT]);
  };
  static_assert(AHEAD == 2, "the prefetched pair is the stage's look-ahead");
  if constexpr (PRE) {
    opnd[0] = pre[0];
    opnd[1] = pre[1];
  } else {
    at_static_for<0, AHEAD>(fetch);
  }
  AT_PIN();
  at_static_for<0, NP>([&](auto kc) {
    constexpr int k = decltype(kc)::value;
    constexpr bool qk = k < QS;
    constexpr int i = qk ? k : k - QS;
    constexpr int in_flight_after = (NP - 1 - k) < (AHEAD - 1) ? (NP - 1 - k) : (AHEAD - 1);
    AT_WAIT_LGKM(in_flight_after);  // operand k has landed
    AT_PIN();
    auto mfma = [&](auto qc, auto lastc) {
      constexpr int qt = decltype(qc)::value;
      constexpr bool settle = decltype(lastc)::value;  // the stage's last MFMA, and results are read right behind it
      if constexpr (qk) {
        if constexpr ((i >> 1) == 0)
          at_mfma_first(s_out[i & 1][qt], opnd[k], qb[qt][0]);
        else if constexpr (settle)
          at_mfma_acc_settled(s_out[i & 1][qt], opnd[k], qb[qt][i >> 1]);
        else
          at_mfma_acc(s_out[i & 1][qt], opnd[k], qb[qt][i >> 1]);
      } else {
        at_mfma_acc(o[i][qt], opnd[k], p_prev[qt]);
      }
    };
    // the two query tiles take turns at going first: across a slot boundary the B operand (Q or P of one query tile)
    // stays the same for two MFMAs in a row, as the A operand does inside a slot (+0.5 % under the power cap)
    mfma(std::integral_constant<int, (k & 1)>{}, std::false_type{});
    if constexpr (k + AHEAD < NP) fetch(std::integral_constant<int, k + AHEAD>{});
#pragma unroll
    for (int u = 0; u < EPS; ++u) {
      const int idx = k * EPS + u;
      // The softmax arithmetic depends only on values known before the stage starts, and the optimiser would
      // otherwise move all of it in front of the stage (out of the MFMAs' shadow): the empty asm ties each
      // element to its slot.
      // (the tie goes through a scalar copy of the scale: S(j) itself must stay where it is, the next step may
      // need it again)
      float sc_here = sc;
      asm volatile("" : "+s"(sc_here));
      x[idx] = __builtin_fmaf(AT_SVAL(s_in, idx), sc_here, neg_m[idx >> 3]);
      if (idx >= 1) e[idx - 1] = __builtin_amdgcn_exp2f(x[idx - 1]);
      if (idx >= 3 && ((idx - 3) & 1) == 0) {
        const int m = (idx - 3) >> 1;
        pk[m] = at_pack2(e[idx - 3], e[idx - 2]);
        // OR of the packed probabilities: any exponent >= 128 (P >= 2, inf, NaN) shows in bit 14 or 30
        // (three words at a time: one three-input instruction)
        if ((m & 3) == 2) det[m >> 2] = pk[m - 2] | pk[m - 1] | pk[m];
        if ((m & 3) == 3) det[m >> 2] |= pk[m];
      }
      // ... and the results to the slot they were produced in (instruction selection lets pure arithmetic float)
      asm volatile("" : "+v"(x[idx]));
      if (idx >= 1) asm volatile("" : "+v"(e[idx - 1]));
      if (idx >= 3 && ((idx - 3) & 1) == 0) {
        if ((((idx - 3) >> 1) & 3) >= 2)
          asm volatile("" : "+v"(pk[(idx - 3) >> 1]), "+v"(det[(idx - 3) >> 3]));
        else
          asm volatile("" : "+v"(pk[(idx - 3) >> 1]));
      }
    }
    AT_PIN();
    mfma(std::integral_constant<int, 1 - (k & 1)>{}, std::integral_constant<bool, SETTLE && !DO_PV && k == NP - 1>{});
    if constexpr (DO_PV && k == NP - 1) {  // row sums of P(j-1) as rounded for the P.V product: ones . P
      at_mfma_acc(o[8][0], ones, p_prev[0]);
      if constexpr (SETTLE)
        at_mfma_acc_settled(o[8][1], ones, p_prev[1]);
      else
        at_mfma_acc(o[8][1], ones, p_prev[1]);
    }
    AT_PIN();
  });
  if constexpr (NEXT >= 0) {
    at_prefetch_qk<NEXT>(ad, pre);
    AT_PIN();
  }
  e[15] = __builtin_amdgcn_exp2f(x[15]);
  pk[7] = at_pack2(e[14], e[15]);
  det[1] |= pk[7];
  static_assert(!(DO_QK && !DO_PV) || SETTLE, "a run's first stage: the next stage's softmax reads S_out at once");
  at_u32x4 w0, w1;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    w0[j] = pk[j];
    w1[j] = pk[4 + j];
  }
  p_out[0] = __builtin_bit_cast(bf16x8, w0);
  p_out[1] = __builtin_bit_cast(bf16x8, w1);
}

// MFMA-only stages (no vector work to hide): first S of a run, last P.V of a run
template <int KH, bool HALF>
__device__ __forceinline__ void at_qk_only(const char* kb, int koff, const bf16x8 (&qb)[2][4], floatx4 (&s_out)[2][2]) {
  constexpr int QS = HALF ? 4 : 8;
  bf16x8 a[8];  // slot i: channel step i / 2, key tile i % 2
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = at_lds128(kb + (koff ^ ((i >> 1) << 6)) + (KH * 32 + (i & 1) * 16) * 256);
  AT_PIN();
#pragma unroll
  for (int i = 0; i < QS; ++i) {
    if (i + 4 < QS) a[i + 4] = at_lds128(kb + (koff ^ (((i + 4) >> 1) << 6)) + (KH * 32 + (i & 1) * 16) * 256);
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      if ((i >> 1) == 0)
        at_mfma_first(s_out[i & 1][qt], a[i], qb[qt][0]);
      else if (i == QS - 1 && qt == 1)  // the last one: the softmax of the next stage reads S_out right away
        at_mfma_acc_settled(s_out[i & 1][qt], a[i], qb[qt][i >> 1]);
      else
        at_mfma_acc(s_out[i & 1][qt], a[i], qb[qt][i >> 1]);
    }
    AT_PIN();
  }
}

template <int KT, bool HALF>
__device__ __forceinline__ void at_pv_only(const char* vb, int voff, const bf16x8 (&p)[2], floatx4 (&o)[9][2],
                                           const bf16x8& ones) {
  constexpr int PS = HALF ? 4 : 8;
  bf16x8 a[8];  // slot i: channel tile i
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = at_lds128(vb + (voff ^ (KT << 6)) + i * 16 * 128);
  AT_PIN();
#pragma unroll
  for (int i = 0; i < PS; ++i) {
    if (i + 4 < PS) a[i + 4] = at_lds128(vb + (voff ^ (KT << 6)) + (i + 4) * 16 * 128);
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) at_mfma_acc(o[i][qt], a[i], p[qt]);
    AT_PIN();
  }
  at_mfma_acc(o[8][0], ones, p[0]);
  at_mfma_acc_settled(o[8][1], ones, p[1]);  // the end of a run: the block sums and the epilogue read O next
}

// causal predicate inside the diagonal block; key_base = offset of the half-tile's first key inside the block
__device__ __forceinline__ void at_causal(floatx4 (&s)[2][2], int key_base, int t) {
  AT_LANE_VIEW(t);
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key_off = key_base + kt * 16 + 4 * g + j;
        s[kt][qt][j] = (key_off <= q_off + qt * 16) ? s[kt][qt][j] : -INFINITY;
      }
}

// Block sizes below 128: the 16 x 16 sub-tiles of a half-tile whose fine block the mask does not keep are taken out
// like the keys the causal predicate hides.  kq: bit 8 * qt + c16 = keep the fine block that holds keys 16 c16 .. 16 c16
// + 15 of the 128-key block for the queries of tile qt (wave-uniform).
__device__ __forceinline__ void at_keep(floatx4 (&s)[2][2], uint32_t kq, int key_base) {
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
      if (((kq >> (8 * qt + (key_base >> 4) + kt)) & 1u) == 0u)
        s[kt][qt] = (floatx4){-INFINITY, -INFINITY, -INFINITY, -INFINITY};
}

// max over the lane's 8 keys of each query tile
__device__ __forceinline__ void at_lanemax(const floatx4 (&s)[2][2], float (&mx)[2]) {
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    float m = at_max3(s[0][qt][0], s[0][qt][1], s[0][qt][2]);
    m = at_max3(m, s[0][qt][3], s[1][qt][0]);
    m = at_max3(m, s[1][qt][1], s[1][qt][2]);
    mx[qt] = at_max2(m, s[1][qt][3]);
  }
}

// ... and over the three partner lanes (lane ^ 16, ^ 32, ^ 48) that hold the other 24 keys of the query
__device__ __forceinline__ float at_groupmax(float mx) {
  uint32_t u = __builtin_bit_cast(uint32_t, mx);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);  // (own, lane ^ 16) in some order
  const float m1 = at_max2(__builtin_bit_cast(float, (uint32_t)a[0]), __builtin_bit_cast(float, (uint32_t)a[1]));
  u = __builtin_bit_cast(uint32_t, m1);
  const auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // (own, lane ^ 32) in some order
  return at_max2(__builtin_bit_cast(float, (uint32_t)b[0]), __builtin_bit_cast(float, (uint32_t)b[1]));
}

// ---- the running max of a query is lazy, its row sum comes off the matrix core ----
// Probabilities are formed against the max as it stood, m_run, which is only ever a lower bound of the true running
// max: they can exceed 1, which costs nothing as long as they stay far from the range limit.  The row sums are taken
// from the probabilities as rounded to bf16 for P.V -- two more MFMAs per step against an all-ones operand,
// accumulated in o[8] -- so numerator and denominator of the softmax see the same values and the result does not
// depend on the largest probability being exactly 1.  No maximum per half-tile: the packed probabilities are OR-ed
// (three instructions per step) and one test of the top exponent bit per step says whether some P(j-1) >= 2, is inf
// or NaN (the first keys of a row, m_run = AT_NO_MAX; a logit more than one octave above the max).  Only then is the
// max taken from S(j-1) -- still intact in the registers the next stage overwrites -- O and the sums are rescaled and
// P(j-1) is formed again; P(j-1) enters O only after this test.
#define AT_NO_MAX (-1.0e30f)          // "no key seen yet": finite, so exp2(S * scale - m) is +inf or 0, never NaN
#define AT_P_TOO_LARGE 0x40004000u    // bf16 pair: exponent >= 128 in either half

// s_prev = S(j-1) (causal predicate applied), p = P(j-1), det = OR of its packed words.  On return p is safe to use.
// PIVOT: l_mark (the row sums at the start of the current key block, see the block sums of pivot heads in the
// kernel) follows every rescale.
// MODE: bit 0 = PIVOT, bit 1 = HALF (see at_fused), bit 2 = FINE (see at_keep)
template <int MODE>
__device__ __forceinline__ void at_commit(const floatx4 (&s_prev)[2][2], bf16x8 (&p)[2], uint32_t (&det)[2],
                                          floatx4 (&o)[9][2], float scale_log2, float (&m_run)[2],
                                          float (&l_mark)[2]) {
  constexpr bool PIVOT = (MODE & 1) != 0, HALF = (MODE & 2) != 0;
  if (__builtin_amdgcn_ballot_w64(((det[0] | det[1]) & AT_P_TOO_LARGE) != 0u) != 0ull) {
    float mx[2];  // (S(j-1) is a whole stage old: no wait states needed before reading it)
    at_lanemax(s_prev, mx);
    const float m_new[2] = {at_max2(m_run[0], at_groupmax(mx[0] * scale_log2)),
                            at_max2(m_run[1], at_groupmax(mx[1] * scale_log2))};
    at_settle_o(o);
    // m_run = AT_NO_MAX on a row's first keys: alpha = 0 (O and the sums are still zero then)
    const float alpha[2] = {__builtin_amdgcn_exp2f(m_run[0] - m_new[0]), __builtin_amdgcn_exp2f(m_run[1] - m_new[1])};
    uint32_t pk[8];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      if constexpr (PIVOT) l_mark[qt] *= alpha[qt];
#pragma unroll
      for (int dt = 0; dt < 9; ++dt) {
        if (HALF && dt >= 4 && dt < 8) continue;  // channel tiles nobody accumulates into
#pragma unroll
        for (int j = 0; j < 4; ++j) o[dt][qt][j] *= alpha[qt];
      }
      float e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        e[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(AT_SVAL(s_prev, 8 * qt + j), scale_log2, -m_new[qt]));
#pragma unroll
      for (int j = 0; j < 4; ++j) pk[4 * qt + j] = at_pack2(e[2 * j], e[2 * j + 1]);
      m_run[qt] = m_new[qt];
    }
    at_settle_o(o);
    p[0] = __builtin_bit_cast(bf16x8, (at_u32x4){pk[0], pk[1], pk[2], pk[3]});
    p[1] = __builtin_bit_cast(bf16x8, (at_u32x4){pk[4], pk[5], pk[6], pk[7]});
    asm volatile("s_nop 4" : "+v"(p[0]), "+v"(p[1]));  // vector writes of P are complete before an MFMA reads them
  }
  det[0] = 0u;
  det[1] = 0u;
}

// One pipeline step.  s_in = S(j) (complete), p_prev = P(j-1) not yet applied to O (HAVE_PREV), det the OR of its
// packed words; s_out still holds S(j-1) on entry and S(j+1) on return, p_out = P(j) with its OR in det.
// The fused stage exists once per step: O never lives in two register sets that would have to be merged.
template <bool DO_QK, bool HAVE_PREV, int KQ, int VB, int KT, int MODE, bool PRE = false, int NEXT = -1>
__device__ __forceinline__ void at_step(const AtAddr& ad, const bf16x8 (&qb)[2][4], floatx4 (&s_out)[2][2],
                                        floatx4 (&s_in)[2][2], bf16x8 (&p_prev)[2], bf16x8 (&p_out)[2],
                                        floatx4 (&o)[9][2], float scale_log2, float (&m_run)[2], uint32_t (&det)[2],
                                        const bf16x8& ones, bool diag, int key_base, int t, float (&l_mark)[2],
                                        bf16x8 (&pre)[2], uint32_t kq = 0xffffu) {
  if (HAVE_PREV) at_commit<MODE>(s_out, p_prev, det, o, scale_log2, m_run, l_mark);
  if (diag) at_causal(s_in, key_base, t);
  if constexpr ((MODE & 4) != 0) at_keep(s_in, kq, key_base);
  const float neg_m[2] = {-m_run[0], -m_run[1]};
  // wait states inside the stage's last MFMA: a run's first stage (S read at once), and for pivot heads the stage
  // behind which the block sums are taken (emit in the kernel: the second stage of a block in the steady state)
  constexpr bool SETTLE = (DO_QK && !HAVE_PREV) || ((MODE & 1) != 0 && DO_QK && HAVE_PREV && KQ == 1);
  at_fused<DO_QK, HAVE_PREV, KQ, VB, KT, PRE, NEXT, (MODE & 2) != 0, SETTLE>(ad, qb, s_out, s_in, p_prev, p_out, o,
                                                                              scale_log2, neg_m, det, ones, pre);
}

// PIVOT = false: every head except the pivots that have a slot in the scheduler area's table (when skip_slotted).
// PIVOT = true: only those pivots; besides the output it leaves, per (query, key block), the softmax mass of the
// block relative to the running max at that time as u = log2(sum) + max, from which at_avg_from_block_sums (sp_attn_avg_kernel) makes
// the block-average map without recomputing any logit.  pivot_u: fp32 [slot][r*(r+1)/2 + c][128 queries].
// HALF: q, k and v are zero beyond channel 64 (see at_fused); channels 64..127 of out are then not written.
// FINE: a block size f = 128 >> fshift below 128.  `mask` is then the OR of the caller's fine mask over 128-token
// blocks (sp_attn_coarsen_kernel) and decides which 128-key blocks a row visits; fine_mask [hq][nbf][nbfw] decides, per
// 16 x 16 sub-tile, what survives of a visited block (at_keep).  Exact, at the cost of computing whole 128 x 128 blocks.
template <bool PIVOT, bool HALF, bool FINE = false>
__global__ __launch_bounds__(AT_FWD_THREADS, 1) void sp_attn_fwd_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const sp_bf16* __restrict__ vt,
    const uint64_t* __restrict__ mask, const int32_t* __restrict__ decision, sp_bf16* __restrict__ out,
    float2* __restrict__ rowstat, int64_t n, int hq, int hkv, int64_t sq_n, int64_t sq_h, int64_t sk_n,
    int64_t sk_h, int nb, int nbw, float scale_log2, int* __restrict__ sched, int skip_slotted,
    float* __restrict__ pivot_u, const uint64_t* __restrict__ fine_mask, int fshift, int nbf, int nbfw) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];  // K ring (4 x 16 KiB) | V^T ring (4 x 16 KiB)
  __shared__ int s_queue, s_ticket;
  constexpr int MODE = (PIVOT ? 1 : 0) | (HALF ? 2 : 0) | (FINE ? 4 : 0);
  if (PIVOT && sched[AT_NPIV_SLOT] == 0) return;  // no pivot in this layer
  const uint8_t* const slots = reinterpret_cast<const uint8_t*>(sched + AT_SLOT_TABLE);
  const uint8_t* const pair_table = reinterpret_cast<const uint8_t*>(sched + AT_PAIR_TABLE);

  const long long clk0 = clock64(), tick0 = wall_clock64();  // see sp_attn_last_launch_clocks
  AtGeom gm;
  at_geometry(gm, hq, hkv, nb);
  gm.order = sched[AT_ORDER_SLOT] != 0 ? reinterpret_cast<const uint16_t*>(sched + 256) : nullptr;
  const int xcd = blockIdx.x & 7;
  int first_try = 0;  // queues before this offset are known to be empty (used by thread 0 only)
  const int t = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // 0..7
  const int grp = wave >> 2;                                 // which row of the pair this wave works on
  const int tq = t & 255;                                    // thread index inside the row's four waves

  // Lane-constant LDS read offsets (bytes) inside a buffer.  With lq = lane % 16 (the lane's row in a 16-row
  // operand tile) and g = lane / 16, the XOR swizzle makes the operand of channel step ks (K) or of key-slot half h
  // (V^T) sit at (offset ^ (index << 6)):
  //   K  : row lq (+16, +32 via immediate), logical chunk 4*ks + g  -> lq*256 + (((4*ks + g) ^ lq) << 4)
  //   V^T: row lq (+16*dt via immediate), logical chunk 4*h + g     -> lq*128 + (((4*h + g) ^ ((lq >> 1) & 7)) << 4)
  // Only these, the two global load offsets and tq stay in registers across the key loop; everything else that
  // depends on the lane is recomputed where it is needed from an opaque copy of tq (AT_LANE_VIEW), so that the
  // compiler does not carry a dozen precomputed lane constants through the loop.
  int koff, voff;
  AtLoadOffsets lo;
  {
    const int lane = t & 63, lq = lane & 15, g = lane >> 4;
    koff = lq * 256 + ((g ^ lq) << 4);
    voff = lq * 128 + ((g ^ ((lq >> 1) & 7)) << 4);
    at_load_offsets(lo, sk_n, wave, lane);
  }
  char* const kring = lds;
  char* const vring = lds + AT_RING * AT_KBUF_BYTES;
  uint32_t* const blist = reinterpret_cast<uint32_t*>(lds + AT_RING * (AT_KBUF_BYTES + AT_VBUF_BYTES));
  const int c_ragged = (n % AT_BS) != 0 ? nb - 1 : -1;  // the only block whose K rows may run past the sequence

  for (;;) {
    __syncthreads();  // previous item's LDS reads are done
    if (t == 0) {
      int found = -1, tk = 0;
      for (int a = first_try; a < 8; ++a) {
        const int xq = (xcd + a) & 7;
        tk = atomicAdd(&sched[PIVOT ? AT_PIVOT_TICKETS + xq : xq * 16], 1);
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
    const int queue = __builtin_amdgcn_readfirstlane(s_queue);
    if (queue < 0) {
      if (!PIVOT && blockIdx.x == 0 && t == 0) {
        long long* clk = reinterpret_cast<long long*>(sched + AT_CLOCK_SLOT);
        clk[0] = clock64() - clk0;
        clk[1] = wall_clock64() - tick0;
      }
      break;
    }
    const int ticket = __builtin_amdgcn_readfirstlane(s_ticket);
    int h_item, pair;
    if (!at_item(gm, queue, ticket, h_item, pair)) continue;
    const int slot = slots[h_item];
    if (PIVOT ? slot == AT_NO_SLOT : (skip_slotted && slot != AT_NO_SLOT)) continue;  // the other launch's head
    // the item's two (head, row): A for waves 0-3, B for waves 4-7
    const bool by_heads = !PIVOT && pair_table[h_item >> 1] != 0;
    const int h_a = by_heads ? (h_item & ~1) : h_item, h_b = by_heads ? (h_item | 1) : h_item;
    const int r_a = by_heads ? 2 * pair + (h_item & 1) : 2 * pair, r_b = by_heads ? r_a : r_a + 1;
    if (r_a >= nb) continue;  // (heads pairing, odd nb: the odd head's last item has no row)
    const bool has_b = r_b < nb;
    const int h = grp ? h_b : h_a;  // this wave's head
    const int r = grp ? r_b : r_a;  // this wave's row
    const bool row_ok = grp == 0 || has_b;
    const int kvh = h_a / gm.group;
    const sp_bf16* kh = k + (int64_t)kvh * sk_h;
    const char* vth = reinterpret_cast<const char*>(vt + (int64_t)kvh * nb * AT_D * AT_BS);
    const uint64_t* mrow_a = mask + ((int64_t)h_a * nb + r_a) * nbw;
    const uint64_t* mrow_b = mask + ((int64_t)h_b * nb + (has_b ? r_b : r_a)) * nbw;

    // ---- the pair's block list: every column kept by either row, ascending, with membership flags ----
    // All waves walk the (uniform) mask words and keep a running count; wave w compacts words w, w+8, ...
    int n_blk = 0;
    {
      const int wmax = (has_b ? r_b : r_a) >> 6;
      const int lane = t & 63;
      for (int wi = 0; wi <= wmax; ++wi) {
        const uint64_t wa = at_trim(mrow_a[wi], wi, r_a);
        const uint64_t wb = has_b ? at_trim(mrow_b[wi], wi, r_b) : 0ull;
        const uint64_t wu = wa | wb;
        if ((wi & 7) == wave && ((wu >> lane) & 1ull)) {
          const int pos = n_blk + __builtin_popcountll(wu & ((1ull << lane) - 1ull));
          blist[pos] = (uint32_t)(wi * 64 + lane) | (((wa >> lane) & 1ull) ? AT_IN_A : 0u) |
                       (((wb >> lane) & 1ull) ? AT_IN_B : 0u);
        }
        n_blk += __builtin_popcountll(wu);
      }
      n_blk = __builtin_amdgcn_readfirstlane(n_blk);
    }
    __syncthreads();

    // Q^T operands: the lane's two queries (one per 16-query tile), 4 channel steps of 8 channels each
    bf16x8 qb[2][4];
    {
      AT_LANE_VIEW(tq);
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        int64_t qrow = (int64_t)r * AT_BS + q_off + qt * 16;
        if (qrow > n - 1) qrow = n - 1;
        const sp_bf16* src = q + (int64_t)h * sq_h + qrow * sq_n + 8 * g;
#pragma unroll
        for (int ks = 0; ks < (HALF ? 2 : 4); ++ks)
          qb[qt][ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(src + 32 * ks));
      }
    }

    // FINE: the two fine mask rows of this wave's query tiles, and the keep bits (at_keep) of a block from them
    const uint64_t* frow[2] = {fine_mask, fine_mask};
    if constexpr (FINE) {
      const int w4 = wave & 3;
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        int fr = (r * AT_BS + 32 * w4 + 16 * qt) >> (7 - fshift);
        if (fr > nbf - 1) fr = nbf - 1;  // (queries beyond the sequence: computed, never stored)
        frow[qt] = fine_mask + ((int64_t)h * nbf + fr) * nbfw;
      }
    }
    // the two 64-bit mask words are requested a block ahead of their use (fine_issue at the top of block b for block
    // b + 1, fine_take when the walk moves on)
    uint64_t fw_next[2] = {~0ull, ~0ull};
    auto fine_issue = [&](int c) {
      if constexpr (FINE) {
        const int fc0 = c << fshift;  // first fine column of the 128-key block; its 1 << fshift bits share a word
        fw_next[0] = frow[0][fc0 >> 6];
        fw_next[1] = frow[1][fc0 >> 6];
      }
    };
    auto fine_take = [&](int c) -> uint32_t {  // kq of column c from the words fine_issue(c) requested
      uint32_t kq = 0xffffu;
      if constexpr (FINE) {
        const int fc0 = c << fshift;
        kq = 0u;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
          const uint32_t fb = (uint32_t)(fw_next[qt] >> (fc0 & 63));
          uint32_t k16 = 0u;
#pragma unroll
          for (int c16 = 0; c16 < 8; ++c16) k16 |= ((fb >> (c16 >> (3 - fshift))) & 1u) << c16;
          kq |= k16 << (8 * qt);
        }
        kq = __builtin_amdgcn_readfirstlane(kq);
      }
      return kq;
    };
    uint32_t kq_cur = 0xffffu;

    floatx4 o[9][2];  // [channel tile][query tile]; o[8]: the row sums (ones . P)
#pragma unroll
    for (int dt = 0; dt < 9; ++dt)
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) o[dt][qt] = (floatx4){0, 0, 0, 0};
    float m_run[2] = {AT_NO_MAX, AT_NO_MAX};
    uint32_t det[2] = {0u, 0u};
    bf16x8 ones = __builtin_bit_cast(bf16x8, (at_u32x4){0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
    asm volatile("" : "+v"(ones));  // one register set for the whole row
    // Pivot heads: block sums.  o[8] - l_mark is the softmax mass of the key block whose last half-tile has just been
    // applied to O, relative to the current running max (both follow every rescale; every lane of a query's group
    // holds the whole sum); it is kept as u = log2(sum) + m_run.
    float l_mark[2] = {0.f, 0.f};
    const int64_t tri_row = (int64_t)slot * ((int64_t)nb * (nb + 1) / 2) + (int64_t)r * (r + 1) / 2;
    float* const pu = PIVOT ? pivot_u + tri_row * AT_BS : nullptr;
    auto emit = [&](int c) {
      if constexpr (PIVOT) {
        // (the sums' last MFMA carried its wait states: at_fused<SETTLE> / at_pv_only)
        AT_LANE_VIEW(tq);
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
          const float tl = o[8][qt][0] - l_mark[qt];
          l_mark[qt] = o[8][qt][0];
          const float u = __builtin_amdgcn_logf(tl) + m_run[qt];
          if (g == 0) pu[(int64_t)c * AT_BS + q_off + qt * 16] = u;
        }
      }
    };

    // Block b of the list is processed as sub-tiles 2b and 2b+1; sub-tile s lives in ring slot s % 4 (K and V^T
    // rings alike).  One wait + barrier + issue per BLOCK: while block b is computed on (K of sub-tiles 2b, 2b+1
    // and V^T of 2b-1, 2b -- the P.V product trails by one sub-tile), K of 2b+2, 2b+3 and V^T of 2b+1, 2b+2 are
    // in flight.  Past the end the last block is fetched again into slots nobody reads any more.
    auto entry = [&](int b) -> uint32_t {
      const int bc = b < n_blk ? b : n_blk - 1;
      return __builtin_amdgcn_readfirstlane(blist[bc]);
    };
    auto issue_k = [&](int c, int hf, int sub) {  // K of sub-tile `sub` = (column c, half hf)
      char* kbuf = kring + (sub & 3) * AT_KBUF_BYTES;
      const int64_t key0 = (int64_t)c * AT_BS + hf * AT_SUB;
      if (c != c_ragged)
        at_issue_k(lo, reinterpret_cast<const char*>(kh + key0 * sk_n), sk_n, kbuf, wave);
      else
        at_issue_k_tail(kh, n, sk_n, key0, kbuf, wave, t);
    };
    auto issue_v = [&](int c, int hf, int sub) {  // V^T of sub-tile `sub` = (column c, half hf)
      at_issue_v(lo, vth + (int64_t)c * (AT_D * AT_BS * 2) + hf * (AT_SUB * 2), vring + (sub & 3) * AT_VBUF_BYTES,
                 wave);
    };
    int c_cur = -1;
    bool mine = false;
    const uint32_t my_flag = grp ? AT_IN_B : AT_IN_A;
    // The list is read one block ahead of its use: e_next is the entry of block b + 1, and the read of block b + 2's
    // goes out at the top of block b, unseen by the compiler (an asynchronous LDS read like the operand fetches),
    // to be picked up when the walk moves on.  Read where it is needed, it cost every wave an LDS round trip right
    // behind each block's barrier, where no other wave has anything to issue either.
    uint32_t e_next = 0u, e_ahead = 0u;
    const uint32_t blist_addr = at_lds_addr(reinterpret_cast<const char*>(blist));
    if (n_blk > 0) {
      const uint32_t e0 = entry(0);
      e_next = entry(1);
      c_cur = (int)(e0 & AT_COL_MASK);
      mine = (e0 & my_flag) != 0u;
      issue_k(c_cur, 0, 0);
      issue_k(c_cur, 1, 1);
      issue_v(c_cur, 0, 0);
      fine_issue(c_cur);
      kq_cur = fine_take(c_cur);
    }

    // The compute walk.  Per block every wave passes `top` exactly once (wait, barrier, issue), whatever its row
    // does with the block.  A row's own blocks come in runs; a run is one straight-line pipeline: start (first S),
    // steady steps while the next block is the row's too, drain on the block after the run (V^T of the run's last
    // sub-tile is resident by then) or after the walk.
    int b = 0;
    const char *kb = kring, *vb = vring;  // K(2b), V^T(2b-1); the second sub-tile's buffers follow in the rings
    const char* vb1 = vring;              // V^T(2b)
    int c_next = 0;  // column of block b+1 (clamped to the last block)
    AtAddr ad;
    auto top = [&]() {
      AT_WAIT_VMCNT0();              // K(2b), K(2b+1), V^T(2b-1), V^T(2b) have landed (own loads)
      __builtin_amdgcn_s_barrier();  // ... everybody's; and every wave is past block b-1
      // (hidden loop invariance: no precomputed copies of these lane constants that could be spilled)
      asm volatile("" : "+v"(lo.k), "+v"(lo.v));
      c_next = (int)(e_next & AT_COL_MASK);
      fine_issue(c_next);
      {
        const int ba = b + 2 < n_blk ? b + 2 : n_blk - 1;
        asm volatile("ds_read_b32 %0, %1" : "=v"(e_ahead) : "v"(blist_addr + 4u * (uint32_t)ba));
      }
      kb = kring + ((2 * b) & 3) * AT_KBUF_BYTES;
      vb = vring + ((2 * b + 3) & 3) * AT_VBUF_BYTES;
      vb1 = vring + ((2 * b) & 3) * AT_VBUF_BYTES;
      asm volatile("" : "+v"(koff), "+v"(voff));
      at_block_addr(ad, kb, vb, vb1, koff, voff);
    };
    // The next block's loads go out in four parts spread over the block's steps: issued in one burst, the eight
    // waves' 64 KiB would queue up in front of the CU's vector-memory path and stall everybody for its duration.
    auto feed = [&](int part) {
      if (part == 0) issue_k(c_next, 0, 2 * b + 2);
      if (part == 1) issue_k(c_next, 1, 2 * b + 3);
      if (part == 2) issue_v(c_cur, 1, 2 * b + 1);
      if (part == 3) issue_v(c_next, 0, 2 * b + 2);
    };
    auto feed_all = [&]() {
      feed(0);
      feed(1);
      feed(2);
      feed(3);
    };
    auto step_walk = [&]() {  // (every call follows a `top` of the block that ends here)
      ++b;
      if (b < n_blk) {
        c_cur = (int)(e_next & AT_COL_MASK);
        mine = (e_next & my_flag) != 0u;
        kq_cur = fine_take(c_cur);
      } else {
        c_cur = -1;
        mine = false;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(e_ahead));  // long since back: issued a whole block ago
      e_next = __builtin_amdgcn_readfirstlane(e_ahead);
    };
    bool finished = false;  // the final wait + barrier has been passed
    while (c_cur >= 0) {
      top();
      if (!mine) {
        feed_all();
        step_walk();
        continue;
      }
      floatx4 sa[2][2], sb[2][2];  // [key tile][query tile]
      bf16x8 pa[2], pb[2];         // [query tile]
      bf16x8 pre[2];               // the next stage's first two LDS operands, in flight (at_prefetch_qk)
      // ---- start of a run: S of the first half-tile, nothing to overlap with yet ----
      feed(0);
      at_qk_only<0, HALF>(kb, koff, qb, sa);
      feed(1);
      at_step<true, false, 1, 0, 0, MODE, false, 2>(ad, qb, sb, sa, pb, pa, o, scale_log2, m_run, det, ones,
                                                     c_cur == r, 0, tq, l_mark, pre, kq_cur);
      feed(2);
      at_step<true, true, 2, 1, 0, MODE, true, 3>(ad, qb, sa, sb, pa, pb, o, scale_log2, m_run, det, ones,
                                                   c_cur == r, 32, tq, l_mark, pre, kq_cur);
      feed(3);
      at_step<true, true, 3, 1, 1, MODE, true, -1>(ad, qb, sb, sa, pb, pa, o, scale_log2, m_run, det, ones,
                                                    c_cur == r, AT_SUB, tq, l_mark, pre, kq_cur);
      int c_prev = c_cur;
      uint32_t kq_prev = kq_cur;
      step_walk();
      // ---- steady state: four half-tile steps per block ----
      while (mine) {  // (mine implies c_cur >= 0)
        top();
        // The instruction arbiter favours the older waves (the even row's), which then finish the block early and
        // idle at the barrier while the odd row's waves run alone at half the matrix-core rate: the odd row gets
        // priority for the first half of the block, which evens the two out.
        at_prefetch_qk<0>(ad, pre);  // (the block's first operands, while the loads and the commit test are set up)
        if (grp) __builtin_amdgcn_s_setprio(1);
        // S(previous block, keys 96..127) -> P;  S(keys 0..31) on the matrix core;  O += V^T(2b-1, keys 0..31) . P
        at_step<true, true, 0, 0, 0, MODE, true, 1>(ad, qb, sa, sb, pa, pb, o, scale_log2, m_run, det, ones,
                                                     c_prev == r, AT_SUB + 32, tq, l_mark, pre, kq_prev);
        feed(0);
        at_step<true, true, 1, 0, 1, MODE, true, 2>(ad, qb, sb, sa, pb, pa, o, scale_log2, m_run, det, ones,
                                                     c_cur == r, 0, tq, l_mark, pre, kq_cur);
        emit(c_prev);  // the previous block's last half-tile went into O (and the sums) in this step
        if (grp) __builtin_amdgcn_s_setprio(0);
        feed(1);
        feed(2);
        at_step<true, true, 2, 1, 0, MODE, true, 3>(ad, qb, sa, sb, pa, pb, o, scale_log2, m_run, det, ones,
                                                     c_cur == r, 32, tq, l_mark, pre, kq_cur);
        feed(3);
        at_step<true, true, 3, 1, 1, MODE, true, -1>(ad, qb, sb, sa, pb, pa, o, scale_log2, m_run, det, ones,
                                                      c_cur == r, AT_SUB, tq, l_mark, pre, kq_cur);
        c_prev = c_cur;
        kq_prev = kq_cur;
        step_walk();
      }
      // ---- drain: the run's last half-tile and its P.V (V^T of sub-tile 2b-1) ----
      if (c_cur >= 0) {
        top();
        feed_all();
        step_walk();
      } else {
        AT_WAIT_VMCNT0();
        __syncthreads();
        finished = true;
        vb = vring + ((2 * b + 3) & 3) * AT_VBUF_BYTES;
        at_block_addr(ad, kb, vb, vb, koff, voff);
      }
      at_step<false, true, 0, 0, 0, MODE>(ad, qb, sa, sb, pa, pb, o, scale_log2, m_run, det, ones,
                                           c_prev == r, AT_SUB + 32, tq, l_mark, pre, kq_prev);
      at_commit<MODE>(sb, pb, det, o, scale_log2, m_run, l_mark);
      at_pv_only<1, HALF>(vb, voff, pb, o, ones);
      emit(c_prev);
    }
    if (!finished) {
      AT_WAIT_VMCNT0();
      __syncthreads();
    }
    at_settle_o(o);
    // every lane of a query's group holds the whole row sum (all rows of the ones . P tile are equal)
    const float l_tot[2] = {o[8][0][0], o[8][1][0]};
    AT_LANE_VIEW(tq);

    // pivot heads: keep the softmax statistics of every query row for the block-average pass
    if (row_ok && rowstat != nullptr && decision != nullptr && decision[h] == SP_DEC_DENSE && g == 0) {
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        const int64_t qrow = (int64_t)r * AT_BS + q_off + qt * 16;
        if (qrow < n) rowstat[(int64_t)h * n + qrow] = make_float2(m_run[qt], l_tot[qt]);
      }
    }

    // ---- epilogue: normalise and store straight from the accumulators.  A lane holds 4 consecutive channels of its
    // query per channel tile: 8-byte stores, 32 contiguous bytes per query row and instruction; the four channel tiles
    // that share a 128-byte line follow each other, and the write-back L2 merges them.  No LDS, no barrier: the
    // workgroup goes on to its next item while the stores drain. ----
    if (row_ok) {
#pragma unroll
      for (int qt = 0; qt < 2; ++qt) {
        const int64_t qrow = (int64_t)r * AT_BS + q_off + qt * 16;
        if (qrow < n) {
          const float inv_l = 1.0f / l_tot[qt];
          sp_bf16* dst = out + (qrow * hq + h) * AT_D + 4 * g;
#pragma unroll
          for (int dt = 0; dt < (HALF ? 4 : 8); ++dt)
            *reinterpret_cast<uint2*>(dst + dt * 16) =
                make_uint2(at_pack2(o[dt][qt][0] * inv_l, o[dt][qt][1] * inv_l),
                           at_pack2(o[dt][qt][2] * inv_l, o[dt][qt][3] * inv_l));
        }
      }
    }
  }
}

// Before the forward launches: clears the queue tickets and gives the first max_pivots heads whose decision is
// DENSE a slot for their block sums (ascending head order); every other head gets AT_NO_SLOT.
__global__ void sp_attn_prep_kernel(int* __restrict__ sched, const int32_t* __restrict__ decision, int hq,
                                    int max_pivots) {
  for (int i = threadIdx.x; i < AT_SLOT_TABLE; i += blockDim.x) sched[i] = 0;
  // pivot launch tickets; pairing table = rows 2p, 2p+1 of a head (sp_attn_pairing_kernel may choose otherwise)
  for (int i = AT_PAIR_TABLE + threadIdx.x; i < AT_PIVOT_TICKETS + 8; i += blockDim.x) sched[i] = 0;
  if (threadIdx.x == 0) {
    uint8_t* slots = reinterpret_cast<uint8_t*>(sched + AT_SLOT_TABLE);
    int cnt = 0;
    for (int h = 0; h < hq; ++h) {
      const bool keep = decision != nullptr && decision[h] == SP_DEC_DENSE && cnt < max_pivots;
      slots[h] = keep ? (uint8_t)cnt++ : (uint8_t)AT_NO_SLOT;
    }
    sched[AT_NPIV_SLOT] = cnt;
    sched[AT_ORDER_SLOT] = 0;
  }
}

// After sp_attn_prep_kernel: chooses, for every two adjacent heads (2i, 2i+1), how the forward kernel pairs query
// blocks into work items.  One workgroup per head pair sums the union sizes both ways over all rows,
//   rows : |row 2p  |  row 2p+1| of each head,      heads : |row r of head 2i  |  row r of head 2i+1|,
// and writes 1 (pair by heads) when that union is strictly smaller and the two heads may share an item: same kv
// head, and neither runs in the pivot launch.  Integer sums: the choice does not depend on the order of anything.
__global__ __launch_bounds__(256) void sp_attn_pairing_kernel(int* __restrict__ sched, const uint64_t* __restrict__ mask,
                                                              int hq, int group, int nb, int nbw, int skip_slotted) {
  __shared__ unsigned long long tot[2];
  const int i = blockIdx.x, h0 = 2 * i, h1 = 2 * i + 1;
  uint8_t* table = reinterpret_cast<uint8_t*>(sched + AT_PAIR_TABLE);
  const uint8_t* slots = reinterpret_cast<const uint8_t*>(sched + AT_SLOT_TABLE);
  const bool eligible = h1 < hq && h0 / group == h1 / group &&
                        !(skip_slotted && (slots[h0] != AT_NO_SLOT || slots[h1] != AT_NO_SLOT));
  if (!eligible) {  // (uniform)
    if (threadIdx.x == 0) table[i] = 0;
    return;
  }
  if (threadIdx.x < 2) tot[threadIdx.x] = 0ull;
  __syncthreads();
  const uint64_t* m0 = mask + (int64_t)h0 * nb * nbw;
  const uint64_t* m1 = mask + (int64_t)h1 * nb * nbw;
  unsigned long long by_rows = 0ull, by_heads = 0ull;
  for (int p = threadIdx.x; 2 * p < nb; p += blockDim.x) {
    const int ra = 2 * p, rb = 2 * p + 1 < nb ? 2 * p + 1 : 2 * p;
    for (int w = 0; w <= (rb >> 6); ++w) {
      const uint64_t a0 = m0[(int64_t)ra * nbw + w], b0 = m0[(int64_t)rb * nbw + w];
      const uint64_t a1 = m1[(int64_t)ra * nbw + w], b1 = m1[(int64_t)rb * nbw + w];
      by_rows += __builtin_popcountll(a0 | b0) + __builtin_popcountll(a1 | b1);
      by_heads += __builtin_popcountll(a0 | a1) + (rb != ra ? __builtin_popcountll(b0 | b1) : 0);
    }
  }
  atomicAdd(&tot[0], by_rows);
  atomicAdd(&tot[1], by_heads);
  __syncthreads();
  if (threadIdx.x == 0) table[i] = tot[1] < tot[0] ? 1 : 0;
}

// After sp_attn_pairing_kernel, for launches of at most AT_ORDER_MAX gangs: ranks the gangs by the work of their items
// -- the blocks the item's two rows visit together, plus a few blocks' worth of fixed time per item -- and writes the
// gang positions in descending order (ties: ascending position) into the order table.  One workgroup; integer
// weights, so the ranking does not depend on the order of anything.
#define AT_ITEM_FIXED 6  // an item's fixed time (ticket, block list, first tiles, epilogue) in units of one block visit
__global__ __launch_bounds__(1024) void sp_attn_order_kernel(int* __restrict__ sched, const uint64_t* __restrict__ mask,
                                                             int hq, int hkv, int nb, int nbw) {
  __shared__ uint32_t weight[AT_ORDER_MAX];
  AtGeom gm;
  at_geometry(gm, hq, hkv, nb);
  const uint8_t* pair_table = reinterpret_cast<const uint8_t*>(sched + AT_PAIR_TABLE);
  uint16_t* order = reinterpret_cast<uint16_t*>(sched + 256);
  for (int pos = threadIdx.x; pos < gm.n_gangs; pos += blockDim.x) {
    int h, j;
    at_gang_of(gm, pos, h, j);
    const bool by_heads = pair_table[h >> 1] != 0;
    const int h_a = by_heads ? (h & ~1) : h, h_b = by_heads ? (h | 1) : h;
    uint32_t wsum = 0;
    for (int slot = 0; slot < gm.gang; ++slot) {
      const int pair = gm.n_pairs - 1 - (j * gm.gang + slot);
      if (pair < 0) break;
      const int r_a = by_heads ? 2 * pair + (h & 1) : 2 * pair, r_b = by_heads ? r_a : r_a + 1;
      if (r_a >= nb) continue;
      const bool has_b = r_b < nb;
      const uint64_t* ma = mask + ((int64_t)h_a * nb + r_a) * nbw;
      const uint64_t* mb = mask + ((int64_t)h_b * nb + (has_b ? r_b : r_a)) * nbw;
      const int wmax = (has_b ? r_b : r_a) >> 6;
      uint32_t cnt = AT_ITEM_FIXED;
      for (int wi = 0; wi <= wmax; ++wi)
        cnt += __builtin_popcountll(at_trim(ma[wi], wi, r_a) | (has_b ? at_trim(mb[wi], wi, r_b) : 0ull));
      wsum += cnt;
    }
    weight[pos] = wsum;
  }
  __syncthreads();
  for (int pos = threadIdx.x; pos < gm.n_gangs; pos += blockDim.x) {
    const uint32_t wp = weight[pos];
    int rank = 0;
    for (int o = 0; o < gm.n_gangs; ++o) {
      const uint32_t wo = weight[o];
      rank += (wo > wp) || (wo == wp && o < pos);
    }
    order[rank] = (uint16_t)pos;
  }
  if (threadIdx.x == 0) sched[AT_ORDER_SLOT] = 1;
}

// ---- pivot heads with a slot: block-averaged attention map from the block sums the forward kernel kept ----
// avg[h][r][c] = mean over the valid queries of block r of  exp2(u[q][c] - m[q]) / l[q]  (m, l: the query's final
// softmax statistics).  One workgroup per (query block, head) of sp_attn_avg_kernel; a wave takes every fourth kept
// block.
__device__ static void at_avg_from_block_sums(const uint64_t* __restrict__ mask, int slot,
                                              const float2* __restrict__ rowstat, const float* __restrict__ pivot_u,
                                              float* __restrict__ avg_attn, int64_t n, int nb, int nbw) {
  const int r = nb - 1 - blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t rem = n - (int64_t)r * AT_BS;
  const int valid_q = rem < AT_BS ? (int)rem : AT_BS;
  float m[2], inv_l[2];
  bool ok[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int qo = lane + 64 * j;
    ok[j] = qo < valid_q;
    const float2 st = rowstat[(int64_t)h * n + (int64_t)r * AT_BS + (ok[j] ? qo : 0)];
    m[j] = st.x;
    inv_l[j] = 1.0f / st.y;
  }
  const float inv_q = 1.0f / (float)valid_q;
  const float* pu = pivot_u + ((int64_t)slot * ((int64_t)nb * (nb + 1) / 2) + (int64_t)r * (r + 1) / 2) * AT_BS;
  float* arow_out = avg_attn + ((int64_t)h * nb + r) * nb;
  AtBlocks it;
  it.init(mask + ((int64_t)h * nb + r) * nbw, r);
  int idx = 0;
  for (int c = it.next(); c >= 0; c = it.next(), ++idx) {
    if ((idx & 3) != wave) continue;
    const float u0 = pu[(int64_t)c * AT_BS + lane], u1 = pu[(int64_t)c * AT_BS + 64 + lane];
    float part = ok[0] ? __builtin_amdgcn_exp2f(u0 - m[0]) * inv_l[0] : 0.f;
    part += ok[1] ? __builtin_amdgcn_exp2f(u1 - m[1]) * inv_l[1] : 0.f;
    part = sp_wave_sum(part);
    if (lane == 0) arow_out[c] = part * inv_q;
  }
}

// ---- pivot heads: block-averaged attention map (shareprefill_attn.py:425-457) ---------------------------
// avg[h][r][c] = mean over the valid queries of block r of the softmax mass that falls into key block c,
// recomputed from the row statistics the forward kernel left behind (the pivots for which the workspace has no
// room to keep block sums; the others are made from their block sums by at_avg_from_block_sums, in the same launch).
// One workgroup per (query block, head); heads that are no pivots leave at once.
__global__ __launch_bounds__(AT_THREADS) void sp_attn_avg_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const uint64_t* __restrict__ mask,
    const int32_t* __restrict__ decision, const float2* __restrict__ rowstat, float* __restrict__ avg_attn, int64_t n,
    int hq, int hkv, int64_t sq_n, int64_t sq_h, int64_t sk_n, int64_t sk_h, int nb, int nbw, float scale_log2,
    const int* __restrict__ sched, const float* __restrict__ pivot_u) {
  __shared__ __attribute__((aligned(16))) sp_bf16 Ks[AT_BS * AT_PITCH];
  __shared__ float wred[2][4];
  const int r = nb - 1 - blockIdx.x, h = blockIdx.y;
  if (decision[h] != SP_DEC_DENSE) return;
  {
    const int slot = reinterpret_cast<const uint8_t*>(sched + AT_SLOT_TABLE)[h];
    if (slot != AT_NO_SLOT) {  // (uniform) the forward pass kept this head's block sums
      at_avg_from_block_sums(mask, slot, rowstat, pivot_u, avg_attn, n, nb, nbw);
      return;
    }
  }
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
  // thread t stages chunk t%16 (16 bytes) of key rows t/16, t/16+16, ...; the next block's tile is fetched into
  // registers while the current one is used
  at_u32x4 kr[8];
  auto fetch = [&](int c) {
#pragma unroll
    for (int i8 = 0; i8 < 8; ++i8) {
      int64_t key = (int64_t)c * AT_BS + i8 * 16 + (t >> 4);
      if (key > n - 1) key = n - 1;
      kr[i8] = *reinterpret_cast<const at_u32x4*>(kh + key * sk_n + (t & 15) * 8);
    }
  };
  int c = it.next();
  if (c >= 0) fetch(c);
  int c_done = -1, par = 0;  // block whose wave partials wait in wred[par ^ 1]
  const float inv_q = 1.0f / (float)valid_q;
  while (c >= 0) {
    __syncthreads();  // the previous block's operand reads are done, its wave partials are written
    if (c_done >= 0 && t == 0)
      arow_out[c_done] = ((wred[par ^ 1][0] + wred[par ^ 1][1]) + (wred[par ^ 1][2] + wred[par ^ 1][3])) * inv_q;
#pragma unroll
    for (int i8 = 0; i8 < 8; ++i8)
      *reinterpret_cast<at_u32x4*>(&Ks[(i8 * 16 + (t >> 4)) * AT_PITCH + (t & 15) * 8]) = kr[i8];
    __syncthreads();
    const int c_next = it.next();
    if (c_next >= 0) fetch(c_next);
    // only the diagonal block and a block that runs past the sequence end need the per-element predicate
    const bool plain = c < r && (int64_t)(c + 1) * AT_BS <= n && valid_q == AT_BS;
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
      if (plain) {
#pragma unroll
        for (int i = 0; i < 16; ++i) part += __builtin_amdgcn_exp2f(__builtin_fmaf(acc[i], scale_log2, -m_row));
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key_off = kt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          const bool ok = q_valid && (c < r || key_off <= q_off) && ((int64_t)c * AT_BS + key_off < n);
          part += ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(acc[i], scale_log2, -m_row)) : 0.f;
        }
      }
    }
    part = sp_wave_sum(part * inv_l);
    if (lane == 0) wred[par][wave] = part;
    c_done = c;
    par ^= 1;
    c = c_next;
  }
  __syncthreads();
  if (c_done >= 0 && t == 0)
    arow_out[c_done] = ((wred[par ^ 1][0] + wred[par ^ 1][1]) + (wred[par ^ 1][2] + wred[par ^ 1][3])) * inv_q;
}

// ---- block sizes below 128 ----------------------------------------------------------------------------
// The caller's mask has one bit per f x f block (f = 128 >> fshift).  The forward kernel walks 128-key blocks: its
// block mask is the OR over every group of (128 / f)^2 fine blocks.  One thread per 64-bit word of the coarse mask.
__global__ __launch_bounds__(256) void sp_attn_coarsen_kernel(const uint64_t* __restrict__ fine, uint64_t* __restrict__ coarse,
                                                              int hq, int nb, int nbw, int nbf, int nbfw, int fshift) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)hq * nb * nbw) return;
  const int wc = (int)(i % nbw), r = (int)((i / nbw) % nb), h = (int)(i / ((int64_t)nbw * nb));
  const int per = 1 << fshift;  // fine blocks per 128 tokens
  uint64_t out = 0ull;
  for (int fi = 0; fi < per; ++fi) {
    const int fr = r * per + fi;
    if (fr >= nbf) break;
    const uint64_t* row = fine + ((int64_t)h * nbf + fr) * nbfw;
    for (int t = 0; t < per; ++t) {  // fine word wc * per + t holds the coarse columns 64 wc + t (64 / per) ...
      const int fw = wc * per + t;
      if (fw >= nbfw) break;
      const uint64_t w = row[fw];
      for (int cb = 0; cb < (64 >> fshift); ++cb)
        if ((w >> (cb << fshift)) & ((1ull << per) - 1ull)) out |= 1ull << (t * (64 >> fshift) + cb);
    }
  }
  coarse[i] = out;
}

// Block-average maps of dense heads at a block size below 128 (shareprefill_attn.py:425-457): the recomputing pass of
// sp_attn_avg_kernel with the sums kept per 16 x 16 cell of a 128 x 128 block, folded to f x f blocks at the end.
// One workgroup per (128-query block, head); only fine blocks the mask keeps are computed into and written.
__global__ __launch_bounds__(AT_THREADS) void sp_attn_avg_fine_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ k, const uint64_t* __restrict__ mask,
    const uint64_t* __restrict__ fine_mask, const int32_t* __restrict__ decision, const float2* __restrict__ rowstat,
    float* __restrict__ avg_attn, int64_t n, int hq, int hkv, int64_t sq_n, int64_t sq_h, int64_t sk_n, int64_t sk_h,
    int nb, int nbw, int nbf, int nbfw, int fshift, float scale_log2) {
  __shared__ __attribute__((aligned(16))) sp_bf16 Ks[AT_BS * AT_PITCH];
  __shared__ float cell[AT_THREADS][8];  // per thread: its query's mass in the eight 16-key groups of the block
  __shared__ float sum16[8][8];          // [16-query group][16-key group]
  const int r = nb - 1 - blockIdx.x, h = blockIdx.y;
  if (decision[h] != SP_DEC_DENSE) return;
  const int kvh = h / (hq / hkv);
  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int lq = lane & 31, g = lane >> 5;
  const int q_off = wave * 32 + lq;
  const int lf = 7 - fshift;   // log2 of the block size
  const int f = 1 << lf, per = 1 << fshift;
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
  const int fr_q = (int)(qrow >> lf);  // this thread's fine row
  const uint64_t* frow = fine_mask + ((int64_t)h * nbf + fr_q) * nbfw;
  AtBlocks it;
  it.init(mask + ((int64_t)h * nb + r) * nbw, r);
  for (int c = it.next(); c >= 0; c = it.next()) {
    __syncthreads();  // the previous block's tile and cells are consumed
    for (int i8 = 0; i8 < 8; ++i8) {
      int64_t key = (int64_t)c * AT_BS + i8 * 16 + (t >> 4);
      if (key > n - 1) key = n - 1;
      *reinterpret_cast<at_u32x4*>(&Ks[(i8 * 16 + (t >> 4)) * AT_PITCH + (t & 15) * 8]) =
          *reinterpret_cast<const at_u32x4*>(kh + key * sk_n + (t & 15) * 8);
    }
    __syncthreads();
    const int fc0 = c << fshift;
    const uint32_t rowbits = (uint32_t)(frow[fc0 >> 6] >> (fc0 & 63)) & ((1u << per) - 1u);  // this query's kept fine columns
    float part[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
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
        const bool ok = q_valid && (c < r || key_off <= q_off) && ((int64_t)c * AT_BS + key_off < n) &&
                        ((rowbits >> (key_off >> lf)) & 1u);
        const float pv = ok ? __builtin_amdgcn_exp2f(__builtin_fmaf(acc[i], scale_log2, -m_row)) : 0.f;
        part[2 * kt + (i >> 3)] += pv;  // keys 8 (i / 4) + 4 g + i % 4 of the 32: below 16 for i < 8
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) cell[t][j] = part[j] * inv_l;
    __syncthreads();
    if (t < 64) {  // cell (16-query group t / 8, 16-key group t % 8): its 16 queries in ascending order
      const int qg = t >> 3, kg = t & 7;
      float sacc = 0.f;
      for (int i = 0; i < 16; ++i) {
        const int qo = 16 * qg + i;  // q_off of the thread that holds it: wave qo / 32, lq qo % 32, both g
        const int tb = (qo >> 5) * 64 + (qo & 31);
        sacc += cell[tb][kg] + cell[tb + 32][kg];
      }
      sum16[qg][kg] = sacc;
    }
    __syncthreads();
    if (t < per * per) {  // fine block (fi, fj) of this 128 x 128 block
      const int fi = t >> fshift, fj = t & (per - 1);
      const int fr = r * per + fi, fc = fc0 + fj;
      if (fr < nbf && fc < nbf && fc <= fr) {
        const uint64_t* rw = fine_mask + ((int64_t)h * nbf + fr) * nbfw;
        if ((rw[fc >> 6] >> (fc & 63)) & 1ull) {
          const int cells = f >> 4;  // 16-wide cells per fine block side
          float tot = 0.f;
          for (int a = 0; a < cells; ++a)
            for (int b2 = 0; b2 < cells; ++b2) tot += sum16[fi * cells + a][fj * cells + b2];
          const int64_t left = n - (int64_t)fr * f;
          const int rows = left < f ? (int)left : f;
          avg_attn[((int64_t)h * nbf + fr) * nbf + fc] = tot / (float)rows;
        }
      }
    }
  }
}

// ---- host ---------------------------------------------------------------------------------------------
// workspace layout: [ repacked V^T : hkv*nb*128*128 bf16 | scheduler area : 1 KiB of slots + 2 KiB order table |
//                     row statistics : hq*n float2 ]
// (the tiles are 128 keys wide whatever the caller's block size)
static size_t at_vt_bytes(int64_t n, int32_t hkv, int32_t d, int32_t bs) {
  (void)bs;
  return (size_t)hkv * (size_t)sp_ceil_div(n, AT_BS) * AT_BS * d * sizeof(sp_bf16);
}
static inline bool at_block_size_ok(int32_t bs) { return bs == 128 || bs == 64 || bs == 32 || bs == 16; }
static inline int at_fshift(int32_t bs) { return bs == 64 ? 1 : bs == 32 ? 2 : bs == 16 ? 3 : 0; }
// block sizes below 128: the 128-block mask the kernels walk, behind the row statistics
static size_t at_coarse_mask_bytes(int64_t n, int32_t hq, int32_t bs) {
  if (bs == AT_BS) return 0;
  const size_t nb = (size_t)sp_ceil_div(n, AT_BS);
  return (size_t)hq * nb * ((nb + 63) / 64) * sizeof(uint64_t);
}

extern "C" size_t sp_attn_workspace_bytes(int64_t n, int32_t hq, int32_t hkv, int32_t d, int32_t bs) {
  if (n <= 0 || hq <= 0 || hkv <= 0 || d <= 0 || bs <= 0) return 0;
  return at_vt_bytes(n, hkv, d, bs) + AT_SCHED_BYTES + (size_t)hq * (size_t)n * sizeof(float2) +
         at_coarse_mask_bytes(n, hq, bs);
}

// block sums of one pivot head: fp32 [nb*(nb+1)/2 lower-triangular blocks][128 queries] (128-token blocks; a call
// with a smaller block size keeps no block sums and ignores workspace beyond the base size)
extern "C" size_t sp_attn_pivot_scratch_bytes(int64_t n, int32_t bs) {
  if (n <= 0 || bs <= 0) return 0;
  const size_t nb = (size_t)sp_ceil_div(n, AT_BS);
  return nb * (nb + 1) / 2 * (size_t)AT_BS * sizeof(float);
}

extern "C" int sp_attn_last_launch_clocks(const void* workspace, int64_t n, int32_t hkv, int32_t d, int32_t bs,
                                          int64_t* cycles_and_ticks, sp_stream_t stream) {
  SP_REQUIRE(workspace && cycles_and_ticks && n > 0 && hkv > 0 && d > 0 && bs > 0, SP_ERR_INVALID_ARGUMENT,
             "sp_attn_last_launch_clocks: bad arguments");
  SP_HIP(hipStreamSynchronize((hipStream_t)stream));
  SP_HIP(hipMemcpy(cycles_and_ticks, (const char*)workspace + at_vt_bytes(n, hkv, d, bs) + AT_CLOCK_SLOT * sizeof(int),
                   2 * sizeof(int64_t), hipMemcpyDeviceToHost));
  return SP_OK;
}

extern "C" int sp_attn_last_launch_pairing(const void* workspace, int64_t n, int32_t hq, int32_t hkv, int32_t d,
                                           int32_t bs, uint8_t* by_heads, sp_stream_t stream) {
  SP_REQUIRE(workspace && by_heads && n > 0 && hq > 0 && hq <= AT_MAX_HEADS && hkv > 0 && d > 0 && bs > 0,
             SP_ERR_INVALID_ARGUMENT, "sp_attn_last_launch_pairing: bad arguments");
  SP_HIP(hipStreamSynchronize((hipStream_t)stream));
  SP_HIP(hipMemcpy(by_heads, (const char*)workspace + at_vt_bytes(n, hkv, d, bs) + AT_PAIR_TABLE * sizeof(int),
                   (size_t)((hq + 1) / 2), hipMemcpyDeviceToHost));
  return SP_OK;
}

extern "C" int sp_attn_repack_v_bf16(const void* v, int64_t n, int32_t hkv, int32_t d, int64_t v_stride_n,
                                     int64_t v_stride_h, int32_t bs, void* workspace, size_t workspace_bytes,
                                     sp_stream_t stream) {
  SP_REQUIRE(v && workspace, SP_ERR_INVALID_ARGUMENT, "sp_attn_repack_v_bf16: null pointer");
  SP_REQUIRE(n > 0 && hkv > 0, SP_ERR_INVALID_ARGUMENT, "sp_attn_repack_v_bf16: bad shape");
  SP_REQUIRE(at_block_size_ok(bs) && d == AT_D, SP_ERR_UNSUPPORTED,
             "sp_attn_repack_v_bf16: block size %d / head_dim %d unsupported (16, 32, 64 or 128 / 128)", bs, d);
  SP_REQUIRE(v_stride_n % 8 == 0 && v_stride_h % 8 == 0 && ((uintptr_t)v % 16) == 0 &&
                 ((uintptr_t)workspace % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_attn_repack_v_bf16: v must be 16-byte aligned, strides multiple of 8");
  SP_REQUIRE(workspace_bytes >= at_vt_bytes(n, hkv, d, bs), SP_ERR_WORKSPACE,
             "sp_attn_repack_v_bf16: workspace too small");
  const int64_t nb = sp_ceil_div(n, AT_BS);
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
  SP_REQUIRE(hq <= AT_MAX_HEADS, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: more than %d query heads",
             AT_MAX_HEADS);
  SP_REQUIRE(softmax_scale > 0.f, SP_ERR_INVALID_ARGUMENT, "sp_block_sparse_attn_fwd_bf16: softmax_scale must be > 0");
  SP_REQUIRE(at_block_size_ok(bs), SP_ERR_UNSUPPORTED,
             "sp_block_sparse_attn_fwd_bf16: block size %d unsupported (16, 32, 64 or 128)", bs);
  SP_REQUIRE(d == AT_D, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: head_dim %d unsupported (only 128)", d);
  SP_REQUIRE(q_stride_n % 8 == 0 && q_stride_h % 8 == 0 && k_stride_n % 8 == 0 && k_stride_h % 8 == 0 &&
                 ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)out % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: tensors must be 16-byte aligned, strides multiple of 8");
  SP_REQUIRE((int64_t)AT_BS * k_stride_n < (1ll << 31), SP_ERR_UNSUPPORTED,
             "sp_block_sparse_attn_fwd_bf16: key token stride %lld too large", (long long)k_stride_n);
  SP_REQUIRE(workspace_bytes >= sp_attn_workspace_bytes(n, hq, hkv, d, bs), SP_ERR_WORKSPACE,
             "sp_block_sparse_attn_fwd_bf16: workspace too small");
  // nb: 128-token blocks, what the kernels walk; nbf: blocks of the caller's size, what `mask` and `avg_attn` index
  const int64_t nb = sp_ceil_div(n, AT_BS), nbf = sp_ceil_div(n, bs);
  const bool fine = bs != AT_BS;
  const int fshift = at_fshift(bs);
  SP_REQUIRE(nbf <= 4096, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: %lld blocks of %d tokens exceed 4096",
             (long long)nbf, bs);
  SP_REQUIRE(nb * hq < (1ll << 31), SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: grid too large");
  SP_REQUIRE(nb <= AT_LIST_MAX, SP_ERR_UNSUPPORTED,
             "sp_block_sparse_attn_fwd_bf16: %lld key blocks exceed the supported %d (sequence too long)", (long long)nb,
             AT_LIST_MAX);
  if (!(flags & SP_ATTN_V_REPACKED)) {
    int rc = sp_attn_repack_v_bf16(v, n, hkv, d, v_stride_n, v_stride_h, bs, workspace, workspace_bytes, stream);
    if (rc != SP_OK) return rc;
  }
  const float scale_log2 = softmax_scale * 1.4426950408889634f;
  char* ws = (char*)workspace;
  int* counter = reinterpret_cast<int*>(ws + at_vt_bytes(n, hkv, d, bs));
  float2* rowstat = reinterpret_cast<float2*>(ws + at_vt_bytes(n, hkv, d, bs) + AT_SCHED_BYTES);
  const bool want_avg = decision != nullptr && avg_attn != nullptr;
  hipStream_t s = (hipStream_t)stream;
  const uint64_t* const fine_mask = mask;  // the caller's mask, at the caller's block size
  const int nbfw = (int)((nbf + 63) / 64);
  if (fine) {
    uint64_t* coarse = reinterpret_cast<uint64_t*>(ws + at_vt_bytes(n, hkv, d, bs) + AT_SCHED_BYTES +
                                                   (size_t)hq * (size_t)n * sizeof(float2));
    const int64_t words = (int64_t)hq * nb * ((nb + 63) / 64);
    hipLaunchKernelGGL(sp_attn_coarsen_kernel, dim3((unsigned)sp_ceil_div(words, 256)), dim3(256), 0, s, fine_mask,
                       coarse, (int)hq, (int)nb, (int)((nb + 63) / 64), (int)nbf, nbfw, fshift);
    SP_LAUNCH_CHECK();
    mask = coarse;  // from here on `mask` is the 128-block mask
  }
  // Workspace beyond the base size holds the block sums of pivot heads, one slab per pivot: those heads run in a
  // launch of their own that keeps the sums, and their block-average maps are made from them; pivots beyond the
  // slabs (or all of them, with a base-size workspace) take the recomputing pass.
  const size_t base_bytes = sp_attn_workspace_bytes(n, hq, hkv, d, bs);
  const size_t base_aligned = (base_bytes + 255) & ~(size_t)255;
  const size_t slab = sp_attn_pivot_scratch_bytes(n, bs);
  int max_pivots = 0;
  if (want_avg && workspace_bytes > base_aligned && !fine) {
    const size_t fit = (workspace_bytes - base_aligned) / slab;
    max_pivots = fit > (size_t)(AT_NO_SLOT - 1) ? AT_NO_SLOT - 1 : (int)fit;
  }
  float* pivot_u = reinterpret_cast<float*>(ws + base_aligned);
  hipLaunchKernelGGL(sp_attn_prep_kernel, dim3(1), dim3(128), 0, s, counter, decision, (int)hq, max_pivots);
  SP_LAUNCH_CHECK();
  if (!(flags & SP_ATTN_PAIR_ROWS)) {  // (otherwise the table stays as sp_attn_prep_kernel left it: rows paired)
    hipLaunchKernelGGL(sp_attn_pairing_kernel, dim3((unsigned)((hq + 1) / 2)), dim3(256), 0, s, counter, mask, (int)hq,
                       (int)(hq / hkv), (int)nb, (int)((nb + 63) / 64), max_pivots > 0 ? 1 : 0);
    SP_LAUNCH_CHECK();
    // few gangs per workgroup and every head's K / V^T within the memory-side cache: deal the gangs heaviest first
    // (measured on dense masks: +6 % at 16K tokens, +4 % at 32K; at 8K and below the ranking launch costs more
    // than the better tail is worth)
    const int64_t n_pairs = (nb + 1) / 2;
    const int64_t gang = n_pairs < AT_GANG ? n_pairs : AT_GANG;
    const int64_t n_gangs = hq * sp_ceil_div(n_pairs, gang);
    if (nb > 64 && nb <= 256 && n_gangs <= AT_ORDER_MAX) {
      hipLaunchKernelGGL(sp_attn_order_kernel, dim3(1), dim3(1024), 0, s, counter, mask, (int)hq, (int)hkv, (int)nb,
                         (int)((nb + 63) / 64));
      SP_LAUNCH_CHECK();
    }
  }
  const size_t lds_bytes = AT_LDS_BYTES;
  // per device, once: the kernels' LDS allowance and the CU count (idempotent, so a race between two host threads
  // at worst repeats it)
  static int cu_of_device[64] = {0};
  int dev = 0;
  SP_HIP(hipGetDevice(&dev));
  SP_REQUIRE(dev >= 0 && dev < 64, SP_ERR_UNSUPPORTED, "sp_block_sparse_attn_fwd_bf16: device index %d", dev);
  if (cu_of_device[dev] == 0) {
    hipDeviceProp_t prop;
    SP_HIP(hipGetDeviceProperties(&prop, dev));
    const void* fwd_kernels[5] = {(const void*)sp_attn_fwd_kernel<false, false>, (const void*)sp_attn_fwd_kernel<true, false>,
                                  (const void*)sp_attn_fwd_kernel<false, true>, (const void*)sp_attn_fwd_kernel<true, true>,
                                  (const void*)sp_attn_fwd_kernel<false, false, true>};
    for (const void* f : fwd_kernels)
      SP_HIP(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    cu_of_device[dev] = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  const int n_cu = cu_of_device[dev];
  const int64_t total = ((nb + 1) / 2) * hq;  // row pairs
  const int grid = (int)(total < (int64_t)n_cu ? ((total + 7) / 8) * 8 : (int64_t)n_cu);
  float2* stats = want_avg ? rowstat : (float2*)nullptr;
  const bool half = (flags & SP_ATTN_HALF_CHANNELS) != 0;
  auto launch_fwd = [&](auto kernel, int skip_slotted, float* block_sums) {
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(AT_FWD_THREADS), lds_bytes, s, (const sp_bf16*)q, (const sp_bf16*)k,
                       (const sp_bf16*)workspace, mask, decision, (sp_bf16*)out, stats, n, hq, hkv, q_stride_n,
                       q_stride_h, k_stride_n, k_stride_h, (int)nb, (int)((nb + 63) / 64), scale_log2, counter,
                       skip_slotted, block_sums, fine_mask, fshift, (int)nbf, nbfw);
  };
  if (fine)  // (one instance: a head_dim below 128 computes its zero channels here)
    launch_fwd(sp_attn_fwd_kernel<false, false, true>, 0, (float*)nullptr);
  else if (half)
    launch_fwd(sp_attn_fwd_kernel<false, true>, max_pivots > 0 ? 1 : 0, (float*)nullptr);
  else
    launch_fwd(sp_attn_fwd_kernel<false, false>, max_pivots > 0 ? 1 : 0, (float*)nullptr);
  SP_LAUNCH_CHECK();
  if (max_pivots > 0) {
    if (half)
      launch_fwd(sp_attn_fwd_kernel<true, true>, 0, pivot_u);
    else
      launch_fwd(sp_attn_fwd_kernel<true, false>, 0, pivot_u);
    SP_LAUNCH_CHECK();
  }
  if (want_avg && fine) {
    hipLaunchKernelGGL(sp_attn_avg_fine_kernel, dim3((unsigned)nb, hq), dim3(AT_THREADS), 0, s, (const sp_bf16*)q,
                       (const sp_bf16*)k, mask, fine_mask, decision, rowstat, avg_attn, n, hq, hkv, q_stride_n,
                       q_stride_h, k_stride_n, k_stride_h, (int)nb, (int)((nb + 63) / 64), (int)nbf, nbfw, fshift,
                       scale_log2);
    SP_LAUNCH_CHECK();
  } else if (want_avg) {
    hipLaunchKernelGGL(sp_attn_avg_kernel, dim3((unsigned)nb, hq), dim3(AT_THREADS), 0, s, (const sp_bf16*)q,
                       (const sp_bf16*)k, mask, decision, rowstat, avg_attn, n, hq, hkv, q_stride_n, q_stride_h,
                       k_stride_n, k_stride_h, (int)nb, (int)((nb + 63) / 64), scale_log2, (const int*)counter,
                       (const float*)pivot_u);
    SP_LAUNCH_CHECK();
  }
  return SP_OK;
}

// Block selection and cross-head pattern sharing on the device, with no host synchronisation.
// Replaces the torch-op chains of shareprefill/attn/attention_sharing.py:169-364 and :94-103 and the
// helpers of shareprefill/attn/utils.py:26-128.
//
// Canonical arithmetic shared with the CPU oracle:
//   * order = (value descending, index ascending), compared on the fp32 bit pattern (sp_sort_key);
//   * cumulative mass = exact integer sums of values truncated to 2^-48 fixed point (sp_to_fixed),
//     so every comparison against a threshold is independent of summation order (integer atomics
//     and scans may associate freely).
// Two primitives:
//   * radix mass descent for long vectors (per-token vectors of length N, the nb*nb pooled map):
//     three passes over the data building (count, mass) histograms over 11/11/10 key bits;
//   * rank sort for short vectors (rows of length nb): rank by pairwise comparison in LDS, scatter to
//     sorted order, integer prefix scan -- a literal sort / cumsum / threshold.
#include <cstring>

#include "sp_common.h"

#define SEL_THREADS 1024
#define SEL_BINS 2048

// ------------------------------------------------------------------------------------------------
// radix mass descent: shared state of the per-vector pick step (one workgroup of SEL_THREADS threads)
// ------------------------------------------------------------------------------------------------
struct SelShared {
  unsigned long long sum[SEL_BINS];
  uint32_t cnt[SEL_BINS];
  unsigned long long sum_above;
  uint32_t cnt_above;
  int32_t bin;
  uint32_t bin_cnt;
  unsigned long long bin_sum;
};

// suffix-inclusive scan of sh.sum over SEL_BINS bins (bin b <- sum of bins >= b), all SEL_THREADS threads.
// Thread t owns bins t and t + SEL_THREADS.  Inside a wave (64 consecutive bins of either half) the suffix sums come
// from lane shuffles; the waves' totals meet in LDS.  Integer sums: any association gives the same result.
__device__ static void sel_suffix_scan(SelShared& sh) {
  __shared__ unsigned long long wave_tot[2][SEL_THREADS / SP_WAVE];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  unsigned long long v0 = sh.sum[t], v1 = sh.sum[t + SEL_THREADS];
#pragma unroll
  for (int off = 1; off < SP_WAVE; off <<= 1) {
    const unsigned long long a0 = __shfl_down(v0, off, SP_WAVE), a1 = __shfl_down(v1, off, SP_WAVE);
    if (lane + off < SP_WAVE) {
      v0 += a0;
      v1 += a1;
    }
  }
  if (lane == 0) {
    wave_tot[0][wave] = v0;
    wave_tot[1][wave] = v1;
  }
  __syncthreads();
  unsigned long long above0 = 0, above1 = 0;  // bins of the same half in higher waves
#pragma unroll
  for (int w = 0; w < SEL_THREADS / SP_WAVE; ++w) {
    if (w > wave) {
      above0 += wave_tot[0][w];
      above1 += wave_tot[1][w];
    }
    above0 += wave_tot[1][w];  // the whole upper half lies above every bin of the lower half
  }
  sh.sum[t] = v0 + above0;
  sh.sum[t + SEL_THREADS] = v1 + above1;
  __syncthreads();
}

// ---- score_cover_idx (attn/utils.py:53-57) on [nb][nb] maps, written into bit masks -----------------
// Multi-workgroup radix mass descent over the LOWER TRIANGLE of each map (entries above the diagonal are
// exactly zero in the reference's maps and cannot be selected; they are ignored here).  Per level: many
// workgroups per vector build LDS histograms of their rows and merge them into a global (count, mass)
// histogram with integer atomics; one workgroup per vector then picks the bin in which the running mass
// crosses the budget.  A row-parallel kernel writes the mask bits.  Only when the boundary falls inside a
// group of equal values that is taken partially (lowest indices first) a sequential kernel ranks them.
#define GSEL_SPLIT 64     // workgroups per vector in the histogram / emit kernels
#define GSEL_THREADS 256

struct GselState {
  unsigned long long rem;   // budget left after the bins / groups above the current prefix
  uint32_t prefix;          // key bits fixed so far
  uint32_t above;           // elements with key above the cut
  uint32_t n_equal, n_take; // boundary group
  int32_t all;              // 1: the whole vector is kept
  int32_t enabled;
  uint32_t pad[8];
};

__device__ static inline bool gsel_enabled(const int32_t* enable, int enable_match, int v) {
  if (!enable) return true;
  const int e = enable[v];
  return enable_match < 0 ? (e != 0) : (e == enable_match);
}

__global__ void sp_gsel_init_kernel(GselState* st, uint32_t* cnt, unsigned long long* sum, const int32_t* enable,
                                    int enable_match, int n_vec, long long t_le, uint64_t* mask, int nb, int nbw) {
  const int v = blockIdx.x;
  for (int i = threadIdx.x; i < SEL_BINS; i += blockDim.x) {
    cnt[(int64_t)v * SEL_BINS + i] = 0;
    sum[(int64_t)v * SEL_BINS + i] = 0;
  }
  if (threadIdx.x == 0) {
    GselState s;
    s.rem = t_le < 0 ? 0ull : (unsigned long long)t_le;
    s.prefix = 0;
    s.above = 0;
    s.n_equal = 0;
    s.n_take = 0;
    s.all = 0;
    s.enabled = (gsel_enabled(enable, enable_match, v) && t_le >= 0) ? 1 : 0;
    for (int i = 0; i < 8; ++i) s.pad[i] = 0;
    st[v] = s;
    if (mask != nullptr && gsel_enabled(enable, enable_match, v))  // block (0,0): the padding id of the reference
      atomicOr(reinterpret_cast<uint32_t*>(mask + (int64_t)v * nb * nbw), 1u);
  }
}

template <int LEVEL>
__global__ __launch_bounds__(GSEL_THREADS) void sp_gsel_hist_kernel(const float* __restrict__ x, int nb,
                                                                    const GselState* __restrict__ st,
                                                                    uint32_t* __restrict__ gcnt,
                                                                    unsigned long long* __restrict__ gsum) {
  __shared__ unsigned long long lsum[SEL_BINS];
  __shared__ uint32_t lcnt[SEL_BINS];
  const int v = blockIdx.y;
  const GselState s = st[v];
  if (!s.enabled || s.all) return;
  constexpr int shift = LEVEL == 0 ? 21 : (LEVEL == 1 ? 10 : 0);
  constexpr int width = LEVEL == 2 ? 10 : 11;
  constexpr int pshift = LEVEL == 0 ? 32 : (LEVEL == 1 ? 21 : 10);
  for (int i = threadIdx.x; i < SEL_BINS; i += GSEL_THREADS) {
    lsum[i] = 0;
    lcnt[i] = 0;
  }
  __syncthreads();
  const float* xv = x + (int64_t)v * nb * nb;
  for (int r = blockIdx.x; r < nb; r += GSEL_SPLIT) {
    const float* row = xv + (int64_t)r * nb;
    for (int c = threadIdx.x; c <= r; c += GSEL_THREADS) {
      const float val = row[c];
      const uint32_t key = sp_sort_key(val);
      if (pshift < 32 && (key >> (pshift & 31)) != s.prefix) continue;
      const uint32_t b = (key >> shift) & ((1u << width) - 1u);
      atomicAdd(&lcnt[b], 1u);
      const unsigned long long fx = sp_to_fixed(val);
      if (fx) atomicAdd(&lsum[b], fx);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < (1 << width); i += GSEL_THREADS) {
    if (lcnt[i]) atomicAdd(&gcnt[(int64_t)v * SEL_BINS + i], lcnt[i]);
    if (lsum[i]) atomicAdd(&gsum[(int64_t)v * SEL_BINS + i], lsum[i]);
  }
}

// One level of the descent on a histogram that sits in sh.sum / sh.cnt: finds the bin in which the running mass
// (from the top bin down) first exceeds the budget left, and moves the state below it.  Called by all SEL_THREADS
// threads of a workgroup with the same `s`; every thread returns with the same updated `s`.  sh may be refilled
// afterwards (the function ends with a barrier).
template <int LEVEL>
__device__ static void sel_pick_level(SelShared& sh, GselState& s) {
  const int t = threadIdx.x;
  constexpr int width = LEVEL == 2 ? 10 : 11;
  const int nbins = 1 << width;
  if (t == 0) {
    sh.bin = -1;
    sh.cnt_above = 0;
  }
  __syncthreads();
  const unsigned long long own0 = sh.sum[t], own1 = sh.sum[t + SEL_THREADS];
  __syncthreads();
  sel_suffix_scan(sh);
#pragma unroll
  for (int rep = 0; rep < 2; ++rep) {
    const int b = t + rep * SEL_THREADS;
    if (b < nbins) {
      const unsigned long long incl = sh.sum[b];
      const unsigned long long excl = (b + 1 < SEL_BINS) ? sh.sum[b + 1] : 0ull;
      if (incl > s.rem && excl <= s.rem) {
        sh.bin = b;
        sh.sum_above = excl;
        sh.bin_sum = rep ? own1 : own0;
        sh.bin_cnt = sh.cnt[b];
      }
    }
  }
  __syncthreads();
  const int bin = sh.bin;
  if (bin < 0) {  // the running mass never exceeds the budget (top level only): keep everything
    s.all = 1;
    __syncthreads();
    return;
  }
  uint32_t c = 0;
#pragma unroll
  for (int rep = 0; rep < 2; ++rep) {
    const int b = t + rep * SEL_THREADS;
    if (b < nbins && b > bin) c += sh.cnt[b];
  }
  if (c) atomicAdd(&sh.cnt_above, c);
  __syncthreads();
  s.prefix = (s.prefix << width) | (uint32_t)bin;
  s.above += sh.cnt_above;
  s.rem -= sh.sum_above;
  if (LEVEL == 2) {
    s.n_equal = sh.bin_cnt;
    const unsigned long long each = sh.bin_sum / (sh.bin_cnt ? sh.bin_cnt : 1u);
    unsigned long long take = each ? s.rem / each : (unsigned long long)s.n_equal;
    if (take > s.n_equal) take = s.n_equal;
    s.n_take = (uint32_t)take;
  }
  __syncthreads();
}

template <int LEVEL>
__global__ __launch_bounds__(SEL_THREADS) void sp_gsel_pick_kernel(GselState* __restrict__ st,
                                                                   uint32_t* __restrict__ gcnt,
                                                                   unsigned long long* __restrict__ gsum) {
  __shared__ SelShared sh;
  const int v = blockIdx.x, t = threadIdx.x;
  GselState s = st[v];
  if (!s.enabled || s.all) return;
  uint32_t* gc = gcnt + (int64_t)v * SEL_BINS;
  unsigned long long* gs = gsum + (int64_t)v * SEL_BINS;
  sh.sum[t] = gs[t];
  sh.sum[t + SEL_THREADS] = gs[t + SEL_THREADS];
  sh.cnt[t] = gc[t];
  sh.cnt[t + SEL_THREADS] = gc[t + SEL_THREADS];
  gs[t] = 0;  // ready for the next level
  gs[t + SEL_THREADS] = 0;
  gc[t] = 0;
  gc[t + SEL_THREADS] = 0;
  sel_pick_level<LEVEL>(sh, s);
  if (t == 0) st[v] = s;
}

// ---- the same descent by ONE workgroup per vector, histograms in LDS only -------------------------------------------
// For short vectors (a few thousand to 16 K entries) the multi-workgroup descent is nothing but launch latency: ten
// launches whose kernels run a few microseconds each.  Here one workgroup of SEL_THREADS threads makes the three
// passes over its vector itself; the arithmetic (keys, fixed-point masses, pick rule, tie rule) is the very same
// code, so both paths select the same entries.
__device__ static inline GselState sel_fresh_state(long long t_le, bool enabled) {
  GselState s;
  s.rem = t_le < 0 ? 0ull : (unsigned long long)t_le;
  s.prefix = 0;
  s.above = 0;
  s.n_equal = 0;
  s.n_take = 0;
  s.all = 0;
  s.enabled = (enabled && t_le >= 0) ? 1 : 0;
  for (int i = 0; i < 8; ++i) s.pad[i] = 0;
  return s;
}

template <int LEVEL>
__device__ static inline void sel_hist_add(SelShared& sh, const GselState& s, float val) {
  constexpr int shift = LEVEL == 0 ? 21 : (LEVEL == 1 ? 10 : 0);
  constexpr int width = LEVEL == 2 ? 10 : 11;
  constexpr int pshift = LEVEL == 0 ? 32 : (LEVEL == 1 ? 21 : 10);
  const uint32_t key = sp_sort_key(val);
  if (pshift < 32 && (key >> (pshift & 31)) != s.prefix) return;
  const uint32_t b = (key >> shift) & ((1u << width) - 1u);
  atomicAdd(&sh.cnt[b], 1u);
  const unsigned long long fx = sp_to_fixed(val);
  if (fx) atomicAdd(&sh.sum[b], fx);
}

__device__ static inline void sel_hist_clear(SelShared& sh) {
  sh.sum[threadIdx.x] = 0;
  sh.sum[threadIdx.x + SEL_THREADS] = 0;
  sh.cnt[threadIdx.x] = 0;
  sh.cnt[threadIdx.x + SEL_THREADS] = 0;
  __syncthreads();
}

// flat vectors (score_cover_topk, the budgets): vectors 0..n0-1 are rows of x0, the others rows of x1
#define GSEL_SMALL_LEN 16384
template <int LEVEL>
__device__ static inline void sel_flat_level(SelShared& sh, GselState& s, const float* __restrict__ xv, int len) {
  sel_hist_clear(sh);
  for (int i = threadIdx.x; i < len; i += SEL_THREADS) sel_hist_add<LEVEL>(sh, s, xv[i]);
  __syncthreads();
  sel_pick_level<LEVEL>(sh, s);
}

__global__ __launch_bounds__(SEL_THREADS) void sp_gsel_count_small_kernel(
    const float* __restrict__ x0, const float* __restrict__ x1, int n0, int len, long long t_le,
    int32_t* __restrict__ out0, int32_t* __restrict__ out1, int bs, int minb, int maxb) {
  __shared__ SelShared sh;
  const int v = blockIdx.x;
  const float* xv = v < n0 ? x0 + (int64_t)v * len : x1 + (int64_t)(v - n0) * len;
  GselState s = sel_fresh_state(t_le, true);
  if (s.enabled) {
    sel_flat_level<0>(sh, s, xv, len);
    if (!s.all) sel_flat_level<1>(sh, s, xv, len);
    if (!s.all) sel_flat_level<2>(sh, s, xv, len);
  }
  if (threadIdx.x == 0) {  // as sp_gsel_count_kernel
    long long m = 0;
    if (t_le >= 0) m = s.all ? (long long)len : (long long)s.above + s.n_take;
    long long r = m + 1;
    if (bs > 0) {
      r = r / bs + 1;
      if (r < minb) r = minb;
      if (r > maxb) r = maxb;
    }
    if (v < n0)
      out0[v] = (int32_t)r;
    else
      out1[v - n0] = (int32_t)r;
  }
}

// lower triangle of an [nb][nb] map (score_cover_idx), nb <= GSEL_SMALL_NB: wave w of the 16 owns rows w, w+16, ...
#define GSEL_SMALL_NB 128
template <int LEVEL>
__device__ static inline void sel_tri_level(SelShared& sh, GselState& s, const float* __restrict__ xv, int nb) {
  sel_hist_clear(sh);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int r = wave; r < nb; r += SEL_THREADS / SP_WAVE)
    for (int c = lane; c <= r; c += SP_WAVE) sel_hist_add<LEVEL>(sh, s, xv[(int64_t)r * nb + c]);
  __syncthreads();
  sel_pick_level<LEVEL>(sh, s);
}

__global__ __launch_bounds__(SEL_THREADS) void sp_gsel_small_kernel(const float* __restrict__ x,
                                                                    const int32_t* __restrict__ enable,
                                                                    int enable_match, int nb, int nbw, long long t_le,
                                                                    uint64_t* __restrict__ mask) {
  __shared__ SelShared sh;
  __shared__ uint32_t row_ties[GSEL_SMALL_NB];
  const int v = blockIdx.x;
  if (!gsel_enabled(enable, enable_match, v)) return;
  const float* xv = x + (int64_t)v * nb * nb;
  uint64_t* mv = mask + (int64_t)v * nb * nbw;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  GselState s = sel_fresh_state(t_le, true);
  if (s.enabled) {
    sel_tri_level<0>(sh, s, xv, nb);
    if (!s.all) sel_tri_level<1>(sh, s, xv, nb);
    if (!s.all) sel_tri_level<2>(sh, s, xv, nb);
  }
  // the boundary group of equal values is taken partially: its n_take lowest indices (row-major) win
  const bool ranked = s.enabled && !s.all && s.n_take != 0 && s.n_take < s.n_equal;
  const bool take_all_equal = s.all || s.n_take >= s.n_equal;
  if (ranked) {
    for (int r = wave; r < nb; r += SEL_THREADS / SP_WAVE) {
      uint32_t cnt = 0;
      for (int c0 = 0; c0 <= r; c0 += SP_WAVE) {
        const int c = c0 + lane;
        cnt += __popcll(__ballot(c <= r && sp_sort_key(xv[(int64_t)r * nb + c]) == s.prefix));
      }
      if (lane == 0) row_ties[r] = cnt;
    }
    __syncthreads();
  }
  for (int r = wave; r < nb; r += SEL_THREADS / SP_WAVE) {
    uint32_t before = 0;  // members of the boundary group in rows above this one (uniform per wave)
    if (ranked)
      for (int i = 0; i < r; ++i) before += row_ties[i];
    for (int c0 = 0; c0 <= r; c0 += SP_WAVE) {
      const int c = c0 + lane;
      bool sel = false, eq = false;
      if (s.enabled && c <= r) {
        const uint32_t key = sp_sort_key(xv[(int64_t)r * nb + c]);
        eq = key == s.prefix;
        sel = s.all || key > s.prefix || (eq && take_all_equal);
      }
      if (ranked) {
        const unsigned long long eqb = __ballot(eq);
        if (eq && before + (uint32_t)__popcll(eqb & ((1ull << lane) - 1ull)) < s.n_take) sel = true;
        before += (uint32_t)__popcll(eqb);
      }
      unsigned long long bal = __ballot(sel);
      if (r == 0 && c0 == 0) bal |= 1ull;  // block (0,0): the padding id of the reference
      // this wave alone writes the words of its rows (the kernels that wrote the mask before have finished)
      if (lane == 0 && bal) mv[(int64_t)r * nbw + (c0 >> 6)] |= bal;
    }
  }
}

__global__ __launch_bounds__(GSEL_THREADS) void sp_gsel_emit_kernel(const float* __restrict__ x, int nb, int nbw,
                                                                    const GselState* __restrict__ st,
                                                                    uint64_t* __restrict__ mask) {
  const int v = blockIdx.y;
  const GselState s = st[v];
  if (!s.enabled) return;
  const bool take_all_equal = s.all || s.n_take >= s.n_equal;
  const float* xv = x + (int64_t)v * nb * nb;
  uint64_t* mv = mask + (int64_t)v * nb * nbw;
  for (int r = blockIdx.x; r < nb; r += GSEL_SPLIT) {
    const float* row = xv + (int64_t)r * nb;
    for (int c0 = 0; c0 <= r; c0 += GSEL_THREADS) {  // uniform trip count per workgroup: every lane votes
      const int c = c0 + threadIdx.x;
      bool sel = false;
      if (c <= r) {
        const uint32_t key = sp_sort_key(row[c]);
        sel = s.all || key > s.prefix || (key == s.prefix && take_all_equal);
      }
      const unsigned long long bal = __ballot(sel);
      if ((threadIdx.x & 63) == 0 && bal)
        atomicOr(reinterpret_cast<unsigned long long*>(mv) + (int64_t)r * nbw + (c >> 6), bal);
    }
  }
}

// Boundary group taken partially: the n_take lowest indices (row-major) of the equal-valued entries win.  The
// rows are cut into GSEL_SPLIT contiguous segments: a first kernel counts each segment's members of the group, the
// second gives every segment the count of the segments before it and ranks inside the segment only.
__device__ static inline void gsel_segment(int nb, int seg, int& r_lo, int& r_hi) {
  const int per = (nb + GSEL_SPLIT - 1) / GSEL_SPLIT;
  r_lo = seg * per < nb ? seg * per : nb;
  r_hi = r_lo + per < nb ? r_lo + per : nb;
}

__device__ static inline bool gsel_ranked_needed(const GselState& s) {
  return s.enabled && !s.all && s.n_take != 0 && s.n_take < s.n_equal;
}

__global__ __launch_bounds__(GSEL_THREADS) void sp_gsel_tie_count_kernel(const float* __restrict__ x, int nb,
                                                                         const GselState* __restrict__ st,
                                                                         uint32_t* __restrict__ tie_cnt) {
  __shared__ uint32_t total;
  const int v = blockIdx.y, seg = blockIdx.x;
  const GselState s = st[v];
  if (!gsel_ranked_needed(s)) return;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  int r_lo, r_hi;
  gsel_segment(nb, seg, r_lo, r_hi);
  const float* xv = x + (int64_t)v * nb * nb;
  uint32_t mine = 0;
  for (int r = r_lo; r < r_hi; ++r)
    for (int c = threadIdx.x; c <= r; c += GSEL_THREADS) mine += sp_sort_key(xv[(int64_t)r * nb + c]) == s.prefix;
  if (mine) atomicAdd(&total, mine);
  __syncthreads();
  if (threadIdx.x == 0) tie_cnt[(int64_t)v * SEL_BINS + seg] = total;
}

__global__ __launch_bounds__(GSEL_THREADS) void sp_gsel_emit_ranked_kernel(const float* __restrict__ x, int nb, int nbw,
                                                                           const GselState* __restrict__ st,
                                                                           const uint32_t* __restrict__ tie_cnt,
                                                                           uint64_t* __restrict__ mask) {
  __shared__ uint32_t wave_cnt[GSEL_THREADS / SP_WAVE];
  const int v = blockIdx.y, seg = blockIdx.x;
  const GselState s = st[v];
  if (!gsel_ranked_needed(s)) return;
  uint32_t running = 0;  // members of the group in front of the current chunk (uniform)
  for (int i = 0; i < seg; ++i) running += tie_cnt[(int64_t)v * SEL_BINS + i];
  if (running >= s.n_take) return;
  int r_lo, r_hi;
  gsel_segment(nb, seg, r_lo, r_hi);
  const float* xv = x + (int64_t)v * nb * nb;
  uint32_t* mv = reinterpret_cast<uint32_t*>(mask + (int64_t)v * nb * nbw);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int r = r_lo; r < r_hi; ++r) {
    for (int c0 = 0; c0 <= r; c0 += GSEL_THREADS) {  // uniform trip count: every lane votes
      const int c = c0 + threadIdx.x;
      const bool eq = c <= r && sp_sort_key(xv[(int64_t)r * nb + c]) == s.prefix;
      const unsigned long long bal = __ballot(eq);
      const uint32_t before = __popcll(bal & ((1ull << lane) - 1ull));
      __syncthreads();  // the previous chunk's counts have been read
      if (lane == 0) wave_cnt[wave] = __popcll(bal);
      __syncthreads();
      uint32_t off = running, tot = 0;
#pragma unroll
      for (int w = 0; w < GSEL_THREADS / SP_WAVE; ++w) {
        if (w < wave) off += wave_cnt[w];
        tot += wave_cnt[w];
      }
      if (eq && off + before < s.n_take)
        atomicOr(&mv[((int64_t)r * nbw + (c >> 6)) * 2 + ((c >> 5) & 1)], 1u << (c & 31));
      running += tot;
      if (running >= s.n_take) return;  // uniform
    }
  }
}

// ---- score_cover_topk (attn/utils.py:47-50) on flat vectors: the same descent, the count instead of the set ----
// (its own launch shape: a flat vector is cut into FLAT_SPLIT strided shares of FLAT_THREADS-wide rows; few fat workgroups,
// all resident at once, instead of 64 x 256 threads: every workgroup pays for clearing and flushing 2048 bins)
#define FLAT_SPLIT 16
#define FLAT_THREADS 1024
template <int LEVEL>
__global__ __launch_bounds__(FLAT_THREADS) void sp_gsel_hist_flat_kernel(const float* __restrict__ x0,
                                                                         const float* __restrict__ x1, int n0,
                                                                         int64_t len,
                                                                         const GselState* __restrict__ st,
                                                                         uint32_t* __restrict__ gcnt,
                                                                         unsigned long long* __restrict__ gsum) {
  __shared__ unsigned long long lsum[SEL_BINS];
  __shared__ uint32_t lcnt[SEL_BINS];
  const int v = blockIdx.y;
  const GselState s = st[v];
  if (!s.enabled || s.all) return;
  constexpr int shift = LEVEL == 0 ? 21 : (LEVEL == 1 ? 10 : 0);
  constexpr int width = LEVEL == 2 ? 10 : 11;
  constexpr int pshift = LEVEL == 0 ? 32 : (LEVEL == 1 ? 21 : 10);
  for (int i = threadIdx.x; i < SEL_BINS; i += FLAT_THREADS) {
    lsum[i] = 0;
    lcnt[i] = 0;
  }
  __syncthreads();
  const float* xv = v < n0 ? x0 + (int64_t)v * len : x1 + (int64_t)(v - n0) * len;  // vectors n0.. live in x1
  for (int64_t i0 = (int64_t)blockIdx.x * FLAT_THREADS; i0 < len; i0 += (int64_t)FLAT_SPLIT * FLAT_THREADS) {
    const int64_t i = i0 + threadIdx.x;
    bool live = i < len;
    uint32_t b = 0;
    unsigned long long fx = 0;
    if (live) {
      const float val = xv[i];
      const uint32_t key = sp_sort_key(val);
      live = !(pshift < 32 && (key >> (pshift & 31)) != s.prefix);
      b = (key >> shift) & ((1u << width) - 1u);
      fx = sp_to_fixed(val);
    }
    if (live) {
      atomicAdd(&lcnt[b], 1u);
      if (fx) atomicAdd(&lsum[b], fx);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < (1 << width); i += FLAT_THREADS) {
    if (lcnt[i]) atomicAdd(&gcnt[(int64_t)v * SEL_BINS + i], lcnt[i]);
    if (lsum[i]) atomicAdd(&gsum[(int64_t)v * SEL_BINS + i], lsum[i]);
  }
}

__global__ void sp_gsel_count_kernel(const GselState* __restrict__ st, int n_vec, long long t_le, int64_t len,
                                     int32_t* __restrict__ out0, int32_t* __restrict__ out1, int n0, int bs,
                                     int minb, int maxb) {
  const int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= n_vec) return;
  const GselState s = st[v];
  long long m = 0;
  if (t_le >= 0) m = s.all ? (long long)len : (long long)s.above + s.n_take;
  long long r = m + 1;
  if (bs > 0) {  // budgets: tokens // bs + 1, clamped (attention_sharing.py:169-176)
    r = r / bs + 1;
    if (r < minb) r = minb;
    if (r > maxb) r = maxb;
  }
  if (v < n0)
    out0[v] = (int32_t)r;
  else
    out1[v - n0] = (int32_t)r;
}

static int gsel_count_run(const float* x0, const float* x1, int n0, int n_vec, int64_t len, float thr, int32_t* out0,
                          int32_t* out1, int bs, int minb, int maxb, void* workspace, size_t workspace_bytes,
                          hipStream_t s, const char* who);

extern "C" size_t sp_cover_select_workspace_bytes(int32_t n_vec) {
  if (n_vec <= 0) return 0;
  return (size_t)n_vec * (sizeof(GselState) + SEL_BINS * (sizeof(uint32_t) + sizeof(unsigned long long)));
}

static int gsel_run(const float* x, const int32_t* enable, int enable_match, int n_vec, int nb, float score,
                    uint64_t* mask, void* workspace, size_t workspace_bytes, hipStream_t s, const char* who) {
  SP_REQUIRE(workspace && workspace_bytes >= sp_cover_select_workspace_bytes(n_vec) && ((uintptr_t)workspace % 8) == 0,
             SP_ERR_WORKSPACE, "%s: workspace missing, misaligned or too small", who);
  const int nbw = (nb + 63) / 64;
  if (nb <= GSEL_SMALL_NB) {  // one workgroup per map does the whole descent and writes the bits
    hipLaunchKernelGGL(sp_gsel_small_kernel, dim3(n_vec), dim3(SEL_THREADS), 0, s, x, enable, enable_match, nb, nbw,
                       (long long)sp_thr_le(score), mask);
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  GselState* st = reinterpret_cast<GselState*>(workspace);
  unsigned long long* gsum = reinterpret_cast<unsigned long long*>(st + n_vec);
  uint32_t* gcnt = reinterpret_cast<uint32_t*>(gsum + (size_t)n_vec * SEL_BINS);
  hipLaunchKernelGGL(sp_gsel_init_kernel, dim3(n_vec), dim3(256), 0, s, st, gcnt, gsum, enable, enable_match, n_vec,
                     (long long)sp_thr_le(score), mask, nb, nbw);
  SP_LAUNCH_CHECK();
  const dim3 hgrid(GSEL_SPLIT, n_vec);
  hipLaunchKernelGGL(sp_gsel_hist_kernel<0>, hgrid, dim3(GSEL_THREADS), 0, s, x, nb, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_pick_kernel<0>, dim3(n_vec), dim3(SEL_THREADS), 0, s, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_hist_kernel<1>, hgrid, dim3(GSEL_THREADS), 0, s, x, nb, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_pick_kernel<1>, dim3(n_vec), dim3(SEL_THREADS), 0, s, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_hist_kernel<2>, hgrid, dim3(GSEL_THREADS), 0, s, x, nb, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_pick_kernel<2>, dim3(n_vec), dim3(SEL_THREADS), 0, s, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_emit_kernel, hgrid, dim3(GSEL_THREADS), 0, s, x, nb, nbw, st, mask);
  // (the histogram counters are free after the last pick: the segments' tie counts go there)
  hipLaunchKernelGGL(sp_gsel_tie_count_kernel, hgrid, dim3(GSEL_THREADS), 0, s, x, nb, st, gcnt);
  hipLaunchKernelGGL(sp_gsel_emit_ranked_kernel, hgrid, dim3(GSEL_THREADS), 0, s, x, nb, nbw, st,
                     (const uint32_t*)gcnt, mask);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// vectors 0..n0-1 are rows of x0 (results to out0), vectors n0..n_vec-1 rows of x1 (results to out1)
static int gsel_count_run(const float* x0, const float* x1, int n0, int n_vec, int64_t len, float thr, int32_t* out0,
                          int32_t* out1, int bs, int minb, int maxb, void* workspace, size_t workspace_bytes,
                          hipStream_t s, const char* who) {
  SP_REQUIRE(workspace && workspace_bytes >= sp_cover_select_workspace_bytes(n_vec) && ((uintptr_t)workspace % 8) == 0,
             SP_ERR_WORKSPACE, "%s: workspace missing, misaligned or too small", who);
  GselState* st = reinterpret_cast<GselState*>(workspace);
  unsigned long long* gsum = reinterpret_cast<unsigned long long*>(st + n_vec);
  uint32_t* gcnt = reinterpret_cast<uint32_t*>(gsum + (size_t)n_vec * SEL_BINS);
  const long long t_le = (long long)sp_thr_le(thr);
  if (len <= GSEL_SMALL_LEN) {  // one workgroup per vector, one launch
    hipLaunchKernelGGL(sp_gsel_count_small_kernel, dim3(n_vec), dim3(SEL_THREADS), 0, s, x0, x1, n0, (int)len, t_le, out0,
                       out1, bs, minb, maxb);
    SP_LAUNCH_CHECK();
    return SP_OK;
  }
  hipLaunchKernelGGL(sp_gsel_init_kernel, dim3(n_vec), dim3(256), 0, s, st, gcnt, gsum, (const int32_t*)nullptr, -1,
                     n_vec, t_le, (uint64_t*)nullptr, 0, 0);
  SP_LAUNCH_CHECK();
  const dim3 hgrid(FLAT_SPLIT, n_vec);
  hipLaunchKernelGGL(sp_gsel_hist_flat_kernel<0>, hgrid, dim3(FLAT_THREADS), 0, s, x0, x1, n0, len, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_pick_kernel<0>, dim3(n_vec), dim3(SEL_THREADS), 0, s, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_hist_flat_kernel<1>, hgrid, dim3(FLAT_THREADS), 0, s, x0, x1, n0, len, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_pick_kernel<1>, dim3(n_vec), dim3(SEL_THREADS), 0, s, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_hist_flat_kernel<2>, hgrid, dim3(FLAT_THREADS), 0, s, x0, x1, n0, len, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_pick_kernel<2>, dim3(n_vec), dim3(SEL_THREADS), 0, s, st, gcnt, gsum);
  hipLaunchKernelGGL(sp_gsel_count_kernel, dim3((n_vec + 63) / 64), dim3(64), 0, s, st, n_vec, t_le, len, out0, out1, n0,
                     bs, minb, maxb);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

extern "C" int sp_cover_count(const float* x, int32_t n_vec, int64_t len, float thr, int32_t* out, void* workspace,
                              size_t workspace_bytes, sp_stream_t stream) {
  SP_REQUIRE(x && out && n_vec > 0 && len > 0, SP_ERR_INVALID_ARGUMENT, "sp_cover_count: bad arguments");
  return gsel_count_run(x, x, n_vec, n_vec, len, thr, out, out, 0, 0, 0, workspace, workspace_bytes,
                        (hipStream_t)stream, "sp_cover_count");
}

// both vectors of every head in one descent: 2*hq vectors
extern "C" int sp_cover_budgets(const float* vert_tok, const float* slash_tok, int32_t hq, int64_t n, int32_t bs,
                                float pattern_threshold, int32_t min_blocks, int32_t max_blocks, int32_t* nv,
                                int32_t* ns, void* workspace, size_t workspace_bytes, sp_stream_t stream) {
  SP_REQUIRE(vert_tok && slash_tok && nv && ns && hq > 0 && n > 0 && bs > 0, SP_ERR_INVALID_ARGUMENT,
             "sp_cover_budgets: bad arguments");
  return gsel_count_run(vert_tok, slash_tok, hq, 2 * hq, n, pattern_threshold, nv, ns, bs, min_blocks, max_blocks,
                        workspace, workspace_bytes, (hipStream_t)stream, "sp_cover_budgets");
}

extern "C" int sp_cover_select_global(const float* x, const int32_t* enable, int32_t n_vec, int32_t nb, float score,
                                      uint64_t* mask, void* workspace, size_t workspace_bytes, sp_stream_t stream) {
  SP_REQUIRE(x && mask && n_vec > 0 && nb > 0, SP_ERR_INVALID_ARGUMENT, "sp_cover_select_global: bad arguments");
  return gsel_run(x, enable, -1, n_vec, nb, score, mask, workspace, workspace_bytes, (hipStream_t)stream,
                  "sp_cover_select_global");
}

// ------------------------------------------------------------------------------------------------
// rank sort for short vectors (length <= RS_MAX), one workgroup of RS_THREADS threads
// ------------------------------------------------------------------------------------------------
#define RS_THREADS 256
#define RS_MAX 4096

// ---- score_cover_idx_each_row (attn/utils.py:60-76) -------------------------------------------------
// keep[r] = first (count(cumsum < thr) + 1) entries of the sorted row, or exactly one if thr is never reached
// Views into the kernel's dynamic LDS, carved for rows of n entries (rs_lds_bytes(n) bytes: 14 KiB at nb = 1024
// instead of the 58 KiB a layout for the longest supported row takes, i.e. eight workgroups per CU instead of two).
struct RowShared {
  uint32_t* keys;                 // [n4], 16-byte aligned
  uint16_t* rank;                 // [n4]
  unsigned long long* sorted_fx;  // [n4]
  unsigned long long* chunk_sum;  // [RS_THREADS]
  uint32_t* below;
  int* n_eff;
};
__host__ __device__ static inline size_t rs_lds_bytes(int n) {
  const size_t n4 = (size_t)((n + 3) & ~3);
  return n4 * 8 + RS_THREADS * 8 + n4 * 4 + n4 * 2 + 16;
}
__device__ static inline RowShared rs_carve(char* base, int n) {
  const size_t n4 = (size_t)((n + 3) & ~3);
  RowShared sh;
  sh.sorted_fx = reinterpret_cast<unsigned long long*>(base);
  sh.chunk_sum = sh.sorted_fx + n4;
  sh.keys = reinterpret_cast<uint32_t*>(sh.chunk_sum + RS_THREADS);
  sh.rank = reinterpret_cast<uint16_t*>(sh.keys + n4);
  sh.below = reinterpret_cast<uint32_t*>(base + n4 * 8 + RS_THREADS * 8 + n4 * 4 + n4 * 2);
  sh.n_eff = reinterpret_cast<int*>(sh.below + 1);
  return sh;
}

// rank[i] for i < m among keys[0 .. m-1], four keys per LDS read; keys[m .. (m + 3) & ~3) must be zero
__device__ static void rs_ranks4(const uint32_t* keys, int m, uint16_t* rank) {
  const int m4 = (m + 3) & ~3;
  for (int i = threadIdx.x; i < m; i += RS_THREADS) {
    const uint32_t ki = keys[i];
    int r = 0;
    for (int j = 0; j < m4; j += 4) {
      const uint4 kj = *reinterpret_cast<const uint4*>(keys + j);
      r += (kj.x > ki) || (kj.x == ki && j < i);
      r += (kj.y > ki) || (kj.y == ki && j + 1 < i);
      r += (kj.z > ki) || (kj.z == ki && j + 2 < i);
      r += (kj.w > ki) || (kj.w == ki && j + 3 < i);
    }
    rank[i] = (uint16_t)r;
  }
}

// Only the row's entries up to its last non-zero key take part in the sort: the zero keys behind it sort last in
// index order whatever stands before them (rank[i] = i), add nothing to any cumulative mass and cannot be the
// crossing entry, so ranks, count and the "never reached -> keep one" rule come out as over the whole row.  Row r of
// a pivot's block-average map ends at column r: a third of the comparisons of the full square on average.
__device__ static int rs_row_keep(const float* __restrict__ row, int n, long long t_lt, const RowShared& sh) {
  if (threadIdx.x == 0) {
    *sh.below = 0;
    *sh.n_eff = 0;
  }
  __syncthreads();
  int last = 0;
  for (int i = threadIdx.x; i < n; i += RS_THREADS) {
    const uint32_t key = sp_sort_key(row[i]);
    sh.keys[i] = key;
    if (key) last = i + 1;
  }
  if (last) atomicMax(sh.n_eff, last);
  __syncthreads();
  const int m = *sh.n_eff;
  for (int i = m + threadIdx.x; i < ((m + 3) & ~3); i += RS_THREADS) sh.keys[i] = 0;  // (past the row's end too)
  for (int i = m + threadIdx.x; i < n; i += RS_THREADS) sh.rank[i] = (uint16_t)i;
  __syncthreads();
  rs_ranks4(sh.keys, m, sh.rank);
  __syncthreads();
  for (int i = threadIdx.x; i < m; i += RS_THREADS) sh.sorted_fx[sh.rank[i]] = sp_to_fixed(row[i]);
  __syncthreads();
  // inclusive scan of sorted_fx in contiguous per-thread chunks
  const int per = (m + RS_THREADS - 1) / RS_THREADS;
  const int lo = min((int)threadIdx.x * per, m), hi = min(lo + per, m);
  unsigned long long s = 0;
  for (int i = lo; i < hi; ++i) s += sh.sorted_fx[i];
  sh.chunk_sum[threadIdx.x] = s;
  __syncthreads();
  unsigned long long off = 0;
  for (int t = 0; t < (int)threadIdx.x; ++t) off += sh.chunk_sum[t];
  uint32_t cnt = 0;
  if (t_lt >= 0) {
    for (int i = lo; i < hi; ++i) {
      off += sh.sorted_fx[i];
      cnt += (off <= (unsigned long long)t_lt);
    }
  }
  if (cnt) atomicAdd(sh.below, cnt);
  __syncthreads();
  const int c = (int)*sh.below;
  return c < m ? c + 1 : 1;
}

__global__ __launch_bounds__(RS_THREADS) void sp_cover_select_rows_kernel(const float* __restrict__ x, int nb, int nbw,
                                                                          long long t_lt,
                                                                          uint64_t* __restrict__ pattern) {
  extern __shared__ __attribute__((aligned(16))) char rs_lds[];
  const RowShared sh = rs_carve(rs_lds, nb);
  const int r = blockIdx.x;
  const int keep = rs_row_keep(x + (int64_t)r * nb, nb, t_lt, sh);
  uint32_t* prow = reinterpret_cast<uint32_t*>(pattern + (int64_t)r * nbw);
  for (int w = threadIdx.x; w < nbw * 2; w += RS_THREADS) {
    uint32_t bits = 0;
    for (int b = 0; b < 32; ++b) {
      const int c = w * 32 + b;
      if (c < nb && c <= r && sh.rank[c] < keep) bits |= 1u << b;
    }
    if (r == 0 && w == 0) bits |= 1u;
    prow[w] = bits;
  }
}

extern "C" int sp_cover_select_rows(const float* x, int32_t nb, float thr, uint64_t* pattern, sp_stream_t stream) {
  SP_REQUIRE(x && pattern && nb > 0, SP_ERR_INVALID_ARGUMENT, "sp_cover_select_rows: bad arguments");
  SP_REQUIRE(nb <= RS_MAX, SP_ERR_UNSUPPORTED, "sp_cover_select_rows: nb=%d exceeds %d", nb, RS_MAX);
  hipLaunchKernelGGL(sp_cover_select_rows_kernel, dim3(nb), dim3(RS_THREADS), rs_lds_bytes(nb), (hipStream_t)stream, x, nb,
                     (nb + 63) / 64, (long long)sp_thr_lt(thr), pattern);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// ------------------------------------------------------------------------------------------------
// sqrt Jensen-Shannon divergence (attn/utils.py:26-30), one wave, fixed summation order
// ------------------------------------------------------------------------------------------------
__device__ static float wave_sqrt_js(const float* __restrict__ p, const float* __restrict__ q, int n, int lane) {
  float sp = 0.f, sq = 0.f;
  for (int i = lane; i < n; i += SP_WAVE) {
    const float a = p[i], b = q[i];
    const float m = (a + b) / 2.f;
    sp += a * logf(a / m);
    sq += b * logf(b / m);
  }
  sp = sp_wave_sum(sp);
  sq = sp_wave_sum(sq);
  return sqrtf(0.5f * sp + 0.5f * sq);
}

// ------------------------------------------------------------------------------------------------
// query-aware test (attention_sharing.py:193-202)
// ------------------------------------------------------------------------------------------------
#define QA_THREADS 1024
__global__ __launch_bounds__(QA_THREADS) void sp_queryaware_test_kernel(
    const sp_bf16* __restrict__ q, const sp_bf16* __restrict__ kbar, const float* __restrict__ vert_blk, int64_t n,
    int hq, int hkv, int d, int64_t sq_n, int64_t sq_h, int bs, int nb, uint32_t flags, float inv_sqrt_d, float thr,
    float* __restrict__ avg_qk, float* __restrict__ js_qa, int32_t* __restrict__ use_qa) {
  extern __shared__ float qa_lds[];
  float* qmean = qa_lds;       // [d]
  float* logit = qa_lds + d;   // [nb]
  __shared__ float red[QA_THREADS / SP_WAVE];
  __shared__ float bcast;
  const int h = blockIdx.x;
  const int kvh = h / (hq / hkv);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // mean over the last bs queries of bf16(q / sqrt(d)), rounded to bf16 (last_q.mean(1), :197-199): thread
  // (row group rg, chunk of 8 channels) sums its rows rg, rg + 16, ..., the 16 partials meet in LDS in a fixed order
  {
    float* part = logit;  // [16][d] partial sums, reused for the logits afterwards (nb >= 1: sized max(nb, 16 d) by the host)
    const int nchunk = d >> 3;
    for (int item = threadIdx.x; item < 16 * nchunk; item += QA_THREADS) {
      const int ch = item % nchunk, rg = item / nchunk;
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int i = rg; i < bs; i += 16) {
        const uint4 raw = *reinterpret_cast<const uint4*>(q + (int64_t)h * sq_h + (n - bs + i) * sq_n + ch * 8);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[2 * j] += sp_round_bf16(__uint_as_float(w[j] << 16) * inv_sqrt_d);
          acc[2 * j + 1] += sp_round_bf16(__uint_as_float(w[j] & 0xffff0000u) * inv_sqrt_d);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) part[rg * d + ch * 8 + j] = acc[j];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < d; c += QA_THREADS) {
      float sum = 0.f;
#pragma unroll
      for (int rg = 0; rg < 16; ++rg) sum += part[rg * d + c];
      qmean[c] = sp_round_bf16(sum / (float)bs);
    }
    __syncthreads();
  }
  // logits against the pooled keys: four threads per key (32 channels each), partials folded in a fixed order
  float lmax = -INFINITY;
  const int quarter = threadIdx.x & 3;
  for (int b0 = 0; b0 < nb; b0 += QA_THREADS / 4) {
    const int b = b0 + (threadIdx.x >> 2);
    float sacc = 0.f;
    if (b < nb) {
      const sp_bf16* kr = kbar + ((int64_t)b * hkv + kvh) * d;
      for (int c = quarter * 8; c < d; c += 32) {
        const uint4 raw = *reinterpret_cast<const uint4*>(kr + c);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          sacc += qmean[c + 2 * j] * __uint_as_float(w[j] << 16);
          sacc += qmean[c + 2 * j + 1] * __uint_as_float(w[j] & 0xffff0000u);
        }
      }
    }
    const float s1 = sacc + __shfl_xor(sacc, 1, SP_WAVE);
    float sfull = s1 + __shfl_xor(s1, 2, SP_WAVE);
    if (b < nb && quarter == 0) {  // (the partial sums that shared `logit` were consumed before the barrier above)
      if (flags & SP_FLAG_LOGITS_BF16) sfull = sp_round_bf16(sfull);
      logit[b] = sfull;
      lmax = fmaxf(lmax, sfull);
    }
  }
  lmax = sp_wave_max(lmax);
  if (lane == 0) red[wave] = lmax;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = red[0];
    for (int w = 1; w < QA_THREADS / SP_WAVE; ++w) m = fmaxf(m, red[w]);
    bcast = m;
  }
  __syncthreads();
  const float gmax = bcast;
  float lsum = 0.f;
  for (int b = threadIdx.x; b < nb; b += QA_THREADS) {
    const float e = expf(logit[b] - gmax);
    logit[b] = e;
    lsum += e;
  }
  lsum = sp_wave_sum(lsum);
  __syncthreads();
  if (lane == 0) red[wave] = lsum;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int w = 0; w < QA_THREADS / SP_WAVE; ++w) s += red[w];
    bcast = s;
  }
  __syncthreads();
  const float gsum = bcast;
  for (int b = threadIdx.x; b < nb; b += QA_THREADS) {
    const float p = logit[b] / gsum;
    logit[b] = p;
    avg_qk[(int64_t)h * nb + b] = p;
  }
  __syncthreads();
  if (wave == 0) {
    const float js = wave_sqrt_js(logit, vert_blk + (int64_t)h * nb, nb, lane);
    if (lane == 0) {
      js_qa[h] = js;
      use_qa[h] = (js < thr) ? 1 : 0;  // NaN compares false
    }
  }
}

extern "C" int sp_queryaware_test_bf16(const void* q, const void* kbar, const float* vert_blk, int64_t n, int32_t hq,
                                       int32_t hkv, int32_t d, int64_t q_stride_n, int64_t q_stride_h, int32_t bs,
                                       uint32_t flags, float queryaware_threshold, float* avg_qk, float* js_qa,
                                       int32_t* use_qa, sp_stream_t stream) {
  SP_REQUIRE(q && kbar && vert_blk && avg_qk && js_qa && use_qa, SP_ERR_INVALID_ARGUMENT,
             "sp_queryaware_test_bf16: null pointer");
  SP_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0 && d % 8 == 0 && n >= bs && bs > 0, SP_ERR_INVALID_ARGUMENT,
             "sp_queryaware_test_bf16: bad shape");
  const int nb = (int)sp_ceil_div(n, bs);
  SP_REQUIRE(d <= 256, SP_ERR_UNSUPPORTED, "sp_queryaware_test_bf16: head_dim %d too large", d);
  SP_REQUIRE(q_stride_n % 8 == 0 && q_stride_h % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)kbar % 16) == 0,
             SP_ERR_UNSUPPORTED, "sp_queryaware_test_bf16: q / kbar must be 16-byte aligned with strides multiple of 8");
  const size_t lds = (size_t)(d + (nb > 16 * d ? nb : 16 * d)) * sizeof(float);
  SP_REQUIRE(lds <= 60000, SP_ERR_UNSUPPORTED, "sp_queryaware_test_bf16: nb=%d too large", nb);
  hipLaunchKernelGGL(sp_queryaware_test_kernel, dim3(hq), dim3(QA_THREADS), lds, (hipStream_t)stream,
                     (const sp_bf16*)q, (const sp_bf16*)kbar, vert_blk, n, hq, hkv, d, q_stride_n, q_stride_h, bs, nb,
                     flags, sp_inv_sqrt_dim(flags, d), queryaware_threshold, avg_qk, js_qa, use_qa);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// ------------------------------------------------------------------------------------------------
// top-k sets of the pooled vertical / slash vectors (attention_sharing.py:231-251, :303-329)
// cols[c] = 1 for the nv best columns (column 0 forced), dists[dd] = 1 for the ns best distances
// (distance 0 forced); slash index i holds distance nb-1-i.
// ------------------------------------------------------------------------------------------------
// Membership in the top k of the order (key descending, index ascending), for every element at once, by selection
// instead of ranking: four 8-bit radix passes over the keys find the k-th key T (a 256-bin histogram in LDS and one
// wave that walks it from the top), then an element is in iff key > T, or key == T and fewer than `take` equal keys
// have a lower index (ballots and per-wave counts give that index order).  O(nb) per workgroup where ranking every
// element against every other was O(nb^2 / threads) -- 50 us of a 1024-thread workgroup at nb = 1024.
// Every thread of the workgroup calls it (nthreads = blockDim.x, a multiple of 64); flags[map(i)] = 1 / 0 for i < nb
// with map(i) = reverse ? nb - 1 - i : i.
__device__ static void vs_topk_flags(const uint32_t* keys, int nb, int k, uint8_t* flags, bool reverse, int nthreads) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t wave_cnt[16];
  __shared__ uint32_t s_prefix, s_take, s_base;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = nthreads >> 6;
  if (k >= nb || k <= 0) {  // (uniform) everything or nothing
    for (int i = threadIdx.x; i < nb; i += nthreads) flags[reverse ? nb - 1 - i : i] = k > 0;
    __syncthreads();
    return;
  }
  if (threadIdx.x == 0) {
    s_prefix = 0u;
    s_take = (uint32_t)k;
  }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int b = threadIdx.x; b < 256; b += nthreads) hist[b] = 0u;
    __syncthreads();
    const uint32_t prefix = s_prefix;
    for (int i = threadIdx.x; i < nb; i += nthreads) {
      const uint32_t key = keys[i];
      if (pass == 0 || (key >> (shift + 8)) == (prefix >> (shift + 8))) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (wave == 0) {  // the bin where the running count from the top reaches the number still to take
      uint32_t c[4], tot = 0;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        c[u] = hist[255 - (4 * lane + u)];  // lane 0 holds the four top bins
        tot += c[u];
      }
      uint32_t incl = tot;  // inclusive scan over lanes
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
      }
      uint32_t above = incl - tot;
      const uint32_t take = s_take;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (above < take && above + c[u] >= take) {  // exactly one (lane, u) satisfies this
          s_prefix = prefix | ((uint32_t)(255 - (4 * lane + u)) << shift);
          s_take = take - above;
        }
        above += c[u];
      }
    }
    __syncthreads();
  }
  const uint32_t T = s_prefix, take = s_take;  // take >= 1 keys equal to T belong, lowest indices first
  if (threadIdx.x == 0) s_base = 0u;
  __syncthreads();
  for (int i0 = 0; i0 < nb; i0 += nthreads) {  // (uniform trip count: every lane votes)
    const int i = i0 + threadIdx.x;
    const uint32_t key = i < nb ? keys[i] : 0u;
    const bool eq = i < nb && key == T;
    const unsigned long long bal = __ballot(eq);
    if (lane == 0) wave_cnt[wave] = __popcll(bal);
    __syncthreads();
    uint32_t before = s_base, tot = 0;
    for (int w = 0; w < nwaves; ++w) {
      if (w < wave) before += wave_cnt[w];
      tot += wave_cnt[w];
    }
    before += __popcll(bal & ((1ull << lane) - 1ull));
    if (i < nb) flags[reverse ? nb - 1 - i : i] = key > T || (eq && before < take);
    __syncthreads();  // counts and base have been read
    if (threadIdx.x == 0) s_base += tot;
    __syncthreads();
  }
}

__device__ static void vs_sets(const float* __restrict__ vert, const float* __restrict__ slash, int nb, int nv,
                               int ns, uint32_t* keys /* LDS [RS_MAX], 16-byte aligned */, uint8_t* cols,
                               uint8_t* dists, int nthreads) {
  const uint32_t inf_key = 0x7f800000u;
  for (int i = threadIdx.x; i < nb; i += nthreads) keys[i] = (i == 0) ? inf_key : sp_sort_key(vert[i]);
  __syncthreads();
  vs_topk_flags(keys, nb, nv, cols, false, nthreads);
  for (int i = threadIdx.x; i < nb; i += nthreads) keys[i] = (i == nb - 1) ? inf_key : sp_sort_key(slash[i]);
  __syncthreads();
  vs_topk_flags(keys, nb, ns, dists, true, nthreads);
}

// ------------------------------------------------------------------------------------------------
// pivot election / share test (attention_sharing.py:204-301): three launches.
//   similarity : one workgroup per head, its sqrt-JS against the cluster's stored pivot (one wave per vector);
//   decide     : one thread per head; the election's ascending order is resolved by looking at the lower heads;
//   keep       : one workgroup per head; the newly elected pivots store their pooled vectors and their own
//                vertical-slash sets.
// ------------------------------------------------------------------------------------------------
#define DEC_THREADS 256
#define DEC_MAX_HEADS 256
// head_cluster[h] names a slot of the state only inside [0, n_clusters); -1 (no shared cluster) and anything a
// caller got wrong must never be used as an index into the slabs
__device__ __forceinline__ bool sp_slot_ok(const sp_cluster_state& st, int c) { return c >= 0 && c < st.n_clusters; }
// similarity of every candidate head against its cluster's stored pivot (pivots of EARLIER layers only: this
// launch precedes the layer's election)
__global__ __launch_bounds__(2 * SP_WAVE) void sp_share_similarity_kernel(
    sp_cluster_state st, const int32_t* __restrict__ head_cluster, const float* __restrict__ vert_blk,
    const float* __restrict__ slash_blk, const int32_t* __restrict__ use_qa, float* __restrict__ js_v,
    float* __restrict__ js_s) {
  const int nb = st.nb;
  const int h = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = head_cluster[h];
  float js = NAN;
  if (sp_slot_ok(st, c) && !use_qa[h] && st.info[c * 8 + 0] >= 0 && st.info[c * 8 + 1] != 0)
    js = wave == 0 ? wave_sqrt_js(st.vert + (int64_t)c * nb, vert_blk + (int64_t)h * nb, nb, lane)
                   : wave_sqrt_js(st.slash + (int64_t)c * nb, slash_blk + (int64_t)h * nb, nb, lane);
  if (lane == 0) (wave == 0 ? js_v : js_s)[h] = js;
}

__global__ __launch_bounds__(DEC_MAX_HEADS) void sp_share_decide_kernel(
    sp_cluster_state st, const int32_t* __restrict__ head_cluster, int layer_idx, int hq,
    const int32_t* __restrict__ use_qa, const int32_t* __restrict__ nv, const int32_t* __restrict__ ns, int minb,
    float sim_thr, double fb_thr, int32_t* __restrict__ decision, const float* __restrict__ js_v,
    const float* __restrict__ js_s, int32_t* __restrict__ nv_f, int32_t* __restrict__ ns_f) {
  // The reference walks the heads in ascending order (attention_sharing.py:209-295): the first head of a shared
  // cluster that is not query-aware and finds no pivot becomes the pivot; its later siblings of the same layer find
  // a pivot without a pattern and fall back; heads of clusters with a pattern take the share test.  One thread per
  // head reaches the same decisions: "first" = no lower head of the same cluster is a candidate too.
  __shared__ int s_slot[DEC_MAX_HEADS];
  __shared__ int s_cand[DEC_MAX_HEADS];
  const int h = threadIdx.x;
  int c = -1, qa = 0;
  bool member = false, candidate = false;
  if (h < hq) {
    c = head_cluster[h];
    qa = use_qa[h];
    member = !qa && sp_slot_ok(st, c);
    candidate = member && st.info[c * 8 + 0] < 0;  // the state as the previous layers left it
  }
  s_slot[h] = c;
  s_cand[h] = candidate ? 1 : 0;
  __syncthreads();  // every read of the pivot slots precedes the writes below
  if (h >= hq) return;
  int dec = SP_DEC_VS;
  if (qa) {
    dec = SP_DEC_QA;
  } else if (candidate) {
    bool first = true;
    for (int h2 = 0; h2 < h; ++h2) first = first && !(s_cand[h2] && s_slot[h2] == c);
    if (first) {
      st.info[c * 8 + 0] = h;
      st.info[c * 8 + 2] = nv[h];
      st.info[c * 8 + 3] = ns[h];
      st.info[c * 8 + 4] = layer_idx;
      dec = SP_DEC_DENSE;
    }
  } else if (member && st.info[c * 8 + 1] != 0) {
    if (js_v[h] < sim_thr && js_s[h] < sim_thr && st.ratio[c] < fb_thr) dec = SP_DEC_SHARE;
  }
  decision[h] = dec;
  const bool reset = (dec == SP_DEC_QA || dec == SP_DEC_SHARE);
  nv_f[h] = reset ? minb : nv[h];
  ns_f[h] = reset ? minb : ns[h];
}

// newly elected pivots (the cluster's pivot is this head, elected in this layer) keep their pooled vectors and
// their own vertical-slash sets (:223-263)
__global__ __launch_bounds__(DEC_THREADS) void sp_share_keep_kernel(
    sp_cluster_state st, const int32_t* __restrict__ head_cluster, int layer_idx,
    const float* __restrict__ vert_blk, const float* __restrict__ slash_blk, const int32_t* __restrict__ decision,
    const int32_t* __restrict__ nv, const int32_t* __restrict__ ns) {
  __shared__ __attribute__((aligned(16))) uint32_t s_keys[RS_MAX];
  const int nb = st.nb;
  const int h = blockIdx.x;
  const int c = head_cluster[h];
  if (!sp_slot_ok(st, c) || decision[h] != SP_DEC_DENSE || st.info[c * 8 + 0] != h || st.info[c * 8 + 4] != layer_idx)
    return;
  for (int i = threadIdx.x; i < nb; i += DEC_THREADS) {
    st.vert[(int64_t)c * nb + i] = vert_blk[(int64_t)h * nb + i];
    st.slash[(int64_t)c * nb + i] = slash_blk[(int64_t)h * nb + i];
  }
  vs_sets(vert_blk + (int64_t)h * nb, slash_blk + (int64_t)h * nb, nb, nv[h], ns[h], s_keys,
          st.cols + (int64_t)c * nb, st.dists + (int64_t)c * nb, DEC_THREADS);
}

// The struct a kernel receives by value.  A caller built against the first layout of the struct (it ended with
// `accum`; struct_bytes 0 or SP_CLUSTER_STATE_V1_BYTES) has no avg_map member: nothing behind `accum` is read.
static sp_cluster_state state_by_value(const sp_cluster_state* st) {
  sp_cluster_state v;
  memset(&v, 0, sizeof v);
  const bool full = st->struct_bytes >= (int32_t)sizeof(sp_cluster_state);
  memcpy(&v, st, full ? sizeof v : (size_t)SP_CLUSTER_STATE_V1_BYTES);
  if (!full) v.avg_map = nullptr;
  return v;
}

static int check_state(const sp_cluster_state* st, int nb, const char* who) {
  SP_REQUIRE(st != nullptr, SP_ERR_INVALID_ARGUMENT, "%s: null cluster state", who);
  SP_REQUIRE(st->struct_bytes == 0 || st->struct_bytes == (int32_t)SP_CLUSTER_STATE_V1_BYTES ||
                 st->struct_bytes >= (int32_t)sizeof(sp_cluster_state),
             SP_ERR_INVALID_ARGUMENT, "%s: cluster state struct_bytes=%d is neither 0, %d nor >= %d", who,
             st->struct_bytes, (int)SP_CLUSTER_STATE_V1_BYTES, (int)sizeof(sp_cluster_state));
  SP_REQUIRE(st->n_clusters >= 0 && st->nb == nb && st->nbw == (nb + 63) / 64, SP_ERR_INVALID_ARGUMENT,
             "%s: cluster state sized for nb=%d, call uses nb=%d", who, st->nb, nb);
  if (st->n_clusters > 0) {
    SP_REQUIRE(st->info && st->ratio && st->vert && st->slash && st->cols && st->dists && st->pattern && st->accum,
               SP_ERR_INVALID_ARGUMENT, "%s: cluster state has null slabs", who);
  }
  return SP_OK;
}

extern "C" int sp_share_decide(const sp_cluster_state* state, const int32_t* head_cluster, int32_t layer_idx,
                               int32_t hq, const float* vert_blk, const float* slash_blk, const int32_t* use_qa,
                               const int32_t* nv, const int32_t* ns, int32_t min_blocks, float similarity_threshold,
                               double fallback_threshold, int32_t* decision, float* js_v, float* js_s,
                               int32_t* nv_final, int32_t* ns_final, sp_stream_t stream) {
  SP_REQUIRE(state, SP_ERR_INVALID_ARGUMENT, "sp_share_decide: null cluster state");
  int rc = check_state(state, state->nb, "sp_share_decide");
  if (rc) return rc;
  SP_REQUIRE(head_cluster && vert_blk && slash_blk && use_qa && nv && ns && decision && js_v && js_s && nv_final &&
                 ns_final,
             SP_ERR_INVALID_ARGUMENT, "sp_share_decide: null pointer");
  SP_REQUIRE(hq > 0 && hq <= DEC_MAX_HEADS, SP_ERR_UNSUPPORTED, "sp_share_decide: hq=%d unsupported (max %d)", hq,
             DEC_MAX_HEADS);
  SP_REQUIRE(state->nb <= RS_MAX, SP_ERR_UNSUPPORTED, "sp_share_decide: nb=%d exceeds %d", state->nb, RS_MAX);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(sp_share_similarity_kernel, dim3(hq), dim3(2 * SP_WAVE), 0, s, state_by_value(state), head_cluster, vert_blk,
                     slash_blk, use_qa, js_v, js_s);
  SP_LAUNCH_CHECK();
  hipLaunchKernelGGL(sp_share_decide_kernel, dim3(1), dim3(DEC_MAX_HEADS), 0, s, state_by_value(state), head_cluster, layer_idx, hq, use_qa,
                     nv, ns, min_blocks, similarity_threshold, fallback_threshold, decision, js_v, js_s, nv_final,
                     ns_final);
  SP_LAUNCH_CHECK();
  hipLaunchKernelGGL(sp_share_keep_kernel, dim3(hq), dim3(DEC_THREADS), 0, s, state_by_value(state), head_cluster, layer_idx, vert_blk,
                     slash_blk, decision, nv, ns);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// ------------------------------------------------------------------------------------------------
// mask construction (attention_sharing.py:303-337 and attn/utils.py:99-128 as a set)
// ------------------------------------------------------------------------------------------------
#define MASK_THREADS 1024
#define MASK_SPLIT 8  // workgroups per head: each ranks the head's vectors itself and writes a share of the rows
__global__ __launch_bounds__(MASK_THREADS) void sp_build_mask_kernel(
    sp_cluster_state st, const int32_t* __restrict__ head_cluster, const int32_t* __restrict__ decision,
    const float* __restrict__ vert_blk, const float* __restrict__ slash_blk, const int32_t* __restrict__ nv_f,
    const int32_t* __restrict__ ns_f, int nb, int nbw, uint64_t* __restrict__ mask) {
  __shared__ __attribute__((aligned(16))) uint32_t s_keys[RS_MAX];
  __shared__ uint8_t s_cols[RS_MAX], s_dists[RS_MAX];
  const int h = blockIdx.x;
  const int dec = decision[h];
  if (dec != SP_DEC_DENSE)
    vs_sets(vert_blk + (int64_t)h * nb, slash_blk + (int64_t)h * nb, nb, nv_f[h], ns_f[h], s_keys, s_cols, s_dists,
            MASK_THREADS);
  const uint64_t* pat = nullptr;
  // a SHARE decision without a valid slot (only a caller's own decision vector can hold one) adds no pattern
  if (dec == SP_DEC_SHARE && sp_slot_ok(st, head_cluster[h])) pat = st.pattern + (int64_t)head_cluster[h] * nb * nbw;
  uint64_t* mh = mask + (int64_t)h * nb * nbw;
  // Both sets as bit strings: colw = the columns, dstw = the distances in the order of the slash index i = nb - 1 - d.
  // Row r, columns c0 .. c0 + 63 then want distance bits i = nb - 1 - r + c0 .. + 63: a 64-bit window of dstw, so a mask
  // word is two shifts and an OR instead of 64 pairs of byte look-ups.
  __shared__ uint64_t colw[RS_MAX / 64], dstw[RS_MAX / 64 + 1];
  if (dec != SP_DEC_DENSE) {
    const int lane = threadIdx.x & 63;
    for (int i0 = 0; i0 < nbw * 64; i0 += MASK_THREADS) {  // (uniform trip count: every lane votes)
      const int i = i0 + threadIdx.x;
      const unsigned long long cb = __ballot(i < nb && s_cols[i] != 0);
      const unsigned long long db = __ballot(i < nb && s_dists[nb - 1 - i] != 0);
      if (lane == 0 && i < nbw * 64) {
        colw[i >> 6] = cb;
        dstw[i >> 6] = db;
      }
    }
    if (threadIdx.x == 0) dstw[nbw] = 0ull;
    __syncthreads();
  }
  const int rows_per = (nb + MASK_SPLIT - 1) / MASK_SPLIT;
  const int r_begin = blockIdx.y * rows_per, r_end = min(nb, r_begin + rows_per);
  for (int idx = r_begin * nbw + threadIdx.x; idx < r_end * nbw; idx += MASK_THREADS) {
    const int r = idx / nbw, w = idx - r * nbw;
    const int c0 = w * 64;
    const int cend = min(c0 + 64, r + 1);
    // the causal part of the word: columns c0 .. cend - 1
    const uint64_t causal = cend <= c0 ? 0ull : ((cend - c0 == 64) ? ~0ull : ((1ull << (cend - c0)) - 1ull));
    uint64_t bits = causal;
    if (dec != SP_DEC_DENSE) {
      bits = 0ull;
      if (causal) {
        const int start = nb - 1 - r + c0;  // >= 0; bits past nb - 1 belong to columns beyond r
        const int k = start >> 6, sh = start & 63;
        uint64_t win = dstw[k] >> sh;
        if (sh) win |= dstw[k + 1] << (64 - sh);
        bits = (colw[w] | win) & causal;
      }
      if (pat) bits |= pat[idx];
    }
    if (idx == 0) bits |= 1ull;
    mh[idx] = bits;
  }
}

extern "C" int sp_build_mask(const sp_cluster_state* state, const int32_t* head_cluster, const int32_t* decision,
                             const float* vert_blk, const float* slash_blk, const int32_t* nv_final,
                             const int32_t* ns_final, int32_t hq, int32_t nb, uint64_t* mask, sp_stream_t stream) {
  int rc = check_state(state, nb, "sp_build_mask");
  if (rc) return rc;
  SP_REQUIRE(head_cluster && decision && vert_blk && slash_blk && nv_final && ns_final && mask,
             SP_ERR_INVALID_ARGUMENT, "sp_build_mask: null pointer");
  SP_REQUIRE(hq > 0 && nb > 0 && nb <= RS_MAX, SP_ERR_UNSUPPORTED, "sp_build_mask: nb=%d unsupported (max %d)", nb,
             RS_MAX);
  hipLaunchKernelGGL(sp_build_mask_kernel, dim3(hq, MASK_SPLIT), dim3(MASK_THREADS), 0, (hipStream_t)stream,
                     state_by_value(state), head_cluster, decision, vert_blk, slash_blk, nv_final, ns_final, nb, (nb + 63) / 64, mask);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// ------------------------------------------------------------------------------------------------
// query-aware heads: pooled block probabilities (attention_sharing.py:350-360)
// ------------------------------------------------------------------------------------------------
#define BP_THREADS 256
__global__ __launch_bounds__(BP_THREADS) void sp_block_probs_kernel(
    const sp_bf16* __restrict__ qbar, const sp_bf16* __restrict__ kbar, const int32_t* __restrict__ decision, int hq,
    int hkv, int d, int nb, uint32_t flags, float inv_sqrt_d, float* __restrict__ probs) {
  extern __shared__ float bp_lds[];
  float* qs = bp_lds;          // [d]
  float* logit = bp_lds + d;   // [nb]
  __shared__ float red[BP_THREADS / SP_WAVE];
  __shared__ float bcast;
  const int r = blockIdx.x, h = blockIdx.y;
  if (decision[h] != SP_DEC_QA) return;
  const int kvh = h / (hq / hkv);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = threadIdx.x; c < d; c += BP_THREADS)
    qs[c] = sp_round_bf16(sp_bf16_to_f32(qbar[((int64_t)r * hq + h) * d + c]) * inv_sqrt_d);
  __syncthreads();
  float lmax = -INFINITY;
  for (int b = threadIdx.x; b <= r; b += BP_THREADS) {
    const sp_bf16* kr = kbar + ((int64_t)b * hkv + kvh) * d;
    float s = 0.f;
    for (int c = 0; c < d; c += 8) {
      const uint4 raw = *reinterpret_cast<const uint4*>(kr + c);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s += qs[c + 2 * j] * __uint_as_float(w[j] << 16);
        s += qs[c + 2 * j + 1] * __uint_as_float(w[j] & 0xffff0000u);
      }
    }
    if (flags & SP_FLAG_LOGITS_BF16) s = sp_round_bf16(s);
    logit[b] = s;
    lmax = fmaxf(lmax, s);
  }
  lmax = sp_wave_max(lmax);
  if (lane == 0) red[wave] = lmax;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = red[0];
    for (int w = 1; w < BP_THREADS / SP_WAVE; ++w) m = fmaxf(m, red[w]);
    bcast = m;
  }
  __syncthreads();
  const float gmax = bcast;
  float lsum = 0.f;
  for (int b = threadIdx.x; b <= r; b += BP_THREADS) {
    const float e = expf(logit[b] - gmax);
    logit[b] = e;
    lsum += e;
  }
  lsum = sp_wave_sum(lsum);
  __syncthreads();
  if (lane == 0) red[wave] = lsum;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int w = 0; w < BP_THREADS / SP_WAVE; ++w) s += red[w];
    bcast = s;
  }
  __syncthreads();
  const float gsum = bcast;
  float* out = probs + ((int64_t)h * nb + r) * nb;
  for (int b = threadIdx.x; b < nb; b += BP_THREADS) out[b] = (b <= r) ? logit[b] / gsum : 0.f;
}

// score = pattern_threshold * nb: the product of the caller's DOUBLE threshold and the block count, evaluated in
// double as Python evaluates it (attention_sharing.py:361), then taken to fp32 as the comparison with an fp32
// tensor takes it (utils.py:56).  A threshold that had been rounded to fp32 first would give a score one fp32 ulp
// away for about a fifth of the block counts.
extern "C" float sp_queryaware_select_score(double pattern_threshold, int32_t nb) {
  volatile double product = pattern_threshold * (double)nb;  // one rounding to double, then one to float
  return (float)product;
}

extern "C" int sp_queryaware_select_bf16(const void* qbar, const void* kbar, const int32_t* decision, int32_t hq,
                                         int32_t hkv, int32_t d, int32_t nb, uint32_t flags, double pattern_threshold,
                                         float* probs, uint64_t* mask, void* workspace, size_t workspace_bytes,
                                         sp_stream_t stream) {
  SP_REQUIRE(qbar && kbar && decision && probs && mask, SP_ERR_INVALID_ARGUMENT,
             "sp_queryaware_select_bf16: null pointer");
  SP_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0 && d % 8 == 0 && nb > 0, SP_ERR_INVALID_ARGUMENT,
             "sp_queryaware_select_bf16: bad shape");
  const size_t lds = (size_t)(d + nb) * sizeof(float);
  SP_REQUIRE(lds <= 60000, SP_ERR_UNSUPPORTED, "sp_queryaware_select_bf16: nb=%d too large", nb);
  if (d == 128) {  // two passes on the matrix core, 128 rows per workgroup
    const int rc = sp_block_probs_mfma_launch(qbar, kbar, decision, hq, hkv, nb, flags, probs, (hipStream_t)stream);
    if (rc != SP_OK) return rc;
  } else {  // one row per workgroup, fp32 dot products
    hipLaunchKernelGGL(sp_block_probs_kernel, dim3(nb, hq), dim3(BP_THREADS), lds, (hipStream_t)stream,
                       (const sp_bf16*)qbar, (const sp_bf16*)kbar, decision, hq, hkv, d, nb, flags,
                       sp_inv_sqrt_dim(flags, d), probs);
    SP_LAUNCH_CHECK();
  }
  const float score = sp_queryaware_select_score(pattern_threshold, nb);
  return gsel_run(probs, decision, SP_DEC_QA, hq, nb, score, mask, workspace, workspace_bytes, (hipStream_t)stream,
                  "sp_queryaware_select_bf16");
}

// ------------------------------------------------------------------------------------------------
// pivot state update (attention_sharing.py:94-103 and the vs_ratio of :278-286, computed eagerly)
// ------------------------------------------------------------------------------------------------
struct PivotRowShared {
  unsigned long long cov, tot;
  unsigned long long pad[RS_THREADS / SP_WAVE];
  int last;
};

// One workgroup per (row, head).  The workgroup that finishes a head's last row (a counter in the cluster's info
// slot 5, which is zero between calls) turns the accumulated masses into the coverage ratio, publishes the pattern
// and leaves counter and accumulators zero again.  Invariant: state.accum and info[.][5] are zero on entry; the
// caller's slabs start zeroed and every completed call restores that.
__global__ __launch_bounds__(RS_THREADS) void sp_pivot_rows_kernel(sp_cluster_state st,
                                                                   const int32_t* __restrict__ head_cluster,
                                                                   const int32_t* __restrict__ decision,
                                                                   const float* __restrict__ avg_attn, int hq,
                                                                   int nb, int nbw, long long t_lt,
                                                                   unsigned long long* __restrict__ accum) {
  __shared__ PivotRowShared sh;
  extern __shared__ __attribute__((aligned(16))) char rs_lds[];
  const RowShared rsh = rs_carve(rs_lds, nb);
  const int r = blockIdx.x, h = blockIdx.y;
  if (decision[h] != SP_DEC_DENSE) return;
  const int c = head_cluster[h];
  if (!sp_slot_ok(st, c)) return;  // a dense head outside every shared cluster keeps no pattern
  // One head per cluster and call: the election flags one, but a caller's own flags may name several heads of a
  // cluster.  The reference stores them one after the other, so the highest head's map is what stays
  // (attention_sharing.py:96-103); here the lower ones leave, or their rows would share the cluster's row counter
  // and accumulators with the highest head's.
  bool later = false;
  for (int h2 = h + 1 + threadIdx.x; h2 < hq; h2 += RS_THREADS)
    later = later || (decision[h2] == SP_DEC_DENSE && head_cluster[h2] == c);
  if (__syncthreads_or(later ? 1 : 0)) return;
  const float* row = avg_attn + ((int64_t)h * nb + r) * nb;
  const int keep = rs_row_keep(row, nb, t_lt, rsh);
  uint32_t* prow = reinterpret_cast<uint32_t*>(st.pattern + ((int64_t)c * nb + r) * nbw);
  for (int w = threadIdx.x; w < nbw * 2; w += RS_THREADS) {
    uint32_t bits = 0;
    for (int b = 0; b < 32; ++b) {
      const int col = w * 32 + b;
      if (col < nb && col <= r && rsh.rank[col] < keep) bits |= 1u << b;
    }
    if (r == 0 && w == 0) bits |= 1u;
    prow[w] = bits;
  }
  // vs_ratio pieces: mass under the pivot's own vertical / slash sets (a block in both counts twice) and the total
  if (threadIdx.x == 0) {
    sh.cov = 0;
    sh.tot = 0;
  }
  __syncthreads();
  const uint8_t* cols = st.cols + (int64_t)c * nb;
  const uint8_t* dists = st.dists + (int64_t)c * nb;
  unsigned long long cov = 0, tot = 0;
  float* keep_row = st.avg_map ? st.avg_map + ((int64_t)c * nb + r) * nb : nullptr;
  for (int col = threadIdx.x; col < nb; col += RS_THREADS) {
    const float val = row[col];
    if (keep_row) keep_row[col] = val;  // the pivot's map itself, for get_pivotal_attn
    const unsigned long long fx = sp_to_fixed(val);
    tot += fx;
    if (col <= r) cov += fx * (unsigned long long)((cols[col] ? 1 : 0) + (dists[r - col] ? 1 : 0));
  }
  if (cov) atomicAdd(&sh.cov, cov);
  if (tot) atomicAdd(&sh.tot, tot);
  __syncthreads();
  if (threadIdx.x == 0) {
    if (sh.cov) atomicAdd(&accum[c * 2 + 0], sh.cov);
    if (sh.tot) atomicAdd(&accum[c * 2 + 1], sh.tot);
    __threadfence();  // this row's pattern words and masses are visible before the row is counted
    sh.last = atomicAdd(&st.info[c * 8 + 5], 1) == nb - 1;
  }
  __syncthreads();
  if (!sh.last) return;
  // ---- the head's last row: every other row of it has been counted, so its atomics and stores are visible ----
  __threadfence();
  // every out-of-range slash / vertical slot of the reference's id list is the padding id 0
  unsigned long long pad = 0;
  for (int i = threadIdx.x; i < nb; i += RS_THREADS) {
    if (cols[i]) pad += (unsigned long long)i;
    if (dists[i]) pad += (unsigned long long)i;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) pad += __shfl_xor(pad, o, SP_WAVE);
  if ((threadIdx.x & 63) == 0) sh.pad[threadIdx.x >> 6] = pad;
  __syncthreads();
  if (threadIdx.x == 0) {
    pad = 0;
    for (int w = 0; w < RS_THREADS / SP_WAVE; ++w) pad += sh.pad[w];
    const unsigned long long acc_cov = atomicAdd(&accum[c * 2 + 0], 0ull), acc_tot = atomicAdd(&accum[c * 2 + 1], 0ull);
    const unsigned long long a00 = sp_to_fixed(avg_attn[(int64_t)h * nb * nb]);
    // one IEEE operation at a time (no fused multiply-add), so the value is reproducible on a CPU
    const double covd = __dadd_rn((double)acc_cov, __dmul_rn((double)pad, (double)a00));
    const double totd = (double)acc_tot;
    st.ratio[c] = totd > 0.0 ? __ddiv_rn(covd, totd) : (double)NAN;
    accum[c * 2 + 0] = 0;
    accum[c * 2 + 1] = 0;
    st.info[c * 8 + 5] = 0;
    __threadfence();
    st.info[c * 8 + 1] = 1;
  }
}

extern "C" int sp_pivot_update(const sp_cluster_state* state, const int32_t* head_cluster, const int32_t* decision,
                               const float* avg_attn, int32_t hq, int32_t nb, float pattern_threshold,
                               sp_stream_t stream) {
  int rc = check_state(state, nb, "sp_pivot_update");
  if (rc) return rc;
  SP_REQUIRE(head_cluster && decision && avg_attn, SP_ERR_INVALID_ARGUMENT, "sp_pivot_update: null pointer");
  SP_REQUIRE(hq > 0 && hq <= 1024 && nb > 0 && nb <= RS_MAX, SP_ERR_UNSUPPORTED,
             "sp_pivot_update: hq=%d nb=%d unsupported", hq, nb);
  if (state->n_clusters == 0) return SP_OK;
  unsigned long long* accum = reinterpret_cast<unsigned long long*>(state->accum);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(sp_pivot_rows_kernel, dim3(nb, hq), dim3(RS_THREADS), rs_lds_bytes(nb), s, state_by_value(state), head_cluster, decision,
                     avg_attn, hq, nb, (nb + 63) / 64, (long long)sp_thr_lt(pattern_threshold), accum);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// ------------------------------------------------------------------------------------------------
// CSR row pointers of a mask (triton_column_count_cumsum, shareprefill_attn.py:226-269)
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void sp_mask_row_pointers_kernel(const uint64_t* __restrict__ mask, int nb, int nbw,
                                                                   int32_t* __restrict__ row_ptr) {
  __shared__ int32_t cnt[RS_MAX];
  const int h = blockIdx.x;
  const uint64_t* mh = mask + (int64_t)h * nb * nbw;
  for (int r = threadIdx.x; r < nb; r += 256) {
    int c = 0;
    for (int w = 0; w < nbw; ++w) c += __popcll(mh[(int64_t)r * nbw + w]);
    cnt[r] = c;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t* out = row_ptr + (int64_t)h * (nb + 1);
    int acc = 0;
    out[0] = 0;
    for (int r = 0; r < nb; ++r) {
      acc += cnt[r];
      out[r + 1] = acc;
    }
  }
}

extern "C" int sp_mask_row_pointers(const uint64_t* mask, int32_t hq, int32_t nb, int32_t* row_ptr,
                                    sp_stream_t stream) {
  SP_REQUIRE(mask && row_ptr && hq > 0 && nb > 0, SP_ERR_INVALID_ARGUMENT, "sp_mask_row_pointers: bad arguments");
  SP_REQUIRE(nb <= RS_MAX, SP_ERR_UNSUPPORTED, "sp_mask_row_pointers: nb=%d exceeds %d", nb, RS_MAX);
  hipLaunchKernelGGL(sp_mask_row_pointers_kernel, dim3(hq), dim3(256), 0, (hipStream_t)stream, mask, nb,
                     (nb + 63) / 64, row_ptr);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

// ------------------------------------------------------------------------------------------------
// The reference's block_idx form of a layer's selection (shareprefill_attn.py:484-486, 528-540): per head a list
// of flat block ids row * nb + col, in any order, padded with values outside the grid (the reference pads with
// nb * (nb + 1)).
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void sp_fill_u64_kernel(uint64_t* __restrict__ p, int64_t n, uint64_t value) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = value;
}

__global__ __launch_bounds__(256) void sp_block_idx_to_mask_kernel(const int64_t* __restrict__ idx, int64_t stride_h,
                                                                   int64_t k, int nb, int nbw,
                                                                   uint64_t* __restrict__ mask) {
  const int h = blockIdx.y;
  const int64_t cells = (int64_t)nb * nb;
  unsigned long long* mh = reinterpret_cast<unsigned long long*>(mask) + (int64_t)h * nb * nbw;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < k; i += (int64_t)gridDim.x * 256) {
    const int64_t id = idx[(int64_t)h * stride_h + i];
    if (id < 0 || id >= cells) continue;  // padding
    const int r = (int)(id / nb), c = (int)(id % nb);
    if (c > r) continue;  // above the diagonal: the kernel's causal mask leaves nothing of such a block
    atomicOr(mh + (int64_t)r * nbw + (c >> 6), 1ull << (c & 63));
  }
}

extern "C" int sp_block_idx_to_mask(const int64_t* block_idx, int64_t idx_stride_h, int64_t k, int32_t hq, int32_t nb,
                                    uint64_t* mask, sp_stream_t stream) {
  SP_REQUIRE(mask && hq > 0 && nb > 0 && k >= 0 && (block_idx || k == 0), SP_ERR_INVALID_ARGUMENT,
             "sp_block_idx_to_mask: bad arguments");
  SP_REQUIRE(hq <= 65535, SP_ERR_UNSUPPORTED, "sp_block_idx_to_mask: hq=%d exceeds 65535", hq);
  const int nbw = (nb + 63) / 64;
  const int64_t words = (int64_t)hq * nb * nbw;
  // a fill kernel rather than a memset node, so that the call can be recorded into a graph
  const unsigned fill_grid = (unsigned)(sp_ceil_div(words, 256) < 4096 ? sp_ceil_div(words, 256) : 4096);
  hipLaunchKernelGGL(sp_fill_u64_kernel, dim3(fill_grid), dim3(256), 0, (hipStream_t)stream, mask, words,
                     (uint64_t)0);
  SP_LAUNCH_CHECK();
  if (k > 0) {
    const unsigned gx = (unsigned)(sp_ceil_div(k, 256) < 1024 ? sp_ceil_div(k, 256) : 1024);
    hipLaunchKernelGGL(sp_block_idx_to_mask_kernel, dim3(gx, hq), dim3(256), 0, (hipStream_t)stream, block_idx,
                       idx_stride_h, k, nb, nbw, mask);
    SP_LAUNCH_CHECK();
  }
  return SP_OK;
}

// CSR row pointers of id lists (count_kernel, shareprefill_attn.py:187-223: a histogram of id / nb, then its running
// sum).  Duplicates count as often as they occur and the order of the ids does not matter, as in the reference.
__global__ __launch_bounds__(256) void sp_block_idx_row_pointers_kernel(const int64_t* __restrict__ idx,
                                                                        int64_t stride_h, int64_t k, int nb,
                                                                        int32_t* __restrict__ row_ptr) {
  __shared__ int32_t cnt[RS_MAX];
  __shared__ int32_t part[256];
  const int h = blockIdx.x;
  const int64_t cells = (int64_t)nb * nb;
  for (int r = threadIdx.x; r < nb; r += 256) cnt[r] = 0;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < k; i += 256) {
    const int64_t id = idx[(int64_t)h * stride_h + i];
    if (id >= 0 && id < cells) atomicAdd(&cnt[(int)(id / nb)], 1);
  }
  __syncthreads();
  // running sum: every thread owns a contiguous run of rows
  const int per = (nb + 255) / 256;
  const int r0 = threadIdx.x * per, r1 = (r0 + per < nb) ? r0 + per : nb;
  int s = 0;
  for (int r = r0; r < r1; ++r) s += cnt[r];
  part[threadIdx.x] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int t = 0; t < 256; ++t) {
      const int v = part[t];
      part[t] = acc;
      acc += v;
    }
  }
  __syncthreads();
  int32_t* out = row_ptr + (int64_t)h * (nb + 1);
  int acc = part[threadIdx.x];
  for (int r = r0; r < r1; ++r) {
    acc += cnt[r];
    out[r + 1] = acc;
  }
  if (threadIdx.x == 0) out[0] = 0;
}

extern "C" int sp_block_idx_row_pointers(const int64_t* block_idx, int64_t idx_stride_h, int64_t k, int32_t hq,
                                         int32_t nb, int32_t* row_ptr, sp_stream_t stream) {
  SP_REQUIRE(row_ptr && hq > 0 && nb > 0 && k >= 0 && (block_idx || k == 0), SP_ERR_INVALID_ARGUMENT,
             "sp_block_idx_row_pointers: bad arguments");
  SP_REQUIRE(nb <= RS_MAX, SP_ERR_UNSUPPORTED, "sp_block_idx_row_pointers: nb=%d exceeds %d", nb, RS_MAX);
  hipLaunchKernelGGL(sp_block_idx_row_pointers_kernel, dim3(hq), dim3(256), 0, (hipStream_t)stream, block_idx,
                     idx_stride_h, k, nb, row_ptr);
  SP_LAUNCH_CHECK();
  return SP_OK;
}

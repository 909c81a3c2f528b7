"""CPU oracle for the SharePrefill prefill-attention path.

TEST INFRASTRUCTURE ONLY.  This module is a CPU (torch + numpy) restatement of
the reference algorithm.  It is imported by tests/, by __graft_entry__.smoke()
and by the cpu_baseline leg of bench.py as the *checker*; nothing in the
shareprefill_amd package imports it and no product code path routes through it.

Every function cites the reference lines it follows (paths relative to the
reference checkout, e.g. shareprefill/attn/utils.py:47-50).

Canonical arithmetic (where the reference leaves behaviour to the backend):

* ordering for every sort / top-k:  value descending, index ascending on ties
  (torch.sort / torch.topk tie order is unspecified).
* cumulative-mass comparisons (utils.py:47-76) are evaluated in exact
  arithmetic on values truncated to unsigned 2^-48 fixed point, so that the
  result does not depend on summation order.  The reference's float cumsum is
  backend-defined (CUDA scan association order); the fixed-point result agrees
  with the literal torch formula except where float rounding decides a tie,
  which tests/test_oracle_pins.py checks on seeded inputs.
* the pivot's vertical-slash coverage ratio (attention_sharing.py:278-286) is
  evaluated as the ratio of two exact fixed-point sums in double precision.

Parity pins (what each function is checked against, besides the HIP path):
  pool_avg ........... float64 mean, constant/linearity invariants
  pool ............... torch's max_pool1d / avg_pool1d library routines on the zero-filled sequence; one-hot cases
  diagonal_sums ...... brute-force double loop; sums to the matrix total
  cover_count ........ literal torch sort+cumsum formula; one-hot / uniform closed forms
  cover_keep_le ...... literal torch formula; brute force on tiny inputs; "excludes crossing entry"
  cover_keep_rows_ge . literal torch formula; "includes crossing entry"; never-reached edge
  sqrt_js ............ scipy.spatial.distance.jensenshannon; NaN on zeros
  vs_id_list ......... brute-force set for nb=5 (ids {0,5,6,10,12,15,16,18,20,22,23,24})
  vs_ratio ........... literal gather-with-duplicates over vs_id_list
  csr_row_pointers ... reference docstring vector [0,5,8,9,13,14] -> [0,1,2,4,6]
  masked_attention ... torch SDPA (full mask), per-block causal attention (diagonal mask)
  masked_attention_ref_roundings ... the fp32 masked_attention within the derived rounding noise; bit-equal to its
                       bf16 rounding on inputs whose probabilities are exact powers of two
  scaled_last_q ...... torch's own bf16-tensor / Python-float division, exhaustively over every bf16 value
  pooled_qk_probs .... fp64 double loop; uniform 1/nb for equal keys; head -> kv head h // g (h % Hkv differs)
  pool_q_head ........ torch's own expression (pad, mean, *bs/(bs-pad)) on CPU bf16, all tail lengths
  block_probs ........ fp64 double loop; row r uniform 1/(r+1) for zero queries; rows sum to 1; upper triangle 0
  decode_attention ... torch SDPA with enable_gqa; one-key and uniform-logit closed forms
  rope_rotate ........ Hugging Face apply_rotary_pos_emb on bf16 CPU tensors (bit-exact); angle 0 / quarter turn
  layer() ............ scripted sharing scenarios (pivot / same-layer sibling / share / fallback)
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np
import torch

FX_BITS = 48
FX_SAT = float(2.0 ** 62)

DEC_VS, DEC_DENSE, DEC_SHARE, DEC_QA = 0, 1, 2, 3


# --------------------------------------------------------------------------- #
# fixed-point cumulative-mass primitives
# --------------------------------------------------------------------------- #
def to_fixed(x) -> np.ndarray:
    """fp32 -> unsigned 2^-48 fixed point (truncating); NaN / negatives -> 0."""
    x = np.asarray(x, dtype=np.float32).astype(np.float64)
    v = np.floor(x * float(2 ** FX_BITS))
    v = np.where(np.isnan(v) | (v < 0), 0.0, v)
    v = np.minimum(v, FX_SAT)
    return v.astype(np.uint64)


def sort_key(x) -> np.ndarray:
    """Order key: the fp32 bit pattern; NaN and anything with the sign bit -> 0."""
    x = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    bits = x.view(np.uint32).copy()
    bad = (bits >> 31 != 0) | np.isnan(x)
    bits[bad] = 0
    return bits


def order_desc(x) -> np.ndarray:
    """Permutation sorting a 1-D vector by (value desc, index asc)."""
    key = sort_key(x).astype(np.int64)
    return np.argsort(-key, kind="stable")


def thr_le(thr: float) -> int:
    """Largest fixed-point sum S with S*2^-48 <= fp32(thr)."""
    t = float(np.float32(thr)) * float(2 ** FX_BITS)
    return int(math.floor(t))


def thr_lt(thr: float) -> int:
    """Largest fixed-point sum S with S*2^-48 < fp32(thr)."""
    t = float(np.float32(thr)) * float(2 ** FX_BITS)
    return int(math.ceil(t)) - 1


def prefix_len(x, t_fx: int) -> int:
    """Number of leading entries of sort_desc(x) whose running sum is <= t_fx."""
    x = np.asarray(x, dtype=np.float32).reshape(-1)
    if t_fx < 0:
        return 0
    o = order_desc(x)
    cs = np.cumsum(to_fixed(x[o]), dtype=np.uint64)
    return int(np.searchsorted(cs, np.uint64(t_fx), side="right"))


def cover_count(x, thr: float) -> int:
    """utils.py:47-50 score_cover_topk: count(cumsum(sort_desc(x)) <= thr) + 1."""
    return prefix_len(x, thr_le(thr)) + 1


def cover_keep_le(x, score: float) -> np.ndarray:
    """utils.py:53-57 score_cover_idx: indices kept (cumsum <= score), crossing entry excluded.

    Returns the kept flat indices in sorted-desc order (the reference replaces the others by 0).
    """
    x = np.asarray(x, dtype=np.float32).reshape(-1)
    m = prefix_len(x, thr_le(score))
    return order_desc(x)[:m]


def cover_keep_rows_ge(a, thr: float) -> np.ndarray:
    """utils.py:60-76 score_cover_idx_each_row: per row keep argmax(cumsum >= thr)+1 entries.

    Returns a bool matrix of kept entries (the reference returns unique flat ids incl. 0).
    A row that never reaches thr keeps exactly one entry (argmax of all-False is 0).
    """
    a = np.asarray(a, dtype=np.float32)
    nr, nc = a.shape
    keep = np.zeros((nr, nc), dtype=bool)
    t = thr_lt(thr)
    for r in range(nr):
        c = prefix_len(a[r], t)
        n_keep = c + 1 if c < nc else 1
        keep[r, order_desc(a[r])[:n_keep]] = True
    return keep


def topk_indices(x, k: int) -> np.ndarray:
    """torch.topk(...).indices with canonical tie order (attention_sharing.py:309-322)."""
    return order_desc(x)[:k]


# --------------------------------------------------------------------------- #
# small float helpers
# --------------------------------------------------------------------------- #
def sqrt_js(p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """utils.py:26-30 square_root_js_divergence (natural log; 0*log 0 -> NaN as in the reference)."""
    p = p.float()
    q = q.float()
    m = (p + q) / 2
    return torch.sqrt(0.5 * (p * torch.log(p / m)).sum(-1) + 0.5 * (q * torch.log(q / m)).sum(-1))


def block_sum(x: torch.Tensor, bs: int) -> torch.Tensor:
    """utils.py:33-44 torch_bhn_sumpool on [..., N] -> [..., ceil(N/bs)], right zero padding."""
    n = x.shape[-1]
    nb = -(-n // bs)
    x = torch.nn.functional.pad(x, (0, nb * bs - n))
    return x.reshape(*x.shape[:-1], nb, bs).sum(-1)


def pool_avg(x: torch.Tensor, bs: int) -> torch.Tensor:
    """utils.py:131-261 triton_bnhd_pool("avg") for x[N,H,D] -> [nb,H,D] in x.dtype.

    Mean over each run of bs tokens, the tail divided by its true length (utils.py:171,187).
    Accumulation is fp32 (the reference accumulates in the input dtype).
    """
    n, h, d = x.shape
    nb = -(-n // bs)
    xf = torch.nn.functional.pad(x.float(), (0, 0, 0, 0, 0, nb * bs - n))
    s = xf.reshape(nb, bs, h, d).sum(1)
    cnt = torch.full((nb,), float(bs))
    cnt[-1] = float(n - (nb - 1) * bs)
    return (s / cnt[:, None, None]).to(x.dtype)


def pool(x: torch.Tensor, bs: int, pool_type: str) -> torch.Tensor:
    """utils.py:131-261 triton_bnhd_pool for x[N,H,D] -> [nb,H,D] in x.dtype, pool types "max", "min", "maxabs", "sum"
    ("avg": pool_avg).  Plain loops over the blocks.

    The reference's kernel loads the tokens of a ragged last block beyond the sequence as zeros (utils.py:168-179,
    other=0) and reduces over all bs slots (:180-191), so the tail's maximum is at least 0 and its minimum at most 0.
    Sums accumulate in fp32 here (the reference's kernel adds in the input dtype)."""
    n, h, d = x.shape
    nb = -(-n // bs)
    out = torch.zeros(nb, h, d, dtype=torch.float32)
    for b in range(nb):
        blk = x[b * bs:(b + 1) * bs].float()
        if blk.shape[0] < bs:
            blk = torch.cat([blk, torch.zeros(bs - blk.shape[0], h, d)])
        if pool_type == "max":
            out[b] = blk.amax(0)
        elif pool_type == "min":
            out[b] = blk.amin(0)
        elif pool_type == "maxabs":
            out[b] = blk.abs().amax(0)
        elif pool_type == "sum":
            out[b] = blk.sum(0)
        else:
            raise KeyError(pool_type)
    return out.to(x.dtype)


def diagonal_sums(p: torch.Tensor) -> torch.Tensor:
    """utils.py:79-86 sum_all_diagonal_matrix for one [n, m] matrix -> [m].

    out[j] = sum_i p[i, j + i - (n-1)] over in-range columns.
    """
    n, m = p.shape
    out = torch.zeros(m, dtype=p.dtype)
    for i in range(n):
        sh = n - 1 - i
        if sh < m:
            out[sh:] += p[i, : m - sh]
    return out


def csr_row_pointers(ids: np.ndarray, nb: int) -> np.ndarray:
    """shareprefill_attn.py:226-269 triton_column_count_cumsum for one sorted id list."""
    ids = np.asarray(ids, dtype=np.int64)
    rows = ids // nb
    cnt = np.bincount(rows[rows < nb], minlength=nb)[:nb]
    return np.concatenate([[0], np.cumsum(cnt)]).astype(np.int32)


# --------------------------------------------------------------------------- #
# vertical-slash expansion
# --------------------------------------------------------------------------- #
def vs_id_list(cols, dists, nb: int) -> np.ndarray:
    """utils.py:99-128 combine_vertical_slash_indices for one head: [slash | vertical] flat ids.

    slash part:  for r in 0..nb-1, for d in dists: (r+d)*nb + r, or 0 when r+d >= nb
    vertical part: for r in 0..nb-1, for c in cols: r*nb + c, or 0 when r < c
    Duplicates and zero padding are kept (they matter for vs_ratio).
    """
    r = np.arange(nb, dtype=np.int64)[:, None]
    d = np.asarray(dists, dtype=np.int64)[None, :]
    c = np.asarray(cols, dtype=np.int64)[None, :]
    sl = (r + d) * nb + r
    sl = np.where(r + d < nb, sl, 0).reshape(-1)
    ve = np.broadcast_to(r * nb + c, (nb, c.shape[1]))
    ve = np.where(r >= c, ve, 0).reshape(-1)
    return np.concatenate([sl, ve])


def vs_mask(cols, dists, nb: int) -> np.ndarray:
    """Set of blocks named by vs_id_list, as a bool [nb, nb] matrix (always contains (0,0))."""
    m = np.zeros((nb, nb), dtype=bool)
    rr = np.arange(nb)
    for c in cols:
        m[rr[rr >= c], c] = True
    for d in dists:
        r = rr[rr + d < nb]
        m[r + d, r] = True
    m[0, 0] = True
    return m


def vs_ratio(avg: np.ndarray, cols, dists) -> float:
    """attention_sharing.py:278-286: sum of avg over vs_id_list WITH multiplicity / sum(avg).

    Closed form: S(slash set) + S(vertical set) + (sum(dists) + sum(cols)) * avg[0,0]
    (each out-of-range slash / vertical slot is the padding id 0).  The two set sums and the total are exact
    fixed-point integers; the final combination is evaluated in double as
    (double(S_sets) + double(pad) * double(avg00)) / double(total), one IEEE operation at a time.
    """
    nb = avg.shape[0]
    fx = to_fixed(avg).astype(object)
    tot = int(fx.sum())
    cov = 0
    rr = np.arange(nb)
    for d in dists:
        r = rr[rr + d < nb]
        cov += int(fx[r + d, r].sum())
    for c in cols:
        r = rr[rr >= c]
        cov += int(fx[r, c].sum())
    pad = int(np.sum(dists)) + int(np.sum(cols))
    if tot == 0:
        return float("nan")
    return (float(cov) + float(pad) * float(int(fx[0, 0]))) / float(tot)


# --------------------------------------------------------------------------- #
# last-block scores (Step A) and pooled estimates (Step C / F)
# --------------------------------------------------------------------------- #
def inv_sqrt_d(d: int) -> np.float32:
    return np.float32(1.0) / np.float32(math.sqrt(d))


def scaled_last_q(q: torch.Tensor, bs: int) -> torch.Tensor:
    """attention_sharing.py:127  last_q = q[-bs:] / sqrt(D), kept in q.dtype.  q: [Hq,N,D]."""
    d = q.shape[-1]
    return (q[:, -bs:].float() * float(inv_sqrt_d(d))).to(q.dtype)


def lastq_scores(q: torch.Tensor, k: torch.Tensor, bs: int, logits_in_input_dtype: bool = True):
    """attention_sharing.py:127-167.  q [Hq,N,D], k [Hkv,N,D] -> vertical[Hq,N], slash[Hq,N] fp32.

    logits_in_input_dtype=True rounds the logits to q.dtype as the reference's einsum does.
    """
    hq, n, d = q.shape
    g = hq // k.shape[0]
    lq = scaled_last_q(q, bs)
    nq = lq.shape[1]
    vert = torch.empty(hq, n, dtype=torch.float32)
    slash = torch.empty(hq, n, dtype=torch.float32)
    ii = torch.arange(nq)
    causal = ii[:, None] >= ii[None, :]
    for h in range(hq):
        s = lq[h].float() @ k[h // g].float().T
        if logits_in_input_dtype:
            s = s.to(q.dtype).float()
        s[:, n - nq:] = s[:, n - nq:].masked_fill(~causal, float("-inf"))
        p = torch.softmax(s, dim=-1, dtype=torch.float32)
        vert[h] = p.mean(0)
        slash[h] = diagonal_sums(p) / nq
    return vert, slash


def pooled_qk_probs(q, kbar, bs, logits_in_input_dtype=True):
    """attention_sharing.py:197-200: softmax_fp32(mean_i(last_q) . avg_k) -> [Hq, nb].  kbar: [nb,Hkv,D]."""
    hq, n, d = q.shape
    g = hq // kbar.shape[1]
    lq = scaled_last_q(q, bs)
    qm = lq.float().mean(1).to(q.dtype)  # [Hq, D]
    out = torch.empty(hq, kbar.shape[0], dtype=torch.float32)
    for h in range(hq):
        s = kbar[:, h // g].float() @ qm[h].float()
        if logits_in_input_dtype:
            s = s.to(q.dtype).float()
        out[h] = torch.softmax(s, dim=-1, dtype=torch.float32)
    return out


def pool_q_head(qh: torch.Tensor, bs: int) -> torch.Tensor:
    """attention_sharing.py:350-356: per-block mean of one head's q[N,D] (zero pad, rescale tail)."""
    n, d = qh.shape
    nb = -(-n // bs)
    pad = nb * bs - n
    x = torch.nn.functional.pad(qh, (0, 0, 0, pad))
    avg = x.float().reshape(nb, bs, d).mean(1).to(qh.dtype)
    if pad:
        last = (avg[-1].float() * bs).to(qh.dtype)
        avg[-1] = (last.float() / (bs - pad)).to(qh.dtype)
    return avg


def block_probs(qbar_h, kbar_h, logits_in_input_dtype=True):
    """attention_sharing.py:357-360: softmax rows of (avg_q/sqrt(D)).avg_k^T with block-causal mask."""
    nb, d = qbar_h.shape
    qs = (qbar_h.float() * float(inv_sqrt_d(d))).to(qbar_h.dtype)
    s = qs.float() @ kbar_h.float().T
    if logits_in_input_dtype:
        s = s.to(qbar_h.dtype).float()
    tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    s = s.masked_fill(~tri, float("-inf"))
    return torch.softmax(s, dim=-1, dtype=torch.float32)


# --------------------------------------------------------------------------- #
# decode step
# --------------------------------------------------------------------------- #
def decode_attention(q, k, v, scale):
    """fp32 attention of one query token per head over the whole cache (no mask), the decode
    branch shareprefill_attn.py:146-155 (flash_attn_func with q_len = 1).

    q [Hq,D], k/v [Hkv,N,D] -> out fp32 [Hq,D]; query head h reads kv head h // (Hq/Hkv).
    """
    hq, d = q.shape
    g = hq // k.shape[0]
    out = torch.zeros(hq, d, dtype=torch.float32)
    for h in range(hq):
        s = (k[h // g].float() @ q[h].float()) * scale
        p = torch.softmax(s, dim=0)
        out[h] = p @ v[h // g].float()
    return out


# --------------------------------------------------------------------------- #
# masked attention (the fp32 output oracle) and the pivot's block-average map
# --------------------------------------------------------------------------- #
def rope_rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x bf16 [..., N, D], cos / sin bf16 [N, D] -> x*cos + rotate_half(x)*sin, bf16.

    The step in front of the attention function: the reference's patched model produces (cos, sin)
    (shareprefill/model_patch.py:121) and the Hugging Face attention layer it patches evaluates this
    expression with elementwise bf16 kernels, each of which computes in fp32 and rounds its result to bf16
    (nearest even).  Restated with those three roundings written out."""
    half = x.shape[-1] // 2
    xf = x.float()
    rot = torch.cat((-xf[..., half:], xf[..., :half]), dim=-1)  # negation and concatenation are exact
    a = (xf * cos.float()).to(torch.bfloat16).float()
    b = (rot * sin.float()).to(torch.bfloat16).float()
    return (a + b).to(torch.bfloat16)


def masked_attention_ref_roundings(q, k, v, mask, bs, scale):
    """The reference kernel's own arithmetic, shareprefill_attn.py:383-471, block by block in ascending key-block
    order: base-2 online softmax with the scale folded (softmax_scale * log2 e, :548-551), the probabilities of a
    block formed against the running maximum and ROUNDED TO bf16 before P.V (:418-420) while the row sum adds them
    unrounded (:409), fp32 accumulator rescaled by exp2(m_old - m_new), final scale exp2(m - lse), output rounded to
    bf16 (:471).  q [Hq,N,D], k/v [Hkv,N,D] bf16 or float, mask bool [Hq,nb,nb] -> out bf16 [Hq,N,D]."""
    hq, n, d = q.shape
    g = hq // k.shape[0]
    nb = -(-n // bs)
    out = torch.zeros(hq, n, d, dtype=torch.bfloat16)
    mask = np.asarray(mask)
    pos = torch.arange(n)
    sc = float(scale) * 1.44269504
    for h in range(hq):
        qh, kh = q[h].float(), k[h // g].float()
        vh = v[h // g].to(torch.bfloat16).float()
        for r in range(nb):
            r0, r1 = r * bs, min((r + 1) * bs, n)
            m = torch.full((r1 - r0,), float("-inf"))
            lse = torch.full((r1 - r0,), float("-inf"))
            acc = torch.zeros(r1 - r0, d)
            for c in np.nonzero(mask[h, r, : r + 1])[0]:
                c0, c1 = c * bs, min((c + 1) * bs, n)
                s = (qh[r0:r1] @ kh[c0:c1].T) * sc
                s = s.masked_fill(pos[None, c0:c1] > pos[r0:r1, None], float("-inf"))
                m_new = torch.maximum(m, s.max(dim=1).values)
                p = torch.exp2(s - m_new[:, None])
                l_blk = p.sum(dim=1)
                acc = acc * torch.exp2(m - m_new)[:, None] + p.to(torch.bfloat16).float() @ vh[c0:c1]
                lse = m_new + torch.log2(torch.exp2(lse - m_new) + l_blk)
                m = m_new
            out[h, r0:r1] = (acc * torch.exp2(m - lse)[:, None]).to(torch.bfloat16)
    return out


def masked_attention(q, k, v, mask, bs, scale, want_avg=None, emulate_bf16=False):
    """fp32 causal block-sparse attention, shareprefill_attn.py:272-471.

    q [Hq,N,D], k/v [Hkv,N,D], mask bool [Hq,nb,nb] -> out fp32 [Hq,N,D].
    want_avg: optional bool[Hq]; for those heads also returns avg[h,r,c] = mean over the
    block's valid queries of the softmax mass falling into key block c (:425-457).
    Only kept blocks are computed.
    emulate_bf16=True: the output comes from masked_attention_ref_roundings instead (the reference kernel's two
    bf16 roundings: probabilities before P.V, and the output), returned as fp32 values of bf16 numbers.
    """
    if emulate_bf16:
        out_b = masked_attention_ref_roundings(q, k, v, mask, bs, scale).float()
        if want_avg is None:
            return out_b, torch.zeros(q.shape[0], -(-q.shape[1] // bs), -(-q.shape[1] // bs))
        return out_b, masked_attention(q, k, v, mask, bs, scale, want_avg)[1]
    hq, n, d = q.shape
    g = hq // k.shape[0]
    nb = -(-n // bs)
    out = torch.zeros(hq, n, d, dtype=torch.float32)
    avg = torch.zeros(hq, nb, nb, dtype=torch.float32)
    mask = np.asarray(mask)
    pos = torch.arange(n)
    for h in range(hq):
        qh = q[h].float()
        kh = k[h // g].float()
        vh = v[h // g].float()
        for r in range(nb):
            cols = np.nonzero(mask[h, r, : r + 1])[0]
            r0, r1 = r * bs, min((r + 1) * bs, n)
            kidx = torch.cat([pos[c * bs: min((c + 1) * bs, n)] for c in cols])
            s = (qh[r0:r1] @ kh[kidx].T) * scale
            s = s.masked_fill(kidx[None, :] > pos[r0:r1, None], float("-inf"))
            p = torch.softmax(s, dim=-1)
            out[h, r0:r1] = p @ vh[kidx]
            if want_avg is not None and bool(want_avg[h]):
                colsum = p.sum(0) / float(r1 - r0)
                off = 0
                for c in cols:
                    w = min((c + 1) * bs, n) - c * bs
                    avg[h, r, c] = colsum[off: off + w].sum()
                    off += w
    return out, avg


# --------------------------------------------------------------------------- #
# cluster table + cross-layer state + one full layer
# --------------------------------------------------------------------------- #
class ClusterTable:
    """attention_sharing.py:368-384: {"clusters": {id: [[layer, head], ...]}, "shared_clusters": [...]}."""

    def __init__(self, clusters: Dict[str, List[List[int]]], shared_clusters):
        self.clusters = clusters
        self.shared = set(shared_clusters)

    def find(self, layer: int, head: int) -> Optional[str]:
        for cid, pairs in self.clusters.items():
            if [layer, head] in pairs:
                return cid
        return None


@dataclass
class PivotState:
    pivot_head: Optional[int] = None
    vert: Optional[torch.Tensor] = None
    slash: Optional[torch.Tensor] = None
    cols: Optional[np.ndarray] = None
    dists: Optional[np.ndarray] = None
    avg: Optional[np.ndarray] = None
    pattern: Optional[np.ndarray] = None  # bool [nb, nb]
    ratio: Optional[float] = None


@dataclass
class LayerResult:
    nv: np.ndarray = None
    ns: np.ndarray = None
    nv_final: np.ndarray = None
    ns_final: np.ndarray = None
    vert_tok: torch.Tensor = None
    slash_tok: torch.Tensor = None
    vert_blk: torch.Tensor = None
    slash_blk: torch.Tensor = None
    kbar: torch.Tensor = None
    avg_qk: torch.Tensor = None
    js_qa: torch.Tensor = None
    js_v: np.ndarray = None
    js_s: np.ndarray = None
    decision: np.ndarray = None
    mask: np.ndarray = None
    qa_probs: Dict[int, torch.Tensor] = field(default_factory=dict)
    out: torch.Tensor = None
    avg: torch.Tensor = None


class OracleSharing:
    """Cross-layer state, attention_sharing.py:41-78; reset at every model forward."""

    def __init__(self, table: ClusterTable):
        self.table = table
        self.reset_state()

    def reset_state(self):
        self.state: Dict[str, PivotState] = {cid: PivotState() for cid in self.table.clusters}

    # -- selection, attention_sharing.py:105-366 ---------------------------------
    def select(self, q, k, layer_idx, bs, min_budget_blocks, max_budget_blocks, pattern_threshold,
               similarity_threshold, fallback_threshold, queryaware_threshold,
               logits_in_input_dtype=True, inject: Optional[dict] = None) -> LayerResult:
        """inject: optional precomputed float intermediates (vert_tok, slash_tok, vert_blk, slash_blk,
        avg_qk, js_qa, js_v, js_s, qa_probs) replacing this function's own float arithmetic, so that
        the integer decisions can be compared bit-for-bit on identical scores."""
        inject = inject or {}
        hq, n, d = q.shape
        nb = -(-n // bs)
        maxb = min(max_budget_blocks, nb)
        minb = min_budget_blocks
        res = LayerResult()

        # Step A (attention_sharing.py:127-167)
        if "vert_tok" in inject:
            res.vert_tok, res.slash_tok = inject["vert_tok"], inject["slash_tok"]
        else:
            res.vert_tok, res.slash_tok = lastq_scores(q, k, bs, logits_in_input_dtype)

        # Step B (:169-180)
        def budget(x):
            b = cover_count(x, pattern_threshold) // bs + 1
            b = max(b, minb)
            return min(b, maxb)

        nv = np.array([budget(res.vert_tok[h].numpy()) for h in range(hq)], dtype=np.int64)
        ns = np.array([budget(res.slash_tok[h].numpy()) for h in range(hq)], dtype=np.int64)
        res.nv, res.ns = nv.copy(), ns.copy()
        res.vert_blk = inject.get("vert_blk", None)
        res.slash_blk = inject.get("slash_blk", None)
        if res.vert_blk is None:
            res.vert_blk = block_sum(res.vert_tok, bs)
            res.slash_blk = block_sum(res.slash_tok, bs)
        vert, slash = res.vert_blk, res.slash_blk

        # Step C (:193-202)
        res.kbar = pool_avg(k.transpose(0, 1).contiguous(), bs)  # [nb, Hkv, D]
        res.avg_qk = inject.get("avg_qk")
        if res.avg_qk is None:
            res.avg_qk = pooled_qk_probs(q, res.kbar, bs, logits_in_input_dtype)
        res.js_qa = inject.get("js_qa")
        if res.js_qa is None:
            res.js_qa = sqrt_js(res.avg_qk, vert)
        use_qa = (res.js_qa < np.float32(queryaware_threshold)).numpy()

        # Step D (:204-295)
        decision = np.full(hq, DEC_VS, dtype=np.int32)
        decision[use_qa] = DEC_QA
        mask = np.zeros((hq, nb, nb), dtype=bool)
        res.js_v = np.full(hq, np.nan, dtype=np.float32)
        res.js_s = np.full(hq, np.nan, dtype=np.float32)
        for h in range(hq):
            if use_qa[h]:
                continue
            cid = self.table.find(layer_idx, h)
            if cid is None or cid not in self.table.shared:
                continue
            st = self.state[cid]
            if st.pivot_head is None:
                st.pivot_head = h
                decision[h] = DEC_DENSE
                mask[h] = np.tril(np.ones((nb, nb), dtype=bool))
                st.vert, st.slash = vert[h].clone(), slash[h].clone()
                st.cols, st.dists = self._vs_sets(vert[h], slash[h], int(nv[h]), int(ns[h]), nb)
            elif st.pattern is not None:
                if "js_v" in inject:
                    jv, js_ = inject["js_v"][h], inject["js_s"][h]
                else:
                    jv = sqrt_js(st.vert, vert[h]).numpy()
                    js_ = sqrt_js(st.slash, slash[h]).numpy()
                res.js_v[h], res.js_s[h] = jv, js_
                if st.ratio is None:
                    st.ratio = vs_ratio(st.avg, st.cols, st.dists)
                if (np.float32(jv) < np.float32(similarity_threshold)
                        and np.float32(js_) < np.float32(similarity_threshold)
                        and st.ratio < fallback_threshold):
                    decision[h] = DEC_SHARE
                    mask[h] |= st.pattern

        # Step E (:297-337)
        for h in range(hq):
            if decision[h] in (DEC_QA, DEC_SHARE):
                nv[h] = minb
                ns[h] = minb
        res.nv_final, res.ns_final = nv, ns
        for h in range(hq):
            cols, dists = self._vs_sets(vert[h], slash[h], int(nv[h]), int(ns[h]), nb)
            mask[h] |= vs_mask(cols, dists, nb)

        # Step F (:339-364)
        for h in range(hq):
            if decision[h] != DEC_QA:
                continue
            if "qa_probs" in inject:
                a = inject["qa_probs"][h]
            else:
                g = hq // k.shape[0]
                a = block_probs(pool_q_head(q[h], bs), res.kbar[:, h // g], logits_in_input_dtype)
            res.qa_probs[h] = a
            kept = cover_keep_le(a.numpy().reshape(-1), pattern_threshold * nb)
            sel = np.zeros(nb * nb, dtype=bool)
            sel[kept] = True
            mask[h] |= sel.reshape(nb, nb) & np.tril(np.ones((nb, nb), dtype=bool))
            mask[h, 0, 0] = True

        res.decision, res.mask = decision, mask
        return res

    @staticmethod
    def _vs_sets(vert_h, slash_h, nv, ns, nb):
        """attention_sharing.py:231-251 / :303-329: force sink column and main diagonal, then top-k."""
        v = vert_h.clone().numpy()
        s = slash_h.clone().numpy()
        v[0] = np.inf
        s[nb - 1] = np.inf
        cols = topk_indices(v, min(nv, nb))
        dists = (nb - 1) - topk_indices(s, min(ns, nb))
        return cols, dists

    # -- state update, attention_sharing.py:94-103 -------------------------------
    def update_pivots(self, layer_idx, decision, avg, pattern_threshold):
        for h in np.nonzero(decision == DEC_DENSE)[0]:
            cid = self.table.find(layer_idx, int(h))
            st = self.state[cid]
            st.avg = np.asarray(avg[h], dtype=np.float32)
            pat = cover_keep_rows_ge(st.avg, pattern_threshold)
            pat &= np.tril(np.ones_like(pat))
            pat[0, 0] = True
            st.pattern = pat

    # -- one layer end-to-end, shareprefill_attn.py:87-155 -----------------------
    def layer(self, q, k, v, layer_idx, bs, min_budget, max_budget, pattern_threshold,
              similarity_threshold, fallback_threshold, queryaware_threshold, scale=None,
              logits_in_input_dtype=True, compute_attention=True, inject=None) -> LayerResult:
        """min_budget / max_budget in tokens (None allowed), converted as shareprefill_attn.py:112-122."""
        d = q.shape[-1]
        scale = (1.0 / math.sqrt(d)) if scale is None else scale
        minb = math.ceil((1 if min_budget is None else min_budget) / bs)
        maxb = math.ceil((2 ** 31 - 1 if max_budget is None else max_budget) / bs)
        res = self.select(q, k, layer_idx, bs, minb, maxb, pattern_threshold, similarity_threshold,
                          fallback_threshold, queryaware_threshold, logits_in_input_dtype, inject)
        if compute_attention:
            want = res.decision == DEC_DENSE
            res.out, res.avg = masked_attention(q, k, v, res.mask, bs, scale, want_avg=want)
            self.update_pivots(layer_idx, res.decision, res.avg.numpy(), pattern_threshold)
        return res


def mask_to_ids(mask_h: np.ndarray) -> np.ndarray:
    """Flat sorted unique block ids (row*nb + col) of one head's mask, shareprefill_attn.py:491-492."""
    nb = mask_h.shape[0]
    r, c = np.nonzero(mask_h)
    return (r.astype(np.int64) * nb + c).astype(np.int64)

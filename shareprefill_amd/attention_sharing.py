"""Cross-layer sparse-pattern sharing state and the per-layer block selection.

Host-side mirror of the reference's AttentionSharing (shareprefill/attn/attention_sharing.py:35-384)
with the same public methods (load_clusters, find_cluster_id, reset_state, get_active_blocks,
update_pivotal_attns, get_pivotal_pattern, get_pivotal_attn).  The data structures differ on purpose:

  * the per-cluster state (pivot head, pooled vectors, vertical-slash sets, coverage ratio, pattern)
    lives in fixed-size device slabs that the HIP kernels read and update, so one layer is a fixed
    sequence of kernel launches with no host synchronisation (the reference synchronises on every
    .nonzero() / .item() / torch.unique of its per-head Python loop);
  * block patterns are bit masks [Hq, nb, ceil(nb/64)] instead of ragged lists of flat block ids;
    ops.mask_to_block_idx converts a mask into the reference's list-of-id-tensors form;
  * keys are never expanded to the query-head count: kernels index KV head h // group.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from . import _lib, ops


@dataclass
class LayerPlan:
    """What the selection decided for one layer (all tensors on the device, nothing synchronised)."""

    layer_idx: int
    nb: int
    mask: torch.Tensor          # int64 [Hq, nb, nbw] block bit mask
    decision: torch.Tensor      # int32 [Hq]: 0 vertical-slash, 1 dense pivot, 2 shared, 3 query-aware
    nv: torch.Tensor            # int32 [Hq] vertical budgets before / after the min-budget reset
    ns: torch.Tensor
    nv_final: torch.Tensor
    ns_final: torch.Tensor
    vert_tok: Optional[torch.Tensor] = None
    slash_tok: Optional[torch.Tensor] = None
    vert_blk: Optional[torch.Tensor] = None
    slash_blk: Optional[torch.Tensor] = None
    kbar: Optional[torch.Tensor] = None
    avg_qk: Optional[torch.Tensor] = None
    js_qa: Optional[torch.Tensor] = None
    js_v: Optional[torch.Tensor] = None
    js_s: Optional[torch.Tensor] = None
    qa_probs: Optional[torch.Tensor] = None
    max_pivots: int = 0         # shared clusters with a head in this layer: no more heads than that can become pivots

    @property
    def use_dense(self) -> torch.Tensor:
        """bool [1, Hq], the reference's second return value (attention_sharing.py:366)."""
        return (self.decision == _lib.SP_DEC_DENSE).unsqueeze(0)

    def _need_mask(self) -> torch.Tensor:
        if self.mask is None:
            raise RuntimeError("this layer's block mask was released when the next layer was planned; set "
                               "AttentionSharing.keep_plans = True to keep every layer's mask")
        return self.mask

    def block_idx(self) -> List[List[torch.Tensor]]:
        """The reference's first return value: [B][Hq] sorted unique flat ids (synchronises)."""
        return [ops.mask_to_block_idx(self._need_mask(), self.nb)]

    def density(self) -> torch.Tensor:
        """Kept blocks / lower-triangular blocks per head (synchronises when read)."""
        kept = ops.mask_row_pointers(self._need_mask())[:, -1].to(torch.float64)
        return kept / (self.nb * (self.nb + 1) / 2)


class AttentionSharing:
    def __init__(self, sharing_lookup_path: str, flags: int = _lib.SP_FLAG_LOGITS_BF16):
        self.sharing_lookup_path = sharing_lookup_path
        self.clusters, self.shared_clusters = self.load_clusters(sharing_lookup_path)
        self.flags = flags
        # (layer, head) -> cluster id; the reference scans the lists linearly (:380-384)
        self._pair_to_cluster: Dict[Tuple[int, int], str] = {}
        for cid, pairs in self.clusters.items():
            for layer, head in pairs:
                self._pair_to_cluster.setdefault((int(layer), int(head)), cid)
        # device slot of every shared cluster, in table order
        self._slot: Dict[str, int] = {}
        for cid in self.clusters:
            if cid in self.shared_clusters:
                self._slot[cid] = len(self._slot)
        self._state: Optional[ops.ClusterState] = None
        self._head_cluster: Dict[Tuple[int, int, str], torch.Tensor] = {}
        # keep every pivot's block-average map in the device state for get_pivotal_attn (fp32 [nb, nb] per shared
        # cluster), unless all of them together exceed pivot_map_limit_bytes
        self.keep_pivot_maps = True
        self.pivot_map_limit_bytes = 4 << 30
        self.keep_debug = False   # keep every float intermediate of every layer (tests)
        self.keep_plans = False   # keep every layer's block mask (64 MiB per layer at 512K tokens) until the reset
        # one LayerPlan per layer planned since the last reset; unless keep_plans / keep_debug is set only the
        # newest one still holds its mask, the older ones keep their few per-head integers
        self.plans: List[LayerPlan] = []
        self._scratch: Dict[Tuple[str, str], torch.Tensor] = {}
        self._max_pivots: Dict[Tuple[int, int], int] = {}
        self.reset_state()

    # ---- table ------------------------------------------------------------------------------------
    @staticmethod
    def load_clusters(file_path: str):
        """{"clusters": {id: [[layer, head], ...]}, "shared_clusters": [ids]} (attention_sharing.py:368-378)."""
        if not os.path.exists(file_path):
            raise FileNotFoundError(f"Sharing lookup file not found: {file_path}")
        with open(file_path, "r") as f:
            info = json.load(f)
        if "clusters" not in info or "shared_clusters" not in info:
            raise ValueError(f"{file_path}: expected the keys 'clusters' and 'shared_clusters'")
        clusters = {str(k): [[int(a), int(b)] for a, b in v] for k, v in info["clusters"].items()}
        return clusters, set(str(c) for c in info["shared_clusters"])

    def find_cluster_id(self, layer: int, head: int) -> Optional[str]:
        return self._pair_to_cluster.get((int(layer), int(head)))

    def _head_cluster_tensor(self, layer_idx: int, hq: int, device) -> torch.Tensor:
        key = (layer_idx, hq, str(device))
        t = self._head_cluster.get(key)
        if t is None:
            slots = [self._slot.get(self._pair_to_cluster.get((layer_idx, h)), -1) for h in range(hq)]
            t = torch.tensor(slots, dtype=torch.int32, device=device)
            self._head_cluster[key] = t
        return t

    # ---- state ------------------------------------------------------------------------------------
    def reset_state(self):
        """Forget every pivot (attention_sharing.py:41-78); called at the start of each model forward."""
        if self._state is not None:
            self._state.reset()
        self.plans = []
        self.dense_layers = 0
        self._dense_heads = 0

    def _ensure_state(self, nb: int, device) -> ops.ClusterState:
        st = self._state
        keep = self.keep_pivot_maps and max(len(self._slot), 1) * nb * nb * 4 <= self.pivot_map_limit_bytes
        if st is None or st.nb != nb or st.device != device or (st.avg_map is not None) != keep:
            st = ops.ClusterState(len(self._slot), nb, device, keep_maps=keep)
            self._state = st
        return st

    def get_pivotal_pattern(self, layer_idx: int, b: int, h: int) -> Optional[torch.Tensor]:
        """Pivot block pattern of the head's cluster as a bit mask [nb, nbw], or None (synchronises)."""
        cid = self.find_cluster_id(layer_idx, h)
        if self._state is None or cid not in self._slot:
            return None
        s = self._slot[cid]
        if int(self._state.info[s, 1]) == 0:
            return None
        return self._state.pattern[s]

    def get_pivotal_attn(self, layer_idx: int, b: int, h: int) -> Optional[torch.Tensor]:
        """The pivot's [nb, nb] block-average attention map of the head's cluster, or None while the cluster has no
        pivot (attention_sharing.py:87-92; synchronises).  The maps live in the device state ([nb, nb] fp32 per
        shared cluster, written by the pivot update); with keep_pivot_maps = False, or when they would exceed
        pivot_map_limit_bytes, they are not kept and this returns None."""
        cid = self.find_cluster_id(layer_idx, h)
        if self._state is None or self._state.avg_map is None or cid not in self._slot:
            return None
        s = self._slot[cid]
        if int(self._state.info[s, 1]) == 0:
            return None
        return self._state.avg_map[s]

    def pivot_summary(self) -> Dict[str, dict]:
        """Host copy of the per-cluster state (synchronises); for logging and tests."""
        out = {}
        if self._state is None:
            return out
        info, ratio = self._state.info.cpu(), self._state.ratio.cpu()
        for cid, s in self._slot.items():
            out[cid] = {"pivot_head": int(info[s, 0]), "has_pattern": bool(info[s, 1]), "nv": int(info[s, 2]),
                        "ns": int(info[s, 3]), "layer": int(info[s, 4]), "vs_ratio": float(ratio[s])}
        return out

    # ---- per-layer selection --------------------------------------------------------------------------
    def plan_layer(self, q: torch.Tensor, k: torch.Tensor, layer_idx: int, block_size: int, min_budget: int,
                   max_budget: int, pattern_threshold: float = 0.9, similarity_threshold: float = 0.5,
                   fallback_threshold: float = 0.9, queryaware_threshold: float = 0.1,
                   scale_dim: Optional[int] = None) -> LayerPlan:
        """q [Hq, N, D], k [Hkv, N, D] bf16 views; budgets in blocks.  Enqueues the whole selection.
        scale_dim: the model's head_dim when q / k have been zero-padded to D (the scores then scale by
        1/sqrt(scale_dim), attention_sharing.py:127 of the reference)."""
        hq, n, d = q.shape
        nb = -(-n // block_size)
        maxb = min(max_budget, nb)
        minb = min_budget  # clamped after maxb exactly as attention_sharing.py:173-176 orders the two clamps
        dev = q.device
        state = self._ensure_state(nb, dev)
        hc = self._head_cluster_tensor(layer_idx, hq, dev)

        flags = self.flags | (_lib.SP_FLAG_SCALE_DIM(scale_dim) if scale_dim and scale_dim != d else 0)
        vert_tok, slash_tok, vert_blk, slash_blk = ops.lastq_scores(q, k, block_size, flags)
        nv, ns = ops.cover_budgets(vert_tok, slash_tok, block_size, pattern_threshold, minb, maxb)
        kbar = ops.pool_avg(k, block_size)
        avg_qk, js_qa, use_qa = ops.queryaware_test(q, kbar, vert_blk, block_size, queryaware_threshold, flags)
        decision, js_v, js_s, nv_f, ns_f = ops.share_decide(state, hc, layer_idx, vert_blk, slash_blk, use_qa, nv, ns,
                                                            minb, similarity_threshold, fallback_threshold)
        mask = ops.build_mask(state, hc, decision, vert_blk, slash_blk, nv_f, ns_f)
        # query-aware heads: pooled Q only for them (head_enable), selection skipped on device for the others
        qbar = ops.pool_avg(q, block_size, tail_mode=_lib.SP_POOL_TAIL_RESCALE, head_enable=use_qa)
        qa_probs = ops.queryaware_select(qbar, kbar, decision, mask, pattern_threshold, flags,
                                         probs=self._qa_scratch(hq, nb, dev))
        plan = LayerPlan(layer_idx, nb, mask, decision, nv, ns, nv_f, ns_f)
        plan.max_pivots = self.max_pivots(layer_idx, hq)
        if self.keep_debug:
            plan.vert_tok, plan.slash_tok, plan.vert_blk, plan.slash_blk = vert_tok, slash_tok, vert_blk, slash_blk
            plan.kbar, plan.avg_qk, plan.js_qa, plan.js_v, plan.js_s = kbar, avg_qk, js_qa, js_v, js_s
            plan.qa_probs = qa_probs.clone()
        if self.plans and not (self.keep_plans or self.keep_debug):
            self.plans[-1].mask = None
        self.plans.append(plan)
        return plan

    def max_pivots(self, layer_idx: int, hq: int) -> int:
        """Shared clusters with a head in this layer: no more heads than that can become pivots in it."""
        key = (layer_idx, hq)
        n = self._max_pivots.get(key)
        if n is None:
            n = len({self._slot[c] for h in range(hq)
                     for c in (self._pair_to_cluster.get((layer_idx, h)),) if c in self._slot})
            self._max_pivots[key] = n
        return n

    def _qa_scratch(self, hq: int, nb: int, device) -> torch.Tensor:
        """fp32 [Hq, nb, nb] scratch of the query-aware selection, owned by this object (one model, one stream of
        layers in order), grow-only, reused by every layer."""
        need = hq * nb * nb * 4
        key = ("qa_probs", str(device))
        buf = self._scratch.get(key)
        if buf is None or buf.numel() < need:
            buf = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
            self._scratch[key] = buf
        return buf[:need].view(torch.float32).view(hq, nb, nb)

    def get_active_blocks(self, q, k, layer_idx, num_heads, block_size, min_budget, max_budget,
                          pattern_threshold=0.9, similarity_threshold=0.5, fallback_threshold=0.9,
                          queryaware_threshold=0.1, gqa_interleave=False, as_ids=False):
        """Reference signature (attention_sharing.py:105-119): q [B, N, Hq, D], k [B, N, Hkv or Hq, D].

        Returns (block bit mask [B, Hq, nb, nbw], use_dense bool [B, Hq]).  With as_ids=True the first value is the
        reference's form instead (attention_sharing.py:366): list[B][Hq] of sorted unique int64 flat block ids
        row * nb + col; building the ragged lists synchronises the stream."""
        if gqa_interleave and k.shape[2] != q.shape[2]:
            # with un-expanded K the reference's second einsum (attention_sharing.py:141-151) gives query head h the kv
            # head h % Hkv; its own attention function never gets here with un-expanded K (it expands first, after
            # which the flag changes nothing), so only this direct call can ask for that mapping
            raise NotImplementedError("gqa_interleave=True with un-expanded K (query head h -> kv head h % Hkv) is not "
                                      "supported; with K expanded to the query head count the flag changes nothing")
        if q.shape[0] != 1:
            raise ValueError("SharePrefill keeps per-cluster state for batch size 1 only")
        model_dim = q.shape[-1]
        if model_dim in (16, 32, 64):  # the kernels are built for head_dim 128: zero-padded q / k give the same scores
            q, k = (torch.nn.functional.pad(t, (0, 128 - model_dim)) for t in (q, k))
        plan = self.plan_layer(q[0].transpose(0, 1), k[0].transpose(0, 1), layer_idx, block_size, min_budget,
                               max_budget, pattern_threshold, similarity_threshold, fallback_threshold,
                               queryaware_threshold, scale_dim=model_dim)
        if as_ids:
            return plan.block_idx(), plan.use_dense
        return plan.mask.unsqueeze(0), plan.use_dense

    def update_pivotal_attns(self, layer_idx, avg_attn, use_dense, pattern_threshold=0.9):
        """Turns this layer's pivot maps into patterns (attention_sharing.py:94-103); avg_attn [B, Hq, nb, nb].

        `use_dense` may be the bool [B, Hq] tensor of the reference or the int32 decision vector."""
        if self._state is None:
            return
        hq = avg_attn.shape[1]
        hc = self._head_cluster_tensor(layer_idx, hq, avg_attn.device)
        if use_dense.dtype == torch.bool:
            # a caller's own flags may name heads outside every shared cluster: those keep no pattern
            decision = (use_dense.reshape(-1) & (hc >= 0)).to(torch.int32) * _lib.SP_DEC_DENSE
        else:
            decision = use_dense.reshape(-1)
        ops.pivot_update(self._state, hc, decision, avg_attn[0], pattern_threshold)

    def note_dense_layer(self, layer_idx: int, hq: int, nb: int) -> None:
        """A layer whose prompt is no longer than the minimum budget ran on the dense causal mask without any
        selection (see shareprefill_attention_core); counted for decision_histogram."""
        self.dense_layers += 1
        self._dense_heads += hq

    # ---- counters -----------------------------------------------------------------------------------------
    def decision_histogram(self) -> Dict[str, int]:
        """Counts of vertical-slash / dense / shared / query-aware heads over the layers planned since the
        last reset (synchronises)."""
        names = {0: "vertical_slash", 1: "dense_pivot", 2: "shared", 3: "query_aware"}
        out = {v: 0 for v in names.values()}
        if self.dense_layers:
            out["all_blocks_kept_no_selection"] = self._dense_heads
        for p in self.plans:
            for code, cnt in zip(*torch.unique(p.decision.cpu(), return_counts=True)):
                out[names[int(code)]] += int(cnt)
        return out


def budget_blocks(min_budget: Optional[int], max_budget: Optional[int], block_size: int) -> Tuple[int, int]:
    """Token budgets -> block budgets (shareprefill/attn/shareprefill_attn.py:112-122)."""
    mn = 1 if min_budget is None else min_budget
    mx = 2 ** 31 - 1 if max_budget is None else max_budget
    return math.ceil(mn / block_size), math.ceil(mx / block_size)

"""The patched attention function (Hugging Face attention-interface signature).

Mirror of shareprefill/attn/shareprefill_attn.py:87-184 of the reference.  Differences, all on purpose:
  * K / V are not expanded to the query-head count and nothing is transposed to contiguous: the HIP
    kernels take the [B, H, N, D] views Hugging Face hands over with their real strides;
  * selection and attention run as a fixed sequence of kernel launches on the current stream, without
    host synchronisation;
  * there is no CPU path: tensors must be on a GPU and the HIP library must be built.
"""

from __future__ import annotations

import logging
import math
from typing import Optional, Tuple

import torch

from . import _lib, ops
from .attention_sharing import budget_blocks

LOGGER = logging.getLogger(__name__)


_dense_masks = {}

KERNEL_HEAD_DIM = 128
PADDED_HEAD_DIMS = (16, 32, 64)  # the reference's other head sizes (shareprefill_attn.py:503-508)


def pad_head_dim(*tensors: torch.Tensor):
    """The kernels are built for head_dim 128.  The reference's smaller head sizes run on them with the head_dim axis
    zero-padded: no dot product changes (q.k gains exact zeros, the extra output channels are P.0 = 0 and are cut
    off again), the softmax scale and the selection's 1/sqrt(head_dim) keep the model's head_dim.  Costs a copy of
    q / k / v; the attention kernel is told that channels 64.. are zero and skips their products (SP_ATTN_HALF_CHANNELS),
    so its arithmetic is that of head_dim 64."""
    d = tensors[0].shape[-1]
    return tuple(torch.nn.functional.pad(t, (0, KERNEL_HEAD_DIM - d)) for t in tensors)



def _dense_causal_mask(hq: int, nb: int, device) -> torch.Tensor:
    """Bit mask with every lower-triangular block set, cached per shape (short prompts ask for it in every layer)."""
    key = (hq, nb, str(device))
    m = _dense_masks.get(key)
    if m is None:
        tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool, device=device))
        m = ops.bool_to_mask(tri).unsqueeze(0).expand(hq, -1, -1).contiguous()
        if nb <= 64:
            _dense_masks[key] = m
    return m


def triton_column_count_cumsum(x: torch.Tensor, num_columns: int) -> torch.Tensor:
    """The reference's helper of this name (shareprefill_attn.py:226-269), here a HIP kernel: x [B, H, K] flat block
    ids of an num_columns x num_columns grid -> int32 [B, H, num_columns + 1], the running count of ids per grid row
    (ids outside the grid are padding).  Its docstring example: ids [0, 5, 8, 9, 13, 14] in a 4 x 4 grid ->
    [0, 1, 2, 4, 6]."""
    if x.dim() != 3:
        raise ValueError("x must be [batch_size, num_heads, activated_block_num]")
    return torch.stack([ops.block_idx_row_pointers(x[b], num_columns) for b in range(x.shape[0])])


def _pad_block_idx(block_idx, batch_size: int, num_heads: int, pad: int, device) -> torch.Tensor:
    """list[B][H] of id tensors -> [B, H, K] padded with `pad` (shareprefill_attn.py:528-540)."""
    if isinstance(block_idx, torch.Tensor):
        assert block_idx.dim() == 3 and block_idx.shape[0] == batch_size and block_idx.shape[1] == num_heads
        return block_idx
    assert (isinstance(block_idx, list) and isinstance(block_idx[0], list)
            and isinstance(block_idx[0][0], torch.Tensor))
    assert len(block_idx) == batch_size and len(block_idx[0]) == num_heads
    flat = [t.reshape(-1).to(device=device, dtype=torch.int64) for row in block_idx for t in row]
    out = torch.nn.utils.rnn.pad_sequence(flat, batch_first=True, padding_value=pad)
    return out.view(batch_size, num_heads, -1)


def triton_block_wise_prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, block_idx,
                                        heads_need_blockwise_attn_mask: torch.Tensor, block_size: int,
                                        grid_offset: int = 0, softmax_scale: Optional[float] = None,
                                        gqa_interleave: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """The reference's kernel wrapper under its own name and arguments (shareprefill_attn.py:474-620), served by the
    HIP block-sparse attention kernel (nothing here is Triton).

    q [B, N, Hq, D], k / v [B, N, Hkv, D] bf16 (any strides with a contiguous head_dim axis); block_idx the
    activated blocks as flat ids row * nb + col, either list[B][Hq] of tensors or one padded tensor [B, Hq, K];
    heads_need_blockwise_attn_mask bool [B, Hq]: the heads whose block-average attention map is wanted.
    Returns (out [B, N, Hq, D] bf16, avg_attn fp32 [B, Hq, nb, nb], zero for the other heads).
    gqa_interleave: query head h reads kv head h % Hkv instead of h // (Hq / Hkv) (shareprefill_attn.py:333-336).
    block_size 16 / 32 / 64 / 128 as in the reference (:509-516); below 128 the kernel walks the 128-token blocks that
    hold an activated block and drops the rest of each per 16 x 16 sub-tile: exact, not tuned.  Only grid_offset == 0
    is built; head_dim 16 / 32 / 64 run zero-padded to 128 (pad_head_dim)."""
    batch_size, q_len, num_q_heads, model_dim = q.shape
    _, k_len, num_kv_heads, _ = k.shape
    assert q.dtype == torch.bfloat16
    assert q_len == k_len
    assert num_q_heads % num_kv_heads == 0
    assert model_dim in PADDED_HEAD_DIMS + (KERNEL_HEAD_DIM,), "only support head_dim in {16, 32, 64, 128}"
    assert block_size in (16, 32, 64, 128), "only support block_size in {16, 32, 64, 128}"
    if model_dim != KERNEL_HEAD_DIM:
        q, k, v = pad_head_dim(q, k, v)
    head_dim = q.shape[-1]
    if grid_offset != 0:
        raise NotImplementedError("grid_offset != 0 is not supported (the SharePrefill path never sets it)")
    nb = -(-q_len // block_size)
    dev = q.device
    idx = _pad_block_idx(block_idx, batch_size, num_q_heads, nb * (nb + 1), dev)
    need = heads_need_blockwise_attn_mask.to(device=dev).reshape(batch_size, num_q_heads) != 0
    scale = 1.0 / math.sqrt(model_dim) if softmax_scale is None else float(softmax_scale)
    g = num_q_heads // num_kv_heads
    interleave = bool(gqa_interleave) and 1 < num_kv_heads < num_q_heads
    # room for the block sums of every head that may want its map (at most 2 GiB of it; the rest recompute)
    slab = _lib.load().sp_attn_pivot_scratch_bytes(q_len, block_size)
    max_pivots = min(num_q_heads, (2 << 30) // slab)
    outs, avgs = [], []
    for b in range(batch_size):
        qb, idx_b, need_b = q[b].transpose(0, 1), idx[b], need[b]
        if interleave:
            # the kernel gives query head h the kv head h // g: put the heads of kv head j (j, j + Hkv, ...) side by side
            qb = qb.reshape(g, num_kv_heads, q_len, head_dim).transpose(0, 1).reshape(num_q_heads, q_len, head_dim)
            idx_b = idx_b.reshape(g, num_kv_heads, -1).transpose(0, 1).reshape(num_q_heads, -1)
            need_b = need_b.reshape(g, num_kv_heads).transpose(0, 1).reshape(num_q_heads)
        mask = ops.block_idx_to_mask(idx_b, nb)
        decision = torch.where(need_b, _lib.SP_DEC_DENSE, _lib.SP_DEC_VS).to(torch.int32)
        avg = torch.zeros(num_q_heads, nb, nb, dtype=torch.float32, device=dev)
        out = ops.block_sparse_attention(qb, k[b].transpose(0, 1), v[b].transpose(0, 1), mask, block_size, scale,
                                         decision=decision, avg_attn=avg, max_pivots=max_pivots,
                                         half_channels=model_dim != KERNEL_HEAD_DIM)
        if interleave:
            out = out.reshape(q_len, num_kv_heads, g, head_dim).transpose(1, 2).reshape(q_len, num_q_heads, head_dim)
            avg = avg.reshape(num_kv_heads, g, nb, nb).transpose(0, 1).reshape(num_q_heads, nb, nb)
        outs.append(out[..., :model_dim])
        avgs.append(avg)
    return torch.stack(outs), torch.stack(avgs)


def shareprefill_attention_core(module, query_states: torch.Tensor, key_states: torch.Tensor,
                                value_states: torch.Tensor, *, gqa_interleave: bool = False
                                ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """query_states [B, Hq, N, D], key/value_states [B, Hkv, Nk, D] -> (attn_output [B, Hq, N, D], avg_attn).

    Prefill (N != 1): vertical/slash estimation, block selection and sharing, block-sparse attention,
    pivot update (shareprefill_attn.py:110-144).  Decode (N == 1): dense attention of the one query over
    all keys (:146-155)."""
    bsz, num_heads, q_len, model_dim = query_states.shape
    config = module.config
    softmax_scale = getattr(module, "scaling", 1.0 / math.sqrt(model_dim))
    # gqa_interleave is accepted and changes nothing, as in the reference: there K and V are expanded to the query
    # head count before anything else, by repeat_interleave (True) or by expand + reshape (False) -- both give query
    # head h the kv head h // g (shareprefill_attn.py:33-40, 77-82) -- and everything after sees one kv head per query
    # head, so neither the selection's einsum (attention_sharing.py:128-151) nor the kernel's head mapping
    # (shareprefill_attn.py:333-336) can tell the two settings apart.  Here K and V stay un-expanded and are indexed h // g.
    del gqa_interleave

    if q_len == 1:
        # decode step (shareprefill_attn.py:146-155): one query against the whole cache, nothing is selected.
        # The HIP kernel is the only path (bf16, head_dim a multiple of 8 up to 128 -- smaller heads are padded inside
        # the kernel, the cache is read as it is -- at most 32 query heads per kv head, 16-byte aligned rows); anything
        # else raises from the entry point's own checks, as every other unsupported shape does.
        if query_states.dtype != torch.bfloat16:
            raise AssertionError(f"SharePrefill attention expects bfloat16 q/k/v, got {query_states.dtype}")
        outs = [ops.decode_attention(query_states[b, :, 0], key_states[b], value_states[b], softmax_scale)
                for b in range(bsz)]
        return torch.stack(outs).unsqueeze(2), None

    if bsz != 1:
        raise ValueError("SharePrefill prefill keeps per-cluster state for batch size 1 only")
    if model_dim in PADDED_HEAD_DIMS:
        query_states, key_states, value_states = pad_head_dim(query_states, key_states, value_states)
    head_dim = query_states.shape[-1]
    assert query_states.dtype == torch.bfloat16, "SharePrefill attention expects bfloat16 q/k/v"
    assert key_states.shape[2] == q_len, "prefill expects q_len == k_len (no cached prefix)"
    _lib.load()

    q, k, v = query_states[0], key_states[0], value_states[0]
    block_size = config.block_size
    nb = -(-q_len // block_size)
    sharing = module.attention_sharing
    minb, maxb = budget_blocks(config.min_budget, config.max_budget, block_size)
    if q_len < block_size or (nb <= minb and nb <= maxb and getattr(config, "dense_short_prompts", True)):
        # (a) Shorter than one block: a single diagonal block, nothing to select (the reference cannot run here).
        # (b) The prompt has no more blocks than the minimum budget, nor than the maximum.  Every head's budgets are
        # then raised to min_budget and cut to min(max_budget, nb) = nb (attention_sharing.py:173-176; with a maximum
        # BELOW nb the cut leaves max_budget columns and distances, a sparse mask, so that case takes the full path),
        # its vertical-slash set is
        # every column and every distance, and whatever the head's decision (pivot, shared, query-aware, fallback) its
        # mask is the whole lower triangle -- in this layer and, with the same prompt, in every later one.  Nothing the
        # selection computes can change an output, so it is skipped and the attention runs on the dense mask: the
        # same result at a fraction of the launches.  What is not produced on this path: decisions, pivot state and
        # the pivots' block-average maps (attn_weights is all zeros).  config.dense_short_prompts = False takes the
        # full path instead.
        avg_attn = torch.zeros(1, num_heads, nb, nb, dtype=torch.float32, device=q.device)
        mask = _dense_causal_mask(num_heads, nb, q.device)
        out = ops.block_sparse_attention(q, k, v, mask, block_size, softmax_scale, pair_rows=True,
                                         half_channels=model_dim != head_dim)
        if q_len >= block_size:
            sharing.note_dense_layer(module.layer_idx, num_heads, nb)
        return out.unsqueeze(0).transpose(1, 2)[..., :model_dim], avg_attn

    # Room for the block sums of this layer's possible pivots (at most 16 GiB of it; pivots beyond that take the
    # recomputing pass).  How many heads can become pivots is known from the table alone.
    slab = _lib.load().sp_attn_pivot_scratch_bytes(q_len, block_size)
    max_pivots = min(sharing.max_pivots(module.layer_idx, num_heads), (16 << 30) // slab)
    ws = ops.attention_workspace(q_len, num_heads, key_states.shape[1], head_dim, block_size, q.device, max_pivots)
    avg_attn = torch.empty(1, num_heads, nb, nb, dtype=torch.float32, device=q.device)
    ops.repack_v(v, block_size, ws[0])
    avg_attn.zero_()
    plan = sharing.plan_layer(q, k, module.layer_idx, block_size, minb, maxb, config.pattern_threshold,
                              config.similarity_threshold, config.fallback_threshold, config.queryaware_threshold,
                              scale_dim=model_dim)
    out = ops.block_sparse_attention(q, k, v, plan.mask, block_size, softmax_scale, decision=plan.decision,
                                     avg_attn=avg_attn[0], max_pivots=max_pivots, workspace=ws,
                                     half_channels=model_dim != head_dim)
    sharing.update_pivotal_attns(module.layer_idx, avg_attn, plan.decision, config.pattern_threshold)
    return out.unsqueeze(0).transpose(1, 2)[..., :model_dim], avg_attn


def shareprefill_attention_forward(module, query_states: torch.Tensor, key_states: torch.Tensor,
                                   value_states: torch.Tensor, attention_mask: Optional[torch.Tensor], *,
                                   scaling: float, dropout: float = 0.0, **kwargs
                                   ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Attention-interface entry (shareprefill_attn.py:158-184): returns (attn_output [B, N, Hq, D] contiguous,
    attn_weights), attn_weights being the block-average map [B, Hq, nb, nb] on prefill and None on decode.
    As in the reference, attention_mask / scaling / dropout are ignored (module.scaling is used) and a
    sliding window is rejected."""
    if kwargs.pop("sliding_window", None) is not None:
        raise NotImplementedError("SharePrefill attention does not support sliding-window mode yet.")
    gqa_interleave = kwargs.pop("gqa_interleave", False)
    attn_output, attn_weights = shareprefill_attention_core(module, query_states, key_states, value_states,
                                                            gqa_interleave=gqa_interleave)
    return attn_output.transpose(1, 2).contiguous(), attn_weights

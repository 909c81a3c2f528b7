"""Kernel wrappers of the reference's attn/utils.py under their own names, served by the HIP library."""

from __future__ import annotations

import torch

from . import ops


def triton_bnhd_pool(x: torch.Tensor, kernel_size: int, pool_type: str = "avg") -> torch.Tensor:
    """x bf16 [B, N, H, D] -> [B, ceil(N / kernel_size), H, D]: every run of kernel_size tokens reduced by pool_type
    (attn/utils.py:211-261; nothing here is Triton): "avg" (the last run divided by its true length; the one the
    selection uses, attention_sharing.py:194-196), "max", "min", "maxabs", "sum", or the slicing mode "last".

    As in the reference's kernel a ragged last run is filled up with zeros, which a maximum / minimum then sees.  Sums
    are kept in fp32 and rounded once (the reference's kernel adds in bf16); an unknown pool_type is a KeyError, as
    from the reference's own dictionary (attn/utils.py:254-256)."""
    if x.dim() != 4:
        raise ValueError("x must be [batch_size, seq_len, num_heads, head_dim]")
    if pool_type == "last":
        if x.shape[1] % kernel_size == 0:
            return x[:, kernel_size - 1::kernel_size, ...]
        return torch.cat((x[:, kernel_size - 1::kernel_size, ...], x[:, -1:, ...]), dim=1)
    assert x.shape[-1] in {16, 32, 64, 128}
    assert kernel_size in {16, 32, 64, 128, 256, 512}
    if pool_type == "avg":
        return torch.stack([ops.pool_avg(x[b].transpose(0, 1), kernel_size) for b in range(x.shape[0])])
    return torch.stack([ops.pool(x[b].transpose(0, 1), kernel_size, pool_type) for b in range(x.shape[0])])


def score_cover_topk(x: torch.Tensor, score: float) -> torch.Tensor:
    """count(cumsum(sort_descending(x)) <= score) + 1 over the last axis (attn/utils.py:47-50), int64 like the
    reference's; x fp32 [..., L] on the GPU."""
    lead = x.shape[:-1]
    flat = x.reshape(-1, x.shape[-1]).to(torch.float32).contiguous()
    return ops.cover_count(flat, float(score)).to(torch.int64).reshape(lead)


__all__ = ["triton_bnhd_pool", "score_cover_topk"]

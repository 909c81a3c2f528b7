"""Kernel wrappers of the reference's attn/utils.py under their own names, served by the HIP library."""

from __future__ import annotations

import torch

from . import ops


def triton_bnhd_pool(x: torch.Tensor, kernel_size: int, pool_type: str = "avg") -> torch.Tensor:
    """x bf16 [B, N, H, D] -> [B, ceil(N / kernel_size), H, D]: the mean of every run of kernel_size tokens, the last
    run divided by its true length (attn/utils.py:211-261; nothing here is Triton).

    Of the reference's pool types only "avg", the one its selection uses (attention_sharing.py:194-196), and the
    slicing mode "last" are built.  The sum is kept in fp32 and rounded once (the reference's kernel adds in bf16)."""
    if x.dim() != 4:
        raise ValueError("x must be [batch_size, seq_len, num_heads, head_dim]")
    if pool_type == "last":
        if x.shape[1] % kernel_size == 0:
            return x[:, kernel_size - 1::kernel_size, ...]
        return torch.cat((x[:, kernel_size - 1::kernel_size, ...], x[:, -1:, ...]), dim=1)
    if pool_type != "avg":
        raise NotImplementedError(f"pool_type {pool_type!r}: only 'avg' and 'last' are built")
    return torch.stack([ops.pool_avg(x[b].transpose(0, 1), kernel_size) for b in range(x.shape[0])])


def score_cover_topk(x: torch.Tensor, score: float) -> torch.Tensor:
    """count(cumsum(sort_descending(x)) <= score) + 1 over the last axis (attn/utils.py:47-50), int64 like the
    reference's; x fp32 [..., L] on the GPU."""
    lead = x.shape[:-1]
    flat = x.reshape(-1, x.shape[-1]).to(torch.float32).contiguous()
    return ops.cover_count(flat, float(score)).to(torch.int64).reshape(lead)


__all__ = ["triton_bnhd_pool", "score_cover_topk"]

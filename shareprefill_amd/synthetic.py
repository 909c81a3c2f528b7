"""Seeded synthetic workloads for the SharePrefill attention layer.

Q, K, V are i.i.d. N(0,1) with planted structure:
  * sink (vertical) tokens: K[:, 0:64] is scaled by 4;
  * slash band: a positional feature shared by Q and K is written into the first
    2*n_pairs channels so that q_i.k_j gains a bump for |i-j| within roughly 256 tokens
    (random-frequency rotary pairs, so the bump depends on i-j only).
Tensors are generated token-major ([N, H, D]) and handed out as the [1, H, N, D] strided
views a Hugging Face attention module passes to its attention function.

Cluster tables use the reference JSON schema
({"clusters": {id: [[layer, head], ...]}, "shared_clusters": [ids]},
shareprefill/attn/attention_sharing.py:368-378).
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    hq: int
    hkv: int
    head_dim: int
    seq_len: int
    n_clusters: int
    seed: int
    block_size: int = 128
    min_budget: int = 1024
    pattern_threshold: float = 0.95
    similarity_threshold: float = 0.5
    fallback_threshold: float = 0.9
    queryaware_threshold: float = 0.1


WORKLOADS: Dict[str, Workload] = {
    "C1": Workload("C1", 8, 2, 128, 8192, 2, 1235),
    "C2": Workload("C2", 32, 8, 128, 32768, 8, 1236),
    "C3": Workload("C3", 32, 8, 128, 131072, 8, 1237),
    "C5": Workload("C5", 28, 4, 128, 262144, 4, 1239),
}

SINK_TOKENS = 64
SINK_SCALE = 4.0
BAND_PAIRS = 16
BAND_WIDTH = 256
BAND_BETA = 2.2
HEAD_GAIN = 1.0


def planted_qkv(hq: int, hkv: int, n: int, d: int, seed: int, device="cpu", dtype=torch.bfloat16,
                q_head_gain: float = 0.0):
    """Returns q [1,hq,n,d], k, v [1,hkv,n,d] (strided views of token-major storage).

    The random draw happens on `device` with a generator seeded by `seed`; a CPU draw and a GPU
    draw with the same seed are different tensors, so parity tests draw on the CPU and copy.
    q_head_gain > 0 gives head h an extra factor (1 + gain*h/hq) on its positional feature,
    which spreads heads between slash-dominated and sink-dominated behaviour.
    """
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    q = torch.randn(n, hq, d, generator=gen, device=device, dtype=torch.float32)
    k = torch.randn(n, hkv, d, generator=gen, device=device, dtype=torch.float32)
    v = torch.randn(n, hkv, d, generator=gen, device=device, dtype=torch.float32)
    k[:SINK_TOKENS] *= SINK_SCALE
    fgen = torch.Generator(device="cpu")
    fgen.manual_seed(seed + 7919)
    pairs = min(BAND_PAIRS, d // 2)  # head sizes below 32 channels carry as many band features as fit
    omega = (torch.rand(BAND_PAIRS, generator=fgen)[:pairs] * (math.pi / (BAND_WIDTH / 2))).to(device)
    pos = torch.arange(n, device=device, dtype=torch.float32)
    ang = pos[:, None] * omega[None, :]
    feat = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1) * BAND_BETA  # [n, 2P]
    gain = 1.0 + q_head_gain * torch.arange(hq, device=device, dtype=torch.float32) / hq
    q[:, :, : 2 * pairs] = feat[:, None, :] * gain[None, :, None]
    k[:, :, : 2 * pairs] = feat[:, None, :]
    q, k, v = (t.to(dtype) for t in (q, k, v))
    return (q.unsqueeze(0).transpose(1, 2), k.unsqueeze(0).transpose(1, 2), v.unsqueeze(0).transpose(1, 2))


def random_cluster_table(hq: int, n_clusters: int, n_layers: int, seed: int) -> dict:
    """Heads randomly permuted (same permutation at every layer) into n_clusters equal groups; all shared."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed + 104729)
    perm = torch.randperm(hq, generator=gen).tolist()
    per = hq // n_clusters
    clusters: Dict[str, List[List[int]]] = {}
    for c in range(n_clusters):
        heads = sorted(perm[c * per:(c + 1) * per])
        clusters[str(c)] = [[layer, h] for layer in range(n_layers) for h in heads]
    return {"clusters": clusters, "shared_clusters": [str(c) for c in range(n_clusters)]}


def write_cluster_table(table: dict, path: str) -> str:
    with open(path, "w") as f:
        json.dump(table, f)
    return path


def workload_inputs(w: Workload, device="cpu", dtype=torch.bfloat16) -> Tuple[torch.Tensor, ...]:
    return planted_qkv(w.hq, w.hkv, w.seq_len, w.head_dim, w.seed, device=device, dtype=dtype,
                       q_head_gain=HEAD_GAIN)

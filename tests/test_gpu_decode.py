"""GPU parity of the decode step (one query token per head against the whole KV cache) with the fp32 oracle.

Tolerance: max-abs <= 2e-2, mean-rel <= 2.5e-3 -- the output is rounded to bf16 (unit roundoff 2^-8 -> 1.3e-3
mean-rel on its own); the kernel itself works in fp32 on the bf16 inputs."""

import math

import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 2.5e-3


def _inputs(hq, hkv, n, seed, token_major=True, d=128):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(hq, d, generator=g).to(torch.bfloat16)
    if token_major:  # the layout of a Hugging Face cache after transpose: [N, Hkv, D] storage viewed as [Hkv, N, D]
        k = torch.randn(n, hkv, d, generator=g).to(torch.bfloat16).transpose(0, 1)
        v = torch.randn(n, hkv, d, generator=g).to(torch.bfloat16).transpose(0, 1)
    else:
        k = torch.randn(hkv, n, d, generator=g).to(torch.bfloat16)
        v = torch.randn(hkv, n, d, generator=g).to(torch.bfloat16)
    return q, k, v


@pytest.mark.parametrize("hq,hkv,n", [(32, 8, 4096), (28, 4, 1000), (8, 8, 129), (4, 1, 1), (16, 2, 70000),
                                      (8, 1, 127), (18, 2, 3000), (64, 4, 2500), (24, 1, 777), (64, 2, 4096)])
@pytest.mark.parametrize("token_major", [True, False])
def test_decode_matches_oracle(gpu_device, hq, hkv, n, token_major):
    from shareprefill_amd import ops

    q, k, v = _inputs(hq, hkv, n, n + hq, token_major)
    scale = 1.0 / math.sqrt(128)
    ref = O.decode_attention(q, k, v, scale)
    out = ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), scale).cpu().float()
    assert (out - ref).abs().max().item() <= MAX_ABS
    assert ((out - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL
    again = ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), scale).cpu().float()
    assert torch.equal(out, again)


@pytest.mark.parametrize("d", [64, 32, 16, 8, 96])
@pytest.mark.parametrize("token_major", [True, False])
def test_decode_smaller_heads_read_the_cache_as_it_is(gpu_device, d, token_major):
    """head_dim below 128 (the reference's 16 / 32 / 64, shareprefill_attn.py:503-508, and any other multiple of 8):
    the kernel pads the rows inside LDS, the cache is neither copied nor padded.  The result must also equal, bit for
    bit, the head_dim-128 call on explicitly zero-padded tensors."""
    from shareprefill_amd import ops

    hq, hkv, n = 12, 4, 3001
    q, k, v = _inputs(hq, hkv, n, 40 + d, token_major, d)
    scale = 1.0 / math.sqrt(d)
    ref = O.decode_attention(q, k, v, scale)
    out = ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), scale)
    assert out.shape == (hq, d)
    o = out.cpu().float()
    assert (o - ref).abs().max().item() <= MAX_ABS
    assert ((o - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL
    pad = lambda t: torch.nn.functional.pad(t, (0, 128 - d)).to(gpu_device)
    wide = ops.decode_attention(pad(q), pad(k), pad(v), scale)
    assert torch.equal(wide[:, :d], out) and float(wide[:, d:].abs().max()) == 0.0


def test_decode_peaked_and_large_logits(gpu_device):
    """A key that dominates (logit far above the rest) and large-magnitude logits: the online softmax across
    tiles and chunks must neither overflow nor lose the winner."""
    from shareprefill_amd import ops

    q, k, v = _inputs(8, 2, 5000, 3)
    k = k.clone()
    k[:, 3333] = (q.float().view(2, 4, 128).mean(1) * 4).to(torch.bfloat16)  # strongly aligned with the queries
    scale = 1.0
    ref = O.decode_attention(q, k, v, scale)
    out = ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), scale).cpu().float()
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max().item() <= 4e-2  # values of magnitude up to ~4: bf16 ulp 0.03
    assert ((out - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL


def test_decode_rejects_unsupported(gpu_device):
    from shareprefill_amd import ops

    q, k, v = _inputs(33, 1, 256, 1)
    with pytest.raises(NotImplementedError):
        ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), 0.1)  # 33 heads per kv head
    q, k, v = _inputs(4, 2, 256, 1)
    qg = torch.zeros(4, 132, dtype=torch.bfloat16, device=gpu_device)[:, 4:]  # rows start 8 bytes off a 16-byte line
    qg.copy_(q)
    with pytest.raises(NotImplementedError):
        ops.decode_attention(qg, k.to(gpu_device), v.to(gpu_device), 0.1)
    q, k, v = _inputs(4, 2, 256, 1)
    with pytest.raises(ValueError):
        ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), 0.0)
    for d in (136, 256):  # wider than the kernel's tiles
        q, k, v = _inputs(4, 2, 256, 1, d=d)
        with pytest.raises(NotImplementedError):
            ops.decode_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), 0.1)

"""GPU parity: last-block scores (vertical / slash vectors and their block sums) against the CPU oracle."""

import pytest
import torch

from oracle import shareprefill_oracle as O
from shareprefill_amd import synthetic

pytestmark = pytest.mark.gpu


def _inputs(hq, hkv, n, seed):
    q, k, _ = synthetic.planted_qkv(hq, hkv, n, 128, seed, q_head_gain=1.0)
    return q[0], k[0]  # [H, N, D] views of token-major storage


@pytest.mark.parametrize("hq,hkv,n", [(4, 2, 1024), (8, 2, 4096), (4, 4, 1000), (2, 1, 128), (4, 1, 2304),
                                      (6, 2, 640), (7, 1, 1111)])  # odd groups: a workgroup half without a head
@pytest.mark.parametrize("bf16_logits", [False, True])
def test_lastq_scores_match_oracle(gpu_device, hq, hkv, n, bf16_logits):
    from shareprefill_amd import _lib, ops

    q, k = _inputs(hq, hkv, n, 11 + n)
    vref, sref = O.lastq_scores(q, k, 128, logits_in_input_dtype=bf16_logits)
    flags = _lib.SP_FLAG_LOGITS_BF16 if bf16_logits else 0
    vt, st, vb, sb = ops.lastq_scores(q.to(gpu_device), k.to(gpu_device), 128, flags)
    vt, st, vb, sb = vt.cpu(), st.cpu(), vb.cpu(), sb.cpu()
    # a logit that lands on the other side of a bf16 rounding boundary (MFMA vs CPU summation order) moves one
    # probability by 2^-8 relative; with fp32 logits only exp/sum rounding remains
    rtol, atol = (3e-2, 1e-6) if bf16_logits else (2e-4, 1e-8)
    assert torch.allclose(vt, vref, rtol=rtol, atol=atol)
    assert torch.allclose(st, sref, rtol=rtol, atol=atol)
    assert torch.allclose(vt.sum(-1), torch.ones(hq), atol=1e-4)
    assert torch.allclose(st.sum(-1), torch.ones(hq), atol=1e-4)
    # block sums are the right-padded 128-token sums of the token vectors the kernel itself wrote
    assert torch.allclose(vb, O.block_sum(vt, 128), rtol=1e-5, atol=1e-9)
    assert torch.allclose(sb, O.block_sum(st, 128), rtol=1e-5, atol=1e-9)


def test_lastq_scores_seeded_random_shapes(gpu_device):
    """Ragged lengths around the tile and chunk boundaries and every group size up to 8 (odd groups leave half of a
    two-head workgroup empty), fp32 logits so that the tight tolerance holds element by element."""
    import numpy as np

    from shareprefill_amd import ops

    rng = np.random.default_rng(20240607)
    lengths = [128, 129, 255, 256, 257, 383, 640, 1000, 1111, 2049, 3000, 4097, 5000, 8191]
    for case in range(24):
        hkv = int(rng.choice([1, 2, 3]))
        g = int(rng.choice([1, 2, 3, 4, 5, 7, 8]))
        n = int(rng.choice(lengths))
        hq = hkv * g
        q, k = _inputs(hq, hkv, n, 1000 + case)
        vref, sref = O.lastq_scores(q, k, 128, logits_in_input_dtype=False)
        vt, st, vb, sb = [x.cpu() for x in ops.lastq_scores(q.to(gpu_device), k.to(gpu_device), 128, 0)]
        tag = f"case {case}: hq {hq} hkv {hkv} n {n}"
        assert torch.allclose(vt, vref, rtol=2e-4, atol=1e-8), tag
        assert torch.allclose(st, sref, rtol=2e-4, atol=1e-8), tag
        assert torch.allclose(vb, O.block_sum(vt, 128), rtol=1e-5, atol=1e-9), tag
        assert torch.allclose(sb, O.block_sum(st, 128), rtol=1e-5, atol=1e-9), tag


@pytest.mark.parametrize("bs", [64, 32, 16])
@pytest.mark.parametrize("hq,hkv,n", [(4, 2, 1024), (6, 2, 1000), (7, 1, 389), (2, 1, 128), (4, 4, 2100), (4, 2, 100),
                                      (2, 2, 64), (3, 1, 127)])  # the last three: prompts shorter than 128 tokens
def test_lastq_scores_smaller_block_sizes(gpu_device, bs, hq, hkv, n):
    """Block sizes below 128 (attention_sharing.py:127: the last bs queries): the same kernels with the rows in front
    of the last bs masked out; token vectors against the oracle with fp32 logits, block sums of bs tokens."""
    from shareprefill_amd import ops

    q, k = _inputs(hq, hkv, n, 77 + n + bs)
    vref, sref = O.lastq_scores(q, k, bs, logits_in_input_dtype=False)
    vt, st, vb, sb = [x.cpu() for x in ops.lastq_scores(q.to(gpu_device), k.to(gpu_device), bs, 0)]
    nb = -(-n // bs)
    assert vb.shape == (hq, nb) and sb.shape == (hq, nb)
    assert torch.allclose(vt, vref, rtol=2e-4, atol=1e-8)
    assert torch.allclose(st, sref, rtol=2e-4, atol=1e-8)
    assert torch.allclose(vt.sum(-1), torch.ones(hq), atol=1e-4)
    assert torch.allclose(vb, O.block_sum(vt, bs), rtol=1e-5, atol=1e-9)
    assert torch.allclose(sb, O.block_sum(st, bs), rtol=1e-5, atol=1e-9)
    # the reference's bf16 logits as well: a logit on the other side of a bf16 rounding boundary (one ulp of a logit
    # of magnitude 8 is 0.03) moves its probability by 3 %, and a slash bin near the end holds few elements
    vref, sref = O.lastq_scores(q, k, bs, logits_in_input_dtype=True)
    vt, st, _, _ = [x.cpu() for x in ops.lastq_scores(q.to(gpu_device), k.to(gpu_device), bs)]
    assert torch.allclose(vt, vref, rtol=8e-2, atol=1e-6)
    assert torch.allclose(st, sref, rtol=8e-2, atol=1e-6)


def test_lastq_scores_head_major_layout_and_determinism(gpu_device):
    from shareprefill_amd import ops

    q, k = _inputs(4, 2, 2048, 5)
    qg, kg = q.to(gpu_device), k.to(gpu_device)
    a = ops.lastq_scores(qg, kg, 128)
    b = ops.lastq_scores(qg.contiguous(), kg.contiguous(), 128)  # [H,N,D] contiguous storage
    c = ops.lastq_scores(qg, kg, 128)
    for x, y, z in zip(a, b, c):
        assert torch.equal(x, y) and torch.equal(x, z)


def test_lastq_scores_rejects_unsupported(gpu_device):
    from shareprefill_amd import ops

    q = torch.zeros(2, 256, 64, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(NotImplementedError):
        ops.lastq_scores(q, q, 128)
    q = torch.zeros(2, 64, 128, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(ValueError):
        ops.lastq_scores(q, q, 128)

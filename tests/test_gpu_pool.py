"""GPU parity: block average pooling (HIP) against the CPU oracle, through the C ABI."""

import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu


def _bf16_ulp_diff(a: torch.Tensor, b: torch.Tensor) -> int:
    ai = a.view(torch.int16).to(torch.int32)
    bi = b.view(torch.int16).to(torch.int32)
    ai = torch.where(ai < 0, -(ai & 0x7FFF), ai)
    bi = torch.where(bi < 0, -(bi & 0x7FFF), bi)
    return int((ai - bi).abs().max())


@pytest.mark.parametrize("n,h,d,layout", [(1024, 8, 128, "nhd"), (1000, 4, 128, "nhd"), (640, 2, 64, "hnd"),
                                          (129, 3, 128, "nhd"), (4096, 32, 128, "nhd")])
def test_pool_avg_matches_oracle(gpu_device, n, h, d, layout):
    from shareprefill_amd import ops

    g = torch.Generator().manual_seed(n + h)
    x = torch.randn(n, h, d, generator=g).to(torch.bfloat16)
    ref = O.pool_avg(x, 128)
    xg = x.to(gpu_device)
    view = xg.transpose(0, 1) if layout == "nhd" else xg.transpose(0, 1).contiguous()
    y = ops.pool_avg(view, 128).cpu()
    assert y.shape == ref.shape
    # fp32 accumulation in a different order: at most one bf16 ulp apart, and almost always equal
    assert _bf16_ulp_diff(y, ref) <= 1
    assert (y != ref).float().mean().item() < 1e-2


def test_pool_avg_rescale_tail_matches_q_pooling(gpu_device):
    from shareprefill_amd import _lib, ops

    g = torch.Generator().manual_seed(7)
    x = torch.randn(300, 2, 128, generator=g).to(torch.bfloat16)
    y = ops.pool_avg(x.to(gpu_device).transpose(0, 1), 128, tail_mode=_lib.SP_POOL_TAIL_RESCALE).cpu()
    for h in range(2):
        ref = O.pool_q_head(x[:, h], 128)
        assert _bf16_ulp_diff(y[:, h].contiguous(), ref) <= 1


def test_pool_avg_constant_and_head_mask(gpu_device):
    from shareprefill_amd import ops

    x = torch.full((512, 4, 128), 0.375, dtype=torch.bfloat16, device=gpu_device)
    out = torch.full((4, 4, 128), -1.0, dtype=torch.bfloat16, device=gpu_device)
    en = torch.tensor([1, 0, 1, 0], dtype=torch.int32, device=gpu_device)
    ops.pool_avg(x.transpose(0, 1), 128, head_enable=en, out=out)
    assert torch.equal(out[:, 0].cpu(), torch.full((4, 128), 0.375, dtype=torch.bfloat16))
    assert torch.equal(out[:, 1].cpu(), torch.full((4, 128), -1.0, dtype=torch.bfloat16))


def test_pool_avg_rejects_bad_arguments(gpu_device):
    from shareprefill_amd import ops

    x = torch.zeros(2, 256, 12, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(NotImplementedError):
        ops.pool_avg(x, 128)
    with pytest.raises(AssertionError):
        ops.pool_avg(torch.zeros(2, 256, 128, dtype=torch.float16, device=gpu_device), 128)

"""GPU test of the decode entry point that allocates nothing (sp_decode_attn_static_bf16).

Called through the C ABI (ctypes) and held to the bar of every other kernel of the path: the result must be
bit-identical to sp_decode_attn_bf16 with a caller's workspace (same kernels, same chunking, sums in the same order),
and within the decode tolerances of the fp32 oracle.  Two calls in a row on the library's built-in scratch, the second
on a smaller input: whatever the first call left in the shared array must not leak into the second."""

import ctypes as C
import math

import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 2.5e-3


def _inputs(hq, hkv, n, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(hq, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(n, hkv, 128, generator=g).to(torch.bfloat16).transpose(0, 1)
    v = torch.randn(n, hkv, 128, generator=g).to(torch.bfloat16).transpose(0, 1)
    return q, k, v


def _call_both(lib, q, k, v, scale, dev):
    """-> (out of the static-scratch entry, out of the workspace entry); raw C-ABI calls on torch's current stream."""
    hq, d = q.shape
    hkv, n, _ = k.shape
    qg, kg, vg = q.to(dev), k.to(dev), v.to(dev)
    out_static = torch.full((hq, d), float("nan"), dtype=torch.bfloat16, device=dev)
    out_ws = torch.full((hq, d), float("nan"), dtype=torch.bfloat16, device=dev)
    need = lib.sp_decode_workspace_bytes(n, hq, hkv)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    args = (C.c_void_p(qg.data_ptr()), C.c_void_p(kg.data_ptr()), C.c_void_p(vg.data_ptr()), n, hq, hkv, d,
            qg.stride(0), kg.stride(1), kg.stride(0), vg.stride(1), vg.stride(0), scale)
    st = lib.sp_decode_attn_static_bf16(*args, C.c_void_p(out_static.data_ptr()), stream)
    assert st == 0, lib.sp_last_error().decode()
    st = lib.sp_decode_attn_bf16(*args, C.c_void_p(out_ws.data_ptr()), C.c_void_p(ws.data_ptr()), need, stream)
    assert st == 0, lib.sp_last_error().decode()
    torch.cuda.synchronize(dev)
    return out_static.cpu(), out_ws.cpu()


def test_static_scratch_decode_matches_workspace_entry_twice(gpu_device):
    from shareprefill_amd import _lib

    lib = _lib.load()
    scale = 1.0 / math.sqrt(128)
    # the larger input first (64 chunks x 32 heads of partials), then a smaller one (fewer chunks, fewer heads) that
    # reuses the front of the same array
    for hq, hkv, n, seed in [(32, 8, 20000, 11), (8, 2, 700, 12)]:
        print(f"static-scratch decode: hq={hq} hkv={hkv} n={n} seed={seed}", flush=True)
        q, k, v = _inputs(hq, hkv, n, seed)
        got, want = _call_both(lib, q, k, v, scale, gpu_device)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), "static-scratch entry differs from the workspace entry"
        ref = O.decode_attention(q, k, v, scale)
        assert (got.float() - ref).abs().max().item() <= MAX_ABS
        assert ((got.float() - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL


def test_static_scratch_decode_rejects_oversize(gpu_device):
    """Partials beyond the built-in 8 MiB are refused with a clear error before anything is launched."""
    from shareprefill_amd import _lib, ops

    lib = _lib.load()
    hq, hkv, n = 256, 8, 70000  # 64 chunks x 256 heads x 520 B = 8.1 MiB
    assert lib.sp_decode_workspace_bytes(n, hq, hkv) > _lib.SP_DECODE_STATIC_SCRATCH_BYTES
    q, k, v = _inputs(hq, hkv, n, 5)
    dev = gpu_device
    with pytest.raises(RuntimeError, match="built-in scratch"):
        ops.decode_attention(q.to(dev), k.to(dev), v.to(dev), 0.1, static_scratch=True)
    # the workspace entry still serves that shape
    out = ops.decode_attention(q.to(dev), k.to(dev), v.to(dev), 0.1).cpu().float()
    ref = O.decode_attention(q, k, v, 0.1)
    assert (out - ref).abs().max().item() <= MAX_ABS

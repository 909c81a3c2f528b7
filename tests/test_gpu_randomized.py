"""GPU: seeded random sweeps over shapes, masks, thresholds and input scales -- attention against the fp32 oracle
(including inputs whose running max keeps moving, which exercises the rescale-and-redo path of the kernel) and the
whole selection against the oracle's integer logic on the GPU's own scores (bit-exact)."""

import importlib.util
import os

import numpy as np
import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu


def test_attention_random_shapes_masks_and_scales(gpu_device):
    from shareprefill_amd import ops

    rng = np.random.default_rng(12345)
    for case in range(40):
        hkv = int(rng.choice([1, 2, 4]))
        hq = hkv * int(rng.choice([1, 2, 4, 7]))
        n = int(rng.choice([128, 200, 256, 384, 640, 1000, 1024, 1280, 1536, 2000]))
        nb = -(-n // 128)
        density = float(rng.choice([0.1, 0.3, 0.6, 0.9, 1.0]))
        gain = float(rng.choice([1.0, 1.0, 3.0, 6.0]))  # large logits: the running max moves often
        gen = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        mk = lambda h, s: (torch.randn(n, h, 128, generator=gen) * s).to(torch.bfloat16).transpose(0, 1)
        q, k, v = mk(hq, gain), mk(hkv, 1.0), mk(hkv, 1.0)
        if rng.random() < 0.3:  # keys growing with position: every tile raises the max
            k = (k.float() * torch.linspace(0.2, 2.0, n)[None, :, None]).to(torch.bfloat16)
        m = np.tril(rng.random((hq, nb, nb)) < density)
        idx = np.arange(nb)
        m[:, idx, idx] = True
        dec = torch.tensor(rng.choice([0, 1, 2, 3], size=hq), dtype=torch.int32)
        avg = torch.zeros(hq, nb, nb, dtype=torch.float32, device=gpu_device)
        scale = float(rng.choice([0.05, 128 ** -0.5, 0.2]))
        out = ops.block_sparse_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device),
                                         ops.bool_to_mask(torch.from_numpy(m)).to(gpu_device), 128, scale,
                                         decision=dec.to(gpu_device), avg_attn=avg,
                                         max_pivots=int(rng.choice([0, 1, hq])))
        out = out.cpu().transpose(0, 1).float()
        ref, avg_ref = O.masked_attention(q, k, v, m, 128, scale, want_avg=(dec == O.DEC_DENSE).numpy())
        what = f"case {case}: hq{hq} hkv{hkv} n{n} density {density} gain {gain} scale {scale:.3f}"
        assert torch.isfinite(out).all(), what
        assert (out - ref).abs().max().item() <= 2e-2, what
        assert ((out - ref).abs().mean() / ref.abs().mean()).item() <= 2.5e-3, what
        assert (avg.cpu() - avg_ref).abs().max().item() <= 1e-3, what
        # no less accurate than the reference kernel's own arithmetic (bf16 probabilities against the running
        # maximum, bf16 output) restated on the CPU, on the same inputs
        emu, _ = O.masked_attention(q, k, v, m, 128, scale, emulate_bf16=True)
        e_ref = ((emu - ref).abs().mean() / ref.abs().mean()).item()
        e_out = ((out - ref).abs().mean() / ref.abs().mean()).item()
        assert e_out <= 1.15 * e_ref + 2e-5, f"{what}: kernel {e_out:.3e}, reference roundings {e_ref:.3e}"


def test_selection_random_shapes_and_thresholds_bit_exact(gpu_device, tmp_path):
    spec = importlib.util.spec_from_file_location(
        "layer_helpers", os.path.join(os.path.dirname(__file__), "test_gpu_layer.py"))
    helpers = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(helpers)
    rng = np.random.default_rng(777)
    seen = np.zeros(4, dtype=np.int64)
    for case in range(24):
        hkv = int(rng.choice([1, 2, 4]))
        hq = hkv * int(rng.choice([2, 4, 7]))
        n = int(rng.choice([1024, 1536, 2048, 3000, 4096, 5120]))
        n_clusters = int(rng.choice([1, 2, max(hq // 2, 1)]))
        if hq % n_clusters:
            n_clusters = 1
        thr = dict(pattern_threshold=float(rng.choice([0.8, 0.9, 0.95, 0.99])),
                   similarity_threshold=float(rng.choice([0.3, 0.5, 0.9])),
                   fallback_threshold=float(rng.choice([0.5, 0.9, 0.99, 1e9])),
                   queryaware_threshold=float(rng.choice([0.0, 0.1, 0.3, 0.6])),
                   min_budget=int(rng.choice([128, 512, 1024])))
        sub = tmp_path / f"case{case}"
        sub.mkdir()
        run = helpers.run_layers(gpu_device, sub, hq=hq, hkv=hkv, n=n, seed=int(rng.integers(1 << 20)),
                                 n_clusters=n_clusters, n_layers=3, with_free=False, **thr)
        helpers.check_forced(run)
        for L in run["layers"]:
            seen += np.bincount(L["dec"], minlength=4)
    assert (seen > 0).all(), f"decision kinds exercised: {seen.tolist()}"  # vertical-slash, pivot, shared, query-aware

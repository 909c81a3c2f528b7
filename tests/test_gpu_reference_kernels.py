"""GPU parity of the kernel wrappers kept under the reference's own names and arguments:
triton_block_wise_prefill_attention / triton_column_count_cumsum (shareprefill/attn/shareprefill_attn.py:226-269,
474-620) and triton_bnhd_pool / score_cover_topk (shareprefill/attn/utils.py:47-50, 211-261), imported the way a user
of the reference imports them.  Index work is compared bit-exactly, attention to max-abs <= 2e-2 and mean-rel
<= 2.5e-3 against the fp32 oracle (the bf16 quantisation floor of this metric is 2.06e-3) and bit-exactly against
the mask form of the same call."""

import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_docstring_vectors.json")


def _ids_from_mask(mask):
    """bool [Hq, nb, nb] -> list[Hq] of int64 id tensors (row * nb + col), the reference's block_idx entries."""
    nb = mask.shape[-1]
    return [torch.from_numpy(np.flatnonzero(mask[h].reshape(-1)).astype(np.int64)) for h in range(mask.shape[0])]


def _random_mask(hq, nb, seed, density=0.4):
    rng = np.random.default_rng(seed)
    m = np.tril(rng.random((hq, nb, nb)) < density)
    idx = np.arange(nb)
    m[:, idx, idx] = True
    m[:, :, 0] = True
    return m


def test_column_count_cumsum_docstring_vectors(gpu_device):
    from shareprefill.attn.shareprefill_attn import triton_column_count_cumsum

    gold = json.load(open(GOLDEN))["csr_row_pointers"]
    x = torch.tensor(gold["block_ids"], device=gpu_device).view(1, 1, -1)
    y = triton_column_count_cumsum(x, gold["grid"])
    assert y.dtype == torch.int32 and y.shape == (1, 1, gold["grid"] + 1)
    assert y.cpu().view(-1).tolist() == gold["row_pointers"]
    # int32 ids (the reference converts to int32 itself) and the reference's padding value
    pad = gold["grid"] * (gold["grid"] + 1)
    x32 = torch.tensor(gold["block_ids"] + [pad, pad], dtype=torch.int32, device=gpu_device).view(1, 1, -1)
    assert triton_column_count_cumsum(x32, gold["grid"]).cpu().view(-1).tolist() == gold["row_pointers"]


@pytest.mark.parametrize("b,h,nb,k", [(1, 1, 1, 1), (2, 3, 7, 19), (1, 5, 300, 4000), (1, 2, 4096, 100000), (1, 2, 9, 0)])
def test_column_count_cumsum_random_ids(gpu_device, b, h, nb, k):
    """Unsorted ids with duplicates and padding: the histogram counts every occurrence (count_kernel:210-214)."""
    from shareprefill.attn.shareprefill_attn import triton_column_count_cumsum

    rng = np.random.default_rng(nb * 31 + k)
    x = rng.integers(0, nb * nb, size=(b, h, k), dtype=np.int64)
    if k:
        x[rng.random((b, h, k)) < 0.2] = nb * (nb + 1)
    y = triton_column_count_cumsum(torch.from_numpy(x).to(gpu_device), nb).cpu().numpy()
    for i in range(b):
        for j in range(h):
            np.testing.assert_array_equal(y[i, j], O.csr_row_pointers(x[i, j], nb))


def test_block_idx_to_mask_round_trip(gpu_device):
    from shareprefill_amd import ops

    gold = json.load(open(GOLDEN))["flat_block_ids"]
    ids = torch.tensor(gold["block_ids"], device=gpu_device).view(1, -1)
    mask = ops.mask_to_bool(ops.block_idx_to_mask(ids, gold["grid"]), gold["grid"])[0].cpu().numpy()
    want = np.zeros((gold["grid"], gold["grid"]), dtype=bool)
    for r, c in gold["blocks_row_col"]:
        want[r, c] = True
    np.testing.assert_array_equal(mask, want)

    for hq, nb in [(3, 5), (4, 130), (2, 1024)]:
        m = _random_mask(hq, nb, nb, 0.3)
        lists = _ids_from_mask(m)
        # shuffled, padded with the reference's value, plus duplicates and ids above the diagonal (dropped)
        rng = np.random.default_rng(nb)
        k = max(len(t) for t in lists) + 7
        padded = np.full((hq, k), nb * (nb + 1), dtype=np.int64)
        for h, t in enumerate(lists):
            row = t.numpy().copy()
            rng.shuffle(row)
            padded[h, :len(row)] = row
            padded[h, len(row)] = row[0]
            if nb > 1:
                padded[h, len(row) + 1] = 0 * nb + (nb - 1)
        got = ops.block_idx_to_mask(torch.from_numpy(padded).to(gpu_device), nb)
        np.testing.assert_array_equal(ops.mask_to_bool(got, nb).cpu().numpy(), m)
        assert torch.equal(got.cpu(), ops.bool_to_mask(torch.from_numpy(m)))
        back = ops.mask_to_block_idx(got, nb)
        for h in range(hq):
            assert torch.equal(back[h].cpu(), lists[h])


@pytest.mark.parametrize("bs", [64, 32, 16])
@pytest.mark.parametrize("hq,hkv,n,density", [(4, 2, 1024, 0.3), (6, 2, 1111, 0.6), (4, 4, 333, 0.1), (7, 1, 640, 1.0)])
def test_block_wise_prefill_attention_smaller_block_sizes(gpu_device, bs, hq, hkv, n, density):
    """The wrapper's other block sizes (shareprefill_attn.py:509-516): ids on the N / bs grid, outputs and the wanted
    heads' block-average maps [nb, nb] against the oracle at that block size; a fully masked stretch of a visited
    128-token block must contribute nothing."""
    from shareprefill.attn.shareprefill_attn import triton_block_wise_prefill_attention

    g = torch.Generator().manual_seed(n + bs)
    mk = lambda h: torch.randn(1, n, h, 128, generator=g).to(torch.bfloat16)
    q, k, v = mk(hq), mk(hkv), mk(hkv)
    nb = -(-n // bs)
    mask = _random_mask(hq, nb, n + bs, density)
    need = torch.zeros(1, hq, dtype=torch.bool)
    need[0, 0] = True
    need[0, hq - 1] = True
    block_idx = [[t.to(gpu_device) for t in _ids_from_mask(mask)]]
    out, avg = triton_block_wise_prefill_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), block_idx,
                                                   need.to(gpu_device), bs)
    assert out.shape == (1, n, hq, 128) and avg.shape == (1, hq, nb, nb)
    qh, kh, vh = (t[0].transpose(0, 1) for t in (q, k, v))
    ref, ref_avg = O.masked_attention(qh, kh, vh, mask, bs, 1.0 / math.sqrt(128), want_avg=need[0].numpy())
    o = out[0].cpu().float().transpose(0, 1)
    assert (o - ref).abs().max().item() <= 2e-2
    assert ((o - ref).abs().mean() / ref.abs().mean()).item() <= 2.5e-3
    a = avg[0].cpu()
    for h in range(hq):
        if need[0, h]:
            assert (a[h] - ref_avg[h]).abs().max().item() <= 2e-3
            np.testing.assert_allclose(a[h].sum(-1).numpy(), 1.0, atol=2e-3)
            assert (a[h][~torch.from_numpy(mask[h])] == 0).all()
        else:
            assert a[h].abs().max().item() == 0.0


@pytest.mark.parametrize("hq,hkv,n,as_tensor", [(4, 2, 1024, False), (8, 2, 1500, True), (4, 4, 640, False)])
def test_block_wise_prefill_attention_reference_signature(gpu_device, hq, hkv, n, as_tensor):
    from shareprefill.attn.shareprefill_attn import triton_block_wise_prefill_attention
    from shareprefill_amd import ops

    g = torch.Generator().manual_seed(n)
    mk = lambda h: torch.randn(1, n, h, 128, generator=g).to(torch.bfloat16)
    q, k, v = mk(hq), mk(hkv), mk(hkv)
    nb = -(-n // 128)
    mask = _random_mask(hq, nb, n)
    need = torch.zeros(1, hq, dtype=torch.bool)
    need[0, 1] = True
    need[0, hq - 1] = True
    lists = [[t.to(gpu_device) for t in _ids_from_mask(mask)]]
    if as_tensor:
        block_idx = torch.nn.utils.rnn.pad_sequence(lists[0], batch_first=True, padding_value=nb * (nb + 1)).unsqueeze(0)
    else:
        block_idx = lists
    out, avg = triton_block_wise_prefill_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), block_idx,
                                                   need.to(gpu_device), 128)
    assert out.shape == (1, n, hq, 128) and out.dtype == torch.bfloat16
    assert avg.shape == (1, hq, nb, nb) and avg.dtype == torch.float32

    qh, kh, vh = (t[0].transpose(0, 1) for t in (q, k, v))
    scale = 1.0 / math.sqrt(128)
    ref, ref_avg = O.masked_attention(qh, kh, vh, mask, 128, scale, want_avg=need[0].numpy())
    o = out[0].cpu().float().transpose(0, 1)
    assert (o - ref).abs().max().item() <= 2e-2
    assert ((o - ref).abs().mean() / ref.abs().mean()).item() <= 2.5e-3
    a = avg[0].cpu()
    for h in range(hq):
        if need[0, h]:
            assert (a[h] - ref_avg[h]).abs().max().item() <= 2e-3
            np.testing.assert_allclose(a[h].sum(-1).numpy(), 1.0, atol=2e-3)
        else:
            assert a[h].abs().max().item() == 0.0
    # the mask form of the same call gives the same bits
    mg = ops.bool_to_mask(torch.from_numpy(mask)).to(gpu_device)
    same = ops.block_sparse_attention(qh.to(gpu_device), kh.to(gpu_device), vh.to(gpu_device), mg, 128, scale)
    assert torch.equal(same, out[0])


def test_block_wise_prefill_attention_interleave_batch_and_scale(gpu_device):
    """gqa_interleave=True: query head h reads kv head h % Hkv (shareprefill_attn.py:333-336); batch 2; an explicit
    softmax_scale."""
    from shareprefill.attn.shareprefill_attn import triton_block_wise_prefill_attention

    b, hq, hkv, n = 2, 6, 2, 700
    g = torch.Generator().manual_seed(5)
    mk = lambda h: torch.randn(b, n, h, 128, generator=g).to(torch.bfloat16)
    q, k, v = mk(hq), mk(hkv), mk(hkv)
    nb = -(-n // 128)
    masks = [_random_mask(hq, nb, 70 + i, 0.5) for i in range(b)]
    need = torch.zeros(b, hq, dtype=torch.bool)
    need[0, 2] = True
    need[1, 3] = True
    block_idx = [[t.to(gpu_device) for t in _ids_from_mask(m)] for m in masks]
    scale = 0.07
    out, avg = triton_block_wise_prefill_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), block_idx,
                                                   need.to(gpu_device), 128, softmax_scale=scale, gqa_interleave=True)
    kv_of = [h % hkv for h in range(hq)]
    for i in range(b):
        # the oracle maps h -> h // g: hand it K / V expanded to one kv head per query head in the interleaved order
        ke = k[i].transpose(0, 1)[kv_of]
        ve = v[i].transpose(0, 1)[kv_of]
        ref, ref_avg = O.masked_attention(q[i].transpose(0, 1), ke, ve, masks[i], 128, scale, want_avg=need[i].numpy())
        o = out[i].cpu().float().transpose(0, 1)
        assert (o - ref).abs().max().item() <= 2e-2
        assert ((o - ref).abs().mean() / ref.abs().mean()).item() <= 2.5e-3
        for h in range(hq):
            if need[i, h]:
                assert (avg[i, h].cpu() - ref_avg[h]).abs().max().item() <= 2e-3
            else:
                assert avg[i, h].abs().max().item() == 0.0
    # without the flag the same call maps h -> h // g and must differ for the heads whose kv head changes
    out2, _ = triton_block_wise_prefill_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), block_idx,
                                                  need.to(gpu_device), 128, softmax_scale=scale)
    g_sz = hq // hkv
    for h in range(hq):
        assert torch.equal(out[:, :, h], out2[:, :, h]) == (h % hkv == h // g_sz)


def test_block_wise_prefill_attention_rejects_what_is_not_built(gpu_device):
    from shareprefill.attn.shareprefill_attn import triton_block_wise_prefill_attention

    q = torch.zeros(1, 256, 2, 128, dtype=torch.bfloat16, device=gpu_device)
    idx = torch.zeros(1, 2, 1, dtype=torch.int64, device=gpu_device)
    need = torch.zeros(1, 2, dtype=torch.bool, device=gpu_device)
    with pytest.raises(NotImplementedError):
        triton_block_wise_prefill_attention(q, q, q, idx, need, 128, grid_offset=64)
    with pytest.raises(AssertionError):
        triton_block_wise_prefill_attention(q.float(), q.float(), q.float(), idx, need, 128)
    with pytest.raises(AssertionError, match="block_size"):  # (the reference asserts the same set, :509-516)
        triton_block_wise_prefill_attention(q, q, q, idx, need, 48)


@pytest.mark.parametrize("b,n,h,d,ks", [(1, 1000, 4, 128, 128), (2, 300, 3, 64, 64), (1, 128, 8, 128, 128)])
def test_bnhd_pool_reference_signature(gpu_device, b, n, h, d, ks):
    from shareprefill.attn.utils import triton_bnhd_pool

    g = torch.Generator().manual_seed(n + d)
    x = torch.randn(b, n, h, d, generator=g).to(torch.bfloat16)
    y = triton_bnhd_pool(x.to(gpu_device), ks)
    m = -(-n // ks)
    assert y.shape == (b, m, h, d) and y.dtype == torch.bfloat16
    for i in range(b):
        want = O.pool_avg(x[i], ks)
        # one bf16 unit in the last place: the sum is fp32 in both, the oracle divides in a different order
        diff = (y[i].cpu().float() - want.float()).abs()
        assert (diff <= want.float().abs() * 2.0 ** -7 + 1e-30).all()
    last = triton_bnhd_pool(x.to(gpu_device), ks, "last").cpu()
    rows = list(range(ks - 1, n, ks)) + ([n - 1] if n % ks else [])
    assert torch.equal(last, x[:, rows])
    # the other pool types (attn/utils.py:180-191): max / min / maxabs are exact, the sum within one bf16 rounding
    for kind in ("max", "min", "maxabs", "sum"):
        got = triton_bnhd_pool(x.to(gpu_device), ks, kind).cpu()
        assert got.shape == (b, m, h, d) and got.dtype == torch.bfloat16
        for i in range(b):
            want = O.pool(x[i], ks, kind)
            if kind == "sum":
                assert ((got[i].float() - want.float()).abs() <= want.float().abs() * 2.0 ** -7 + 1e-30).all()
            else:
                assert torch.equal(got[i], want), kind
    with pytest.raises(KeyError):
        triton_bnhd_pool(x.to(gpu_device), ks, "median")


def test_score_cover_topk_reference_signature(gpu_device):
    from shareprefill.attn.utils import score_cover_topk

    g = torch.Generator().manual_seed(3)
    x = torch.softmax(torch.randn(2, 3, 5000, generator=g) * 3, dim=-1)
    got = score_cover_topk(x.to(gpu_device), 0.9)
    assert got.shape == (2, 3) and got.dtype == torch.int64
    want = [[O.cover_count(x[i, j].numpy(), 0.9) for j in range(3)] for i in range(2)]
    assert got.cpu().tolist() == want


@pytest.mark.parametrize("d", [64, 32, 16])
def test_block_wise_prefill_attention_small_head_dims(gpu_device, d):
    """head_dim 16 / 32 / 64 (shareprefill_attn.py:503-508) run zero-padded on the head_dim-128 kernel; the default
    softmax scale stays 1/sqrt(d)."""
    from shareprefill.attn.shareprefill_attn import triton_block_wise_prefill_attention

    hq, hkv, n = 4, 2, 900
    g = torch.Generator().manual_seed(d)
    mk = lambda h: torch.randn(1, n, h, d, generator=g).to(torch.bfloat16)
    q, k, v = mk(hq), mk(hkv), mk(hkv)
    nb = -(-n // 128)
    mask = _random_mask(hq, nb, d, 0.5)
    need = torch.tensor([[True, False, False, True]])
    block_idx = [[t.to(gpu_device) for t in _ids_from_mask(mask)]]
    out, avg = triton_block_wise_prefill_attention(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), block_idx,
                                                   need.to(gpu_device), 128)
    assert out.shape == (1, n, hq, d)
    qh, kh, vh = (t[0].transpose(0, 1) for t in (q, k, v))
    ref, ref_avg = O.masked_attention(qh, kh, vh, mask, 128, 1.0 / math.sqrt(d), want_avg=need[0].numpy())
    o = out[0].cpu().float().transpose(0, 1)
    assert (o - ref).abs().max().item() <= 2e-2
    assert ((o - ref).abs().mean() / ref.abs().mean()).item() <= 2.5e-3
    for h in range(hq):
        if need[0, h]:
            assert (avg[0, h].cpu() - ref_avg[h]).abs().max().item() <= 2e-3


def _reference_side_binding():
    """The ctypes stub that the integration notes at the repository root show to a maintainer of the reference (the
    module they would add as shareprefill/attn/hip_backend.py), taken from the notes themselves -- the Python block
    that opens the library -- and executed against the in-tree library, so that the text shown there is the code tested here."""
    import types

    from shareprefill_amd import _lib

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    blocks = [b[:b.index("```")] for b in text.split("```python")[1:]]
    code = next(b for b in blocks if 'C.CDLL("libshareprefill_hip.so")' in b)
    code = code.replace('C.CDLL("libshareprefill_hip.so")', f"C.CDLL({_lib.LIB_PATH!r})")
    mod = types.ModuleType("hip_backend")
    exec(compile(code, "hip_backend.py", "exec"), mod.__dict__)
    return mod


def test_ctypes_binding_for_the_reference(gpu_device):
    """The self-contained ctypes stub a maintainer of the reference would add gives the results of the package's own
    front ends."""
    from shareprefill_amd import ops

    rb = _reference_side_binding()

    hq, hkv, n = 4, 2, 1100
    g = torch.Generator().manual_seed(8)
    mk = lambda h: torch.randn(1, n, h, 128, generator=g).to(torch.bfloat16).to(gpu_device)
    q, k, v = mk(hq), mk(hkv), mk(hkv)
    nb = -(-n // 128)
    mask = _random_mask(hq, nb, 8, 0.5)
    pooled = rb.hip_bnhd_pool(k, 128)
    assert torch.equal(pooled[0], ops.pool_avg(k[0].transpose(0, 1), 128))
    block_idx = [[t.to(gpu_device) for t in _ids_from_mask(mask)]]
    use_dense = torch.tensor([[False, True, False, False]], device=gpu_device)
    out, avg = rb.hip_block_wise_prefill_attention(q, k, v, block_idx, use_dense, 128, 128 ** -0.5)
    mg = ops.bool_to_mask(torch.from_numpy(mask)).to(gpu_device)
    assert torch.equal(rb.ids_to_mask(block_idx, nb), mg)
    dec = use_dense[0].to(torch.int32)
    avg_want = torch.zeros(hq, nb, nb, dtype=torch.float32, device=gpu_device)
    want = ops.block_sparse_attention(q[0].transpose(0, 1), k[0].transpose(0, 1), v[0].transpose(0, 1), mg, 128,
                                      128 ** -0.5, decision=dec, avg_attn=avg_want)
    assert torch.equal(out[0], want)
    assert torch.equal(avg[0], avg_want) and float(avg[0, 1].sum()) > 0

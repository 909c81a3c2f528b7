"""Pins for the CPU oracle: each oracle function is checked against something that is not the oracle's
own formula -- the reference's docstring vectors, the literal torch expression the reference evaluates,
closed forms, library routines (scipy, torch SDPA) and brute force on tiny inputs."""

import math

import numpy as np
import pytest
import torch

from oracle import shareprefill_oracle as O


# ----- literal restatements of the reference's torch expressions, used only as checkers -----------
def literal_cover_topk(x, score):  # utils.py:47-50
    c = torch.cumsum(torch.sort(x, dim=-1, descending=True, stable=True).values, dim=-1)
    return int(torch.sum(c <= score, dim=-1)) + 1


def literal_cover_idx(x, score):  # utils.py:53-57
    xs, idx = torch.sort(x, dim=-1, descending=True, stable=True)
    c = torch.cumsum(xs, dim=-1)
    return idx[~(c > score)]


def literal_each_row(a, score):  # utils.py:60-76
    xs, idx = torch.sort(a, dim=-1, descending=True, stable=True)
    c = torch.cumsum(xs, dim=-1)
    t = (c >= score).float().argmax(dim=-1) + 1
    keep = torch.zeros_like(a, dtype=torch.bool)
    for r in range(a.shape[0]):
        keep[r, idx[r, : int(t[r])]] = True
    return keep.numpy()


def rand_probs(n, seed, sharp=3.0):
    g = torch.Generator().manual_seed(seed)
    return torch.softmax(torch.randn(n, generator=g) * sharp, dim=-1)


# ----- reference docstring vectors (tests/golden/reference_docstring_vectors.json) ------------------
def golden_vectors():
    import json
    import os

    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_docstring_vectors.json")) as f:
        return json.load(f)


def test_csr_docstring_vector():
    v = golden_vectors()["csr_row_pointers"]  # shareprefill_attn.py:235-236
    assert O.csr_row_pointers(np.array(v["block_ids"]), v["grid"]).tolist() == v["row_pointers"]
    assert np.diff(v["row_pointers"]).tolist() == v["blocks_per_row"]


def test_csr_ignores_padding_ids():
    nb = 4
    ids = np.array([0, 5, 8, 13, 14, nb * (nb + 1), nb * (nb + 1)])
    assert O.csr_row_pointers(ids, nb).tolist() == [0, 1, 2, 3, 5]


def test_flat_id_docstring_vector():
    v = golden_vectors()["flat_block_ids"]  # shareprefill_attn.py:491-492
    m = np.zeros((v["grid"], v["grid"]), dtype=bool)
    for r, c in v["blocks_row_col"]:
        m[r, c] = True
    assert O.mask_to_ids(m).tolist() == v["block_ids"]


# ----- pooling --------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [256, 300, 129])
def test_pool_avg_is_block_mean(n):
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, 3, 16, generator=g)
    y = O.pool_avg(x, 128)
    nb = -(-n // 128)
    assert y.shape == (nb, 3, 16)
    for b in range(nb):
        ref = x[b * 128: min((b + 1) * 128, n)].double().mean(0)
        assert torch.allclose(y[b].double(), ref, atol=1e-6)


def test_pool_avg_constant_and_linear():
    x = torch.full((300, 2, 16), 0.375)
    assert torch.equal(O.pool_avg(x, 128), torch.full((3, 2, 16), 0.375))
    g = torch.Generator().manual_seed(0)
    a, b = torch.randn(256, 2, 16, generator=g), torch.randn(256, 2, 16, generator=g)
    assert torch.allclose(O.pool_avg(a + 2 * b, 128), O.pool_avg(a, 128) + 2 * O.pool_avg(b, 128), atol=1e-5)


@pytest.mark.parametrize("n,ks", [(256, 128), (300, 128), (100, 16), (1000, 512), (33, 32)])
def test_pool_types_against_the_library_pooling_routines(n, ks):
    """The reference kernel's other pool types (attn/utils.py:180-191) against torch's own pooling routines run on the
    sequence filled up with zeros to a whole number of blocks, which is what the kernel's masked load does to a ragged
    last block (utils.py:168-179) -- so a negative tail has maximum 0, a positive tail minimum 0."""
    g = torch.Generator().manual_seed(n + ks)
    x = (torch.randn(n, 2, 16, generator=g) * 3).to(torch.bfloat16)
    nb = -(-n // ks)
    seq = torch.nn.functional.pad(x.float(), (0, 0, 0, 0, 0, nb * ks - n)).permute(1, 2, 0).reshape(1, 32, nb * ks)
    F = torch.nn.functional
    lib = {"max": F.max_pool1d(seq, ks, ks), "min": -F.max_pool1d(-seq, ks, ks), "maxabs": F.max_pool1d(seq.abs(), ks, ks),
           "sum": F.avg_pool1d(seq, ks, ks) * ks}
    for kind, want in lib.items():
        got = O.pool(x, ks, kind)
        assert got.shape == (nb, 2, 16) and got.dtype == torch.bfloat16
        want = want.reshape(2, 16, nb).permute(2, 0, 1)
        if kind == "sum":
            assert torch.allclose(got.float(), want, rtol=2 ** -7, atol=1e-3)
        else:
            assert torch.equal(got.float(), want), kind
    with pytest.raises(KeyError):
        O.pool(x, ks, "median")


def test_pool_types_see_the_zero_fill_of_a_ragged_tail():
    x = torch.full((40, 1, 16), -2.0, dtype=torch.bfloat16)
    assert float(O.pool(x, 32, "max")[0].max()) == -2.0 and float(O.pool(x, 32, "max")[1].max()) == 0.0
    assert float(O.pool(-x, 32, "min")[1].min()) == 0.0 and float(O.pool(x, 32, "min")[1].min()) == -2.0
    assert float(O.pool(x, 32, "maxabs")[1].max()) == 2.0 and float(O.pool(x, 32, "sum")[1].max()) == -16.0
    one = torch.zeros(64, 1, 16, dtype=torch.bfloat16)
    one[37, 0, 5] = -7.0
    assert float(O.pool(one, 32, "min")[1, 0, 5]) == -7.0 and float(O.pool(one, 32, "maxabs")[1, 0, 5]) == 7.0
    assert float(O.pool(one, 32, "max").abs().max()) == 0.0


def test_pool_q_head_tail_rescale():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(300, 16, generator=g)
    y = O.pool_q_head(x, 128)
    assert torch.allclose(y[2], x[256:].mean(0), atol=1e-5)
    assert torch.allclose(y[0], x[:128].mean(0), atol=1e-6)


# ----- anti-diagonal sums ---------------------------------------------------------------------------
def test_diagonal_sums_bruteforce():
    g = torch.Generator().manual_seed(1)
    n, m = 8, 40
    p = torch.rand(n, m, generator=g, dtype=torch.float64)
    out = O.diagonal_sums(p)
    ref = torch.zeros(m, dtype=torch.float64)
    for j in range(m):
        for i in range(n):
            c = j + i - (n - 1)
            if 0 <= c < m:
                ref[j] += p[i, c]
    assert torch.allclose(out, ref, atol=1e-12)
    # last entry is the main diagonal of the trailing n x n square
    assert math.isclose(out[m - 1].item(), sum(p[i, m - n + i].item() for i in range(n)), rel_tol=1e-12)


def test_lastq_scores_invariants_and_bruteforce():
    g = torch.Generator().manual_seed(2)
    hq, hkv, n, d, bs = 4, 2, 512, 16, 128
    q = torch.randn(hq, n, d, generator=g)
    k = torch.randn(hkv, n, d, generator=g)
    vert, slash = O.lastq_scores(q, k, bs, logits_in_input_dtype=False)
    assert torch.allclose(vert.sum(-1), torch.ones(hq), atol=1e-5)
    assert torch.allclose(slash.sum(-1), torch.ones(hq), atol=1e-5)
    h = 3
    s = (q[h, -bs:].double() / math.sqrt(d)) @ k[h // 2].double().T
    for i in range(bs):
        s[i, n - bs + i + 1:] = -math.inf
    p = torch.softmax(s, -1)
    assert torch.allclose(vert[h].double(), p.mean(0), atol=1e-6)
    diag = sum(p[i, n - bs + i].item() for i in range(bs)) / bs
    assert math.isclose(slash[h, n - 1].item(), diag, rel_tol=1e-4)
    j = 200  # distance n-1-j behind each query
    ref = sum(p[i, j + i - (bs - 1)].item() for i in range(bs) if 0 <= j + i - (bs - 1) < n) / bs
    assert math.isclose(slash[h, j].item(), ref, rel_tol=1e-4, abs_tol=1e-9)


# ----- cumulative-mass selection -------------------------------------------------------------------
def test_cover_count_closed_forms():
    onehot = np.zeros(1000, dtype=np.float32)
    onehot[123] = 1.0
    assert O.cover_count(onehot, 0.95) == 1
    n = 1024  # uniform 2^-10: exactly representable, cumsum exact
    uni = np.full(n, 1.0 / n, dtype=np.float32)
    for thr in (0.5, 0.9, 0.95, 0.99):
        assert O.cover_count(uni, thr) == math.floor(float(np.float32(thr)) * n) + 1


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("thr", [0.9, 0.95, 0.99])
def test_cover_count_matches_literal_torch(seed, thr):
    x = rand_probs(4096 + 37 * seed, seed)
    assert O.cover_count(x.numpy(), thr) == literal_cover_topk(x, thr)


def test_cover_count_is_smallest_prefix_exceeding():
    x = rand_probs(300, 5).numpy()
    m = O.cover_count(x, 0.9)
    s = np.sort(x.astype(np.float64))[::-1]
    assert s[: m - 1].sum() <= 0.9 + 1e-9
    assert s[:m].sum() > 0.9 - 1e-9


@pytest.mark.parametrize("seed", range(8))
def test_cover_keep_le_matches_literal_and_excludes_crossing(seed):
    nb = 16
    g = torch.Generator().manual_seed(seed)
    a = torch.softmax(torch.randn(nb, nb, generator=g) * 2, -1).reshape(-1)
    score = 0.9 * nb
    kept = O.cover_keep_le(a.numpy(), score)
    lit = literal_cover_idx(a, score)
    assert sorted(kept.tolist()) == sorted(lit.tolist())
    assert a[kept].double().sum().item() <= score + 1e-6
    rest = np.setdiff1d(np.arange(nb * nb), kept)
    assert a[kept].double().sum().item() + a[rest].max().item() > score - 1e-6


def test_cover_keep_le_largest_exceeds_score_keeps_nothing():
    x = np.array([0.7, 0.2, 0.1], dtype=np.float32)
    assert O.cover_keep_le(x, 0.5).size == 0


def test_cover_keep_le_tie_order_is_index_ascending():
    x = np.array([0.25, 0.25, 0.25, 0.25], dtype=np.float32)
    assert O.cover_keep_le(x, 0.5).tolist() == [0, 1]
    assert O.cover_keep_le(x, 0.74).tolist() == [0, 1]
    assert O.cover_keep_le(x, 0.75).tolist() == [0, 1, 2]


@pytest.mark.parametrize("seed", range(8))
def test_cover_keep_rows_matches_literal_and_includes_crossing(seed):
    g = torch.Generator().manual_seed(100 + seed)
    a = torch.softmax(torch.randn(12, 20, generator=g) * 2, -1)
    keep = O.cover_keep_rows_ge(a.numpy(), 0.9)
    assert np.array_equal(keep, literal_each_row(a, 0.9))
    for r in range(a.shape[0]):
        sel = a[r][torch.from_numpy(keep[r])].double()
        assert sel.sum().item() >= 0.9 - 1e-6
        assert sel.sum().item() - sel.min().item() < 0.9 + 1e-6


def test_cover_keep_rows_never_reaching_keeps_one():
    a = np.array([[0.3, 0.4, 0.1], [0.5, 0.45, 0.05]], dtype=np.float32)
    keep = O.cover_keep_rows_ge(a, 0.9)
    assert keep[0].tolist() == [False, True, False]  # total 0.8 < 0.9: argmax of all-False -> 1 entry
    assert keep[1].tolist() == [True, True, False]


def test_fixed_point_conversion():
    x = np.array([1.0, 0.5, 2.0 ** -48, 2.0 ** -49, 0.0, -1.0, np.nan, 3.0 * 2.0 ** -30], dtype=np.float32)
    fx = O.to_fixed(x)
    assert fx.tolist() == [2 ** 48, 2 ** 47, 1, 0, 0, 0, 0, 3 * 2 ** 18]
    assert O.thr_le(0.5) == 2 ** 47 and O.thr_lt(0.5) == 2 ** 47 - 1


# ----- JS divergence ----------------------------------------------------------------------------------
def test_sqrt_js_vs_scipy():
    from scipy.spatial.distance import jensenshannon

    p, q = rand_probs(257, 1, 1.0), rand_probs(257, 2, 1.0)
    assert math.isclose(O.sqrt_js(p, q).item(), jensenshannon(p.numpy(), q.numpy()), rel_tol=1e-4)
    assert O.sqrt_js(p, p).item() == 0.0
    assert math.isclose(O.sqrt_js(p, q).item(), O.sqrt_js(q, p).item(), rel_tol=1e-6)


def test_sqrt_js_zero_entry_is_nan_and_compares_false():
    p = torch.tensor([0.5, 0.5, 0.0])
    q = torch.tensor([0.25, 0.25, 0.5])
    v = O.sqrt_js(p, q)
    assert torch.isnan(v)
    assert not bool(v < 0.5)


# ----- vertical-slash expansion ---------------------------------------------------------------------
def test_vs_id_list_bruteforce_nb5():
    ids = O.vs_id_list(cols=[0, 3], dists=[0, 2], nb=5)
    assert set(ids.tolist()) == {0, 5, 6, 10, 12, 15, 16, 18, 20, 22, 23, 24}
    assert len(ids) == 5 * 4
    # layout: slash part first (row-major over r, then d), then the vertical part
    assert ids[:10].tolist() == [0, 10, 6, 16, 12, 22, 18, 0, 24, 0]
    assert ids[10:].tolist() == [0, 0, 5, 0, 10, 0, 15, 18, 20, 23]


@pytest.mark.parametrize("seed", range(4))
def test_vs_mask_equals_id_set(seed):
    rng = np.random.default_rng(seed)
    nb = 11
    cols = np.concatenate([[0], rng.choice(np.arange(1, nb), 3, replace=False)])
    dists = np.concatenate([[0], rng.choice(np.arange(1, nb), 2, replace=False)])
    ids = set(O.vs_id_list(cols, dists, nb).tolist())
    m = O.vs_mask(cols, dists, nb)
    assert ids == set(O.mask_to_ids(m).tolist())
    assert all(m[r, r] and m[r, 0] for r in range(nb))
    assert not np.triu(m, 1).any()


def test_vs_ratio_counts_duplicates_hand_example():
    # 3x3 map, cols {0,2}, dists {0,1}.  id list (slash | vertical):
    #   slash: r=0:(0,0)->0,(1,0)->3 ; r=1:(1,1)->4,(2,1)->7 ; r=2:(2,2)->8, pad 0
    #   vert : r=0: 0, pad 0 ; r=1: 3, pad 0 ; r=2: 6, 8
    avg = np.array([[1.0, 0, 0], [0.5, 0.5, 0], [0.25, 0.25, 0.5]], dtype=np.float32)
    ids = O.vs_id_list([0, 2], [0, 1], 3)
    assert ids.tolist() == [0, 3, 4, 7, 8, 0, 0, 0, 3, 0, 6, 8]
    lit = avg.reshape(-1)[ids].astype(np.float64).sum() / avg.astype(np.float64).sum()
    assert math.isclose(lit, (1 + .5 + .5 + .25 + .5 + 1 + 1 + 1 + .5 + 1 + .25 + .5) / 3.0)
    assert math.isclose(O.vs_ratio(avg, [0, 2], [0, 1]), lit, rel_tol=1e-12)
    assert O.vs_ratio(avg, [0, 2], [0, 1]) > 1.0


@pytest.mark.parametrize("seed", range(4))
def test_vs_ratio_matches_literal_gather(seed):
    rng = np.random.default_rng(seed)
    nb = 9
    avg = np.tril(rng.random((nb, nb))).astype(np.float32)
    avg /= avg.sum(1, keepdims=True)
    cols = np.concatenate([[0], rng.choice(np.arange(1, nb), 3, replace=False)])
    dists = np.concatenate([[0], rng.choice(np.arange(1, nb), 3, replace=False)])
    ids = O.vs_id_list(cols, dists, nb)
    lit = avg.reshape(-1)[ids].astype(np.float64).sum() / avg.astype(np.float64).sum()
    assert math.isclose(O.vs_ratio(avg, cols, dists), lit, rel_tol=1e-9)


# ----- masked attention -------------------------------------------------------------------------------
def test_masked_attention_full_mask_is_sdpa_causal():
    g = torch.Generator().manual_seed(4)
    hq, hkv, n, d, bs = 4, 2, 300, 32, 128
    q, k, v = (torch.randn(h, n, d, generator=g) for h in (hq, hkv, hkv))
    nb = 3
    mask = np.tril(np.ones((nb, nb), dtype=bool))[None].repeat(hq, 0)
    out, avg = O.masked_attention(q, k, v, mask, bs, 1 / math.sqrt(d), want_avg=np.ones(hq, bool))
    ke, ve = k.repeat_interleave(2, 0), v.repeat_interleave(2, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(q[None], ke[None], ve[None], is_causal=True)[0]
    assert torch.allclose(out, ref, atol=2e-5)
    assert torch.allclose(avg.sum(-1), torch.ones(hq, nb), atol=1e-5)
    s = (q[1] @ ke[1].T) / math.sqrt(d)
    s = s.masked_fill(torch.triu(torch.ones(n, n, dtype=torch.bool), 1), -math.inf)
    p = torch.softmax(s, -1)
    assert math.isclose(avg[1, 2, 1].item(), p[256:300, 128:256].sum().item() / 44, rel_tol=1e-4)


def test_masked_attention_diagonal_mask_is_per_block_causal():
    g = torch.Generator().manual_seed(5)
    n, d, bs = 256, 16, 128
    q, k, v = (torch.randn(1, n, d, generator=g) for _ in range(3))
    mask = np.eye(2, dtype=bool)[None]
    out, _ = O.masked_attention(q, k, v, mask, bs, 0.25)
    for b in range(2):
        sl = slice(b * bs, (b + 1) * bs)
        ref = torch.nn.functional.scaled_dot_product_attention(q[:, sl][None], k[:, sl][None], v[:, sl][None],
                                                               is_causal=True, scale=0.25)[0]
        assert torch.allclose(out[:, sl], ref, atol=2e-5)


# ----- sharing scenarios on a toy table ----------------------------------------------------------------
def _toy(seed=0, n=1024, hq=4, hkv=2, d=32):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(hq, n, d, generator=g)
    k = torch.randn(hkv, n, d, generator=g)
    v = torch.randn(hkv, n, d, generator=g)
    k[:, :8] *= 3
    return q, k, v


TOY_TABLE = {"clusters": {"a": [[0, 0], [0, 1], [1, 0], [1, 1]], "b": [[0, 2], [0, 3], [1, 2], [1, 3]]},
             "shared_clusters": ["a"]}
KW = dict(bs=128, min_budget=128, max_budget=None, pattern_threshold=0.9, similarity_threshold=0.5,
          fallback_threshold=1e9, queryaware_threshold=0.0)


def test_decode_attention_is_sdpa_with_gqa_and_closed_forms():
    g = torch.Generator().manual_seed(11)
    hq, hkv, n, d = 8, 2, 300, 16
    q = torch.randn(hq, d, generator=g)
    k = torch.randn(hkv, n, d, generator=g)
    v = torch.randn(hkv, n, d, generator=g)
    out = O.decode_attention(q, k, v, 0.3)
    ref = torch.nn.functional.scaled_dot_product_attention(q[None, :, None, :], k[None], v[None], scale=0.3,
                                                           enable_gqa=True)[0, :, 0]
    assert torch.allclose(out, ref, atol=1e-5)
    # a single key: the output is that key's value, whatever the logit
    one = O.decode_attention(q, k[:, :1], v[:, :1], 7.0)
    assert torch.allclose(one, v[:, 0].repeat_interleave(hq // hkv, 0), atol=1e-6)
    # equal logits (zero query): the plain mean of the values
    mean = O.decode_attention(torch.zeros(hq, d), k, v, 1.0)
    assert torch.allclose(mean, v.mean(1).repeat_interleave(hq // hkv, 0), atol=1e-5)
    # a transposed head mapping (h % hkv instead of h // g) must differ
    wrong = torch.stack([torch.softmax((k[h % hkv] @ q[h]) * 0.3, 0) @ v[h % hkv] for h in range(hq)])
    assert not torch.allclose(out, wrong, atol=1e-3)


def _rope_tables(n, d, theta=10000.0, dtype=torch.bfloat16):
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = torch.arange(n, dtype=torch.float32)[:, None] * inv[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def test_rope_rotate_is_the_hugging_face_expression_and_closed_forms():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    g = torch.Generator().manual_seed(21)
    hq, hkv, n, d = 4, 2, 77, 32
    q = (torch.randn(1, hq, n, d, generator=g) * 3).to(torch.bfloat16)
    k = (torch.randn(1, hkv, n, d, generator=g) * 3).to(torch.bfloat16)
    cos, sin = _rope_tables(n, d)
    q_hf, k_hf = apply_rotary_pos_emb(q, k, cos[None], sin[None])  # the elementwise bf16 evaluation, on the CPU
    assert torch.equal(O.rope_rotate(q[0], cos, sin), q_hf[0])
    assert torch.equal(O.rope_rotate(k[0], cos, sin), k_hf[0])
    # angle 0: identity; quarter turn (cos 0, sin 1): rotate_half itself
    one, zero = torch.ones(n, d, dtype=torch.bfloat16), torch.zeros(n, d, dtype=torch.bfloat16)
    assert torch.equal(O.rope_rotate(q[0], one, zero), q[0])
    quarter = O.rope_rotate(q[0], zero, one)
    assert torch.equal(quarter[..., : d // 2], -q[0][..., d // 2:]) and torch.equal(quarter[..., d // 2:], q[0][..., : d // 2])
    # a rotation: the (i, i + d/2) pairs keep their length, and q.k depends on the position difference only
    # (both within the bf16 roundings of the three steps)
    rq = O.rope_rotate(q[0], cos, sin).float()
    pair_len = lambda x: (x[..., : d // 2] ** 2 + x[..., d // 2:] ** 2).sqrt()
    assert torch.allclose(pair_len(rq), pair_len(q[0].float()), rtol=2e-2, atol=2e-2)
    x = torch.randn(d, generator=g).to(torch.bfloat16)
    same = O.rope_rotate(x.expand(1, n, d), cos, sin).float()[0]  # the same vector at every position
    d5 = (same[5:] * same[:-5]).sum(-1)  # <R(p+5) x, R(p) x> must not depend on p
    assert (d5 - d5[0]).abs().max().item() < 0.05 * d5.abs().max().item() + 0.3
    # swapping the sign of the rotation (a transposed rotate_half) must differ
    wrong = (q[0].float() * cos.float() - torch.cat((-q[0].float()[..., d // 2:], q[0].float()[..., : d // 2]), -1)
             * sin.float()).to(torch.bfloat16)
    assert not torch.equal(wrong, q_hf[0])


def test_sharing_scenarios():
    q, k, v = _toy()
    sh = O.OracleSharing(O.ClusterTable(TOY_TABLE["clusters"], TOY_TABLE["shared_clusters"]))
    r0 = sh.layer(q, k, v, 0, **KW)
    # (i) first non-QA head of the shared cluster becomes the dense pivot; (ii) its same-layer sibling does not share
    assert r0.decision.tolist() == [O.DEC_DENSE, O.DEC_VS, O.DEC_VS, O.DEC_VS]
    nb = 8
    assert np.array_equal(r0.mask[0], np.tril(np.ones((nb, nb), bool)))
    assert sh.state["a"].pivot_head == 0 and sh.state["a"].pattern is not None
    # (v) the non-shared cluster never elects a pivot
    assert sh.state["b"].pivot_head is None
    # every row holds its sink column and its diagonal block
    for h in range(4):
        assert all(r0.mask[h, r, 0] and r0.mask[h, r, r] for r in range(nb))
    # (iii) next layer: identical inputs -> JS = 0 -> both cluster members share (fallback disabled by 1e9)
    r1 = sh.layer(q, k, v, 1, **KW)
    assert r1.decision.tolist() == [O.DEC_SHARE, O.DEC_SHARE, O.DEC_VS, O.DEC_VS]
    assert r1.js_v[0] == 0.0 and r1.js_s[0] == 0.0
    assert (r1.mask[0] & sh.state["a"].pattern).sum() == sh.state["a"].pattern.sum()
    assert r1.nv_final[0] == 1 and r1.ns_final[0] == 1


def test_sharing_blocked_by_fallback_and_similarity():
    q, k, v = _toy()
    sh = O.OracleSharing(O.ClusterTable(TOY_TABLE["clusters"], TOY_TABLE["shared_clusters"]))
    kw = dict(KW)
    sh.layer(q, k, v, 0, **kw)
    kw["fallback_threshold"] = 0.0  # vs_ratio >= 0 always -> never share
    r1 = sh.layer(q, k, v, 1, **kw)
    assert O.DEC_SHARE not in r1.decision.tolist()
    # (iv) a dissimilar head falls back: similarity threshold 0 can never be met (JS >= 0)
    sh.reset_state()
    kw = dict(KW, similarity_threshold=0.0)
    sh.layer(q, k, v, 0, **kw)
    r1 = sh.layer(q, k, v, 1, **kw)
    assert O.DEC_SHARE not in r1.decision.tolist()


def test_query_aware_head_never_becomes_pivot():
    q, k, v = _toy()
    sh = O.OracleSharing(O.ClusterTable(TOY_TABLE["clusters"], TOY_TABLE["shared_clusters"]))
    kw = dict(KW, queryaware_threshold=10.0)  # every head with a finite JS is query-aware
    r0 = sh.layer(q, k, v, 0, **kw)
    assert all(d == O.DEC_QA for d in r0.decision.tolist())
    assert sh.state["a"].pivot_head is None
    assert r0.mask[:, 0, 0].all()
    assert not np.triu(r0.mask[0], 1).any()


def test_reset_state_clears_pivots():
    q, k, v = _toy()
    sh = O.OracleSharing(O.ClusterTable(TOY_TABLE["clusters"], TOY_TABLE["shared_clusters"]))
    sh.layer(q, k, v, 0, **KW)
    sh.reset_state()
    assert sh.state["a"].pivot_head is None and sh.state["a"].pattern is None


# ----- float stages of the query-aware path ------------------------------------------------------------
def _all_bf16_values():
    """Every one of the 65536 bf16 bit patterns, as a [65536] bf16 tensor."""
    return torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def _same_bits_or_both_nan(a, b):
    a, b = a.contiguous(), b.contiguous()
    same = a.view(torch.int16) == b.view(torch.int16)
    return bool((same | (torch.isnan(a.float()) & torch.isnan(b.float()))).all())


@pytest.mark.parametrize("d", [16, 32, 64, 128, 256])
def test_scaled_last_q_is_torchs_tensor_by_float_division_exhaustively(d):
    """attention_sharing.py:127 evaluates `q[:, -bs:] / math.sqrt(D)` on a bf16 tensor.  Checked against that very
    expression (torch divides in fp32 and rounds to bf16) on EVERY bf16 value, so the multiply-by-reciprocal the
    oracle and the kernels use instead of a true division is shown to give the same bits, also for D = 32 and 128
    where sqrt(D) is no power of two."""
    allv = _all_bf16_values()
    bs = 128
    q = allv.reshape(-1, bs, d)  # [Hq, N = bs, D]: the last block is the whole tensor
    ref = q[:, -bs:] / math.sqrt(d)
    assert ref.dtype == torch.bfloat16
    assert _same_bits_or_both_nan(O.scaled_last_q(q, bs), ref)
    # and only the last bs tokens are taken
    q2 = torch.cat([torch.ones(q.shape[0], 5, d, dtype=torch.bfloat16), q], dim=1)
    assert _same_bits_or_both_nan(O.scaled_last_q(q2, bs), ref)


def test_pool_q_head_is_the_reference_expression_on_bf16():
    """attention_sharing.py:350-356 literally (zero pad, view, mean, rescale the tail in place) on CPU bf16 tensors,
    for every tail length; the tail's `* bs / (bs - pad)` is two bf16 roundings, which the oracle must reproduce."""
    g = torch.Generator().manual_seed(21)
    bs, d = 128, 16
    for n in [128, 129, 200, 255, 256, 257, 300, 383]:
        q = (torch.randn(n, d, generator=g) * 3).to(torch.bfloat16)
        nb = math.ceil(n / bs)
        pad_q = nb * bs - n
        avg_q = torch.nn.functional.pad(q, (0, 0, 0, pad_q), value=0).view(nb, bs, d).mean(1)
        avg_q[-1, :] = avg_q[-1, :] * bs / (bs - pad_q)
        got = O.pool_q_head(q, bs)
        assert got.dtype == torch.bfloat16
        # the block means may differ by fp32 summation order (one bf16 ulp, rarely); the tail arithmetic on top of
        # an identical mean must be identical, which the exhaustive check below covers
        diff = (got.float() - avg_q.float()).abs()
        assert (diff <= 2.0 ** -7 * avg_q.float().abs() + 1e-30).all()
        assert (got.view(torch.int16) != avg_q.view(torch.int16)).float().mean().item() <= 0.02
    # tail rescale alone, exhaustively: every bf16 mean value x every pad
    allv = _all_bf16_values()
    for pad in range(1, bs):
        want = allv * bs / (bs - pad)
        # the oracle's arithmetic for that step: fp32 product rounded to bf16, fp32 quotient rounded to bf16
        mine = ((allv.float() * bs).to(torch.bfloat16).float() / (bs - pad)).to(torch.bfloat16)
        assert _same_bits_or_both_nan(mine, want), pad
    # and pool_q_head applies exactly that step to the tail block's mean
    q = (torch.randn(130, d, generator=g)).to(torch.bfloat16)
    tail_mean = torch.nn.functional.pad(q[128:], (0, 0, 0, 126)).float().mean(0).to(torch.bfloat16)
    want = tail_mean * 128 / 2
    assert _same_bits_or_both_nan(O.pool_q_head(q, 128)[1], want)


def test_pooled_qk_probs_fp64_bruteforce_and_closed_forms():
    """attention_sharing.py:197-200: softmax over the nb pooled keys of (mean of the last block's scaled queries) .
    pooled key, query head h reading kv head h // g (repeat_interleave, :193-194)."""
    g = torch.Generator().manual_seed(22)
    hq, hkv, n, d, bs = 4, 2, 512, 16, 128
    nb = n // bs
    q = torch.randn(hq, n, d, generator=g)
    k = torch.randn(hkv, n, d, generator=g)
    kbar = O.pool_avg(k.transpose(0, 1).contiguous(), bs)  # [nb, Hkv, D]
    got = O.pooled_qk_probs(q, kbar, bs, logits_in_input_dtype=False)
    assert got.shape == (hq, nb) and got.dtype == torch.float32
    ref = torch.zeros(hq, nb, dtype=torch.float64)
    for h in range(hq):
        qm = [sum(q[h, n - bs + i, c].item() / math.sqrt(d) for i in range(bs)) / bs for c in range(d)]
        logits = [sum(qm[c] * kbar[j, h // 2, c].item() for c in range(d)) for j in range(nb)]
        mx = max(logits)
        e = [math.exp(x - mx) for x in logits]
        for j in range(nb):
            ref[h, j] = e[j] / sum(e)
    assert torch.allclose(got.double(), ref, atol=2e-6)
    assert torch.allclose(got.sum(-1), torch.ones(hq), atol=1e-6)
    # a head mapping h % Hkv would give heads 1 and 2 each other's keys: the two mappings must be distinguishable here
    wrong = torch.stack([ref[h] for h in (0, 2, 1, 3)])
    assert (wrong - ref).abs().max().item() > 1e-3
    # identical pooled keys -> every block gets 1/nb, whatever the queries
    kconst = kbar[:1].expand(nb, hkv, d).contiguous()
    assert torch.allclose(O.pooled_qk_probs(q, kconst, bs, logits_in_input_dtype=False),
                          torch.full((hq, nb), 1.0 / nb), atol=1e-6)
    # one pooled key aligned with the mean query and far longer than the others takes all the mass
    kb2 = kbar.clone()
    kb2[2, 0] = 1000.0 * q[0, -bs:].mean(0)
    p = O.pooled_qk_probs(q, kb2, bs, logits_in_input_dtype=False)
    assert p[0].argmax().item() == 2 and p[0, 2].item() > 0.999
    # only the last block's queries matter
    q2 = q.clone()
    q2[:, : n - bs] = 0
    assert torch.equal(O.pooled_qk_probs(q2, kbar, bs, logits_in_input_dtype=False), got)


def test_pooled_qk_probs_bf16_logit_rounding_is_the_einsums():
    """With bf16 inputs the reference's einsum returns bf16 logits (attention_sharing.py:197-199): compared with that
    very einsum on CPU bf16 tensors (fp32 accumulation order may move a logit by one bf16 ulp, rarely)."""
    g = torch.Generator().manual_seed(23)
    hq, hkv, n, d, bs = 8, 2, 2048, 64, 128
    q = torch.randn(hq, n, d, generator=g).to(torch.bfloat16)
    k = torch.randn(hkv, n, d, generator=g).to(torch.bfloat16)
    kbar = O.pool_avg(k.transpose(0, 1).contiguous(), bs)
    last_q = (q[:, -bs:] / math.sqrt(d)).transpose(0, 1)[None]          # [1, bs, Hq, D] as in the reference
    avg_k = kbar[None].repeat_interleave(hq // hkv, 2)                   # [1, nb, Hq, D]
    lit = torch.einsum("bihd, bjhd -> bhij", last_q.mean(1, keepdim=True), avg_k).squeeze(2)
    lit = torch.softmax(lit, dim=-1, dtype=torch.float32)[0]
    got = O.pooled_qk_probs(q, kbar, bs, logits_in_input_dtype=True)
    assert torch.allclose(got, lit, rtol=2.0 ** -6, atol=1e-7)  # one bf16 ulp of a logit of size <= 2 moves p by <= 2^-7
    assert ((got - lit).abs() > 1e-6 * lit).float().mean().item() <= 0.05


def test_block_probs_fp64_bruteforce_and_closed_forms():
    """attention_sharing.py:357-360: rows of softmax((avg_q / sqrt(D)) . avg_k^T) under the block-causal mask."""
    g = torch.Generator().manual_seed(24)
    nb, d = 7, 16
    qbar = torch.randn(nb, d, generator=g)
    kbar = torch.randn(nb, d, generator=g)
    got = O.block_probs(qbar, kbar, logits_in_input_dtype=False)
    assert got.shape == (nb, nb) and got.dtype == torch.float32
    for r in range(nb):
        logits = [sum(qbar[r, c].item() / math.sqrt(d) * kbar[j, c].item() for c in range(d)) for j in range(r + 1)]
        mx = max(logits)
        e = [math.exp(x - mx) for x in logits]
        for j in range(nb):
            want = e[j] / sum(e) if j <= r else 0.0
            assert math.isclose(got[r, j].item(), want, rel_tol=1e-5, abs_tol=1e-8), (r, j)
    assert torch.allclose(got.sum(-1), torch.ones(nb), atol=1e-6)
    assert (torch.triu(got, 1) == 0).all()
    assert got[0, 0].item() == 1.0
    # zero queries: row r is uniform over its r + 1 visible blocks
    z = O.block_probs(torch.zeros(nb, d), kbar, logits_in_input_dtype=False)
    for r in range(nb):
        assert torch.allclose(z[r, : r + 1], torch.full((r + 1,), 1.0 / (r + 1)), atol=1e-7)
    # transposed operands (k . q^T) must be caught: the matrix is not symmetric
    swapped = O.block_probs(kbar, qbar, logits_in_input_dtype=False)
    assert (swapped - got).abs().max().item() > 1e-3
    # the scale matters: dropping 1/sqrt(D) changes the result
    unscaled = O.block_probs(qbar * math.sqrt(d), kbar, logits_in_input_dtype=False)
    assert (unscaled - got).abs().max().item() > 1e-3


def test_block_probs_bf16_is_the_reference_expression():
    """bf16 inputs: the literal expression of attention_sharing.py:357-360 on CPU bf16 tensors."""
    g = torch.Generator().manual_seed(25)
    nb, d = 24, 128
    avg_q = torch.randn(nb, d, generator=g).to(torch.bfloat16)
    avg_k = torch.randn(nb, d, generator=g).to(torch.bfloat16)
    tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    attn = torch.einsum("id, jd -> ij", avg_q / math.sqrt(d), avg_k).masked_fill_(~tri, float("-inf"))
    lit = torch.softmax(attn, dim=-1, dtype=torch.float32)
    got = O.block_probs(avg_q, avg_k, logits_in_input_dtype=True)
    assert torch.allclose(got, lit, rtol=2.0 ** -5, atol=1e-7)
    assert ((got - lit).abs() > 1e-6 * lit).float().mean().item() <= 0.05


# ----- the reference kernel's own roundings ---------------------------------------------------------------
def test_masked_attention_ref_roundings_against_fp32_and_exact_case():
    """masked_attention_ref_roundings (shareprefill_attn.py:383-471 with its bf16 roundings) must sit within the
    rounding noise of the fp32 oracle: the output rounding alone gives mean|d|/mean|x| ~ 1.4e-3, the bf16
    probabilities add ~1.6e-3 in quadrature (2.06e-3 together); anything systematic (a dropped block, a wrong
    rescale) shows in the bias, which rounding noise does not have.  On inputs whose probabilities are exact powers
    of two the probability rounding vanishes and the result must equal the bf16 rounding of the fp32 oracle."""
    g = torch.Generator().manual_seed(26)
    hq, hkv, n, d, bs = 4, 2, 700, 64, 128
    q, k, v = (torch.randn(h, n, d, generator=g).to(torch.bfloat16) for h in (hq, hkv, hkv))
    nb = math.ceil(n / bs)
    mask = np.tril(torch.rand(hq, nb, nb, generator=g).numpy() < 0.6)
    mask[:, np.arange(nb), np.arange(nb)] = True
    mask[:, :, 0] = True
    scale = 1.0 / math.sqrt(d)
    ref, _ = O.masked_attention(q, k, v, mask, bs, scale)
    emu, _ = O.masked_attention(q, k, v, mask, bs, scale, emulate_bf16=True)
    mean_rel = ((emu - ref).abs().mean() / ref.abs().mean()).item()
    only_out = ((ref.to(torch.bfloat16).float() - ref).abs().mean() / ref.abs().mean()).item()
    assert 1.2e-3 <= only_out <= 1.6e-3
    assert only_out <= mean_rel <= 2.4e-3
    assert abs((emu - ref).mean().item()) / ref.abs().mean().item() <= 1e-4
    assert (emu - ref).abs().max().item() <= 2e-2
    # exact case: integer logits in base-2 units (softmax_scale = ln 2, q and k with entries in {-1, 0, 1})
    qi = torch.randint(-1, 2, (hq, n, d), generator=g).float() * (torch.rand(hq, n, d, generator=g) < 0.15)
    ki = torch.randint(-1, 2, (hkv, n, d), generator=g).float() * (torch.rand(hkv, n, d, generator=g) < 0.3)
    ref, _ = O.masked_attention(qi, ki, v, mask, bs, math.log(2.0))
    emu = O.masked_attention_ref_roundings(qi, ki, v, mask, bs, math.log(2.0))
    want = ref.to(torch.bfloat16)
    neq = (emu.view(torch.int16) != want.view(torch.int16))
    assert neq.float().mean().item() <= 2e-3          # a value within fp32 noise of a rounding boundary may flip
    assert ((emu.float() - ref).abs().mean() / ref.abs().mean()).item() <= only_out * 1.05

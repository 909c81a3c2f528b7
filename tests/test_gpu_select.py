"""GPU parity (bit-exact): cumulative-mass selection, budgets, top-k sets and masks against the CPU oracle
on identical fp32 score inputs."""

import numpy as np
import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu


def _probs(rows, n, seed, sharp=3.0):
    g = torch.Generator().manual_seed(seed)
    return torch.softmax(torch.randn(rows, n, generator=g) * sharp, dim=-1)


@pytest.mark.parametrize("n", [1000, 8192, 131072])
@pytest.mark.parametrize("thr", [0.5, 0.9, 0.95, 0.99])
def test_cover_count_bit_exact(gpu_device, n, thr):
    from shareprefill_amd import ops

    x = _probs(6, n, n, sharp=4.0)
    x[1] = 1.0 / n                       # all ties
    x[2] = 0.0
    x[2, 17] = 1.0                       # one-hot
    x[3, : n // 2] = 0.0                 # exact zeros
    x[3] /= x[3].sum()
    got = ops.cover_count(x.to(gpu_device).contiguous(), thr).cpu().tolist()
    want = [O.cover_count(x[i].numpy(), thr) for i in range(x.shape[0])]
    assert got == want


def test_cover_count_threshold_edges(gpu_device):
    from shareprefill_amd import ops

    x = _probs(2, 4096, 3).to(gpu_device).contiguous()
    assert ops.cover_count(x, -1.0).cpu().tolist() == [1, 1]
    assert ops.cover_count(x, 2.0).cpu().tolist() == [4097, 4097]   # never exceeded: every entry counted
    assert ops.cover_count(x, 0.0).cpu().tolist() == [O.cover_count(x[i].cpu().numpy(), 0.0) for i in range(2)]


@pytest.mark.parametrize("hq,n", [(8, 8192), (4, 1000)])
def test_budgets_bit_exact(gpu_device, hq, n):
    from shareprefill_amd import ops

    v, s = _probs(hq, n, 1, 5.0), _probs(hq, n, 2, 2.0)
    nb = -(-n // 128)
    nv, ns = ops.cover_budgets(v.to(gpu_device), s.to(gpu_device), 128, 0.95, 8, nb)

    def want(x):
        return [min(max(O.cover_count(x[h].numpy(), 0.95) // 128 + 1, 8), nb) for h in range(hq)]

    assert nv.cpu().tolist() == want(v) and ns.cpu().tolist() == want(s)


@pytest.mark.parametrize("nb", [16, 64, 100, 256, 1024, 2048])
@pytest.mark.parametrize("thr", [0.9, 0.95])
def test_cover_select_global_bit_exact(gpu_device, nb, thr):
    from shareprefill_amd import ops

    g = torch.Generator().manual_seed(nb)
    logits = torch.randn(3, nb, nb, generator=g) * 2
    tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    a = torch.softmax(logits.masked_fill(~tri, float("-inf")), dim=-1)
    a[2] = torch.softmax(torch.zeros(nb, nb).masked_fill(~tri, float("-inf")), dim=-1)  # uniform rows: heavy ties
    score = float(np.float32(thr * nb))
    mask = torch.zeros(3, nb, (nb + 63) // 64, dtype=torch.int64, device=gpu_device)
    en = torch.tensor([1, 1, 1], dtype=torch.int32, device=gpu_device)
    ops.cover_select_global(a.to(gpu_device).contiguous(), score, mask, en)
    got = ops.mask_to_bool(mask, nb).cpu().numpy()
    for v in range(3):
        kept = O.cover_keep_le(a[v].numpy().reshape(-1), score)
        want = np.zeros(nb * nb, dtype=bool)
        want[kept] = True
        want = want.reshape(nb, nb) & tri.numpy()
        want[0, 0] = True
        assert np.array_equal(got[v], want), f"vector {v}"


def test_cover_select_global_skips_disabled(gpu_device):
    from shareprefill_amd import ops

    a = torch.softmax(torch.zeros(2, 16, 16), -1).to(gpu_device)
    mask = torch.zeros(2, 16, 1, dtype=torch.int64, device=gpu_device)
    ops.cover_select_global(a, 8.0, mask, torch.tensor([0, 1], dtype=torch.int32, device=gpu_device))
    assert int(mask[0].abs().sum()) == 0 and int(mask[1].abs().sum()) != 0


@pytest.mark.parametrize("nb", [8, 64, 100, 1024])
def test_cover_select_rows_bit_exact(gpu_device, nb):
    from shareprefill_amd import ops

    g = torch.Generator().manual_seed(nb + 1)
    tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    a = torch.softmax((torch.randn(nb, nb, generator=g) * 3).masked_fill(~tri, float("-inf")), dim=-1)
    a[nb // 2] *= 0.5                     # a row that never reaches the threshold keeps one entry
    a[nb - 1] = a[nb - 1].mean()          # all ties
    got = ops.mask_to_bool(ops.cover_select_rows(a.to(gpu_device).contiguous(), 0.9), nb).cpu().numpy()
    want = O.cover_keep_rows_ge(a.numpy(), 0.9) & tri.numpy()
    want[0, 0] = True
    assert np.array_equal(got, want)


def _table_tensor(table, layer, hq, gpu):
    ids = {cid: i for i, cid in enumerate(sorted(table["shared_clusters"]))}
    hc = torch.full((hq,), -1, dtype=torch.int32)
    for cid, pairs in table["clusters"].items():
        for lay, h in pairs:
            if lay == layer and cid in ids:
                hc[h] = ids[cid]
    return hc.to(gpu), ids


def test_decide_and_mask_match_oracle_on_identical_scores(gpu_device):
    """Feeds the same pooled vectors / budgets to sp_share_decide + sp_build_mask and to the oracle."""
    from shareprefill_amd import ops

    hq, nb, minb = 8, 40, 3
    g = torch.Generator().manual_seed(9)
    vert = torch.softmax(torch.randn(hq, nb, generator=g) * 2, -1)
    slash = torch.softmax(torch.randn(hq, nb, generator=g) * 2, -1)
    nv = torch.randint(minb, 12, (hq,), generator=g, dtype=torch.int32)
    ns = torch.randint(minb, 12, (hq,), generator=g, dtype=torch.int32)
    use_qa = torch.tensor([0, 0, 1, 0, 0, 0, 0, 1], dtype=torch.int32)
    table = {"clusters": {"a": [[0, 0], [0, 1], [0, 2]], "b": [[0, 3], [0, 4]], "c": [[0, 5], [0, 6], [0, 7]]},
             "shared_clusters": ["a", "c"]}
    hc, ids = _table_tensor(table, 0, hq, gpu_device)
    state = ops.ClusterState(len(ids), nb, gpu_device)
    dev = lambda t: t.to(gpu_device).contiguous()
    dec, jv, js, nvf, nsf = ops.share_decide(state, hc, 0, dev(vert), dev(slash), dev(use_qa), dev(nv), dev(ns),
                                             minb, 0.5, 0.9)
    # heads 0 and 5 are the first non-query-aware heads of the shared clusters -> dense pivots
    assert dec.cpu().tolist() == [O.DEC_DENSE, O.DEC_VS, O.DEC_QA, O.DEC_VS, O.DEC_VS, O.DEC_DENSE, O.DEC_VS, O.DEC_QA]
    assert nvf.cpu().tolist() == [int(nv[h]) if h not in (2, 7) else minb for h in range(hq)]
    mask = ops.mask_to_bool(ops.build_mask(state, hc, dec, dev(vert), dev(slash), nvf, nsf), nb).cpu().numpy()
    for h in range(hq):
        if dec[h] == O.DEC_DENSE:
            want = np.tril(np.ones((nb, nb), bool))
        else:
            cols, dists = O.OracleSharing._vs_sets(vert[h], slash[h], int(nvf[h]), int(nsf[h]), nb)
            want = O.vs_mask(cols, dists, nb)
        assert np.array_equal(mask[h], want), f"head {h}"
    # the pivot's stored sets are its own top-k sets with its own budgets
    for cid, h in (("a", 0), ("c", 5)):
        cols, dists = O.OracleSharing._vs_sets(vert[h], slash[h], int(nv[h]), int(ns[h]), nb)
        c = ids[cid]
        assert sorted(torch.nonzero(state.cols[c]).reshape(-1).cpu().tolist()) == sorted(cols.tolist())
        assert sorted(torch.nonzero(state.dists[c]).reshape(-1).cpu().tolist()) == sorted(dists.tolist())
        assert torch.equal(state.vert[c].cpu(), vert[h])
        assert state.info[c].cpu().tolist()[:5] == [h, 0, int(nv[h]), int(ns[h]), 0]


def test_row_pointers_docstring_vector(gpu_device):
    """shareprefill_attn.py:235-236: ids [0,5,8,9,13,14] on a 4x4 grid -> [0,1,2,4,6]."""
    import json
    import os

    from shareprefill_amd import ops

    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_docstring_vectors.json")) as f:
        v = json.load(f)["csr_row_pointers"]
    b = torch.zeros(1, v["grid"], v["grid"], dtype=torch.bool)
    for i in v["block_ids"]:
        b[0, i // v["grid"], i % v["grid"]] = True
    m = ops.bool_to_mask(b).to(gpu_device)
    assert ops.mask_row_pointers(m).cpu().tolist() == [v["row_pointers"]]
    assert ops.mask_to_block_idx(m, v["grid"])[0].cpu().tolist() == v["block_ids"]


def test_heads_without_a_cluster_slot_never_touch_the_state(gpu_device):
    """head_cluster[h] = -1 (no shared cluster) is legal for every head, also for one a caller marks dense or
    shared in its own decision vector, and values >= n_clusters are a caller's mistake: neither may be used as an
    index into the state slabs.  The state is surrounded by canaries here; a dense head with slot -1 (which would
    write accum[-2], the pattern slab before slot 0 and ratio[-1]) and one with slot n_clusters must leave every slab
    and every canary as it was, while the one dense head with a valid slot is processed."""
    from shareprefill_amd import ops

    hq, nb, c = 6, 40, 2
    nbw = 1
    g = torch.Generator().manual_seed(19)
    state = ops.ClusterState(c, nb, gpu_device)

    def guarded(shape, dtype, fill):
        """a slab with one slot of canary in front and one behind; returns (whole buffer, view of the middle)"""
        buf = torch.full((c + 2, *shape), fill, dtype=dtype, device=gpu_device)
        return buf, buf[1:c + 1]

    bufs = {}
    for name, shape, dtype, fill in (("info", (8,), torch.int32, 77), ("ratio", (), torch.float64, 7.5),
                                     ("vert", (nb,), torch.float32, 7.5), ("slash", (nb,), torch.float32, 7.5),
                                     ("cols", (nb,), torch.uint8, 7), ("dists", (nb,), torch.uint8, 7),
                                     ("pattern", (nb, nbw), torch.int64, 77), ("accum", (2,), torch.int64, 77)):
        bufs[name], mid = guarded(shape, dtype, fill)
        mid.copy_(getattr(state, name))
        setattr(state, name, mid)
    state.struct = ops.ClusterStateStruct(c, nb, nbw, 0, *(getattr(state, n).data_ptr() for n in
                                          ("info", "ratio", "vert", "slash", "cols", "dists", "pattern", "accum")))
    state.reset()
    hc = torch.tensor([-1, 0, 2, -1, 1, 57], dtype=torch.int32, device=gpu_device)
    vert = torch.softmax(torch.randn(hq, nb, generator=g) * 2, -1).to(gpu_device)
    slash = torch.softmax(torch.randn(hq, nb, generator=g) * 2, -1).to(gpu_device)
    nv = torch.full((hq,), 4, dtype=torch.int32, device=gpu_device)
    use_qa = torch.zeros(hq, dtype=torch.int32, device=gpu_device)
    dec, _, _, nvf, nsf = ops.share_decide(state, hc, 0, vert, slash, use_qa, nv, nv, 3, 0.5, 0.9)
    # only the heads with slots 0 and 1 can become pivots; slot 2 and 57 do not exist, -1 is "no cluster"
    assert dec.cpu().tolist() == [O.DEC_VS, O.DEC_DENSE, O.DEC_VS, O.DEC_VS, O.DEC_DENSE, O.DEC_VS]
    before = {k: v.clone() for k, v in bufs.items()}
    # a caller's own decision vector: dense and shared heads without a valid slot
    mine = torch.tensor([O.DEC_DENSE, O.DEC_VS, O.DEC_DENSE, O.DEC_SHARE, O.DEC_VS, O.DEC_DENSE], dtype=torch.int32,
                        device=gpu_device)
    tri = torch.tril(torch.ones(nb, nb, device=gpu_device))
    avg = (tri / tri.sum(-1, keepdim=True)).expand(hq, nb, nb).contiguous()
    ops.pivot_update(state, hc, mine, avg, 0.9)
    mask = ops.mask_to_bool(ops.build_mask(state, hc, mine, vert, slash, nvf, nsf), nb)
    torch.cuda.synchronize()
    for k, v in bufs.items():
        assert torch.equal(v, before[k]), f"slab {k} changed although no head had a valid slot"
    assert mask[0].cpu().equal(tri.bool().cpu())          # dense is dense, with or without a slot
    assert mask[3, :, 0].all() and not torch.triu(mask[3], 1).any()  # SHARE without a slot: its own vertical-slash set
    # the same call with the valid pivots does update their slots and nothing else
    ops.pivot_update(state, hc, dec, avg, 0.9)
    torch.cuda.synchronize()
    assert state.info[:, 1].cpu().tolist() == [1, 1]
    for k, v in bufs.items():
        assert torch.equal(v[0], before[k][0]) and torch.equal(v[-1], before[k][-1]), f"canary of {k} overwritten"


def _straddling_threshold(probs: np.ndarray, nb: int):
    """A double threshold pt for which the score fp32(pt * nb) that the reference forms (attention_sharing.py:361,
    utils.py:56) and the score fp32(fp32(pt) * nb) that a float argument would give lie on the two sides of one of
    the running sums of `probs`, so the two scores select different sets.  Returns (pt, kept right, kept wrong)."""
    order = O.order_desc(probs)
    sums = np.cumsum(O.to_fixed(probs[order]), dtype=np.uint64)
    nonzero = int((probs > 0).sum())  # entries above the diagonal are exact zeros: they sort last and add nothing
    for m in range(nonzero // 3, nonzero - 1):
        s = int(sums[m]) / float(2 ** 48)
        lo = np.float32(s)
        if float(lo) > s:
            lo = np.nextafter(lo, np.float32(0))
        hi = np.nextafter(lo, np.float32(np.inf))
        for u in np.linspace(0.30, 0.70, 161):
            pt = (float(lo) + u * (float(hi) - float(lo))) / nb
            right, wrong = np.float32(pt * nb), np.float32(float(np.float32(pt)) * nb)
            if right != wrong and {float(right), float(wrong)} == {float(lo), float(hi)}:
                kr, kw = O.prefix_len(probs, O.thr_le(float(right))), O.prefix_len(probs, O.thr_le(float(wrong)))
                if kr != kw and 0.3 < pt < 1.0:
                    return pt, kr, kw
    raise AssertionError("no straddling threshold found")


@pytest.mark.parametrize("nb", [13, 21, 100])
def test_queryaware_select_compares_with_the_double_product_score(gpu_device, nb):
    """The query-aware selection's score is fp32(double(pattern_threshold) * nb).  The thresholds here are chosen, per
    head, so that one running sum of the head's own block probabilities lies between that score and the one a
    threshold rounded to fp32 first would give (one fp32 ulp apart): the selection must keep exactly the entries the
    oracle keeps with the reference's score, and the negative control shows that the other score keeps a different
    number of entries."""
    from shareprefill_amd import _lib, ops

    hq, hkv, d = 4, 2, 128
    g = torch.Generator().manual_seed(1000 + nb)
    qbar = (torch.randn(nb, hq, d, generator=g) * 1.5).to(torch.bfloat16).to(gpu_device)
    kbar = (torch.randn(nb, hkv, d, generator=g) * 1.5).to(torch.bfloat16).to(gpu_device)
    tri = np.tril(np.ones((nb, nb), dtype=bool))
    all_qa = torch.full((hq,), _lib.SP_DEC_QA, dtype=torch.int32, device=gpu_device)
    mask0 = torch.zeros(hq, nb, (nb + 63) // 64, dtype=torch.int64, device=gpu_device)
    probs = ops.queryaware_select(qbar, kbar, all_qa, mask0, 0.9).cpu().numpy()   # the probabilities do not depend on it
    for h in range(hq):
        ph = probs[h].reshape(-1)
        pt, kept_right, kept_wrong = _straddling_threshold(ph, nb)
        assert kept_right != kept_wrong
        only = torch.zeros(hq, dtype=torch.int32, device=gpu_device)
        only[h] = _lib.SP_DEC_QA
        mask = torch.zeros(hq, nb, (nb + 63) // 64, dtype=torch.int64, device=gpu_device)
        ops.queryaware_select(qbar, kbar, only, mask, pt)
        got = ops.mask_to_bool(mask, nb).cpu().numpy()
        want = np.zeros(nb * nb, dtype=bool)
        want[O.cover_keep_le(ph, pt * nb)] = True
        want = want.reshape(nb, nb) & tri
        want[0, 0] = True
        assert np.array_equal(got[h], want), f"head {h}, threshold {pt!r}"
        assert not got[[x for x in range(hq) if x != h]].any()
        other = np.zeros(nb * nb, dtype=bool)
        other[O.cover_keep_le(ph, float(np.float32(float(np.float32(pt)) * nb)))] = True
        other = other.reshape(nb, nb) & tri
        other[0, 0] = True
        assert not np.array_equal(other, want), "negative control: the fp32-rounded threshold must select another set"


def test_pivot_update_with_several_dense_heads_of_one_cluster_keeps_the_highest(gpu_device):
    """A caller's own flags may mark several heads of one cluster dense.  The reference stores their maps one after
    the other (attention_sharing.py:96-103), so the highest head's stays; here the rows of the lower heads leave
    at once instead of sharing the cluster's row counter and accumulators.  The state after the call is exactly that
    of a call with the highest head alone, and counter and accumulators are zero again."""
    from shareprefill_amd import ops

    hq, nb = 6, 48
    g = torch.Generator().manual_seed(23)
    tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    avg = torch.softmax((torch.randn(hq, nb, nb, generator=g) * 2).masked_fill(~tri, float("-inf")), -1)
    avg = avg.to(gpu_device).contiguous()
    hc = torch.tensor([0, 0, 1, 0, -1, 1], dtype=torch.int32, device=gpu_device)

    def run(decision):
        state = ops.ClusterState(2, nb, gpu_device, keep_maps=True)
        state.info[0, 0], state.info[1, 0] = 3, 5
        state.cols[:, :3] = 1
        state.dists[:, :2] = 1
        ops.pivot_update(state, hc, torch.tensor(decision, dtype=torch.int32, device=gpu_device), avg, 0.9)
        torch.cuda.synchronize()
        return state

    many = run([1, 1, 1, 1, 1, 1])
    last = run([0, 0, 0, 1, 0, 1])
    for name in ("info", "ratio", "pattern", "accum", "avg_map"):
        assert torch.equal(getattr(many, name), getattr(last, name)), name
    assert many.info[:, 1].cpu().tolist() == [1, 1] and many.info[:, 5].cpu().tolist() == [0, 0]
    assert int(many.accum.abs().sum()) == 0
    for slot, h in ((0, 3), (1, 5)):
        want = O.cover_keep_rows_ge(avg[h].cpu().numpy(), 0.9) & tri.numpy()
        want[0, 0] = True
        assert np.array_equal(ops.mask_to_bool(many.pattern[slot], nb).cpu().numpy(), want)
        assert torch.equal(many.avg_map[slot], avg[h])

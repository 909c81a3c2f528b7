"""GPU checks at the full benchmark size (C3: B1 Hq32 Hkv8 D128 N131072, nb 1024), where the CPU oracle cannot
run the whole layer: size-independent properties of every stage, plus exact-tolerance spot checks of single
query blocks against a plain fp32 torch computation of the same rows.

Properties used: softmax mass conservation of the last-query scores (vertical and slash vectors each sum to 1),
block sums equal to sums of tokens, budget bounds and monotonicity, masks lower-triangular with sink column and
diagonal kept, row pointers equal to popcounts, the id-list view round-tripping to the mask, rows of a pivot's
block-average map summing to 1, linearity of attention in V, run-to-run bit reproducibility, and the closed form of
every output row for zero queries (the mean of the kept values).
"""

import math
import types

import pytest
import torch

from shareprefill_amd import synthetic

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 2.5e-3  # see tests/test_gpu_attention.py for the mean-rel floor of a bf16 result


def _two_layers(gpu_device, tmp_path_factory, name):
    from shareprefill_amd import AttentionSharing, shareprefill_attention_forward

    w = synthetic.WORKLOADS[name]
    q, k, v = synthetic.workload_inputs(w, device=gpu_device)
    table = synthetic.random_cluster_table(w.hq, w.n_clusters, 2, w.seed)
    path = synthetic.write_cluster_table(table, str(tmp_path_factory.mktemp(name.lower()) / "table.json"))
    sharing = AttentionSharing(path)
    sharing.keep_plans = True  # both layers' masks are inspected below
    cfg = types.SimpleNamespace(block_size=128, min_budget=w.min_budget, max_budget=None,
                                pattern_threshold=w.pattern_threshold, similarity_threshold=w.similarity_threshold,
                                fallback_threshold=w.fallback_threshold, queryaware_threshold=w.queryaware_threshold)
    outs, plans, avgs = [], [], []
    for layer in (0, 1):
        mod = types.SimpleNamespace(config=cfg, attention_sharing=sharing, layer_idx=layer, scaling=128 ** -0.5)
        out, avg = shareprefill_attention_forward(mod, q, k, v, None, scaling=128 ** -0.5)
        outs.append(out)
        avgs.append(avg)
        plans.append(sharing.plans[-1])
    torch.cuda.synchronize()
    return types.SimpleNamespace(w=w, q=q, k=k, v=v, outs=outs, plans=plans, avgs=avgs, nb=w.seq_len // 128)


@pytest.fixture(scope="module")
def c3(gpu_device, tmp_path_factory):
    return _two_layers(gpu_device, tmp_path_factory, "C3")


@pytest.fixture(scope="module")
def c5(gpu_device, tmp_path_factory):
    """Qwen2.5-7B head shapes at 262144 tokens: 28 query heads on 4 kv heads (groups of 7: an odd head per group is
    paired by rows, and head pairs never cross kv heads), nb 2048."""
    return _two_layers(gpu_device, tmp_path_factory, "C5")


@pytest.fixture
def full_size_case(request):
    return request.getfixturevalue(request.param)


def test_scores_conserve_mass_and_block_sums(c3):
    from shareprefill_amd import ops

    vt, st, vb, sb = ops.lastq_scores(c3.q[0], c3.k[0], 128)
    ones = torch.ones(c3.w.hq, dtype=torch.float64, device=vt.device)
    assert torch.allclose(vt.double().sum(1), ones, atol=2e-4)
    assert torch.allclose(st.double().sum(1), ones, atol=2e-4)
    assert torch.allclose(vt.view(c3.w.hq, c3.nb, 128).sum(2), vb, rtol=1e-4, atol=1e-7)
    assert torch.allclose(st.view(c3.w.hq, c3.nb, 128).sum(2), sb, rtol=1e-4, atol=1e-7)
    assert (vt >= 0).all() and (st >= 0).all()
    # same call again: bit-identical (every sum runs in a fixed order)
    vt2, st2, vb2, sb2 = ops.lastq_scores(c3.q[0], c3.k[0], 128)
    assert torch.equal(vt, vt2) and torch.equal(st, st2) and torch.equal(vb, vb2) and torch.equal(sb, sb2)
    # budgets: within [min_budget blocks, nb], monotone in the threshold
    prev = None
    for thr in (0.5, 0.9, 0.95, 0.99):
        nv, ns = ops.cover_budgets(vt, st, 128, thr, 8, c3.nb)
        assert int(nv.min()) >= 8 and int(nv.max()) <= c3.nb and int(ns.min()) >= 8 and int(ns.max()) <= c3.nb
        if prev is not None:
            assert (nv >= prev[0]).all() and (ns >= prev[1]).all()
        prev = (nv, ns)


def test_scores_match_the_oracle_at_full_size_on_sampled_heads(c3):
    """The oracle's last-query scores finish for single heads at 131072 tokens (a 128 x N product each): four heads
    element by element, with fp32 logits (only exp / sum rounding left) and with the reference's bf16 logits."""
    from oracle import shareprefill_oracle as O
    from shareprefill_amd import ops

    w = c3.w
    g = w.hq // w.hkv
    for flags, bf16_logits, rtol, atol in ((0, False, 5e-4, 1e-9), (1, True, 3e-2, 1e-7)):
        vt, st, _, _ = ops.lastq_scores(c3.q[0], c3.k[0], 128, flags)
        for h in (0, 5, 17, w.hq - 1):
            qh = c3.q[0][h:h + 1].cpu()
            kh = c3.k[0][h // g:h // g + 1].cpu()
            vref, sref = O.lastq_scores(qh, kh, 128, logits_in_input_dtype=bf16_logits)
            assert torch.allclose(vt[h].cpu(), vref[0], rtol=rtol, atol=atol), f"vertical, head {h}, bf16 {bf16_logits}"
            assert torch.allclose(st[h].cpu(), sref[0], rtol=rtol, atol=atol), f"slash, head {h}, bf16 {bf16_logits}"


@pytest.mark.parametrize("full_size_case", ["c3", "c5"], indirect=True)
def test_decode_and_pooling_at_full_size(full_size_case):
    """The two HBM-bound steps at the benchmark lengths against plain fp32 evaluations on the device: the decode step
    of the last token over the whole cache (131072 / 262144 keys) with the real queries, with zero queries (the mean
    of V) and with one-hot values (a distribution), and the block means of K."""
    from shareprefill_amd import ops

    c = full_size_case
    w, nb = c.w, c.nb
    g = w.hq // w.hkv
    k, v = c.k[0], c.v[0]                                   # [Hkv, N, D]
    scale = 128 ** -0.5
    for q1 in (c.q[0][:, -1], torch.zeros(w.hq, 128, dtype=torch.bfloat16, device=k.device)):
        out = ops.decode_attention(q1.contiguous(), k, v, scale).float()
        logits = torch.einsum("hgd,hnd->hgn", q1.float().view(w.hkv, g, 128), k.float()) * scale
        ref = torch.einsum("hgn,hnd->hgd", torch.softmax(logits, -1), v.float()).reshape(w.hq, 128)
        assert (out - ref).abs().max().item() <= MAX_ABS
        assert ((out - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL
    eye = torch.eye(128, dtype=torch.bfloat16, device=k.device)
    v1 = eye.repeat(w.seq_len // 128, 1)[None].expand(w.hkv, -1, -1)
    rows = ops.decode_attention(c.q[0][:, -1].contiguous(), k, v1, scale).float()
    assert bool((rows >= 0).all()) and (rows.sum(-1) - 1.0).abs().max().item() <= 2.0 ** -8 + 1e-4
    kbar = ops.pool_avg(k, 128).float()                     # [nb, Hkv, D]
    want = k.float().view(w.hkv, nb, 128, 128).mean(2).transpose(0, 1)
    assert (kbar - want).abs().max().item() <= 2.0 ** -8 * max(1.0, want.abs().max().item())
    assert ((kbar - want).abs() <= 2.0 ** -8 * want.abs() + 1e-6).all()


def test_masks_are_causal_keep_sink_and_diagonal_and_match_their_views(c3):
    from shareprefill_amd import ops

    nb = c3.nb
    for plan in c3.plans:
        mb = ops.mask_to_bool(plan.mask, nb)
        assert not torch.triu(mb, diagonal=1).any()
        idx = torch.arange(nb, device=mb.device)
        vs_or_dense = (plan.decision == 0) | (plan.decision == 1) | (plan.decision == 2)
        assert mb[vs_or_dense][:, :, 0].all()
        assert mb[vs_or_dense][:, idx, idx].all()
        assert mb[:, 0, 0].all()
        ptr = ops.mask_row_pointers(plan.mask)
        assert torch.equal(ptr[:, 1:] - ptr[:, :-1], mb.sum(2).to(ptr.dtype))
        assert torch.equal(ops.bool_to_mask(mb), plan.mask)
        ids = plan.block_idx()[0]
        for h in (0, c3.w.hq - 1):
            flat = torch.zeros(nb * nb, dtype=torch.bool, device=mb.device)
            flat[ids[h].long()] = True
            assert torch.equal(flat.view(nb, nb), mb[h])
    dense = c3.plans[0].decision == 1
    assert int(dense.sum()) == c3.w.n_clusters  # one pivot per shared cluster in layer 0
    tri = torch.tril(torch.ones(nb, nb, dtype=torch.bool, device=dense.device))
    assert (ops.mask_to_bool(c3.plans[0].mask, nb)[dense] == tri).all()


def test_pivot_average_maps_are_row_stochastic(c3):
    avg = c3.avgs[0][0]
    dense = c3.plans[0].decision == 1
    rows = avg[dense].double().sum(-1)
    assert torch.allclose(rows, torch.ones_like(rows), atol=5e-3)
    assert (avg[~dense] == 0).all()
    assert not torch.triu(avg[dense], diagonal=1).any()


def _rows_reference(q, k, v, mask_row, h, r, hkv_group, scale):
    """fp32 masked attention of query block r of head h against all keys (plain torch on the GPU)."""
    n = q.shape[2]
    qs = q[0, h, r * 128:(r + 1) * 128].float()
    kf, vf = k[0, h // hkv_group].float(), v[0, h // hkv_group].float()
    s = (qs @ kf.t()) * scale
    keep = mask_row.repeat_interleave(128)[:n]
    qpos = torch.arange(r * 128, (r + 1) * 128, device=q.device)[:, None]
    kpos = torch.arange(n, device=q.device)[None, :]
    s = s.masked_fill(~(keep[None, :] & (kpos <= qpos)), float("-inf"))
    return torch.softmax(s, dim=-1) @ vf


def test_attention_rows_match_fp32_reference_at_full_size(c3):
    from shareprefill_amd import ops

    w, nb = c3.w, c3.nb
    scale = 1.0 / math.sqrt(128)
    for layer in (0, 1):
        mb = ops.mask_to_bool(c3.plans[layer].mask, nb)
        out = c3.outs[layer][0]  # [N, Hq, D]
        for h, r in ((0, nb - 1), (5, nb - 2), (w.hq - 1, 511), (17, 640), (9, 0), (30, 1)):
            ref = _rows_reference(c3.q, c3.k, c3.v, mb[h, r], h, r, w.hq // w.hkv, scale)
            got = out[r * 128:(r + 1) * 128, h].float()
            assert (got - ref).abs().max().item() <= MAX_ABS
            assert ((got - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL


def test_attention_is_linear_in_v_and_reproducible(c3):
    from shareprefill_amd import ops

    w = c3.w
    mask = c3.plans[1].mask
    scale = 1.0 / math.sqrt(128)
    g = torch.Generator(device=c3.v.device).manual_seed(7)
    v2 = torch.randn(c3.v.shape, device=c3.v.device, dtype=torch.float32, generator=g).to(torch.bfloat16)
    v2 = v2.transpose(1, 2).contiguous().transpose(1, 2)  # token-major storage like the workload's tensors
    o1 = ops.block_sparse_attention(c3.q[0], c3.k[0], c3.v[0], mask, 128, scale)
    o1b = ops.block_sparse_attention(c3.q[0], c3.k[0], c3.v[0], mask, 128, scale)
    assert torch.equal(o1, o1b)
    o2 = ops.block_sparse_attention(c3.q[0], c3.k[0], v2[0], mask, 128, scale)
    vsum = (c3.v.float() + v2.float()).to(torch.bfloat16)
    o12 = ops.block_sparse_attention(c3.q[0], c3.k[0], vsum[0], mask, 128, scale)
    lhs, rhs = o12.float(), o1.float() + o2.float()
    # bf16 roundings of the outputs (2^-9 of their magnitude) plus those of v1+v2 and of the probabilities inside
    # the three products (2^-9 of sum p|v|, |v| up to ~5 -- not of the possibly cancelling result)
    scale_of = o1.float().abs() + o2.float().abs() + lhs.abs()
    assert ((lhs - rhs).abs() <= 2.0 ** -7 * scale_of + 5e-2).all()
    assert ((lhs - rhs).abs().mean() / rhs.abs().mean()).item() <= 1e-2
    assert torch.equal(o1, c3.outs[1][0])  # the layer call produced exactly this


@pytest.mark.parametrize("full_size_case", ["c3", "c5"], indirect=True)
def test_zero_queries_give_the_mean_of_the_kept_values_in_every_row(full_size_case):
    """With q = 0 every logit is 0, every probability 1 (exact in bf16), so each output row is the plain mean of V over
    the keys its mask keeps and causality allows -- a closed form for ALL rows of the full-size masks (131072 x 32 at
    C3, 262144 x 28 at C5), from
    block sums of V: out[i] = (sum of V over kept blocks left of the diagonal + sum of V[128 r .. i]) / their count.
    What it pins at full size: which blocks every row visits (a skipped or doubled block changes the mean by 1 / count),
    the causal edge inside the diagonal block, the row sums, the head -> kv head mapping and the output layout."""
    from shareprefill_amd import ops

    c3 = full_size_case  # (either full-size fixture)
    w, nb = c3.w, c3.nb
    g = w.hq // w.hkv
    vf = c3.v[0].float()                                   # [Hkv, N, D]
    blk = vf.view(w.hkv, nb, 128, 128).sum(2)              # [Hkv, nb, D] block sums
    within = vf.view(w.hkv, nb, 128, 128).cumsum(2)        # [Hkv, nb, 128, D] running sums inside each block
    pos = torch.arange(1, 129, device=vf.device, dtype=torch.float32)
    for layer in (0, 1):
        mask = c3.plans[layer].mask
        q0 = torch.zeros_like(c3.q[0])
        out = ops.block_sparse_attention(q0, c3.k[0], c3.v[0], mask, 128, 128 ** -0.5).float()  # [N, Hq, D]
        mb = ops.mask_to_bool(mask, nb)
        assert bool(mb.diagonal(dim1=1, dim2=2).all())  # the closed form below counts the diagonal block of every row
        left = torch.tril(mb, -1).float()                  # [Hq, nb, nb] kept blocks left of the diagonal
        worst = 0.0
        for h in range(w.hq):
            kv = h // g
            num = (left[h] @ blk[kv])[:, None, :] + within[kv]          # [nb, 128, D]
            cnt = left[h].sum(1)[:, None] * 128.0 + pos[None, :]        # [nb, 128]
            want = (num / cnt[:, :, None]).reshape(w.seq_len, 128)
            got = out[:, h]
            # the output's own bf16 rounding (unit roundoff 2^-8) and fp32 summation order over up to 262144 values
            err = (got - want).abs()
            assert (err <= 2.0 ** -8 * want.abs() + 2e-4).all(), f"layer {layer} head {h}: {err.max().item():.3e}"
            worst = max(worst, (err.mean() / want.abs().mean()).item())
            if h == 3:  # negative control: the closed form with one kept block of row 700 dropped must NOT pass
                r = 700
                c = int(torch.nonzero(left[h, r])[0])
                num_bad = num[r] - blk[kv][c][None, :]
                bad = num_bad / (cnt[r] - 128.0)[:, None]
                assert not ((got[r * 128:(r + 1) * 128] - bad).abs() <= 2.0 ** -8 * bad.abs() + 2e-4).all()
        assert worst <= 2.5e-3


@pytest.mark.parametrize("full_size_case", ["c3", "c5"], indirect=True)
def test_one_hot_values_make_every_output_row_a_distribution(full_size_case):
    """V[j] = unit vector of channel j mod 128 (exact in bf16): an output row is then the row's probability mass by
    in-block key offset, so with the real queries and keys every one of the rows (all heads, all tokens) must be non-negative and
    sum to 1 -- the normalisation (running maximum, rescales, row sums, the causal edge) checked on every row."""
    from shareprefill_amd import ops

    c3 = full_size_case  # (either full-size fixture)
    w = c3.w
    eye = torch.eye(128, dtype=torch.bfloat16, device=c3.q.device)
    v1 = eye.repeat(w.seq_len // 128, 1)[None].expand(w.hkv, -1, -1)           # [Hkv, N, D] view, nothing copied per head
    for layer in (0, 1):
        out = ops.block_sparse_attention(c3.q[0], c3.k[0], v1, c3.plans[layer].mask, 128, 128 ** -0.5).float()
        assert bool((out >= 0).all())
        rows = out.sum(-1)                                                      # [N, Hq]
        # 128 bf16 roundings (unit roundoff 2^-8) of the non-negative parts of a sum that is 1: at most 2^-8 of it when
        # every rounding goes the same way (rows with a handful of keys come close), far less on average
        dev = (rows - 1.0).abs()
        assert dev.max().item() <= 2.0 ** -8 + 1e-4, f"layer {layer}: {dev.max().item():.3e}"
        assert dev.mean().item() <= 5e-4 and abs(rows.mean().item() - 1.0) <= 2e-5


@pytest.mark.parametrize("max_pivots", [8, 0])
def test_zero_queries_give_closed_form_block_average_maps(c3, max_pivots):
    """Same inputs (q = 0, every probability 1): a dense pivot's block-average map is known in closed form for all
    1024 x 1024 entries -- query i of block r spreads its mass evenly over its 128 r + i + 1 keys, so
    avg[r, c < r] = mean_i 128 / (128 r + i + 1) and avg[r, r] = mean_i (i + 1) / (128 r + i + 1).
    max_pivots = 8: the maps come from the block sums kept during the forward pass; 0: from the recomputing pass."""
    from shareprefill_amd import ops

    w, nb = c3.w, c3.nb
    plan = c3.plans[0]
    dense = torch.nonzero(plan.decision == 1).reshape(-1).tolist()
    assert len(dense) == w.n_clusters
    avg = torch.zeros(w.hq, nb, nb, dtype=torch.float32, device=c3.q.device)
    ops.block_sparse_attention(torch.zeros_like(c3.q[0]), c3.k[0], c3.v[0], plan.mask, 128, 128 ** -0.5,
                               decision=plan.decision, avg_attn=avg, max_pivots=max_pivots)
    i = torch.arange(1, 129, device=avg.device, dtype=torch.float64)
    r = torch.arange(nb, device=avg.device, dtype=torch.float64)
    cnt = 128.0 * r[:, None] + i[None, :]                       # [nb, 128] keys seen by query i of block r
    off = (128.0 / cnt).mean(1)                                 # value of every block left of the diagonal in row r
    diag = (i[None, :] / cnt).mean(1)
    want = torch.tril(off[:, None].expand(nb, nb), -1) + torch.diag(diag)
    for h in range(w.hq):
        if h in dense:
            got = avg[h].double()
            assert (got - want).abs().max().item() <= 2e-6, f"head {h}"
            assert torch.allclose(got.sum(1), torch.ones(nb, dtype=torch.float64, device=avg.device), atol=1e-5)
        else:
            assert float(avg[h].abs().max()) == 0.0


def test_maximum_supported_length_selection_bit_exact_and_rows_within_tolerance(gpu_device, tmp_path):
    """524288 tokens = 4096 key blocks, the longest sequence the block lists and rank tables are sized for (two query
    heads on one kv head, one shared cluster, two layers): budgets, decisions, masks and the pivot's pattern
    identical to the oracle's integer logic on the GPU's own scores, and single query blocks of both layers -- the
    dense pivot of layer 0 included -- against the plain fp32 torch evaluation."""
    import importlib.util
    import os

    from shareprefill_amd import ops

    spec = importlib.util.spec_from_file_location(
        "layer_helpers_max", os.path.join(os.path.dirname(__file__), "test_gpu_layer.py"))
    helpers = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(helpers)
    n, hq, hkv = 4096 * 128, 2, 1
    run = helpers.run_layers(gpu_device, tmp_path, hq=hq, hkv=hkv, n=n, seed=91, n_clusters=1, with_free=False)
    helpers.check_forced(run)
    assert run["nb"] == 4096
    assert (run["layers"][0]["dec"] == 1).sum() == 1  # the cluster's pivot runs dense
    q, k, v = (run[x][None].to(gpu_device) for x in ("q", "k", "v"))
    scale = 1.0 / math.sqrt(128)
    for L in run["layers"]:
        mb = torch.from_numpy(L["mask"]).to(gpu_device)
        out = L["out"][0].to(gpu_device)  # [N, Hq, D]
        for h, r in ((0, 4095), (1, 4095), (0, 2048), (1, 4094), (0, 0), (1, 63)):
            ref = _rows_reference(q, k, v, mb[h, r], h, r, hq // hkv, scale)
            got = out[r * 128:(r + 1) * 128, h].float()
            assert (got - ref).abs().max().item() <= MAX_ABS
            assert ((got - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL
    # one more key block is refused, not mangled
    with pytest.raises(NotImplementedError):
        qq = torch.zeros(1, 4097 * 128, 128, dtype=torch.bfloat16, device=gpu_device)
        mm = torch.zeros(1, 4097, 65, dtype=torch.int64, device=gpu_device)
        ops.block_sparse_attention(qq, qq, qq, mm, 128, scale)


def _layer_helpers():
    import importlib.util
    import os

    spec = importlib.util.spec_from_file_location(
        "layer_helpers_full", os.path.join(os.path.dirname(__file__), "test_gpu_layer.py"))
    helpers = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(helpers)
    return helpers


@pytest.mark.parametrize("name", ["C3", "C5"])
def test_sharing_and_query_aware_heads_at_full_size_bit_exact(gpu_device, tmp_path, name):
    """The share test, the pattern OR of the mask construction and the query-aware selection over nb^2 = 1 M (C3,
    131072 tokens) and 4.2 M (C5, 262144 tokens, GQA 7:1) block probabilities, at the benchmark shapes.  With the
    library's default thresholds no head of these synthetic inputs shares or goes query-aware, so the thresholds are
    placed where they do: fallback_threshold is lifted (a local-attention pivot has vs_ratio >= (nb-1)/nb) and
    queryaware_threshold is put between the heads' own sqrt-JS values so that a quarter of the heads take the
    query-aware path.  Two layers (pivot election, then sharing): budgets, decisions, masks, pivot patterns and
    coverage ratios must equal the oracle's integer logic on the GPU's own scores, every decision kind must occur,
    and single query blocks of a shared and of a query-aware head are held to the attention tolerances."""
    import numpy as np

    from oracle import shareprefill_oracle as O

    helpers = _layer_helpers()
    w = synthetic.WORKLOADS[name]
    kw = dict(hq=w.hq, hkv=w.hkv, n=w.seq_len, seed=w.seed, n_clusters=w.n_clusters, with_free=False,
              pattern_threshold=w.pattern_threshold)
    print(f"full-size sharing / query-aware parity: {name} probe layer", flush=True)
    probe = helpers.run_layers(gpu_device, tmp_path, n_layers=1, with_forced=False, **kw)
    js = np.sort(probe["layers"][0]["plan"].js_qa.cpu().numpy())
    assert np.isfinite(js).all()
    n_qa = w.hq // 4
    assert js[n_qa] > js[n_qa - 1], "the two sqrt-JS values around the threshold coincide"
    qat = float((js[n_qa - 1].astype(np.float64) + js[n_qa].astype(np.float64)) / 2)
    del probe
    torch.cuda.empty_cache()
    print(f"full-size sharing / query-aware parity: {name} two layers, queryaware_threshold {qat:.6f}", flush=True)
    run = helpers.run_layers(gpu_device, tmp_path, fallback_threshold=1e9, queryaware_threshold=qat, **kw)
    helpers.check_forced(run)
    d0, d1 = run["layers"][0]["dec"], run["layers"][1]["dec"]
    assert (d0 == O.DEC_QA).sum() == n_qa and (d1 == O.DEC_QA).sum() == n_qa
    assert (d0 == O.DEC_DENSE).sum() >= 1 and (d0 == O.DEC_SHARE).sum() == 0
    assert (d1 == O.DEC_SHARE).sum() >= 1, "no head shared its cluster pivot's pattern in the second layer"
    assert (d1 == O.DEC_VS).sum() + (d1 == O.DEC_SHARE).sum() + n_qa == w.hq
    # a shared head's mask is the pivot's pattern OR its own minimum-budget vertical-slash set: strictly more than
    # the latter alone
    nb = run["nb"]
    h_share = int(np.nonzero(d1 == O.DEC_SHARE)[0][0])
    h_qa = int(np.nonzero(d1 == O.DEC_QA)[0][0])
    assert run["layers"][1]["mask"][h_share].sum() > 3 * nb
    q, k, v = (run[x][None].to(gpu_device) for x in ("q", "k", "v"))
    scale = 1.0 / math.sqrt(128)
    L = run["layers"][1]
    mb = torch.from_numpy(L["mask"]).to(gpu_device)
    out = L["out"][0].to(gpu_device)  # [N, Hq, D]
    for h in (h_share, h_qa):
        for r in (nb - 1, nb // 2 + 1, 3):
            ref = _rows_reference(q, k, v, mb[h, r], h, r, w.hq // w.hkv, scale)
            got = out[r * 128:(r + 1) * 128, h].float()
            assert (got - ref).abs().max().item() <= MAX_ABS
            assert ((got - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL
    # the float stages of the query-aware path at this size against the oracle's own evaluation (they are cheap for
    # the oracle: pooled rows, the last query block, one [nb, nb] product per head)
    plan = L["plan"]
    g = w.hq // w.hkv
    kref = O.pool_avg(run["k"].transpose(0, 1).contiguous(), 128)                  # [nb, Hkv, D]
    kb = plan.kbar.cpu().float()
    assert (kb - kref.float()).abs().max().item() <= 2 ** -8 * max(1.0, kref.float().abs().max().item())
    avg_ref = O.pooled_qk_probs(run["q"], kref, 128)
    assert torch.allclose(plan.avg_qk.cpu(), avg_ref, rtol=2e-2, atol=1e-7)
    js_ref = O.sqrt_js(avg_ref, plan.vert_blk.cpu())
    assert torch.allclose(plan.js_qa.cpu(), js_ref, rtol=2e-2, atol=1e-4)
    for h in [int(x) for x in np.nonzero(d1 == O.DEC_QA)[0][:2]]:
        want = O.block_probs(O.pool_q_head(run["q"][h], 128), kref[:, h // g])
        got = plan.qa_probs[h].cpu()
        assert torch.allclose(got.sum(-1), torch.ones(nb), atol=1e-5) and bool((torch.triu(got, 1) == 0).all())
        assert torch.allclose(got, want, rtol=6e-2, atol=1e-6), f"head {h}: block probabilities"
        assert ((got - want).abs().sum() / want.abs().sum()).item() <= 5e-3

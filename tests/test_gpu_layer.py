"""GPU parity of the whole SharePrefill layer (scores -> budgets -> query-aware test -> pivot / share
decision -> mask -> block-sparse attention -> pivot update) through the patched attention function.

Two comparisons per layer:
  * forced: the oracle's integer logic is fed the float intermediates the GPU produced; decisions, budgets,
    masks, pivot patterns and coverage ratios must then be IDENTICAL (bit-exact selection on identical scores);
  * free: the oracle computes everything itself; float stages agree to tolerance, and on these seeded inputs
    (no value sits on a decision boundary) the decisions and masks agree as well.
Attention outputs are checked against the fp32 masked-attention oracle on the GPU's mask.
"""

import types

import numpy as np
import pytest
import torch

from oracle import shareprefill_oracle as O
from shareprefill_amd import synthetic

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_REL = 2e-2, 2.5e-3  # see tests/test_gpu_attention.py for the mean-rel floor of a bf16 result


class FakeAttention:
    """The attributes the attention function reads from a Hugging Face attention module."""

    def __init__(self, cfg, sharing, layer_idx, head_dim, hq, hkv):
        self.config = cfg
        self.attention_sharing = sharing
        self.layer_idx = layer_idx
        self.scaling = head_dim ** -0.5
        self.num_heads = hq
        self.num_key_value_groups = hq // hkv
        self.training = False
        self.attention_dropout = 0.0


def run_layers(gpu, tmp_path, hq, hkv, n, seed, n_clusters, n_layers=2, with_free=True, with_forced=True, d=128,
               shared=None, table=None, layer_ids=None, reseed=False, **thr):
    """table: a cluster table to use instead of a random one; layer_ids: the layer indices to run, in order (default
    0 .. n_layers - 1); reseed: draw new q / k / v for every layer (seed + layer index) instead of one set."""
    from shareprefill_amd import AttentionSharing, shareprefill_attention_forward, ops

    # dense_short_prompts off: these tests compare the selection itself, also where the prompt is so short that every
    # mask comes out dense and the attention function would skip it
    kw = dict(block_size=128, min_budget=1024, max_budget=None, pattern_threshold=0.95, similarity_threshold=0.5,
              fallback_threshold=0.9, queryaware_threshold=0.1, dense_short_prompts=False)
    kw.update(thr)
    if table is None:
        table = synthetic.random_cluster_table(hq, n_clusters, n_layers, seed)
    if shared is not None:  # only these clusters share (the shipped Llama table shares one of its 44)
        table["shared_clusters"] = list(shared)
    path = synthetic.write_cluster_table(table, str(tmp_path / "table.json"))
    q, k, v = synthetic.planted_qkv(hq, hkv, n, d, seed, q_head_gain=1.0)
    sharing = AttentionSharing(path)
    sharing.keep_debug = True
    cfg = types.SimpleNamespace(**kw)
    oracle_forced = O.OracleSharing(O.ClusterTable(table["clusters"], table["shared_clusters"]))
    oracle_free = O.OracleSharing(O.ClusterTable(table["clusters"], table["shared_clusters"]))
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    bs = kw["block_size"]
    nb = -(-n // bs)
    results = []
    for layer in (range(n_layers) if layer_ids is None else layer_ids):
        if reseed:
            q, k, v = synthetic.planted_qkv(hq, hkv, n, d, seed + layer, q_head_gain=1.0)
            qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
        mod = FakeAttention(cfg, sharing, layer, d, hq, hkv)
        out, avg = shareprefill_attention_forward(mod, qg, kg, vg, None, scaling=mod.scaling)
        plan = sharing.plans[-1]
        assert out.shape == (1, n, hq, d) and out.is_contiguous() and out.dtype == torch.bfloat16
        assert avg.shape == (1, hq, nb, nb) and avg.dtype == torch.float32
        gpu_mask = ops.mask_to_bool(plan.mask, nb).cpu().numpy()
        dec = plan.decision.cpu().numpy()
        inject = dict(vert_tok=plan.vert_tok.cpu(), slash_tok=plan.slash_tok.cpu(), vert_blk=plan.vert_blk.cpu(),
                      slash_blk=plan.slash_blk.cpu(), avg_qk=plan.avg_qk.cpu(), js_qa=plan.js_qa.cpu(),
                      js_v=plan.js_v.cpu().numpy(), js_s=plan.js_s.cpu().numpy(),
                      qa_probs={h: plan.qa_probs[h].cpu() for h in range(hq)})
        okw = dict(bs=bs, min_budget=kw["min_budget"], max_budget=kw["max_budget"],
                   pattern_threshold=kw["pattern_threshold"], similarity_threshold=kw["similarity_threshold"],
                   fallback_threshold=kw["fallback_threshold"], queryaware_threshold=kw["queryaware_threshold"])
        forced = None
        if with_forced:
            forced = oracle_forced.layer(q[0], k[0], v[0], layer, compute_attention=False, inject=inject, **okw)
            oracle_forced.update_pivots(layer, forced.decision, avg[0].cpu().numpy(), kw["pattern_threshold"])
        free = None
        if with_free:
            free = oracle_free.layer(q[0], k[0], v[0], layer, compute_attention=False, **okw)
            oracle_free.update_pivots(layer, free.decision, avg[0].cpu().numpy(), kw["pattern_threshold"])
        results.append(dict(layer=layer, out=out.cpu(), avg=avg.cpu(), plan=plan, mask=gpu_mask, dec=dec,
                            forced=forced, free=free, q=q[0], k=k[0], v=v[0]))
    return dict(q=q[0], k=k[0], v=v[0], table=table, sharing=sharing, oracle_forced=oracle_forced,
                oracle_free=oracle_free, layers=results, nb=nb, kw=kw, d=d)


def check_forced(run):
    sharing = run["sharing"]
    for L in run["layers"]:
        plan, forced = L["plan"], L["forced"]
        assert plan.nv.cpu().tolist() == forced.nv.tolist(), "vertical budgets"
        assert plan.ns.cpu().tolist() == forced.ns.tolist(), "slash budgets"
        assert L["dec"].tolist() == forced.decision.tolist(), "decisions"
        assert plan.nv_final.cpu().tolist() == forced.nv_final.tolist()
        assert plan.ns_final.cpu().tolist() == forced.ns_final.tolist()
        for h in range(L["mask"].shape[0]):
            assert np.array_equal(L["mask"][h], forced.mask[h]), f"layer {L['layer']} head {h}: mask differs"
    # pivot state after the last layer: pattern bits and coverage ratio
    summary = sharing.pivot_summary()
    state = sharing._state
    for cid, st in run["oracle_forced"].state.items():
        if cid not in sharing._slot:
            continue
        got = summary[cid]
        assert got["pivot_head"] == (-1 if st.pivot_head is None else st.pivot_head)
        if st.pattern is not None:
            from shareprefill_amd import ops

            pat = ops.mask_to_bool(state.pattern[sharing._slot[cid]], run["nb"]).cpu().numpy()
            assert np.array_equal(pat, st.pattern), f"cluster {cid}: pattern differs"
            assert got["vs_ratio"] == O.vs_ratio(st.avg, st.cols, st.dists), f"cluster {cid}: vs_ratio"
            # the reference's getters (attention_sharing.py:80-92), asked through any member (layer, head) of the cluster
            layer_m, head_m = run["table"]["clusters"][cid][-1]
            kept = sharing.get_pivotal_attn(layer_m, 0, head_m)
            assert kept is not None and np.array_equal(kept.cpu().numpy(), st.avg), f"cluster {cid}: pivot map"
            kept_pat = sharing.get_pivotal_pattern(layer_m, 0, head_m)
            assert np.array_equal(ops.mask_to_bool(kept_pat, run["nb"]).cpu().numpy(), st.pattern)
        else:
            layer_m, head_m = run["table"]["clusters"][cid][-1]
            assert sharing.get_pivotal_attn(layer_m, 0, head_m) is None
            assert sharing.get_pivotal_pattern(layer_m, 0, head_m) is None


def check_free(run, expect_same_masks=True):
    for L in run["layers"]:
        plan, free = L["plan"], L["free"]
        assert torch.allclose(plan.vert_tok.cpu(), free.vert_tok, rtol=3e-2, atol=1e-6)
        assert torch.allclose(plan.slash_tok.cpu(), free.slash_tok, rtol=3e-2, atol=1e-6)
        assert torch.allclose(plan.vert_blk.cpu(), free.vert_blk, rtol=1e-2, atol=1e-6)
        assert torch.allclose(plan.slash_blk.cpu(), free.slash_blk, rtol=1e-2, atol=1e-6)
        assert torch.allclose(plan.avg_qk.cpu(), free.avg_qk, rtol=2e-2, atol=1e-7)
        assert torch.allclose(plan.js_qa.cpu(), free.js_qa, rtol=2e-2, atol=1e-4)
        kb, kr = plan.kbar.cpu().float(), free.kbar.float()
        assert (kb - kr).abs().max().item() <= 2 ** -8 * max(1.0, kr.abs().max().item())
        # block probabilities of the query-aware heads (sp_block_probs_kernel) against the oracle's own evaluation:
        # a logit may land on the neighbouring bf16 value (pooled q / k differ by an ulp, fp32 sums in another
        # order), which moves a probability by up to 2^-7 of itself per unit of logit magnitude
        for h, want in free.qa_probs.items():
            if L["dec"][h] != O.DEC_QA:
                continue
            got = plan.qa_probs[h].cpu()
            assert torch.allclose(got.sum(-1), torch.ones(got.shape[0]), atol=1e-5)
            assert (torch.triu(got, 1) == 0).all()
            assert torch.allclose(got, want, rtol=6e-2, atol=1e-6), f"layer {L['layer']} head {h}: block probabilities"
            assert ((got - want).abs().sum() / want.abs().sum()).item() <= 5e-3
        if expect_same_masks:
            assert L["dec"].tolist() == free.decision.tolist()
            differing = sum(int((L["mask"][h] != free.mask[h]).sum()) for h in range(L["mask"].shape[0]))
            assert differing <= 0.002 * L["mask"].sum(), f"{differing} mask bits differ from the free-running oracle"


def check_outputs(run):
    for L in run["layers"]:
        q, k, v = L["q"], L["k"], L["v"]
        want = L["dec"] == O.DEC_DENSE
        ref, avg_ref = O.masked_attention(q, k, v, L["mask"], run["kw"]["block_size"], run["d"] ** -0.5, want_avg=want)
        out = L["out"][0].transpose(0, 1).float()
        assert (out - ref).abs().max().item() <= MAX_ABS
        assert ((out - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL
        for h in np.nonzero(want)[0]:
            assert torch.allclose(L["avg"][0, h], avg_ref[h], rtol=3e-2, atol=2e-5)
            assert torch.allclose(L["avg"][0, h].sum(-1), torch.ones(run["nb"]), atol=2e-3)
        for h in np.nonzero(~want)[0]:
            assert float(L["avg"][0, h].abs().sum()) == 0.0


def test_layer_default_thresholds_small(gpu_device, tmp_path):
    run = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=2048, seed=21, n_clusters=2)
    check_forced(run)
    check_free(run)
    check_outputs(run)
    d0 = run["layers"][0]["dec"]
    assert (d0 == O.DEC_DENSE).sum() == 2  # one pivot per shared cluster in the first layer


@pytest.mark.parametrize("bs,n,hq,hkv", [(64, 2048, 8, 2), (64, 1100, 6, 2), (32, 1536, 8, 2), (32, 999, 4, 4),
                                         (16, 1024, 8, 2), (16, 777, 7, 1), (16, 100, 4, 2), (32, 127, 4, 2)])
def test_layer_smaller_block_sizes(gpu_device, tmp_path, bs, n, hq, hkv):
    """block_size 64 / 32 / 16 (shareprefill_attn.py:509-516): the selection runs on N / bs blocks, the attention
    kernel walks the 128-token blocks that hold a kept block and drops the rest of them per 16 x 16 sub-tile.  Three
    layers (pivot election, sharing tests, pivot update), budgets / decisions / masks / pivot state forced against
    the oracle, float stages and outputs to the bars of the 128 case, with thresholds under which heads share and go
    query-aware."""
    n_clusters = 2 if hq % 2 == 0 else 1
    seen = []
    for qa_thr in (0.0, 1e9):  # nobody query-aware: pivots and their sharers; then every head query-aware
        run = run_layers(gpu_device, tmp_path, hq=hq, hkv=hkv, n=n, seed=500 + bs + n, n_clusters=n_clusters,
                         n_layers=3, block_size=bs, min_budget=4 * bs, fallback_threshold=1e9,
                         similarity_threshold=0.9, queryaware_threshold=qa_thr)
        assert run["nb"] == -(-n // bs)
        check_forced(run)
        check_free(run, expect_same_masks=False)
        check_outputs(run)
        seen.append(np.concatenate([L["dec"] for L in run["layers"]]))
    assert (seen[0] == O.DEC_DENSE).any() and (seen[0] == O.DEC_SHARE).any() and (seen[1] == O.DEC_QA).any()
    # default thresholds as well
    run = run_layers(gpu_device, tmp_path, hq=hq, hkv=hkv, n=n, seed=600 + bs + n, n_clusters=n_clusters,
                     block_size=bs, min_budget=8 * bs)
    check_forced(run)
    check_outputs(run)


@pytest.mark.parametrize("d,n", [(64, 2048), (32, 1100), (16, 1536)])
def test_layer_small_head_dims(gpu_device, tmp_path, d, n):
    """The reference's other head sizes (shareprefill_attn.py:503-508) run zero-padded to 128 on the same kernels: the
    oracle works on the unpadded tensors with 1/sqrt(d), so every comparison below also checks that the padding
    changes nothing (kbar is compared on the model's d channels, the padded ones must be zero)."""
    run = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=n, seed=100 + d, n_clusters=2, d=d, min_budget=512)
    for L in run["layers"]:
        kbar = L["plan"].kbar
        assert kbar.shape[-1] == 128 and float(kbar[..., d:].abs().max()) == 0.0
        L["plan"].kbar = kbar[..., :d]
    check_forced(run)
    check_free(run)
    check_outputs(run)


def test_layer_c1_shape(gpu_device, tmp_path):
    """B1 Hq8 Hkv2 D128 N8192, 2 clusters of 4: the CPU-runnable parity configuration (inputs in bf16)."""
    w = synthetic.WORKLOADS["C1"]
    run = run_layers(gpu_device, tmp_path, hq=w.hq, hkv=w.hkv, n=w.seq_len, seed=w.seed, n_clusters=w.n_clusters,
                     pattern_threshold=w.pattern_threshold)
    check_forced(run)
    check_free(run)
    check_outputs(run)


def test_layer_c2_shape_masks_bit_exact(gpu_device, tmp_path):
    """B1 Hq32 Hkv8 D128 N32768 (Llama-3.1-8B head shapes, nb 256), 8 clusters of 4, two layers: budgets, decisions,
    masks, pivot patterns and coverage ratios identical to the oracle's integer logic on the GPU's own scores.
    (The fp32 attention oracle does not finish at this size; outputs at large sizes: tests/test_gpu_fullsize.py.)"""
    w = synthetic.WORKLOADS["C2"]
    run = run_layers(gpu_device, tmp_path, hq=w.hq, hkv=w.hkv, n=w.seq_len, seed=w.seed, n_clusters=w.n_clusters,
                     with_free=False, pattern_threshold=w.pattern_threshold)
    check_forced(run)
    assert (run["layers"][0]["dec"] == O.DEC_DENSE).sum() == w.n_clusters


def test_layer_c3_shape_masks_bit_exact(gpu_device, tmp_path):
    """The benchmark's own size, B1 Hq32 Hkv8 D128 N131072 (nb 1024): same bit-exact comparison of the selection."""
    w = synthetic.WORKLOADS["C3"]
    run = run_layers(gpu_device, tmp_path, hq=w.hq, hkv=w.hkv, n=w.seq_len, seed=w.seed, n_clusters=w.n_clusters,
                     with_free=False, pattern_threshold=w.pattern_threshold)
    check_forced(run)
    assert (run["layers"][0]["dec"] == O.DEC_DENSE).sum() == w.n_clusters


def test_layer_c5_shape_masks_bit_exact(gpu_device, tmp_path):
    """Qwen2.5-7B head shapes at 262144 tokens (Hq28 Hkv4, GQA 7:1, nb 2048, 4 clusters of 7): the selection scan
    and the mask sharing at 2048 query blocks, bit-exact against the oracle's integer logic."""
    w = synthetic.WORKLOADS["C5"]
    run = run_layers(gpu_device, tmp_path, hq=w.hq, hkv=w.hkv, n=w.seq_len, seed=w.seed, n_clusters=w.n_clusters,
                     with_free=False, pattern_threshold=w.pattern_threshold)
    check_forced(run)
    assert (run["layers"][0]["dec"] == O.DEC_DENSE).sum() == w.n_clusters


def test_layer_sharing_and_query_aware_paths(gpu_device, tmp_path):
    """fallback_threshold lifted so similar heads DO share in layer 1; queryaware_threshold set between the
    heads' JS values so that some heads take the query-aware path."""
    probe = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=4096, seed=33, n_clusters=2, n_layers=1)
    js = np.sort(probe["layers"][0]["plan"].js_qa.cpu().numpy())
    qat = float((js[2] + js[3]) / 2)  # three heads below the threshold
    run = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=4096, seed=33, n_clusters=2, fallback_threshold=1e9,
                     queryaware_threshold=qat)
    check_forced(run)
    check_free(run)
    check_outputs(run)
    d0, d1 = run["layers"][0]["dec"], run["layers"][1]["dec"]
    assert (d0 == O.DEC_QA).sum() == 3 and (d1 == O.DEC_QA).sum() == 3
    assert (d0 == O.DEC_SHARE).sum() == 0          # a fresh pivot's siblings cannot share in the same layer
    assert (d1 == O.DEC_SHARE).sum() >= 1          # next layer: same inputs -> JS = 0 -> shared
    hist = run["sharing"].decision_histogram()
    assert hist["dense_pivot"] == 2 and hist["shared"] == int((d1 == O.DEC_SHARE).sum())


def test_prompt_within_the_minimum_budget_skips_selection_with_identical_output(gpu_device, tmp_path):
    """1024 tokens = 8 blocks = the minimum budget: every head's mask is the whole lower triangle whatever it decides
    (the oracle says so too), so the attention function runs the dense mask directly.  Same bits as the full path,
    no plan, zero attn_weights."""
    full = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=1024, seed=44, n_clusters=2, fallback_threshold=1e9)
    check_forced(full)
    tri = np.tril(np.ones((8, 8), dtype=bool))
    for L in full["layers"]:
        assert all(np.array_equal(L["mask"][h], tri) for h in range(8))
        assert all(np.array_equal(L["forced"].mask[h], tri) for h in range(8))
    sub = tmp_path / "fast"
    sub.mkdir()
    fast = run_layers(gpu_device, sub, hq=8, hkv=2, n=1024, seed=44, n_clusters=2, fallback_threshold=1e9,
                      n_layers=0)
    from shareprefill_amd import shareprefill_attention_forward

    sharing = fast["sharing"]
    cfg = types.SimpleNamespace(**{**fast["kw"], "dense_short_prompts": True})
    q, k, v = (fast[x][None].to(gpu_device) for x in ("q", "k", "v"))
    for layer in range(2):
        mod = FakeAttention(cfg, sharing, layer, 128, 8, 2)
        out, avg = shareprefill_attention_forward(mod, q, k, v, None, scaling=mod.scaling)
        assert torch.equal(out.cpu(), full["layers"][layer]["out"])
        assert float(avg.abs().sum()) == 0.0 and avg.shape == (1, 8, 8, 8)
    assert sharing.plans == [] and sharing.decision_histogram()["all_blocks_kept_no_selection"] == 16
    # one block more than the budget: the selection runs
    cfg9 = types.SimpleNamespace(**{**fast["kw"], "dense_short_prompts": True, "min_budget": 896})
    shareprefill_attention_forward(FakeAttention(cfg9, sharing, 0, 128, 8, 2), q, k, v, None, scaling=128 ** -0.5)
    assert len(sharing.plans) == 1


def test_layer_ragged_length(gpu_device, tmp_path):
    run = run_layers(gpu_device, tmp_path, hq=4, hkv=2, n=1000, seed=5, n_clusters=2, fallback_threshold=1e9,
                     min_budget=256)
    check_forced(run)
    check_free(run, expect_same_masks=False)
    check_outputs(run)


@pytest.mark.parametrize("n", [128, 129, 200, 256, 257, 383, 385])
@pytest.mark.parametrize("qat", [0.1, 10.0])
def test_layer_of_one_to_four_blocks(gpu_device, tmp_path, n, qat):
    """The whole selection (not the dense short-prompt shortcut) on prompts of one to four blocks, ragged and not, with
    the minimum budget at one block; queryaware_threshold 10 sends every head down the query-aware path.  Degenerate
    sizes for every kernel: one-entry vectors, a single diagonal block, pivots whose map is 1 x 1."""
    run = run_layers(gpu_device, tmp_path, hq=4, hkv=2, n=n, seed=n, n_clusters=2, min_budget=128,
                     fallback_threshold=1e9, queryaware_threshold=qat)
    check_forced(run)
    if n > 128:
        # (with a single block both distributions of the query-aware test are [1] up to rounding, and their sqrt-JS is
        # the square root of rounding noise around zero: 0, 2e-4 or NaN by the last bit of a sum, here as in the
        # reference -- nothing to compare; every mask is the one block whatever it decides)
        check_free(run, expect_same_masks=False)
    check_outputs(run)


@pytest.mark.parametrize("shared", [[], ["1"], ["0", "3"]])
def test_layer_with_few_or_no_shared_clusters(gpu_device, tmp_path, shared):
    """Tables in which only some clusters share, or none does (no device slot at all): heads outside the shared
    clusters never become pivots and never share, whatever the thresholds."""
    run = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=3000, seed=77, n_clusters=4, n_layers=3, shared=shared,
                     fallback_threshold=1e9, min_budget=512)
    check_forced(run)
    check_free(run)
    check_outputs(run)
    dense_per_layer = [int((L["dec"] == O.DEC_DENSE).sum()) for L in run["layers"]]
    assert dense_per_layer[0] == len(shared) and sum(dense_per_layer[1:]) == 0
    member = {h for cid in shared for layer, h in run["table"]["clusters"][cid]}
    for L in run["layers"]:
        for h in range(8):
            if h not in member:
                assert L["dec"][h] in (O.DEC_VS, O.DEC_QA)


@pytest.mark.parametrize("min_budget,max_budget,thr", [(512, 1536, 0.95), (128, 128, 0.99), (2048, 1024, 0.9), (None, None, 0.5),
                                                       (1, 100000, 0.999)])
def test_layer_budget_clamps(gpu_device, tmp_path, min_budget, max_budget, thr):
    """min_budget / max_budget in tokens, converted and clamped as shareprefill_attn.py:112-122 and
    attention_sharing.py:169-176 do: a maximum below what the threshold asks for, a maximum of one block, a minimum
    above the maximum (the maximum wins: it is applied last), no limits at all, and limits that never bind."""
    run = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=4096, seed=31, n_clusters=2, min_budget=min_budget,
                     max_budget=max_budget, pattern_threshold=thr, fallback_threshold=1e9)
    check_forced(run)
    check_free(run, expect_same_masks=False)
    check_outputs(run)
    if max_budget is not None:
        cap = min(-(-max_budget // 128), run["nb"])
        for L in run["layers"]:
            assert int(L["plan"].nv.max()) <= cap and int(L["plan"].ns.max()) <= cap


@pytest.mark.parametrize("hq,hkv,n_clusters", [(1, 1, 1), (3, 3, 1), (5, 1, 1), (12, 4, 3), (6, 6, 2), (9, 3, 3)])
def test_layer_head_counts(gpu_device, tmp_path, hq, hkv, n_clusters):
    """One head, no grouping, odd groups, groups of three: the kv-head mapping of every kernel and the work-item
    pairing (two adjacent heads only inside one kv group; an odd head pairs its own rows)."""
    run = run_layers(gpu_device, tmp_path, hq=hq, hkv=hkv, n=1500, seed=10 * hq + hkv, n_clusters=n_clusters,
                     min_budget=256, fallback_threshold=1e9)
    check_forced(run)
    check_free(run, expect_same_masks=False)
    check_outputs(run)


def test_reference_style_interfaces(gpu_device, tmp_path):
    """get_active_blocks / update_pivotal_attns with the reference's argument layout, and the id-list view."""
    from shareprefill_amd import AttentionSharing, ops

    hq, hkv, n = 4, 2, 1024
    table = synthetic.random_cluster_table(hq, 2, 2, 3)
    path = synthetic.write_cluster_table(table, str(tmp_path / "t.json"))
    q, k, v = synthetic.planted_qkv(hq, hkv, n, 128, 3)
    sharing = AttentionSharing(path)
    qn, kn = q.transpose(1, 2).to(gpu_device), k.transpose(1, 2).to(gpu_device)  # [B, N, H, D]
    mask, use_dense = sharing.get_active_blocks(qn, kn, 0, hq, 128, 8, 2 ** 24, 0.9, 0.5, 0.9, 0.1)
    assert mask.shape == (1, hq, 8, 1) and use_dense.shape == (1, hq) and use_dense.dtype == torch.bool
    ids = sharing.plans[-1].block_idx()[0]
    dense_heads = torch.nonzero(use_dense[0]).reshape(-1).cpu().tolist()
    assert len(dense_heads) == 2
    for h in dense_heads:  # all lower-triangular ids, attention_sharing.py:217-219
        assert ids[h].cpu().tolist() == [r * 8 + c for r in range(8) for c in range(r + 1)]
    with pytest.raises(NotImplementedError):  # un-expanded K: the reference would map head h to kv head h % Hkv
        sharing.get_active_blocks(qn, kn, 0, hq, 128, 8, 2 ** 24, gqa_interleave=True)
    # K expanded to the query head count, as the reference's attention function passes it: the flag changes nothing
    sharing.reset_state()
    k_exp = kn.repeat_interleave(hq // kn.shape[2], dim=2)
    mask_i, dense_i = sharing.get_active_blocks(qn, k_exp, 0, hq, 128, 8, 2 ** 24, 0.9, 0.5, 0.9, 0.1, gqa_interleave=True)
    assert torch.equal(mask_i, mask) and torch.equal(dense_i, use_dense)
    with pytest.raises(ValueError):
        sharing.get_active_blocks(qn.expand(2, -1, -1, -1), kn.expand(2, -1, -1, -1), 0, hq, 128, 8, 2 ** 24)
    sharing.reset_state()
    assert all(v["pivot_head"] == -1 for v in sharing.pivot_summary().values())


def test_forward_rejects_sliding_window_and_handles_short_and_decode(gpu_device, tmp_path):
    from shareprefill_amd import AttentionSharing, shareprefill_attention_forward

    table = synthetic.random_cluster_table(4, 2, 1, 0)
    path = synthetic.write_cluster_table(table, str(tmp_path / "t.json"))
    cfg = types.SimpleNamespace(block_size=128, min_budget=1024, max_budget=None, pattern_threshold=0.9,
                                similarity_threshold=0.5, fallback_threshold=0.9, queryaware_threshold=0.1)
    mod = FakeAttention(cfg, AttentionSharing(path), 0, 128, 4, 2)
    g = torch.Generator().manual_seed(0)
    mk = lambda h, n: torch.randn(1, n, h, 128, generator=g).to(torch.bfloat16).transpose(1, 2).to(gpu_device)
    q, k, v = mk(4, 100), mk(2, 100), mk(2, 100)
    with pytest.raises(NotImplementedError):
        shareprefill_attention_forward(mod, q, k, v, None, scaling=1.0, sliding_window=4096)
    out, w = shareprefill_attention_forward(mod, q, k, v, None, scaling=1.0)   # shorter than a block: dense causal
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float().repeat_interleave(2, 1),
                                                           v.float().repeat_interleave(2, 1), is_causal=True)
    assert (out.transpose(1, 2).float() - ref).abs().max().item() <= MAX_ABS
    # gqa_interleave: accepted, and (as in the reference, which expands K / V the same way under both settings)
    # without any effect
    out_i, _ = shareprefill_attention_forward(mod, q, k, v, None, scaling=1.0, gqa_interleave=True)
    assert torch.equal(out_i, out)
    out1, w1 = shareprefill_attention_forward(mod, q[:, :, -1:], k, v, None, scaling=1.0)  # decode step
    assert w1 is None and out1.shape == (1, 1, 4, 128)
    assert (out1[0, 0].float() - ref[0, :, -1].float()).abs().max().item() <= MAX_ABS


@pytest.mark.parametrize("nb,thr", [(13, 0.95), (21, 0.95), (37, 0.95), (12, 0.9), (23, 0.9), (14, 0.99), (29, 0.99)])
def test_layer_all_query_aware_at_block_counts_where_a_float_threshold_would_differ(gpu_device, tmp_path, nb, thr):
    """Block counts at which fp32(double(pattern_threshold) * nb), the score the reference's query-aware selection
    compares with (attention_sharing.py:361), differs from what a threshold rounded to fp32 first would give (never the
    case for powers of two, which every other test of this path uses).  queryaware_threshold 10 sends every head down
    the query-aware path; the forced comparison holds the masks to the oracle's, which forms the score from the
    Python float."""
    assert np.float32(thr * nb) != np.float32(float(np.float32(thr)) * nb)
    run = run_layers(gpu_device, tmp_path, hq=8, hkv=2, n=nb * 128, seed=nb, n_clusters=2, min_budget=256,
                     pattern_threshold=thr, fallback_threshold=1e9, queryaware_threshold=10.0)
    assert all((L["dec"] == O.DEC_QA).all() for L in run["layers"])
    check_forced(run)
    check_free(run, expect_same_masks=False)
    check_outputs(run)


def test_short_prompt_shortcut_needs_the_maximum_budget_to_reach_the_prompt_too(gpu_device, tmp_path):
    """min_budget 2048 tokens (16 blocks) above max_budget 1024 (8 blocks) on a prompt of 12 blocks: the budgets are
    raised to 16 and then cut to 8 (attention_sharing.py:173-176), so vertical-slash and fallback heads keep 8 of 12
    columns and distances -- a sparse mask, although the prompt has no more blocks than the minimum budget.  The
    dense short-prompt shortcut must not be taken: with it enabled the layer gives the full path's decisions, masks
    (the oracle's) and output bits."""
    from shareprefill_amd import shareprefill_attention_forward

    kw = dict(hq=8, hkv=2, n=1500, seed=91, n_clusters=2, min_budget=2048, max_budget=1024, fallback_threshold=1e9)
    full = run_layers(gpu_device, tmp_path, **kw)
    check_forced(full)
    check_outputs(full)
    tri = np.tril(np.ones((12, 12), dtype=bool))
    assert any(not np.array_equal(L["mask"][h], tri) for L in full["layers"] for h in range(8)), "masks must be sparse"
    from shareprefill_amd import AttentionSharing

    fast = full
    sharing = AttentionSharing(synthetic.write_cluster_table(full["table"], str(tmp_path / "same_table.json")))
    cfg = types.SimpleNamespace(**{**fast["kw"], "dense_short_prompts": True})
    q, k, v = (fast[x][None].to(gpu_device) for x in ("q", "k", "v"))
    for layer in range(2):
        out, avg = shareprefill_attention_forward(FakeAttention(cfg, sharing, layer, 128, 8, 2), q, k, v, None,
                                                  scaling=128 ** -0.5)
        assert torch.equal(out.cpu(), full["layers"][layer]["out"]), f"layer {layer}"
        assert torch.equal(avg.cpu(), full["layers"][layer]["avg"])
    assert len(sharing.plans) == 2 and sharing.dense_layers == 0
    # with the maximum at or above the prompt the shortcut is taken again
    cfg_ok = types.SimpleNamespace(**{**fast["kw"], "dense_short_prompts": True, "max_budget": 1536})
    sharing.reset_state()
    shareprefill_attention_forward(FakeAttention(cfg_ok, sharing, 0, 128, 8, 2), q, k, v, None, scaling=128 ** -0.5)
    assert sharing.plans == [] and sharing.dense_layers == 1


def test_layers_of_the_shipped_llama_table_elect_and_reuse_the_pivot_of_its_one_shared_cluster(gpu_device, tmp_path):
    """The table the reference ships for Llama-3.1-8B-Instruct: 44 clusters over 32 layers x 32 heads of which ONE
    ("9": 42 heads in layers 14 to 30) is shared (attention_sharing.py:204-295 only ever look at shared clusters).
    Layers 14, 15, 17, 22 and 30 run with the layer indices of the table on 8192 planted tokens, new q / k / v per
    layer: the pivot is elected at the cluster's first layer (14, head 17), a layer without members (15) changes
    nothing, the members of layers 17, 22 (nine of them in one layer) and 30 -- sixteen layers after the election --
    take the share test against that pivot's stored vectors and reuse its pattern; every head outside the cluster
    stays on the vertical-slash path.  Decisions, budgets, masks, the pivot's pattern, map and coverage ratio are the
    oracle's (forced comparison); outputs against the fp32 masked attention for the last layer."""
    import json

    from shareprefill_amd import SharePrefillConfig, ops

    path = SharePrefillConfig(model_name="Llama-3.1-8B-Instruct").sharing_lookup_path
    with open(path) as f:
        table = json.load(f)
    members = {}
    for layer, head in table["clusters"]["9"]:
        members.setdefault(layer, []).append(head)
    assert table["shared_clusters"] == ["9"] and min(members) == 14 and members[14] == [17] and 15 not in members
    layer_ids = [14, 15, 17, 22, 30]
    run = run_layers(gpu_device, tmp_path, hq=32, hkv=8, n=8192, seed=400, n_clusters=0, table=table,
                     layer_ids=layer_ids, reseed=True, with_free=False, fallback_threshold=1e9)
    sharing = run["sharing"]
    assert len(sharing._slot) == 1 and sharing.max_pivots(14, 32) == 1 and sharing.max_pivots(15, 32) == 0
    check_forced(run)
    by_layer = {L["layer"]: L for L in run["layers"]}
    assert np.nonzero(by_layer[14]["dec"] == O.DEC_DENSE)[0].tolist() == [17]
    summary = sharing.pivot_summary()["9"]
    assert summary["pivot_head"] == 17 and summary["layer"] == 14 and summary["has_pattern"]
    shared_heads = 0
    for layer in layer_ids[1:]:
        dec = by_layer[layer]["dec"]
        assert not (dec == O.DEC_DENSE).any()
        share = set(np.nonzero(dec == O.DEC_SHARE)[0].tolist())
        assert share <= set(members.get(layer, []))
        shared_heads += len(share)
        # a shared head's mask holds the pivot's pattern
        pat = ops.mask_to_bool(sharing._state.pattern[0], run["nb"]).cpu().numpy()
        for h in share:
            assert (by_layer[layer]["mask"][h] & pat == pat).all()
    assert not (by_layer[15]["dec"] == O.DEC_SHARE).any()
    assert len(set(np.nonzero(by_layer[22]["dec"] == O.DEC_SHARE)[0].tolist())) >= 2, "several members in one layer"
    assert (by_layer[30]["dec"] == O.DEC_SHARE).tolist().count(True) == 1 and by_layer[30]["dec"][21] == O.DEC_SHARE
    assert shared_heads >= 4
    L = by_layer[30]  # heads 20 .. 23 = the group of kv head 5, with the shared head 21 among them
    ref, _ = O.masked_attention(L["q"][20:24], L["k"][5:6], L["v"][5:6], L["mask"][20:24], 128, 128 ** -0.5)
    out = L["out"][0].transpose(0, 1)[20:24].float()
    assert (out - ref).abs().max().item() <= MAX_ABS
    assert ((out - ref).abs().mean() / ref.abs().mean()).item() <= MEAN_REL

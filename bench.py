"""Benchmark of the SharePrefill prefill-attention layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--pattern-threshold 0.95]

A step is one pass of the whole layer (last-block scores, budgets, K pooling, query-aware test, pivot /
share decision, mask build, Q pooling + query-aware selection, V repack, block-sparse attention, pivot
update) over one synthetic Q/K/V batch that is already resident in HBM.  The layer timed is layer 1, after
one untimed call of layer 0 has elected the cluster pivots (sharing can only start in the layer after the
pivot's, shareprefill/attn/shareprefill_attn.py:141-143).  Prints ONE JSON line.

The default run carries the whole metric in that one line: the 128K layer (value, roofline of the attention kernel),
the pattern_threshold sweep 0.9 / 0.95 / 0.99 with the dense causal baseline, a second timed variant of the same layer
whose thresholds make heads share and go query-aware (`sharing_layer`), the end-to-end TTFT of the whole
Llama-3.1-8B architecture at 131072 tokens (`ttft`), and the CPU baseline.  --no-sweep / --no-ttft / --no-extras /
--no-cpu-baseline drop parts of it.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import tempfile
import time
import types

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FLOP_PER_BLOCK = 4 * 128 * 128 * 128       # QK^T + PV of one kept 128x128 block at head_dim 128
PEAK_BF16_TFLOPS = 2500.0                  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="C3", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--seq-len", type=int, default=131072, help="C4 only: prompt length")
    ap.add_argument("--pattern-threshold", type=float, default=None)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the stage breakdown / dense baseline / sweep")
    ap.add_argument("--sweep", action="store_true", help="(default now) time pattern_threshold 0.9, 0.95 and 0.99")
    ap.add_argument("--no-sweep", action="store_true", help="skip the pattern_threshold sweep")
    ap.add_argument("--no-ttft", action="store_true",
                    help="skip the end-to-end TTFT block (whole Llama-3.1-8B architecture, 131072 tokens, 1 warm-up + 1 "
                         "timed forward) that the default C3 run appends")
    ap.add_argument("--fuse-rope", action="store_true",
                    help="C4 only: rotary embedding by the one-pass in-place HIP kernel instead of the model's "
                         "elementwise kernels (bit-identical)")
    ap.add_argument("--length-sweep", default=None,
                    help="C4 only: comma-separated prompt lengths; adds TTFT per length for the SharePrefill path and for "
                         "the model's stock causal attention (torch SDPA), the protocol of eval/efficiency/latency.py")
    return ap.parse_args()


def event_ms(fn, reps=3):
    import torch

    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        ts.append(a.elapsed_time(b))
    return sum(ts) / len(ts)


def cpu_baseline(w, q, k, v, mask_bool, decision, kept_blocks, pt):
    """Times the CPU oracle (torch-CPU restatement of the reference mask logic + block-sparse attention over
    kept blocks) on a bounded sample and scales it to one layer: the selection float work on 2 of the heads,
    the attention on 6 (head, query-block) rows spread over the heads and the sequence."""
    import numpy as np
    import torch

    from oracle import shareprefill_oracle as O

    hq, n, bs = w.hq, w.seq_len, w.block_size
    nb = n // bs
    g = hq // w.hkv
    heads = [0, hq - 1]
    qc = q[0][heads].cpu()
    kc = k[0][[h // g for h in heads]].cpu()
    t0 = time.perf_counter()
    for i in range(len(heads)):
        vt, st = O.lastq_scores(qc[i:i + 1], kc[i:i + 1], bs)
        O.cover_count(vt[0].numpy(), pt)
        O.cover_count(st[0].numpy(), pt)
        O.block_sum(vt, bs), O.block_sum(st, bs)
        O.pool_avg(kc[i].unsqueeze(1), bs)
    t_sel = (time.perf_counter() - t0) / len(heads) * hq
    # attention sample: rows at 1/6, 2/6 ... of the sequence, heads spread
    rows = [(int(hq * (i + 0.5) / 6), int(nb * (i + 1) / 6) - 1) for i in range(6)]
    blocks = 0
    t_att = 0.0
    for h, r in rows:
        qh = q[0][h:h + 1, r * bs:(r + 1) * bs].cpu()
        kh, vh = k[0][h // g:h // g + 1, : (r + 1) * bs].cpu(), v[0][h // g:h // g + 1, : (r + 1) * bs].cpu()
        cols = np.nonzero(mask_bool[h, r, : r + 1])[0]
        t1 = time.perf_counter()
        kidx = torch.cat([torch.arange(c * bs, (c + 1) * bs) for c in cols])
        s = (qh[0].float() @ kh[0][kidx].float().T) * (w.head_dim ** -0.5)
        pos = torch.arange(r * bs, (r + 1) * bs)
        s = s.masked_fill(kidx[None, :] > pos[:, None], float("-inf"))
        p = torch.softmax(s, -1)
        _ = p @ vh[0][kidx].float()
        t_att += time.perf_counter() - t1
        blocks += len(cols)
    per_block = t_att / max(blocks, 1)
    total_ms = (t_sel + per_block * kept_blocks) * 1e3
    return {"value": round(total_ms, 1), "unit": "ms", "cores": torch.get_num_threads(), "kind": "port, extrapolated",
            "extrapolated": True,
            "sample": f"EXTRAPOLATED from a bounded sample: selection float stages on heads {heads} (x{hq // len(heads)}), fp32 block-sparse attention on "
                      f"{len(rows)} (head, query-block) rows = {blocks} kept blocks at {per_block * 1e3:.3f} ms/block, "
                      f"scaled to {kept_blocks} kept blocks; extrapolated"}


# Bytes one steady-state sp_attn_fwd_kernel launch moves past the L2 caches, from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE scaled by the V-repack kernel's known 256 MiB (profiles/attention_layer_C3_hbm_traffic.txt).  A counter
# run cannot happen inside this script, so the figure is tied to the kernel source it was measured on: it is
# reported only while shareprefill_amd/csrc/sp_attn.hip still has that hash, and is null (with a note) after any
# change to the kernel until the profile is taken again.
MEASURED_ATTN_TRAFFIC = {
    ("C3", 0.95): {"bytes": int((102.5 + 1.0) * 2 ** 30), "sp_attn_hip_sha256_16": "8d0a005a12007b26",
                   "profile": "profiles/attention_layer_C3_hbm_traffic.txt"},
}


def measured_traffic(workload, pt):
    """-> (bytes or None, note)"""
    import hashlib

    rec = MEASURED_ATTN_TRAFFIC.get((workload, pt))
    if rec is None:
        return None, "no counter profile for this workload"
    with open(os.path.join(ROOT, "shareprefill_amd", "csrc", "sp_attn.hip"), "rb") as f:
        sha = hashlib.sha256(f.read()).hexdigest()[:16]
    if sha != rec["sp_attn_hip_sha256_16"]:
        return None, f"kernel source changed since {rec['profile']} was taken (sha {rec['sp_attn_hip_sha256_16']} -> {sha})"
    return rec["bytes"], f"FETCH_SIZE + WRITE_SIZE past L2 (memory-side cache + HBM), {rec['profile']}, kernel source sha {sha}"


def library_gemm_tflops(dev, n=8192, reps=200):
    """bf16 GEMM rate of the vendor library (torch.matmul) on N(0,1) data: what a tuned dense kernel sustains on
    this chip with operands that toggle -- a calibration point beside the nominal peak, nothing the path uses."""
    import torch

    g = torch.Generator(device=dev).manual_seed(1)
    a = torch.randn(n, n, device=dev, dtype=torch.bfloat16, generator=g)
    b = torch.randn(n, n, device=dev, dtype=torch.bfloat16, generator=g)
    for _ in range(3):
        a @ b
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        a @ b
    torch.cuda.synchronize()
    return 2.0 * n ** 3 * reps / (time.perf_counter() - t0) / 1e12


def c4_line(args):
    """TTFT of the full Llama-3.1-8B architecture (random-init bf16, 32 layers, hidden 4096, Hq32 Hkv8, RoPE theta
    5e5, vocab 128256) on uniform-random token ids, SharePrefill patched into every layer with the shipped
    Llama-3.1-8B-Instruct table; one prefill forward with last-token logits only."""
    import torch
    from transformers import LlamaConfig, LlamaForCausalLM

    from shareprefill_amd import SharePrefill

    dev = torch.device("cuda:0")
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=128256, max_position_embeddings=131072,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0}, rms_norm_eps=1e-5,
                      tie_word_embeddings=False)
    torch.manual_seed(1238)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    with torch.device(dev):
        model = LlamaForCausalLM(cfg)
    torch.set_default_dtype(old)
    model.eval()
    model = SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct", pattern_threshold=0.95, similarity_threshold=0.5,
                         fallback_threshold=0.95, block_size=128, min_budget=1024, fuse_rope=args.fuse_rope)(model)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1238)
    ids = torch.randint(0, cfg.vocab_size, (1, args.seq_len), generator=gen, device=dev)
    model.attention_sharing.keep_plans = True  # every layer's mask (4 MiB at 128K) stays for the density below

    def fwd():
        with torch.no_grad():
            return model(ids, use_cache=False, logits_to_keep=1).logits

    for _ in range(max(args.warmup, 1)):
        fwd()
    torch.cuda.synchronize()
    steps = max(1, min(args.steps, 3))
    t0 = time.perf_counter()
    for _ in range(steps):
        out = fwd()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    sharing = model.attention_sharing
    dens = torch.stack([p.density() for p in sharing.plans]).mean().item()
    line = {"metric": "ttft_s_llama31_8b_arch_prefill", "value": round(sec, 3), "unit": "s", "n_gpus": 1,
            "steps": steps, "warmup": max(args.warmup, 1), "ms_per_step": round(sec * 1e3, 1),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"C4: Llama-3.1-8B architecture, random-init bf16, {args.seq_len} uniform-random token "
                                   "ids, SharePrefill in all 32 layers (shipped Llama-3.1-8B-Instruct table, "
                                   "pattern 0.95, similarity 0.5, fallback 0.95, min_budget 1024), logits_to_keep=1",
                       "fuse_rope": bool(args.fuse_rope)},
            "tokens_per_s": round(args.seq_len / sec, 1), "mean_block_density": round(dens, 4),
            "decisions": sharing.decision_histogram(), "finite_logits": bool(torch.isfinite(out).all())}
    if getattr(args, "both_rope", False):
        # the same model and prompt with the other rotary-embedding setting (the fused one-pass kernel is bit-identical
        # to the model's elementwise evaluation): 1 warm-up + the same number of timed forwards
        from shareprefill_amd import unpatch_model

        unpatch_model(model)
        model = SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct", pattern_threshold=0.95,
                             similarity_threshold=0.5, fallback_threshold=0.95, block_size=128, min_budget=1024,
                             fuse_rope=not args.fuse_rope)(model)
        fwd()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fwd()
        torch.cuda.synchronize()
        line["other_rope_setting"] = {"fuse_rope": not args.fuse_rope, "value": round((time.perf_counter() - t0) / steps, 3),
                                      "unit": "s", "steps": steps, "warmup": 1}
    if args.length_sweep:
        # the reference's latency protocol (eval/efficiency/latency.py:21-108): same model, growing prompts,
        # sparse path against the stock dense causal attention
        sweep = []
        for length in [int(x) for x in args.length_sweep.split(",") if x]:
            ids_l = torch.randint(0, cfg.vocab_size, (1, length), generator=gen, device=dev)
            row = {"seq_len": length}
            for name, impl in (("shareprefill_s", "shareprefill"), ("dense_sdpa_s", "sdpa")):
                model.config._attn_implementation = impl
                try:
                    with torch.no_grad():
                        model(ids_l, use_cache=False, logits_to_keep=1)
                        torch.cuda.synchronize()
                        t1 = time.perf_counter()
                        model(ids_l, use_cache=False, logits_to_keep=1)
                        torch.cuda.synchronize()
                    row[name] = round(time.perf_counter() - t1, 4)
                except Exception as exc:  # e.g. the dense path running out of memory at the longest prompts
                    row[name] = None
                    row[name + "_error"] = type(exc).__name__
                    torch.cuda.empty_cache()
            model.config._attn_implementation = "shareprefill"
            if row.get("shareprefill_s") and row.get("dense_sdpa_s"):
                row["speedup"] = round(row["dense_sdpa_s"] / row["shareprefill_s"], 3)
            sweep.append(row)
        line["length_sweep"] = sweep
    del model
    import gc

    gc.collect()
    torch.cuda.empty_cache()
    return line


def run_c4(args):
    print(json.dumps(c4_line(args)))


def sharing_layer_variant(args, w, pt, q, k, v, table):
    """The same layer on the same inputs with thresholds under which heads DO share and go query-aware (with the
    library defaults none of these synthetic heads does: a pivot with local attention has vs_ratio >= (nb-1)/nb >
    fallback_threshold 0.9, and no head's sqrt-JS is below queryaware_threshold 0.1): fallback_threshold lifted,
    queryaware_threshold placed between the heads' own sqrt-JS values so that a quarter of them are query-aware.
    Layer 0 once (pivot election), then warm-up and timed calls of layer 1; plus the time of the stages that only
    these head kinds use."""
    import torch

    from shareprefill_amd import AttentionSharing, _lib, ops, shareprefill_attention_forward

    nb = w.seq_len // w.block_size
    tri = w.hq * nb * (nb + 1) // 2
    scale = w.head_dim ** -0.5
    with tempfile.TemporaryDirectory() as tmp:
        from shareprefill_amd import synthetic

        sh = AttentionSharing(synthetic.write_cluster_table(table, os.path.join(tmp, "table.json")))

    def cfg(fallback, qat):
        return types.SimpleNamespace(block_size=w.block_size, min_budget=w.min_budget, max_budget=None,
                                     pattern_threshold=pt, similarity_threshold=w.similarity_threshold,
                                     fallback_threshold=fallback, queryaware_threshold=qat)

    def run(layer, c):
        mod = types.SimpleNamespace(config=c, attention_sharing=sh, layer_idx=layer, scaling=scale)
        return shareprefill_attention_forward(mod, q, k, v, None, scaling=scale)

    sh.keep_debug = True
    run(0, cfg(w.fallback_threshold, w.queryaware_threshold))
    js = torch.sort(sh.plans[-1].js_qa.double().cpu()).values
    n_qa = max(w.hq // 4, 1)
    qat = float((js[n_qa - 1] + js[n_qa]) / 2)
    c2 = cfg(1e9, qat)
    sh.keep_debug = False
    sh.reset_state()
    _, avg0 = run(0, c2)
    plan0 = sh.plans[-1]
    for _ in range(2):
        run(1, c2)
    torch.cuda.synchronize()
    steps = max(1, min(args.steps, 10))
    tm = ops.KernelTimer()
    ops.kernel_timer = tm
    t0 = time.perf_counter()
    for _ in range(steps):
        run(1, c2)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    ops.kernel_timer = None
    attn_ms = sum(tm.durations_ms("attn")) / steps
    names = {0: "vertical_slash", 1: "dense_pivot", 2: "shared", 3: "query_aware"}

    def hist(plan):
        return {names[int(c)]: int(n) for c, n in zip(*torch.unique(plan.decision.cpu(), return_counts=True))}

    plan1 = sh.plans[-1]
    kept = int(ops.mask_row_pointers(plan1.mask)[:, -1].sum())
    out = {"thresholds": {"pattern": pt, "similarity": w.similarity_threshold, "fallback": 1e9,
                          "queryaware": round(qat, 6)},
           "steps": steps, "layer_ms": round(ms, 3), "attn_ms": round(attn_ms, 3), "kept_blocks": kept,
           "density": round(kept / tri, 4), "decisions": hist(plan1), "layer0_decisions": hist(plan0),
           "attn_tflops": round(kept * FLOP_PER_BLOCK / attn_ms / 1e9, 1),
           "attn_frac_of_peak": round(kept * FLOP_PER_BLOCK / attn_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
           "layer_frac_of_peak": round(kept * FLOP_PER_BLOCK / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    # stages that only shared / query-aware / pivot heads use, timed alone on this layer's own intermediates
    sh.keep_debug = True
    run(1, c2)
    p = sh.plans[-1]
    sh.keep_debug = False
    state = sh._state
    hc = sh._head_cluster_tensor(1, w.hq, q.device)
    use_qa = (p.decision == _lib.SP_DEC_QA).to(torch.int32)
    minb = math.ceil(w.min_budget / w.block_size)
    qh = q[0]
    stage = {}
    stage["share_decide"] = event_ms(lambda: ops.share_decide(state, hc, 1, p.vert_blk, p.slash_blk, use_qa, p.nv, p.ns,
                                                              minb, w.similarity_threshold, 1e9))
    stage["build_mask"] = event_ms(lambda: ops.build_mask(state, hc, p.decision, p.vert_blk, p.slash_blk, p.nv_final,
                                                          p.ns_final))
    scratch_mask = p.mask.clone()

    def qa_select():
        qbar = ops.pool_avg(qh, w.block_size, tail_mode=_lib.SP_POOL_TAIL_RESCALE, head_enable=use_qa)
        ops.queryaware_select(qbar, p.kbar, p.decision, scratch_mask, pt, probs=sh._qa_scratch(w.hq, nb, q.device))

    stage["queryaware_select_incl_q_pooling"] = event_ms(qa_select)
    hc0 = sh._head_cluster_tensor(0, w.hq, q.device)
    # the layer-0 pivots' update (row patterns + coverage ratio); repeating it rewrites the same values
    stage["pivot_update_layer0_pivots"] = event_ms(lambda: ops.pivot_update(state, hc0, plan0.decision, avg0[0], pt))
    out["stage_ms"] = {a: round(b, 3) for a, b in stage.items()}
    out["n_pivots_layer0"] = int((plan0.decision == _lib.SP_DEC_DENSE).sum())
    return out


def timed_layer_point(w, q, k, v, table, pt, steps=5, n_tokens=None, with_stages=False):
    """Layer 0 once (pivot election), one warm-up and `steps` timed calls of layer 1 at pattern_threshold pt on the
    workload's inputs (cut to their first n_tokens tokens when given): kept blocks, layer and attention-launch time,
    fractions of the bf16 peak on kept blocks; with_stages adds the time of every stage outside the attention launch."""
    import torch

    from shareprefill_amd import AttentionSharing, ops, shareprefill_attention_forward, synthetic

    if n_tokens is not None:
        q, k, v = q[:, :, :n_tokens], k[:, :, :n_tokens], v[:, :, :n_tokens]
    n = q.shape[2]
    nb = -(-n // w.block_size)
    tri = w.hq * nb * (nb + 1) // 2
    scale = w.head_dim ** -0.5
    with tempfile.TemporaryDirectory() as tmp:
        sh = AttentionSharing(synthetic.write_cluster_table(table, os.path.join(tmp, "table.json")))
    cfg = types.SimpleNamespace(block_size=w.block_size, min_budget=w.min_budget, max_budget=None, pattern_threshold=pt,
                                similarity_threshold=w.similarity_threshold, fallback_threshold=w.fallback_threshold,
                                queryaware_threshold=w.queryaware_threshold)

    def run(layer):
        mod = types.SimpleNamespace(config=cfg, attention_sharing=sh, layer_idx=layer, scaling=scale)
        return shareprefill_attention_forward(mod, q, k, v, None, scaling=scale)

    run(0)
    run(1)
    torch.cuda.synchronize()
    tm = ops.KernelTimer()
    ops.kernel_timer = tm
    t0 = time.perf_counter()
    for _ in range(steps):
        run(1)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    ops.kernel_timer = None
    ams = sum(tm.durations_ms("attn")) / steps
    plan = sh.plans[-1]
    kept = int(ops.mask_row_pointers(plan.mask)[:, -1].sum())
    flop_per_block = 4.0 * w.block_size * w.block_size * w.head_dim  # (FLOP_PER_BLOCK at the path's block size 128)
    out = {"pattern_threshold": pt, "tokens": n, "kept_blocks": kept, "density": round(kept / tri, 4),
           "layer_ms": round(ms, 3), "attn_ms": round(ams, 3),
           "attn_tflops": round(kept * flop_per_block / ams / 1e9, 1),
           "attn_frac_of_peak": round(kept * flop_per_block / ams / 1e9 / PEAK_BF16_TFLOPS, 4),
           "layer_frac_of_peak": round(kept * flop_per_block / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    if with_stages:
        qh, kh, vh = q[0], k[0], v[0]
        minb = math.ceil(w.min_budget / w.block_size)
        st = {}
        st["lastq_scores"] = event_ms(lambda: ops.lastq_scores(qh, kh, w.block_size))
        vt, st_, vb, sb = ops.lastq_scores(qh, kh, w.block_size)
        st["cover_budgets"] = event_ms(lambda: ops.cover_budgets(vt, st_, w.block_size, pt, minb, nb))
        st["pool_k"] = event_ms(lambda: ops.pool_avg(kh, w.block_size))
        kbar = ops.pool_avg(kh, w.block_size)
        st["queryaware_test"] = event_ms(lambda: ops.queryaware_test(qh, kbar, vb, w.block_size, w.queryaware_threshold))
        st["attention_launch"] = ams
        st["everything_else"] = max(0.0, ms - sum(st.values()))
        out["stage_ms"] = {a: round(b, 3) for a, b in st.items()}
    return out


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (the SharePrefill layer has no multi-GPU path); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == "C4":
        import torch

        if not torch.cuda.is_available():
            print("bench.py: no GPU visible", file=sys.stderr)
            sys.exit(2)
        run_c4(args)
        return

    import torch

    from shareprefill_amd import AttentionSharing, _lib, ops, shareprefill_attention_forward, synthetic

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    _lib.load()
    dev = torch.device("cuda:0")
    w = synthetic.WORKLOADS[args.workload]
    pt = w.pattern_threshold if args.pattern_threshold is None else args.pattern_threshold
    q, k, v = synthetic.workload_inputs(w, device=dev)
    table = synthetic.random_cluster_table(w.hq, w.n_clusters, 2, w.seed)
    with tempfile.TemporaryDirectory() as tmp:
        sharing = AttentionSharing(synthetic.write_cluster_table(table, os.path.join(tmp, "table.json")))
    nb = w.seq_len // w.block_size

    def make_cfg(thr):
        return types.SimpleNamespace(block_size=w.block_size, min_budget=w.min_budget, max_budget=None,
                                     pattern_threshold=thr, similarity_threshold=w.similarity_threshold,
                                     fallback_threshold=w.fallback_threshold,
                                     queryaware_threshold=w.queryaware_threshold)

    def module(layer, thr):
        return types.SimpleNamespace(config=make_cfg(thr), attention_sharing=sharing, layer_idx=layer,
                                     scaling=w.head_dim ** -0.5)

    def run_layer(layer, thr):
        return shareprefill_attention_forward(module(layer, thr), q, k, v, None, scaling=w.head_dim ** -0.5)

    def prime(thr):
        sharing.reset_state()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        run_layer(0, thr)
        b.record()
        b.synchronize()
        return a.elapsed_time(b)

    # ---- layer 0 once (pivot election), then W warm-up and K timed steps of layer 1 -----------------
    layer0_ms = prime(pt)
    plan0 = sharing.plans[-1]
    kept0 = int(ops.mask_row_pointers(plan0.mask)[:, -1].sum())  # now: the mask is released when layer 1 is planned
    for _ in range(args.warmup):
        run_layer(1, pt)
    torch.cuda.synchronize()
    timer = ops.KernelTimer()
    ops.kernel_timer = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_layer(1, pt)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops.kernel_timer = None
    ms_per_step = elapsed / args.steps * 1e3
    plan = sharing.plans[-1]
    kept = int(ops.mask_row_pointers(plan.mask)[:, -1].sum())
    tri = w.hq * nb * (nb + 1) // 2
    density = kept / tri
    attn_ms = timer.durations_ms("attn")
    attn_avg_ms = sum(attn_ms) / len(attn_ms)
    flop = kept * FLOP_PER_BLOCK
    attn_tflops = flop / (attn_avg_ms * 1e-3) / 1e12
    layer_tflops = flop / (ms_per_step * 1e-3) / 1e12
    hist = {}
    names = {0: "vertical_slash", 1: "dense_pivot", 2: "shared", 3: "query_aware"}
    for code, cnt in zip(*torch.unique(plan.decision.cpu(), return_counts=True)):
        hist[names[int(code)]] = int(cnt)
    hist0 = {}
    for code, cnt in zip(*torch.unique(plan0.decision.cpu(), return_counts=True)):
        hist0[names[int(code)]] = int(cnt)

    line = {
        "metric": "sparse_attn_prefill_ms_per_layer_128k" if args.workload == "C3" else
                  f"sparse_attn_prefill_ms_per_layer_{args.workload}",
        "value": round(ms_per_step, 3), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{w.name}: B1 Hq{w.hq} Hkv{w.hkv} D{w.head_dim} N{w.seq_len} bf16, block 128, "
                               f"min_budget {w.min_budget}, pattern_threshold {pt}, similarity {w.similarity_threshold}, "
                               f"fallback {w.fallback_threshold}, queryaware {w.queryaware_threshold}, "
                               f"{w.n_clusters} shared clusters; layer 1 timed after pivot-election layer 0",
                   "generator": f"seed {w.seed}, sink {synthetic.SINK_TOKENS} tok x{synthetic.SINK_SCALE}, band "
                                f"{synthetic.BAND_PAIRS} rotary pairs beta {synthetic.BAND_BETA} width "
                                f"{synthetic.BAND_WIDTH}, head gain {synthetic.HEAD_GAIN}"},
        "kept_blocks": kept, "density": round(density, 4), "decisions": hist,
        "layer_tflops_on_kept_blocks": round(layer_tflops, 1),
        "layer_frac_of_bf16_peak": round(layer_tflops / PEAK_BF16_TFLOPS, 4),
        "layer0": {"ms": round(layer0_ms, 3), "decisions": hist0,
                   "density": round(kept0 / tri, 4)},
        "roofline": {"bound": "mfma", "kernel": "sp_attn_fwd_kernel", "achieved": round(attn_tflops, 1),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(attn_tflops / PEAK_BF16_TFLOPS, 4),
                     "avg_launch_ms": round(attn_avg_ms, 3), "launches": len(attn_ms),
                     "traffic": measured_traffic(args.workload, pt)[0],
                     "traffic_note": measured_traffic(args.workload, pt)[1],
                     "sclk_mhz": round(ops.attention_clock_mhz(w.seq_len, w.hkv, w.head_dim, w.block_size, dev))},
    }
    pairing = ops.attention_pairing(w.seq_len, w.hq, w.hkv, w.head_dim, w.block_size, dev)
    line["item_pairing"] = {"head_pairs_by_heads": sum(pairing), "head_pairs_by_rows": len(pairing) - sum(pairing)}

    if not args.no_extras:
        qh, kh, vh = q[0], k[0], v[0]
        stages = {}
        stages["lastq_scores"] = event_ms(lambda: ops.lastq_scores(qh, kh, 128))
        vt, st_, vb, sb = ops.lastq_scores(qh, kh, 128)
        stages["cover_budgets"] = event_ms(lambda: ops.cover_budgets(vt, st_, 128, pt, 8, nb))
        stages["pool_k"] = event_ms(lambda: ops.pool_avg(kh, 128))
        stages["pool_q_all_heads"] = event_ms(lambda: ops.pool_avg(qh, 128))
        kbar = ops.pool_avg(kh, 128)
        stages["queryaware_test"] = event_ms(lambda: ops.queryaware_test(qh, kbar, vb, 128, w.queryaware_threshold))
        ws = ops._workspace("attn_vt", _lib.load().sp_attn_workspace_bytes(w.seq_len, w.hq, w.hkv, w.head_dim, 128), dev)
        lib = _lib.load()
        stages["repack_v"] = event_ms(lambda: lib.sp_attn_repack_v_bf16(
            vh.data_ptr(), w.seq_len, w.hkv, w.head_dim, vh.stride(1), vh.stride(0), 128, ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream().cuda_stream))
        stages["attention"] = attn_avg_ms
        stages["other_selection_and_host"] = max(0.0, ms_per_step - sum(
            stages[x] for x in ("lastq_scores", "cover_budgets", "pool_k", "queryaware_test", "repack_v", "attention")))
        line["stage_ms"] = {a: round(b, 3) for a, b in stages.items()}
        kbytes = w.seq_len * w.hkv * w.head_dim * 2 + nb * w.hkv * w.head_dim * 2
        qbytes = w.seq_len * w.hq * w.head_dim * 2 + nb * w.hq * w.head_dim * 2
        line["pooling"] = {"k_GBps": round(kbytes / stages["pool_k"] / 1e6, 1),
                           "q_GBps": round(qbytes / stages["pool_q_all_heads"] / 1e6, 1),
                           "peak_GBps": PEAK_HBM_GBS,
                           "q_frac": round(qbytes / stages["pool_q_all_heads"] / 1e6 / PEAK_HBM_GBS, 4)}
        # dense causal baseline at the same shape (every lower-triangular block kept)
        dense_mask = torch.tril(torch.ones(nb, nb, dtype=torch.bool, device=dev))
        dense_mask = ops.bool_to_mask(dense_mask).unsqueeze(0).expand(w.hq, -1, -1).contiguous()
        tm = ops.KernelTimer()
        ops.kernel_timer = tm
        for _ in range(2):
            ops.block_sparse_attention(qh, kh, vh, dense_mask, 128, w.head_dim ** -0.5)
        torch.cuda.synchronize()
        ops.kernel_timer = None
        dms = tm.durations_ms("attn")[-1]
        line["dense_causal_baseline"] = {"ms": round(dms, 3), "blocks": tri,
                                         "tflops": round(tri * FLOP_PER_BLOCK / dms / 1e9, 1),
                                         "frac": round(tri * FLOP_PER_BLOCK / dms / 1e9 / PEAK_BF16_TFLOPS, 4)}
        # decode step over the same cache (one query token per head; HBM-bound: K and V read once)
        q1 = qh[:, -1].contiguous()
        dec_ms = event_ms(lambda: ops.decode_attention(q1, kh, vh, w.head_dim ** -0.5), reps=5)
        sdpa_ms = event_ms(lambda: torch.nn.functional.scaled_dot_product_attention(
            q1[None, :, None, :], k, v, scale=w.head_dim ** -0.5, enable_gqa=True), reps=5)
        dec_bytes = 2 * w.seq_len * w.hkv * w.head_dim * 2
        kc, vc = kh.contiguous(), vh.contiguous()  # [Hkv, N, D] contiguous: the layout of a Hugging Face KV cache
        dec_hm_ms = event_ms(lambda: ops.decode_attention(q1, kc, vc, w.head_dim ** -0.5), reps=5)
        line["decode_step"] = {"ms": round(dec_hm_ms, 4), "GBps": round(dec_bytes / dec_hm_ms / 1e6, 1),
                               "frac_of_hbm_peak": round(dec_bytes / dec_hm_ms / 1e6 / PEAK_HBM_GBS, 4),
                               "layout": "k, v [Hkv, N, D] contiguous",
                               "token_major_kv_ms": round(dec_ms, 4), "torch_sdpa_ms": round(sdpa_ms, 4)}
        del kc, vc
        # the step in front of the layer: rotary embedding of q and k, one in-place pass against the model's
        # elementwise evaluation (bytes = q and k read and written once)
        from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
        cs = torch.randn(2, w.seq_len, w.head_dim, device=dev, dtype=torch.float32).clamp_(-1, 1).to(torch.bfloat16)
        rope_bytes = 2 * (w.hq + w.hkv) * w.seq_len * w.head_dim * 2
        qr, kr = q.clone(), k.clone()  # (same strides; the workload's own tensors stay as they are)
        rope_ms = event_ms(lambda: ops.rope_inplace(qr[0], kr[0], cs[0], cs[1]), reps=5)
        stock_rope = getattr(apply_rotary_pos_emb, "_shareprefill_original", apply_rotary_pos_emb)
        with torch.no_grad():
            rope_torch_ms = event_ms(lambda: stock_rope(qr, kr, cs[0][None], cs[1][None]), reps=3)
        line["rope_step"] = {"ms": round(rope_ms, 4), "GBps": round(rope_bytes / rope_ms / 1e6, 1),
                             "frac_of_hbm_peak": round(rope_bytes / rope_ms / 1e6 / PEAK_HBM_GBS, 4),
                             "elementwise_torch_ms": round(rope_torch_ms, 4)}
        del cs, qr, kr
        # what back-to-back MFMAs alone sustain on this chip (power-managed clocks): the practical ceiling
        line["mfma_sustained_tflops"] = {"random_operands_changing_every_instruction": round(ops.mfma_probe_tflops(2), 1),
                                         "random_operands_held_in_registers": round(ops.mfma_probe_tflops(1), 1),
                                         "constant_operands": round(ops.mfma_probe_tflops(0), 1),
                                         "library_gemm_8192_random_data": round(library_gemm_tflops(dev), 1),
                                         "nominal_peak": PEAK_BF16_TFLOPS}
        # the attention kernel against what MFMAs alone sustain on this chip under the same power limit
        sustained = line["mfma_sustained_tflops"]["random_operands_changing_every_instruction"]
        line["mfma_sustained_tflops"]["attention_kernel_over_sustained"] = round(attn_tflops / sustained, 4)
        if not args.no_sweep:
            sweep = []
            for thr in (0.9, 0.95, 0.99):
                prime(thr)
                run_layer(1, thr)
                torch.cuda.synchronize()
                tm = ops.KernelTimer()
                ops.kernel_timer = tm
                t1 = time.perf_counter()
                for _ in range(3):
                    run_layer(1, thr)
                torch.cuda.synchronize()
                ms = (time.perf_counter() - t1) / 3 * 1e3
                ops.kernel_timer = None
                kb = int(ops.mask_row_pointers(sharing.plans[-1].mask)[:, -1].sum())
                ams = sum(tm.durations_ms("attn")) / 3
                sweep.append({"pattern_threshold": thr, "density": round(kb / tri, 4), "layer_ms": round(ms, 3),
                              "attn_ms": round(ams, 3), "attn_tflops": round(kb * FLOP_PER_BLOCK / ams / 1e9, 1),
                              "attn_frac_of_peak": round(kb * FLOP_PER_BLOCK / ams / 1e9 / PEAK_BF16_TFLOPS, 4),
                              "layer_frac_of_peak": round(kb * FLOP_PER_BLOCK / ms / 1e9 / PEAK_BF16_TFLOPS, 4)})
            line["threshold_sweep"] = sweep
            # The regime the method exists for: the reference's minimum mask is 8 vertical + 8 slash blocks per row
            # (attention_sharing.py:169-176), which a pattern_threshold near zero leaves alone (every budget clamps to
            # min_budget); 0.65 gives about a tenth of the blocks with this generator.  Same layer, same inputs.
            line["low_density"] = [timed_layer_point(w, q, k, v, table, thr, steps=5, with_stages=True)
                                   for thr in (0.01, 0.65)]
            # shorter prompts of the same workload (the lengths most of the reference's latency protocol covers,
            # eval/efficiency/latency.py:90-108): its first 16384 and 32768 tokens, and the 32768-token configuration
            line["shorter_prompts"] = [timed_layer_point(w, q, k, v, table, pt, steps=10, n_tokens=t, with_stages=True)
                                       for t in (16384, 32768)]
            w2 = synthetic.WORKLOADS["C2"]
            q2, k2, v2 = synthetic.workload_inputs(w2, device=dev)
            c2 = timed_layer_point(w2, q2, k2, v2, synthetic.random_cluster_table(w2.hq, w2.n_clusters, 2, w2.seed),
                                   w2.pattern_threshold, steps=10, with_stages=True)
            c2["workload"] = "C2: B1 Hq32 Hkv8 D128 N32768 bf16, seed %d" % w2.seed
            line["c2_layer"] = c2
            # the reference's other block sizes (shareprefill_attn.py:509-516) on the same inputs: a compatibility path
            # on the 128-token kernels, timed so that its cost is on record (TFLOP/s counted on the kept fine blocks)
            import dataclasses

            small = []
            for bs in (64, 32, 16):
                wb = dataclasses.replace(w2, block_size=bs)
                pnt = timed_layer_point(wb, q2, k2, v2, synthetic.random_cluster_table(w2.hq, w2.n_clusters, 2, w2.seed),
                                        w2.pattern_threshold, steps=5)
                pnt["block_size"] = bs
                small.append(pnt)
            line["c2_smaller_block_sizes"] = small
            del q2, k2, v2
        line["sharing_layer"] = sharing_layer_variant(args, w, pt, q, k, v, table)

    if not args.no_cpu_baseline:
        mask_bool = ops.mask_to_bool(plan.mask, nb).cpu().numpy()
        line["cpu_baseline"] = cpu_baseline(w, q, k, v, mask_bool, plan.decision.cpu().numpy(), kept, pt)
    else:
        line["cpu_baseline"] = None
    if args.workload == "C3" and not args.no_ttft and not args.no_extras:
        # the metric's third part: end-to-end TTFT of the whole architecture at the same 131072 tokens
        del q, k, v
        ops.release_workspaces()
        torch.cuda.empty_cache()
        targs = argparse.Namespace(**vars(args))
        targs.seq_len, targs.warmup, targs.steps = 131072, 1, 3  # 1 warm-up, mean of 3 timed forwards
        targs.length_sweep = "1024,4096,16384"
        targs.both_rope = True
        targs.fuse_rope = True  # bit-identical to the model's own rotary embedding; the other setting is timed as well
        c4 = c4_line(targs)
        line["ttft"] = {"value": c4["value"], "unit": "s", "steps": c4["steps"], "warmup": c4["warmup"],
                        "tokens_per_s": c4["tokens_per_s"], "mean_block_density": c4["mean_block_density"],
                        "decisions": c4["decisions"], "finite_logits": c4["finite_logits"],
                        "workload": c4["config"]["workload"], "fuse_rope": c4["config"]["fuse_rope"],
                        "other_rope_setting": c4.get("other_rope_setting"),
                        "length_sweep": c4.get("length_sweep")}
    print(json.dumps(line))


if __name__ == "__main__":
    main()

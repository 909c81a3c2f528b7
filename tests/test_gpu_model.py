"""GPU: SharePrefill(...)(model) on a small random-init Hugging Face Llama: the patched model runs prefill through
the HIP path (no N x N mask is built), matches the eager model when the budgets keep every block, and can decode."""

import json

import pytest
import torch

pytestmark = pytest.mark.gpu


def small_llama(layers=2, hq=4, hkv=2, head_dim=128):
    from transformers import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(hidden_size=hq * head_dim, intermediate_size=1024, num_hidden_layers=layers,
                      num_attention_heads=hq, num_key_value_heads=hkv, head_dim=head_dim, vocab_size=512,
                      max_position_embeddings=8192)
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg)


def table(tmp_path, layers, hq):
    t = {"clusters": {"0": [[l, h] for l in range(layers) for h in range(hq // 2)],
                      "1": [[l, h] for l in range(layers) for h in range(hq // 2, hq)]}, "shared_clusters": ["0", "1"]}
    p = tmp_path / "table.json"
    p.write_text(json.dumps(t))
    return str(p)


def test_patched_model_matches_eager_when_every_block_is_kept(gpu_device, tmp_path):
    from shareprefill_amd import SharePrefill

    n = 1024
    ids = torch.randint(0, 512, (1, n), generator=torch.Generator().manual_seed(1)).to(gpu_device)
    ref_model = small_llama().to(gpu_device, torch.bfloat16)
    ref_model.config._attn_implementation = "eager"
    with torch.no_grad():
        ref = ref_model(ids).logits.float()
    model = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), min_budget=8192)(
        small_llama().to(gpu_device, torch.bfloat16))
    with torch.no_grad():
        out = model(ids, use_cache=False).logits.float()
    assert out.shape == ref.shape
    assert (out - ref).abs().max().item() < 0.15 and ((out - ref).abs().mean() / ref.abs().mean()).item() < 2e-2
    hist = model.attention_sharing.decision_histogram()
    # 1024 tokens lie within min_budget: both layers ran on the dense mask without any selection
    assert hist["all_blocks_kept_no_selection"] == 8 and model.attention_sharing.plans == []
    # ... and with that shortcut switched off the selection decides, and keeps every block just the same
    model_full = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), min_budget=8192, dense_short_prompts=False)(
        small_llama().to(gpu_device, torch.bfloat16))
    with torch.no_grad():
        out_full = model_full(ids, use_cache=False).logits.float()
    assert torch.equal(out_full, out)
    hist = model_full.attention_sharing.decision_histogram()
    assert sum(hist.values()) == 8 and hist["dense_pivot"] <= 2  # 2 layers x 4 heads, at most one pivot per cluster
    # a second forward resets the sharing state and gives the same result
    with torch.no_grad():
        out2 = model(ids, use_cache=False).logits.float()
    assert torch.equal(out, out2)


def test_patched_model_sparse_prefill_and_generate(gpu_device, tmp_path):
    from shareprefill_amd import SharePrefill

    model = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), pattern_threshold=0.9, min_budget=256)(
        small_llama().to(gpu_device, torch.bfloat16))
    ids = torch.randint(0, 512, (1, 2048), generator=torch.Generator().manual_seed(2)).to(gpu_device)
    model.attention_sharing.keep_plans = True  # every layer's mask is read below
    with torch.no_grad():
        logits = model(ids, use_cache=False, logits_to_keep=1).logits
    assert logits.shape == (1, 1, 512) and torch.isfinite(logits).all()
    dens = [p.density().cpu() for p in model.attention_sharing.plans]
    assert len(dens) == 2 and all((d > 0).all() and (d <= 1).all() for d in dens)
    with torch.no_grad():
        gen = model.generate(ids[:, :300], max_new_tokens=4, do_sample=False)
    assert gen.shape == (1, 304)


def test_patched_model_with_head_dim_64(gpu_device, tmp_path):
    """Llama-3.2-1B-style heads (head_dim 64, one of the reference's head sizes, shareprefill_attn.py:503-508): prefill
    with every block kept matches the eager model, a sparse prefill runs the selection, and decode works."""
    from shareprefill_amd import SharePrefill

    ids = torch.randint(0, 512, (1, 1536), generator=torch.Generator().manual_seed(6)).to(gpu_device)
    ref_model = small_llama(head_dim=64).to(gpu_device, torch.bfloat16)
    ref_model.config._attn_implementation = "eager"
    with torch.no_grad():
        ref = ref_model(ids).logits.float()
    model = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), min_budget=8192, dense_short_prompts=False)(
        small_llama(head_dim=64).to(gpu_device, torch.bfloat16))
    with torch.no_grad():
        out = model(ids, use_cache=False).logits.float()
    assert (out - ref).abs().max().item() < 0.15 and ((out - ref).abs().mean() / ref.abs().mean()).item() < 2e-2
    assert sum(model.attention_sharing.decision_histogram().values()) == 8
    sparse = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), pattern_threshold=0.9, min_budget=256)(
        small_llama(head_dim=64).to(gpu_device, torch.bfloat16))
    with torch.no_grad():
        logits = sparse(ids, use_cache=False, logits_to_keep=1).logits
        gen = sparse.generate(ids[:, :300], max_new_tokens=3, do_sample=False)
        want = ref_model.generate(ids[:, :300], max_new_tokens=3, do_sample=False)
    assert torch.isfinite(logits).all() and gen.shape == (1, 303)
    # 300 tokens lie within the minimum budget (dense prefill), decode is dense: the greedy tokens are the eager model's
    assert torch.equal(gen, want)


@pytest.mark.parametrize("block_size,head_dim", [(64, 128), (32, 128), (16, 64)])
def test_patched_model_with_smaller_block_sizes(gpu_device, tmp_path, block_size, head_dim):
    """block_size 64 / 32 / 16 through SharePrefill(...)(model) (shareprefill_configurations.py:37,
    shareprefill_attn.py:509-516), the last together with a head_dim of 64: with budgets that keep every block the
    patched model matches the eager one; with sparse budgets the selection runs on the finer grid, and the dense
    short-prompt shortcut and decode work."""
    from shareprefill_amd import SharePrefill

    ids = torch.randint(0, 512, (1, 1100), generator=torch.Generator().manual_seed(block_size)).to(gpu_device)
    ref_model = small_llama(head_dim=head_dim).to(gpu_device, torch.bfloat16)
    ref_model.config._attn_implementation = "eager"
    with torch.no_grad():
        ref = ref_model(ids).logits.float()
    for shortcut in (True, False):
        model = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), min_budget=8192, block_size=block_size,
                             dense_short_prompts=shortcut)(small_llama(head_dim=head_dim).to(gpu_device, torch.bfloat16))
        with torch.no_grad():
            out = model(ids, use_cache=False).logits.float()
        assert (out - ref).abs().max().item() < 0.15 and ((out - ref).abs().mean() / ref.abs().mean()).item() < 2e-2
    assert sum(model.attention_sharing.decision_histogram().values()) == 8
    sparse = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), pattern_threshold=0.9, min_budget=2 * block_size,
                          block_size=block_size)(small_llama(head_dim=head_dim).to(gpu_device, torch.bfloat16))
    sparse.attention_sharing.keep_plans = True
    with torch.no_grad():
        logits = sparse(ids, use_cache=False, logits_to_keep=1).logits
    assert torch.isfinite(logits).all()
    nb = -(-1100 // block_size)
    plans = sparse.attention_sharing.plans
    assert len(plans) == 2 and all(p.mask.shape[1] == nb for p in plans)
    assert all((p.density().cpu() < 1).any() for p in plans)
    with torch.no_grad():
        gen = sparse.generate(ids[:, :block_size + 5], max_new_tokens=3, do_sample=False)
    assert gen.shape == (1, block_size + 8)


def test_patched_qwen2_model_prefill_and_generate(gpu_device, tmp_path):
    """The patch is model-agnostic (any module with ALL_ATTENTION_FUNCTIONS): Qwen2's attention layer passes
    sliding_window=None for its full-attention layers and has q/k/v biases."""
    from transformers import Qwen2Config, Qwen2ForCausalLM

    from shareprefill_amd import SharePrefill

    cfg = Qwen2Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=512, max_position_embeddings=8192, use_sliding_window=False)
    torch.manual_seed(0)
    ref_model = Qwen2ForCausalLM(cfg).to(gpu_device, torch.bfloat16)
    ref_model.config._attn_implementation = "eager"
    ids = torch.randint(0, 512, (1, 1024), generator=torch.Generator().manual_seed(4)).to(gpu_device)
    with torch.no_grad():
        ref = ref_model(ids).logits.float()
    torch.manual_seed(0)
    model = SharePrefill(sharing_lookup_path=table(tmp_path, 2, 4), min_budget=8192, fuse_rope=True)(
        Qwen2ForCausalLM(cfg).to(gpu_device, torch.bfloat16))
    from transformers.models.qwen2 import modeling_qwen2
    try:
        with torch.no_grad():
            out = model(ids, use_cache=False).logits.float()
            gen = model.generate(ids[:, :200], max_new_tokens=3, do_sample=False)
    finally:
        stock = getattr(modeling_qwen2.apply_rotary_pos_emb, "_shareprefill_original", None)
        if stock is not None:
            modeling_qwen2.apply_rotary_pos_emb = stock
    assert (out - ref).abs().max().item() < 0.15 and ((out - ref).abs().mean() / ref.abs().mean()).item() < 2e-2
    assert gen.shape == (1, 203)


def test_llama31_8b_architecture_at_131072_tokens(gpu_device):
    """The end-to-end configuration of the benchmark at its real layer shape and length: Llama-3.1-8B architecture
    (hidden 4096, Hq32 Hkv8 head_dim 128, intermediate 14336, RoPE theta 5e5, vocab 128256, random-init bf16) cut to
    two decoder layers, 131072 uniform-random token ids, patched with the shipped Llama-3.1-8B-Instruct table.
      * budgets that keep every block: the last-token logits must match the stock model's (torch SDPA) -- the patch,
        the strided q/k/v hand-over, the fused rotary pass and the attention kernel at 1024 key blocks, end to end;
      * the benchmark's thresholds: finite logits, every head of both layers decided, density within (0, 1]."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from shareprefill_amd import SharePrefill, unpatch_model

    n = 131072
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=2, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=128256, max_position_embeddings=n,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0}, rms_norm_eps=1e-5,
                      tie_word_embeddings=False)
    torch.manual_seed(1238)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(gpu_device):
            model = LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    model.eval()
    gen = torch.Generator(device=gpu_device).manual_seed(1238)
    ids = torch.randint(0, cfg.vocab_size, (1, n), generator=gen, device=gpu_device)
    print("C4-shaped model test: stock SDPA forward", flush=True)
    model.config._attn_implementation = "sdpa"
    with torch.no_grad():
        ref = model(ids, use_cache=False, logits_to_keep=1).logits.float()
    print("C4-shaped model test: patched forward, every block kept", flush=True)
    SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct", pattern_threshold=0.95, min_budget=n, fuse_rope=True,
                 dense_short_prompts=False)(model)
    from transformers.models.llama import modeling_llama
    try:
        with torch.no_grad():
            out = model(ids, use_cache=False, logits_to_keep=1).logits.float()
        assert out.shape == ref.shape == (1, 1, cfg.vocab_size)
        assert torch.isfinite(out).all()
        # two layers of bf16 arithmetic in a different summation order
        assert (out - ref).abs().max().item() < 0.1 and ((out - ref).abs().mean() / ref.abs().mean()).item() < 2e-2
        hist = model.attention_sharing.decision_histogram()
        assert sum(hist.values()) == 64
        print("C4-shaped model test: patched forward, benchmark thresholds", flush=True)
        unpatch_model(model)
        SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct", pattern_threshold=0.95, similarity_threshold=0.5,
                     fallback_threshold=0.95, block_size=128, min_budget=1024)(model)
        model.attention_sharing.keep_plans = True
        with torch.no_grad():
            out2 = model(ids, use_cache=False, logits_to_keep=1).logits.float()
        assert torch.isfinite(out2).all()
        hist = model.attention_sharing.decision_histogram()
        assert sum(hist.values()) == 64
        dens = [p.density().cpu() for p in model.attention_sharing.plans]
        assert len(dens) == 2 and all((d > 0).all() and (d <= 1).all() for d in dens)
    finally:
        stock = getattr(modeling_llama.apply_rotary_pos_emb, "_shareprefill_original", None)
        if stock is not None:
            modeling_llama.apply_rotary_pos_emb = stock


def test_llama31_8b_architecture_all_32_layers_at_131072_tokens(gpu_device):
    """The end-to-end configuration as stated: the whole Llama-3.1-8B architecture (32 layers, hidden 4096, Hq32 Hkv8,
    head_dim 128, intermediate 14336, RoPE theta 5e5, vocab 128256, random-init bf16, 16 GB of weights), 131072
    uniform-random token ids, SharePrefill in every layer with the shipped Llama-3.1-8B-Instruct table (44 clusters,
    one shared, its members in layers 14 to 30) and the thresholds of the reference's latency script
    (eval/efficiency/run_latency.sh:12).  One prefill forward: finite last-token logits, all 32 x 32 heads decided,
    every layer's block density within (0, 1], and a second forward (state reset in between) gives the same logits
    bit for bit."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from shareprefill_amd import SharePrefill

    n = 131072
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=128256, max_position_embeddings=n,
                      rope_parameters={"rope_type": "default", "rope_theta": 500000.0}, rms_norm_eps=1e-5,
                      tie_word_embeddings=False)
    torch.manual_seed(1238)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(gpu_device):
            model = LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    model.eval()
    gen = torch.Generator(device=gpu_device).manual_seed(1238)
    ids = torch.randint(0, cfg.vocab_size, (1, n), generator=gen, device=gpu_device)
    SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct", pattern_threshold=0.95, similarity_threshold=0.5,
                 fallback_threshold=0.95, block_size=128, min_budget=1024)(model)
    sharing = model.attention_sharing
    assert len(sharing.clusters) == 44 and len(sharing._slot) == 1
    sharing.keep_plans = True
    print("C4 test: 32-layer patched forward", flush=True)
    with torch.no_grad():
        out = model(ids, use_cache=False, logits_to_keep=1).logits.float()
    assert out.shape == (1, 1, cfg.vocab_size) and torch.isfinite(out).all()
    assert [p.layer_idx for p in sharing.plans] == list(range(32))
    hist = sharing.decision_histogram()
    assert sum(hist.values()) == 1024
    for p in sharing.plans:
        d = p.density().cpu()
        assert d.shape == (32,) and (d > 0).all() and (d <= 1).all()
        assert int(p.decision.min()) >= 0 and int(p.decision.max()) <= 3
    # heads outside the one shared cluster can neither become pivots nor share
    members = {(l, h) for l, h in sharing.clusters["9"]}
    for p in sharing.plans:
        for h in torch.nonzero((p.decision == 1) | (p.decision == 2)).reshape(-1).cpu().tolist():
            assert (p.layer_idx, h) in members
    print("C4 test: second forward", flush=True)
    sharing.keep_plans = False
    with torch.no_grad():
        out2 = model(ids, use_cache=False, logits_to_keep=1).logits.float()
    assert torch.equal(out, out2)
    assert len(sharing.plans) == 32

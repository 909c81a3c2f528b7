"""GPU: sp_rope_inplace_bf16 through the C ABI against the oracle (bit-exact), against the Hugging Face elementwise
evaluation on the same device (bit-exact), at the benchmark's full size, and inside a patched model."""

import json

import pytest
import torch

from oracle import shareprefill_oracle as O

pytestmark = pytest.mark.gpu


def tables(n, d, device, theta=500000.0, offset=0):
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = (torch.arange(n, dtype=torch.float32) + offset)[:, None] * inv[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    return emb.cos().to(torch.bfloat16).to(device), emb.sin().to(torch.bfloat16).to(device)


@pytest.mark.parametrize("hq,hkv,n,d", [(4, 2, 1, 128), (8, 2, 77, 128), (3, 1, 513, 64), (32, 8, 2050, 128),
                                        (2, 2, 130, 16), (5, 0, 9, 128), (0, 3, 9, 32)])
def test_matches_oracle_bit_exact_on_projection_layout(gpu_device, hq, hkv, n, d):
    from shareprefill_amd import ops

    g = torch.Generator().manual_seed(100 + n)
    # the layout the attention layer hands over: one [N, (Hq + 2 Hkv) * D] projection viewed per head
    proj = (torch.randn(n, (hq + hkv) * d + 16, generator=g) * 2.5).to(torch.bfloat16)
    qv = proj[:, : hq * d].view(n, hq, d).transpose(0, 1)
    kv = proj[:, hq * d: (hq + hkv) * d].view(n, hkv, d).transpose(0, 1)
    cos, sin = tables(n, d, "cpu")
    want_q, want_k = O.rope_rotate(qv, cos, sin), O.rope_rotate(kv, cos, sin)
    dev = proj.to(gpu_device)
    q = dev[:, : hq * d].view(n, hq, d).transpose(0, 1)
    k = dev[:, hq * d: (hq + hkv) * d].view(n, hkv, d).transpose(0, 1)
    ops.rope_inplace(q, k, cos.to(gpu_device), sin.to(gpu_device))
    assert torch.equal(q.cpu(), want_q) and torch.equal(k.cpu(), want_k)
    assert torch.equal(dev[:, (hq + hkv) * d:].cpu(), proj[:, (hq + hkv) * d:])  # nothing else was touched


def test_special_values_and_argument_checks(gpu_device):
    from shareprefill_amd import ops

    n, d = 40, 128
    x = torch.zeros(2, n, d, dtype=torch.bfloat16)
    x[0, :, 0] = float("inf")
    x[0, :, 1] = -0.0
    x[0, :, 2] = 1e-38   # bf16 subnormal range: the products stay exact in fp32
    x[1, :, 70] = 3.0e38
    x[1, :, 5] = -2.5
    cos, sin = tables(n, d, "cpu", offset=1000)
    want = O.rope_rotate(x, cos, sin)
    q = x.to(gpu_device)
    k = x[:1].to(gpu_device).clone()
    ops.rope_inplace(q, k, cos.to(gpu_device), sin.to(gpu_device))
    got = q.cpu()
    finite = torch.isfinite(want.float())
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float()))
    assert torch.equal(got[finite].view(torch.int16), want[finite].view(torch.int16))  # signed zeros included
    with pytest.raises(ValueError):
        ops.rope_inplace(q, k, cos.to(gpu_device)[:, :64], sin.to(gpu_device)[:, :64])
    with pytest.raises(ValueError):
        ops.rope_inplace(q, k[:, :-1], cos.to(gpu_device), sin.to(gpu_device))
    with pytest.raises(AssertionError):
        ops.rope_inplace(q.float(), k, cos.to(gpu_device), sin.to(gpu_device))
    bad = torch.zeros(2, n, 24, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(NotImplementedError):
        ops.rope_inplace(bad, bad.clone(), torch.zeros(n, 24, dtype=torch.bfloat16, device=gpu_device),
                         torch.zeros(n, 24, dtype=torch.bfloat16, device=gpu_device))


def test_full_size_equals_the_elementwise_evaluation_on_the_device(gpu_device):
    """C3 shapes (Hq32 Hkv8 D128 N131072): the one-pass kernel against transformers' apply_rotary_pos_emb run on the
    same GPU, bit for bit; a second application with the negated angle returns the input within the roundings."""
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    from shareprefill_amd import ops

    hq, hkv, n, d = 32, 8, 131072, 128
    g = torch.Generator(device=gpu_device).manual_seed(5)
    proj = torch.randn(n, (hq + hkv) * d, device=gpu_device, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q = proj[:, : hq * d].view(1, n, hq, d).transpose(1, 2)
    k = proj[:, hq * d:].view(1, n, hkv, d).transpose(1, 2)
    cos, sin = tables(n, d, gpu_device)
    rope = getattr(apply_rotary_pos_emb, "_shareprefill_original", apply_rotary_pos_emb)
    want_q, want_k = rope(q, k, cos[None], sin[None])
    keep = proj.clone()
    ops.rope_inplace(q[0], k[0], cos, sin)
    assert torch.equal(q, want_q) and torch.equal(k, want_k)
    del want_q, want_k
    ops.rope_inplace(q[0], k[0], cos, -sin)
    err = (proj.float() - keep.float()).abs()
    assert err.max().item() <= 2.0 ** -5 * keep.float().abs().max().item()
    assert (err.mean() / keep.float().abs().mean()).item() < 1e-2


def test_patched_model_with_fused_rope_gives_identical_logits(gpu_device, tmp_path):
    from transformers import LlamaConfig, LlamaForCausalLM
    from transformers.models.llama import modeling_llama

    from shareprefill_amd import SharePrefill

    def build():
        cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                          num_key_value_heads=2, head_dim=128, vocab_size=512, max_position_embeddings=8192)
        torch.manual_seed(0)
        return LlamaForCausalLM(cfg).to(gpu_device, torch.bfloat16)

    t = {"clusters": {"0": [[l, h] for l in range(2) for h in range(2)],
                      "1": [[l, h] for l in range(2) for h in range(2, 4)]}, "shared_clusters": ["0", "1"]}
    path = tmp_path / "table.json"
    path.write_text(json.dumps(t))
    ids = torch.randint(0, 512, (1, 1500), generator=torch.Generator().manual_seed(3)).to(gpu_device)
    stock = modeling_llama.apply_rotary_pos_emb
    assert not hasattr(stock, "_shareprefill_original")
    try:
        plain = SharePrefill(sharing_lookup_path=str(path), min_budget=256)(build())
        with torch.no_grad():
            ref = plain(ids, use_cache=False).logits
        fused = SharePrefill(sharing_lookup_path=str(path), min_budget=256, fuse_rope=True)(build())
        assert modeling_llama.apply_rotary_pos_emb._shareprefill_original is stock
        with torch.no_grad():
            out = fused(ids, use_cache=False).logits
            gen = fused.generate(ids[:, :200], max_new_tokens=3, do_sample=False)
        assert torch.equal(out, ref)
        assert gen.shape == (1, 203)
        # with autograd on, the in-place path must not be taken (the projection output is needed for backward)
        q = torch.randn(1, 2, 8, 128, device=gpu_device, dtype=torch.bfloat16, requires_grad=True)
        cos, sin = tables(8, 128, gpu_device)
        q2, _ = modeling_llama.apply_rotary_pos_emb(q, q, cos[None], sin[None])
        assert q2 is not q and q2.requires_grad
    finally:
        modeling_llama.apply_rotary_pos_emb = stock

"""CPU-only checks: the C-ABI library loads and exports every symbol the header declares, the ctypes
signatures cover the header, host-side configuration / table loading / patching behave like the reference's
(shareprefill/shareprefill_patch.py, shareprefill_configurations.py, attn/attention_sharing.py:368-384)."""

import ctypes
import json
import os
import re
import types

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "shareprefill_hip.h")
DIAG_HEADER = os.path.join(ROOT, "include", "shareprefill_hip_diag.h")  # measurement aids, not the drop-in boundary


def header_functions(paths=(HEADER, DIAG_HEADER)):
    names = set()
    for path in paths:
        text = re.sub(r"/\*.*?\*/", "", open(path).read(), flags=re.S)
        names |= set(re.findall(r"\b(sp_[a-z0-9_]+)\s*\(", text))
    return sorted(names - {"sp_cluster_state"})


def test_library_exports_every_declared_symbol():
    from shareprefill_amd import _lib

    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m shareprefill_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = header_functions()
    assert len(names) >= 19
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes signature table and header disagree"
    # the measurement aids live in a header of their own: the boundary header declares none of them
    diag = {"sp_diag_mfma_bf16", "sp_diag_mfma_flops", "sp_attn_last_launch_clocks", "sp_attn_last_launch_pairing"}
    assert set(header_functions((DIAG_HEADER,))) == diag
    assert not diag & set(header_functions((HEADER,)))


def test_library_identity_and_error_string():
    from shareprefill_amd import _lib

    lib = _lib.load()
    assert lib.sp_version() >= 1
    assert lib.sp_arch() == b"gfx950"
    # argument validation happens on the host before any GPU call: usable without a GPU
    st = lib.sp_pool_avg_bf16(None, None, 128, 1, 128, 128, 128, 128, 0, None, None)
    assert st == -1 and b"null" in lib.sp_last_error()
    with pytest.raises(ValueError):
        _lib.check(st, "sp_pool_avg_bf16")
    # 1024 key tiles in chunks of 32 (the launch's own chunking at this size) + the folded row statistics
    assert lib.sp_lastq_scores_workspace_bytes(131072, 32, 128) == (32 * 32 * 128 + 32 * 128) * 8
    assert lib.sp_lastq_scores_workspace_bytes(4096, 32, 128) == (32 * 16 * 128 + 32 * 128) * 8  # two tiles per chunk
    assert lib.sp_attn_workspace_bytes(131072, 32, 8, 128, 128) == 8 * 131072 * 128 * 2 + 3072 + 32 * 131072 * 8


def test_cluster_state_struct_matches_header_layout():
    from shareprefill_amd._lib import ClusterStateStruct

    assert ctypes.sizeof(ClusterStateStruct) == 16 + 9 * 8
    assert [f[0] for f in ClusterStateStruct._fields_][4:] == ["info", "ratio", "vert", "slash", "cols", "dists",
                                                              "pattern", "accum", "avg_map"]
    # the header declares the same members in the same order
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "shareprefill_hip.h")).read()
    body = header[header.index("typedef struct sp_cluster_state {"):header.index("} sp_cluster_state;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = re.findall(r"(\w+);", body)
    assert names == [f[0] for f in ClusterStateStruct._fields_]


def test_cluster_state_struct_size_guards_the_members_added_later():
    """struct_bytes tells the library which layout the caller was compiled against: the first one ended with `accum`
    (80 bytes), so avg_map is read only from a struct that declares itself long enough; any other size is refused
    (argument checks run on the host, before any GPU call)."""
    from shareprefill_amd import _lib
    from shareprefill_amd._lib import ClusterStateStruct

    lib = _lib.load()
    assert ctypes.sizeof(ClusterStateStruct) == 88
    header = open(HEADER).read()
    assert "#define SP_CLUSTER_STATE_V1_BYTES 80" in header
    one = ctypes.c_void_p(16)  # never dereferenced: the calls below fail their checks before any launch
    for size, ok in ((0, True), (80, True), (88, True), (96, True), (84, False), (40, False), (-1, False)):
        st = ClusterStateStruct(1, 4, 1, size, one, one, one, one, one, one, one, one, None)
        rc = lib.sp_pivot_update(ctypes.byref(st), None, None, None, 1, 4, 0.9, None)
        msg = lib.sp_last_error()
        assert rc == -1
        assert (b"struct_bytes" not in msg) == ok, (size, msg)


def test_queryaware_selection_score_is_the_double_product_taken_to_fp32():
    """attention_sharing.py:361 forms pattern_threshold * num_blocks from the Python float (double) and utils.py:56
    compares the fp32 running sums with it, i.e. with fp32(double(pt) * nb).  The entry point takes the threshold as a
    double and must form exactly that value -- for every block count the kernels accept.  Rounding the threshold to
    fp32 first (what a `float` argument does) gives another value for hundreds of block counts: the negative control."""
    import numpy as np

    from shareprefill_amd import _lib

    lib = _lib.load()
    for pt in (0.5, 0.9, 0.95, 0.99, 0.999, 0.1, 1.0 / 3.0):
        differs_when_rounded_first = 0
        for nb in range(1, 4097):
            want = float(np.float32(pt * nb))
            assert lib.sp_queryaware_select_score(pt, nb) == want, (pt, nb)
            differs_when_rounded_first += float(np.float32(float(np.float32(pt)) * nb)) != want
        if pt in (0.9, 0.95, 0.99):
            assert differs_when_rounded_first > 400  # 1326 / 818 / 497 of 4096
    # the binding hands the Python float over unrounded
    assert _lib.SIGNATURES["sp_queryaware_select_bf16"][1][8] is ctypes.c_double


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from shareprefill_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    with pytest.raises(_lib.SharePrefillLibraryError, match="no CPU fallback"):
        _lib.load(str(tmp_path / "missing.so"))
    monkeypatch.setattr(_lib, "_lib", None)


def test_cpu_tensors_are_rejected_not_silently_computed():
    from shareprefill_amd import ops

    x = torch.zeros(2, 256, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU"):
        ops.pool_avg(x, 128)


# ---- configuration ---------------------------------------------------------------------------------
def test_config_defaults_and_registry():
    from shareprefill_amd import SharePrefillConfig

    c = SharePrefillConfig(model_name="meta-llama/Llama-3.1-8B-Instruct")
    assert (c.pattern_threshold, c.similarity_threshold, c.fallback_threshold, c.queryaware_threshold) == (
        0.9, 0.5, 0.9, 0.1)
    assert (c.block_size, c.min_budget, c.max_budget) == (128, 1024, None)
    assert c.sharing_lookup_path.endswith("Llama-3.1-8B-Instruct_code_debug_hiera-40.0-2.json")
    assert os.path.exists(c.sharing_lookup_path)
    with pytest.raises(AssertionError):
        SharePrefillConfig(model_name="org/unknown-model")
    with pytest.raises(AssertionError):
        SharePrefillConfig(attn_type="other", model_name="x")
    with pytest.raises(AssertionError):
        SharePrefillConfig()
    assert SharePrefillConfig(sharing_lookup_path="/x/y.json").sharing_lookup_path == "/x/y.json"


def test_shipped_table_properties():
    from shareprefill_amd import AttentionSharing, SharePrefillConfig

    path = SharePrefillConfig(model_name="Llama-3.1-8B-Instruct").sharing_lookup_path
    clusters, shared = AttentionSharing.load_clusters(path)
    pairs = [tuple(p) for v in clusters.values() for p in v]
    assert len(clusters) == 44 and len(pairs) == 1024 and len(set(pairs)) == 1024
    assert shared == {"9"} and len(clusters["9"]) == 42
    assert {l for l, _ in clusters["9"]} <= set(range(14, 31))
    sh = AttentionSharing(path)
    for cid, v in clusters.items():
        for layer, head in v[:3]:
            assert sh.find_cluster_id(layer, head) == cid
    assert sh.find_cluster_id(99, 0) is None


def test_table_loader_errors(tmp_path):
    from shareprefill_amd import AttentionSharing

    with pytest.raises(FileNotFoundError):
        AttentionSharing(str(tmp_path / "nope.json"))
    bad = tmp_path / "bad.json"
    bad.write_text(json.dumps({"clusters": {}}))
    with pytest.raises(ValueError):
        AttentionSharing(str(bad))


def test_budget_conversion():
    from shareprefill_amd.attention_sharing import budget_blocks

    assert budget_blocks(1024, None, 128) == (8, (2 ** 31 - 1 + 127) // 128)
    assert budget_blocks(None, 1000, 128) == (1, 8)
    assert budget_blocks(129, 4096, 128) == (2, 32)


# ---- patching a Hugging Face model -------------------------------------------------------------------
def tiny_llama():
    from transformers import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                      num_key_value_heads=1, head_dim=128, vocab_size=128, max_position_embeddings=4096)
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg)


def tiny_table(tmp_path):
    t = {"clusters": {"0": [[0, 0], [1, 0]], "1": [[0, 1], [1, 1]]}, "shared_clusters": ["0"]}
    p = tmp_path / "table.json"
    p.write_text(json.dumps(t))
    return str(p)


def test_patch_installs_reference_hooks(tmp_path):
    from shareprefill_amd import AttentionSharing, SharePrefill, shareprefill_attention_forward
    from transformers.models.llama import modeling_llama

    model = tiny_llama()
    patched = SharePrefill(sharing_lookup_path=tiny_table(tmp_path), pattern_threshold=0.95, min_budget=256)(model)
    assert patched is model
    assert model.config._attn_implementation == "shareprefill"
    assert modeling_llama.ALL_ATTENTION_FUNCTIONS["shareprefill"] is shareprefill_attention_forward
    assert isinstance(model.attention_sharing, AttentionSharing)
    assert callable(model.reset_attention_sharing) and callable(model._init_attention_sharing)
    # thresholds are pushed onto the shared HF config, every attention module sees the same state object
    assert model.config.pattern_threshold == 0.95 and model.config.min_budget == 256 and model.config.block_size == 128
    for layer in model.model.layers:
        assert layer.self_attn.attention_sharing is model.attention_sharing
        assert layer.self_attn.config is model.config


def test_patched_forward_resets_state_and_has_no_cpu_path(tmp_path):
    from shareprefill_amd import SharePrefill

    model = SharePrefill(sharing_lookup_path=tiny_table(tmp_path))(tiny_llama()).to(torch.bfloat16)
    calls = []
    orig = model.attention_sharing.reset_state
    model.attention_sharing.reset_state = lambda: (calls.append(1), orig())[1]
    ids = torch.randint(0, 128, (1, 256))
    # the attention function reaches the HIP ops, which refuse CPU tensors: no silent fallback
    with pytest.raises(ValueError, match="GPU"):
        model(ids)
    assert len(calls) == 1


def test_fuse_rope_replaces_the_module_function_and_leaves_other_calls_alone(tmp_path):
    """fuse_rope=True swaps the model module's apply_rotary_pos_emb for a wrapper that takes the in-place HIP pass
    only for bf16 GPU tensors without autograd; CPU / fp32 / autograd calls get the original function's result."""
    from shareprefill_amd import SharePrefill
    from transformers.models.llama import modeling_llama

    stock = modeling_llama.apply_rotary_pos_emb
    try:
        SharePrefill(sharing_lookup_path=tiny_table(tmp_path))(tiny_llama())
        assert modeling_llama.apply_rotary_pos_emb is stock  # off by default
        SharePrefill(sharing_lookup_path=tiny_table(tmp_path), fuse_rope=True)(tiny_llama())
        wrapped = modeling_llama.apply_rotary_pos_emb
        assert wrapped is not stock and wrapped._shareprefill_original is stock
        SharePrefill(sharing_lookup_path=tiny_table(tmp_path), fuse_rope=True)(tiny_llama())
        assert modeling_llama.apply_rotary_pos_emb is wrapped  # not wrapped twice
        g = torch.Generator().manual_seed(0)
        q, k = torch.randn(1, 4, 9, 32, generator=g), torch.randn(1, 2, 9, 32, generator=g)
        cos, sin = torch.randn(1, 9, 32, generator=g), torch.randn(1, 9, 32, generator=g)
        for cast in (torch.float32, torch.bfloat16):
            a = wrapped(q.to(cast), k.to(cast), cos.to(cast), sin.to(cast))
            b = stock(q.to(cast), k.to(cast), cos.to(cast), sin.to(cast))
            assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        qg = q.clone().requires_grad_(True)
        out, _ = wrapped(qg, k, cos, sin)
        assert out.requires_grad and out is not qg
    finally:
        modeling_llama.apply_rotary_pos_emb = stock


def test_patch_rejects_unsupported_models_and_types(tmp_path):
    from shareprefill_amd import SharePrefill

    with pytest.raises(TypeError):
        SharePrefill(sharing_lookup_path=tiny_table(tmp_path))(torch.nn.Linear(2, 2))
    sp = SharePrefill(sharing_lookup_path=tiny_table(tmp_path))
    sp.config.attn_type = "flash"
    with pytest.raises(ValueError):
        sp(tiny_llama())


def test_attention_forward_argument_errors(tmp_path):
    from shareprefill_amd import AttentionSharing, shareprefill_attention_forward

    cfg = types.SimpleNamespace(block_size=128, min_budget=1024, max_budget=None, pattern_threshold=0.9,
                                similarity_threshold=0.5, fallback_threshold=0.9, queryaware_threshold=0.1)
    mod = types.SimpleNamespace(config=cfg, attention_sharing=AttentionSharing(tiny_table(tmp_path)), layer_idx=0,
                                scaling=0.1)
    q = torch.zeros(1, 2, 256, 128, dtype=torch.bfloat16)
    k = torch.zeros(1, 1, 256, 128, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        shareprefill_attention_forward(mod, q, k, k, None, scaling=0.1, sliding_window=128)
    with pytest.raises(ValueError):  # gqa_interleave is accepted (it changes nothing, as in the reference): batch 2 is what fails
        shareprefill_attention_forward(mod, q.expand(2, -1, -1, -1), k.expand(2, -1, -1, -1), k.expand(2, -1, -1, -1),
                                       None, scaling=0.1, gqa_interleave=True)
    with pytest.raises(ValueError):
        shareprefill_attention_forward(mod, q.expand(2, -1, -1, -1), k.expand(2, -1, -1, -1), k.expand(2, -1, -1, -1),
                                       None, scaling=0.1)
    with pytest.raises(AssertionError):
        shareprefill_attention_forward(mod, q.float(), k.float(), k.float(), None, scaling=0.1)
    with pytest.raises(AssertionError):
        shareprefill_attention_forward(mod, q, k[:, :, :128], k[:, :, :128], None, scaling=0.1)


def test_synthetic_tables_and_generator_are_seeded():
    from shareprefill_amd import synthetic

    a = synthetic.random_cluster_table(32, 8, 2, 5)
    assert a == synthetic.random_cluster_table(32, 8, 2, 5)
    assert sorted(h for c in a["clusters"].values() for l, h in c if l == 0) == list(range(32))
    q1, k1, v1 = synthetic.planted_qkv(4, 2, 512, 128, 3)
    q2, _, _ = synthetic.planted_qkv(4, 2, 512, 128, 3)
    assert torch.equal(q1, q2) and q1.shape == (1, 4, 512, 128) and q1.stride(3) == 1 and q1.stride(1) == 128


def test_reference_import_name_resolves_to_this_package():
    """`from shareprefill import SharePrefill` (shareprefill/__init__.py:15-17 of the reference) and the reference's
    module paths give the classes of this package."""
    import shareprefill
    import shareprefill_amd
    from shareprefill import SharePrefill, SharePrefillConfig
    from shareprefill.attn.attention_sharing import AttentionSharing
    from shareprefill.attn.shareprefill_attn import shareprefill_attention_forward
    from shareprefill.shareprefill_patch import shareprefill_patch

    assert SharePrefill is shareprefill_amd.SharePrefill and SharePrefillConfig is shareprefill_amd.SharePrefillConfig
    assert AttentionSharing is shareprefill_amd.AttentionSharing
    assert shareprefill_attention_forward is shareprefill_amd.shareprefill_attention_forward
    assert callable(shareprefill_patch) and shareprefill.attn.AttentionSharing is AttentionSharing


def test_unpatch_restores_the_model(tmp_path):
    from shareprefill_amd import SharePrefill, unpatch_model

    model = tiny_llama()
    before_impl = model.config._attn_implementation
    before_forward = model.forward.__func__
    SharePrefill(sharing_lookup_path=tiny_table(tmp_path), fuse_rope=True)(model)
    assert model.config._attn_implementation == "shareprefill" and model.forward.__func__ is not before_forward
    from transformers.models.llama import modeling_llama
    try:
        assert unpatch_model(model) is model
        assert model.config._attn_implementation == before_impl
        assert model.forward.__func__ is before_forward
        assert not hasattr(model.model.layers[0].self_attn, "attention_sharing")
        ids = torch.randint(0, 128, (1, 16))
        assert model(ids).logits.shape == (1, 16, 128)  # runs on the CPU again: nothing of the patch is left
        unpatch_model(model)  # a second call is a no-op
    finally:
        stock = getattr(modeling_llama.apply_rotary_pos_emb, "_shareprefill_original", None)
        if stock is not None:
            modeling_llama.apply_rotary_pos_emb = stock


def test_fused_rope_is_taken_only_inside_a_patched_forward(tmp_path, monkeypatch):
    """The module-level wrapper that fuse_rope=True installs hands every call to the stock function unless a forward
    of a model patched with fuse_rope=True is on the stack: unpatched models of the architecture are not affected,
    and call forms the wrapper does not know (keywords, extra arguments) go to the stock function as they are."""
    from shareprefill_amd import SharePrefill, ops, shareprefill_patch as sp
    from transformers.models.llama import modeling_llama

    stock = modeling_llama.apply_rotary_pos_emb
    calls = []
    monkeypatch.setattr(ops, "rope_inplace", lambda *a: calls.append(a))
    try:
        model = SharePrefill(sharing_lookup_path=tiny_table(tmp_path), fuse_rope=True)(tiny_llama())
        wrapped = modeling_llama.apply_rotary_pos_emb
        g = torch.Generator().manual_seed(0)
        q, k = torch.randn(1, 4, 9, 32, generator=g), torch.randn(1, 2, 9, 32, generator=g)
        cos, sin = torch.randn(1, 9, 32, generator=g), torch.randn(1, 9, 32, generator=g)
        a = wrapped(q, k, cos=cos, sin=sin)          # keyword form: straight to the stock function
        b = stock(q, k, cos, sin)
        assert torch.equal(a[0], b[0])
        a = wrapped(q, k, cos, sin, unsqueeze_dim=1)
        assert torch.equal(a[0], b[0]) and not calls
        # outside a patched forward the depth counter is zero
        assert getattr(sp._fused_rope_depth, "n", 0) == 0
        seen = []
        monkeypatch.setattr(model.model, "forward", lambda *a, **kw: seen.append(sp._fused_rope_depth.n) or 1 / 0)
        with pytest.raises(ZeroDivisionError):
            model(torch.zeros(1, 4, dtype=torch.long))
        assert seen == [1] and sp._fused_rope_depth.n == 0  # set during the forward, restored when it raises
        plain = SharePrefill(sharing_lookup_path=tiny_table(tmp_path))(tiny_llama())
        seen.clear()
        monkeypatch.setattr(plain.model, "forward", lambda *a, **kw: seen.append(getattr(sp._fused_rope_depth, "n", 0)) or 1 / 0)
        with pytest.raises(ZeroDivisionError):
            plain(torch.zeros(1, 4, dtype=torch.long))
        assert seen == [0]  # a model patched without fuse_rope never switches the fused pass on
    finally:
        modeling_llama.apply_rotary_pos_emb = stock


def test_update_pivotal_attns_masks_dense_flags_of_heads_without_a_slot(tmp_path, monkeypatch):
    """A caller's bool use_dense may name heads outside every shared cluster (attention_sharing.py:94-103 would store
    a pattern for any cluster id): those flags are dropped on the host before the device update."""
    from shareprefill_amd import AttentionSharing, ops

    sharing = AttentionSharing(tiny_table(tmp_path))  # head 0 in shared cluster "0", head 1 in unshared "1"
    sharing._state = types.SimpleNamespace()
    monkeypatch.setattr(sharing, "_head_cluster_tensor", lambda layer, hq, dev: torch.tensor([0, -1], dtype=torch.int32))
    got = {}
    monkeypatch.setattr(ops, "pivot_update", lambda st, hc, dec, avg, thr: got.update(dec=dec.tolist()))
    avg = torch.zeros(1, 2, 4, 4)
    sharing.update_pivotal_attns(0, avg, torch.tensor([[True, True]]), 0.9)
    assert got["dec"] == [1, 0]
    sharing.update_pivotal_attns(0, avg, torch.tensor([1, 1], dtype=torch.int32), 0.9)  # decision vector: as given
    assert got["dec"] == [1, 1]


def test_plans_release_older_masks_unless_asked_to_keep_them(tmp_path):
    from shareprefill_amd import AttentionSharing
    from shareprefill_amd.attention_sharing import LayerPlan

    sharing = AttentionSharing(tiny_table(tmp_path))
    mk = lambda i: LayerPlan(i, 2, torch.zeros(2, 2, 1, dtype=torch.int64), torch.zeros(2, dtype=torch.int32),
                             None, None, None, None)
    # plan_layer's bookkeeping, without the device work
    for i in range(3):
        if sharing.plans and not (sharing.keep_plans or sharing.keep_debug):
            sharing.plans[-1].mask = None
        sharing.plans.append(mk(i))
    assert [p.mask is None for p in sharing.plans] == [True, True, False]
    with pytest.raises(RuntimeError, match="keep_plans"):
        sharing.plans[0].block_idx()
    assert sharing.decision_histogram()["vertical_slash"] == 6  # the per-head decisions are kept


# ---- host helpers of the reference-named kernel wrappers (no GPU needed) ----------------------------------------
def test_pad_block_idx_list_and_tensor_forms():
    """list[B][H] of id tensors -> [B, H, K] padded with the reference's value (shareprefill_attn.py:528-540)."""
    from shareprefill_amd.shareprefill_attn import _pad_block_idx

    nb = 4
    pad = nb * (nb + 1)
    lists = [[torch.tensor([0, 5, 8]), torch.tensor([0])], [torch.tensor([], dtype=torch.int64), torch.tensor([0, 15])]]
    out = _pad_block_idx(lists, 2, 2, pad, torch.device("cpu"))
    assert out.shape == (2, 2, 3) and out.dtype == torch.int64
    assert out.tolist() == [[[0, 5, 8], [0, pad, pad]], [[pad, pad, pad], [0, 15, pad]]]
    t = torch.zeros(2, 2, 5, dtype=torch.int64)
    assert _pad_block_idx(t, 2, 2, pad, torch.device("cpu")) is t
    with pytest.raises(AssertionError):
        _pad_block_idx(lists, 1, 2, pad, torch.device("cpu"))


def test_pad_head_dim_appends_zero_channels():
    from shareprefill_amd.shareprefill_attn import KERNEL_HEAD_DIM, PADDED_HEAD_DIMS, pad_head_dim

    assert KERNEL_HEAD_DIM == 128 and PADDED_HEAD_DIMS == (16, 32, 64)
    x = torch.randn(1, 2, 5, 64).to(torch.bfloat16)
    y = torch.randn(1, 1, 5, 64).to(torch.bfloat16)
    px, py = pad_head_dim(x, y)
    assert px.shape == (1, 2, 5, 128) and py.shape == (1, 1, 5, 128)
    assert torch.equal(px[..., :64], x) and float(px[..., 64:].abs().max()) == 0.0
    # a zero-padded dot product is the dot product (fp64 holds these sums of bf16 products exactly, in any order)
    assert torch.equal((px.double() @ px.double().transpose(-1, -2)), (x.double() @ x.double().transpose(-1, -2)))


def test_scale_dim_flag_field():
    from shareprefill_amd import _lib

    assert _lib.SP_FLAG_SCALE_DIM(64) == 8 << 8 and _lib.SP_FLAG_SCALE_DIM(16) == 2 << 8
    assert (_lib.SP_FLAG_SCALE_DIM(32) & _lib.SP_FLAG_LOGITS_BF16) == 0
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "shareprefill_hip.h")).read()
    assert "#define SP_FLAG_SCALE_DIM(head_dim) ((((uint32_t)(head_dim)) / 8u) << 8)" in header


def test_reference_import_paths_resolve_to_the_package():
    import shareprefill
    from shareprefill.attn import utils as ref_utils
    from shareprefill.attn.shareprefill_attn import (shareprefill_attention_forward, triton_block_wise_prefill_attention,
                                                     triton_column_count_cumsum)
    import shareprefill_amd

    assert shareprefill.SharePrefill is shareprefill_amd.SharePrefill
    assert ref_utils.triton_bnhd_pool is shareprefill_amd.utils.triton_bnhd_pool
    assert triton_block_wise_prefill_attention is shareprefill_amd.shareprefill_attn.triton_block_wise_prefill_attention
    assert callable(triton_column_count_cumsum) and callable(shareprefill_attention_forward)

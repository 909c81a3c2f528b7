"""SharePrefill(...)(model): patches a Hugging Face decoder-only model to use the SharePrefill attention.

Mirror of shareprefill/shareprefill_patch.py:31-169 of the reference for the installed transformers:
  * registers the attention function under "shareprefill" in the model module's ALL_ATTENTION_FUNCTIONS
    and selects it through config._attn_implementation (:85-94);
  * attaches _init_attention_sharing / reset_attention_sharing / attention_sharing to the model (:96-140);
  * wraps model.forward so the sharing state is reset at every forward (:156-166).
Beyond the reference, `SharePrefill(..., fuse_rope=True)` routes the model module's apply_rotary_pos_emb (five
elementwise kernels per tensor in front of the attention function) to one in-place HIP pass with identical bits
while a forward of a model patched that way is running; every other caller of that module function (an unpatched
model of the same architecture, say) still gets the original.  `unpatch_model(model)` undoes the patch.
The reference also swaps in a copy of LlamaModel.forward that avoids the 4-D causal mask
(model_patch.py:41-170); transformers >= 5 already passes no mask to an attention implementation that has
no mask function registered, so nothing N x N is ever built and no forward is replaced.
"""

from __future__ import annotations

import functools
import importlib
import logging
import threading

import torch

from . import ops
from .attention_sharing import AttentionSharing
from .shareprefill_attn import shareprefill_attention_forward
from .shareprefill_configurations import SharePrefillConfig

LOGGER = logging.getLogger(__name__)

_CONFIG_FIELDS = ("sharing_lookup_path", "pattern_threshold", "similarity_threshold", "fallback_threshold",
                  "block_size", "min_budget", "max_budget", "queryaware_threshold")


class SharePrefill:
    def __init__(self, attn_type: str = "shareprefill", model_name: str = None, sharing_lookup_path: str = None,
                 pattern_threshold: float = 0.9, similarity_threshold: float = 0.5, fallback_threshold: float = 0.9,
                 queryaware_threshold: float = 0.1, block_size: int = 128, min_budget: int = 1024,
                 max_budget: int = None, **kwargs):
        self.config = SharePrefillConfig(
            attn_type=attn_type, model_name=model_name, sharing_lookup_path=sharing_lookup_path,
            pattern_threshold=pattern_threshold, similarity_threshold=similarity_threshold,
            fallback_threshold=fallback_threshold, queryaware_threshold=queryaware_threshold,
            block_size=block_size, min_budget=min_budget, max_budget=max_budget, **kwargs)

    def __call__(self, model):
        return self.patch_model(model)

    def patch_model(self, model):
        if self.config.attn_type not in self.config.SUPPORTED_ATTENTION_TYPES:
            raise ValueError(f"The attention type {self.config.attn_type} is not supported.")
        return shareprefill_patch(model, self.config)


_fused_rope_depth = threading.local()  # > 0 while a forward of a model patched with fuse_rope=True is running


def _fused_rope(original):
    """apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim=1) -> (q_embed, k_embed) with the rotation done in place
    by the HIP kernel when (a) the call comes from inside the forward of a model patched with fuse_rope=True and
    (b) it has the shape the attention layer produces at inference (bf16 GPU tensors [B, H, N, D] that nothing
    else needs, no autograd).  Any other call -- other models of the architecture, other argument forms -- goes to
    the original function unchanged."""

    @functools.wraps(original)
    def apply_rotary_pos_emb(*args, **kwargs):
        if getattr(_fused_rope_depth, "n", 0) <= 0 or len(args) != 4 or (kwargs and set(kwargs) != {"unsqueeze_dim"}):
            return original(*args, **kwargs)
        q, k, cos, sin = args
        unsqueeze_dim = kwargs.get("unsqueeze_dim", 1)
        if not all(isinstance(t, torch.Tensor) for t in args):
            return original(*args, **kwargs)
        fusable = (unsqueeze_dim == 1 and q.dim() == 4 and k.dim() == 4 and cos.dim() == 3 and q.is_cuda
                   and q.dtype == k.dtype == cos.dtype == sin.dtype == torch.bfloat16
                   and not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad))
                   and q.shape[-1] % 16 == 0 and q.stride(3) == 1 and k.stride(3) == 1
                   and cos.shape == sin.shape == (q.shape[0], q.shape[2], q.shape[3]) and k.shape[2] == q.shape[2]
                   and cos.stride(2) == 1 and sin.stride() == cos.stride()
                   and all(st % 8 == 0 for st in (*q.stride()[:3], *k.stride()[:3], cos.stride(1)))
                   and all(t.data_ptr() % 16 == 0 for t in (q, k, cos, sin)))
        if not fusable:
            return original(*args, **kwargs)
        for b in range(q.shape[0]):
            ops.rope_inplace(q[b], k[b], cos[b], sin[b])
        return q, k

    apply_rotary_pos_emb._shareprefill_original = original
    return apply_rotary_pos_emb


def shareprefill_patch(model, config: SharePrefillConfig):
    try:
        attention_cls = model.model.layers[0].self_attn.__class__
    except AttributeError as exc:
        raise TypeError("SharePrefill expects a decoder-only architecture exposing "
                        "`model.model.layers[*].self_attn`.") from exc

    attention_module = importlib.import_module(attention_cls.__module__)
    attention_functions = getattr(attention_module, "ALL_ATTENTION_FUNCTIONS", None)
    if attention_functions is None:
        raise TypeError("Expected the attention module to define ALL_ATTENTION_FUNCTIONS for integration.")
    attention_functions["shareprefill"] = shareprefill_attention_forward
    prev_attn_implementation = getattr(model.config, "_attn_implementation", None)
    model.config._attn_implementation = "shareprefill"
    if config.extra.get("fuse_rope", False):
        rope = getattr(attention_module, "apply_rotary_pos_emb", None)
        if rope is None:
            raise TypeError(f"fuse_rope=True: {attention_module.__name__} has no apply_rotary_pos_emb to replace")
        if not hasattr(rope, "_shareprefill_original"):
            attention_module.apply_rotary_pos_emb = _fused_rope(rope)

    def _init_attention_sharing(self):
        self.attention_sharing = AttentionSharing(config.sharing_lookup_path)
        return self.attention_sharing

    def reset_attention_sharing(self):
        """New inference pass: rebuild the state if the lookup table changed, else clear it; push the
        thresholds onto the shared HF config, where the attention function reads them (:106-134)."""
        changed = (not hasattr(self, "attention_sharing")
                   or getattr(self.config, "sharing_lookup_path", None) != config.sharing_lookup_path)
        if changed:
            self.attention_sharing = AttentionSharing(config.sharing_lookup_path)
        else:
            self.attention_sharing.reset_state()
        for name in _CONFIG_FIELDS:
            setattr(self.config, name, getattr(config, name))
        # not in the reference: prompts no longer than min_budget run on the dense mask without any selection
        self.config.dense_short_prompts = bool(config.extra.get("dense_short_prompts", True))
        for m in self.modules():
            if isinstance(m, attention_cls):
                m.attention_sharing = self.attention_sharing
        return self.attention_sharing

    model.__class__._init_attention_sharing = _init_attention_sharing
    model.__class__.reset_attention_sharing = reset_attention_sharing
    model.attention_sharing = model._init_attention_sharing()

    model._shareprefill_fuse_rope = bool(config.extra.get("fuse_rope", False))
    if not getattr(model, "_shareprefill_wrapped", False):
        original = model.forward.__func__ if hasattr(model.forward, "__func__") else model.forward
        model._shareprefill_prev = {"forward": model.__dict__.get("forward"),
                                    "attn_implementation": prev_attn_implementation}

        @functools.wraps(original)
        def wrapped(self, *args, **kwargs):
            self.reset_attention_sharing()
            if not getattr(self, "_shareprefill_fuse_rope", False):
                return original(self, *args, **kwargs)
            _fused_rope_depth.n = getattr(_fused_rope_depth, "n", 0) + 1
            try:
                return original(self, *args, **kwargs)
            finally:
                _fused_rope_depth.n -= 1

        model.forward = wrapped.__get__(model, model.__class__)
        model._shareprefill_wrapped = True

    model.reset_attention_sharing()
    LOGGER.info("Patched model for shareprefill.")
    return model


def unpatch_model(model):
    """Undoes shareprefill_patch on this model object: the forward wrapper goes, the attention implementation the
    config named before comes back, the sharing state is dropped.  The "shareprefill" entry of the architecture's
    attention-function table and the module-level rotary wrapper stay (both are inert for unpatched models)."""
    if not getattr(model, "_shareprefill_wrapped", False):
        return model
    prev = getattr(model, "_shareprefill_prev", {})
    if prev.get("forward") is None:
        model.__dict__.pop("forward", None)
    else:
        model.forward = prev["forward"]
    if prev.get("attn_implementation") is not None:
        model.config._attn_implementation = prev["attn_implementation"]
    for name in ("_shareprefill_wrapped", "_shareprefill_prev", "_shareprefill_fuse_rope", "attention_sharing"):
        model.__dict__.pop(name, None)
    for m in model.modules():
        m.__dict__.pop("attention_sharing", None)
    return model

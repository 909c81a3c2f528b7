"""SharePrefill(...)(model): patches a Hugging Face decoder-only model to use the SharePrefill attention.

Mirror of shareprefill/shareprefill_patch.py:31-169 of the reference for the installed transformers:
  * registers the attention function under "shareprefill" in the model module's ALL_ATTENTION_FUNCTIONS
    and selects it through config._attn_implementation (:85-94);
  * attaches _init_attention_sharing / reset_attention_sharing / attention_sharing to the model (:96-140);
  * wraps model.forward so the sharing state is reset at every forward (:156-166).
The reference also swaps in a copy of LlamaModel.forward that avoids the 4-D causal mask
(model_patch.py:41-170); transformers >= 5 already passes no mask to an attention implementation that has
no mask function registered, so nothing N x N is ever built and no forward is replaced.
"""

from __future__ import annotations

import functools
import importlib
import logging

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
    model.config._attn_implementation = "shareprefill"

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
        for m in self.modules():
            if isinstance(m, attention_cls):
                m.attention_sharing = self.attention_sharing
        return self.attention_sharing

    model.__class__._init_attention_sharing = _init_attention_sharing
    model.__class__.reset_attention_sharing = reset_attention_sharing
    model.attention_sharing = model._init_attention_sharing()

    if not getattr(model, "_shareprefill_wrapped", False):
        original = model.forward.__func__ if hasattr(model.forward, "__func__") else model.forward

        @functools.wraps(original)
        def wrapped(self, *args, **kwargs):
            self.reset_attention_sharing()
            return original(self, *args, **kwargs)

        model.forward = wrapped.__get__(model, model.__class__)
        model._shareprefill_wrapped = True

    model.reset_attention_sharing()
    LOGGER.info("Patched model for shareprefill.")
    return model

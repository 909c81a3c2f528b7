"""The reference's import name for the MI355X implementation:

    from shareprefill import SharePrefill                      # shareprefill/__init__.py:15-17 of the reference
    model = SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct")(model)

Everything lives in the `shareprefill_amd` package; this package only re-exports it under the names a user of the
reference imports (the top-level classes, and the module paths shareprefill.shareprefill_patch,
shareprefill.shareprefill_configurations, shareprefill.attn.attention_sharing, shareprefill.attn.shareprefill_attn,
shareprefill.attn.utils).
"""

import sys
import types

import shareprefill_amd
from shareprefill_amd import (AttentionSharing, SharePrefill, SharePrefillConfig, attention_sharing,
                              shareprefill_attention_forward, shareprefill_attn, shareprefill_configurations,
                              shareprefill_patch, utils)

__all__ = ["SharePrefill", "SharePrefillConfig", "AttentionSharing", "shareprefill_attention_forward"]

attn = types.ModuleType(__name__ + ".attn", "Selection state and attention function (shareprefill/attn/ of the reference).")
attn.attention_sharing = attention_sharing
attn.shareprefill_attn = shareprefill_attn
attn.utils = utils
attn.AttentionSharing = AttentionSharing
attn.shareprefill_attention_forward = shareprefill_attention_forward
sys.modules[attn.__name__] = attn
sys.modules[attn.__name__ + ".attention_sharing"] = attention_sharing
sys.modules[attn.__name__ + ".shareprefill_attn"] = shareprefill_attn
sys.modules[attn.__name__ + ".utils"] = utils
sys.modules[__name__ + ".shareprefill_patch"] = shareprefill_patch
sys.modules[__name__ + ".shareprefill_configurations"] = shareprefill_configurations

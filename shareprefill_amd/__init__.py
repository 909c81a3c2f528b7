"""shareprefill_amd: the SharePrefill prefill-attention path for AMD MI355X (gfx950).

    from shareprefill_amd import SharePrefill
    model = SharePrefill(model_name="meta-llama/Llama-3.1-8B-Instruct", pattern_threshold=0.95)(model)

Host code is Python on PyTorch-ROCm; the device side is libshareprefill_hip.so (hand-written HIP, C ABI in
include/shareprefill_hip.h), built with `python -m shareprefill_amd.build`.  There is no CPU fallback.
"""

from .attention_sharing import AttentionSharing
from .shareprefill_attn import shareprefill_attention_forward
from .shareprefill_configurations import SharePrefillConfig
from . import attention_sharing, shareprefill_attn, shareprefill_configurations, shareprefill_patch, utils
from .shareprefill_patch import SharePrefill, unpatch_model

__all__ = ["SharePrefill", "SharePrefillConfig", "AttentionSharing", "shareprefill_attention_forward", "unpatch_model"]

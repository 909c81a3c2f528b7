"""Configuration object of the SharePrefill patch (reference: shareprefill/shareprefill_configurations.py:24-77).

Field names and defaults are the reference's; they are the public API.  One difference: the reference
evaluates model_name.split("/") before looking at an explicit sharing_lookup_path, so model_name=None
fails even when a path is given (:67-72); here an explicit path needs no model name."""

from __future__ import annotations

import os
from pathlib import Path
from typing import Optional

from .clusters.sharing_lookup_registry import SHARING_LOOKUP_REGISTRY

PACKAGE_DIR = Path(__file__).resolve().parent


class SharePrefillConfig:
    SUPPORTED_ATTENTION_TYPES = ["shareprefill"]

    def __init__(self, attn_type: str = "shareprefill", model_name: Optional[str] = None,
                 sharing_lookup_path: Optional[str] = None, pattern_threshold: float = 0.9,
                 similarity_threshold: float = 0.5, fallback_threshold: float = 0.9,
                 queryaware_threshold: float = 0.1, block_size: int = 128, min_budget: Optional[int] = 1024,
                 max_budget: Optional[int] = None, **kwargs):
        assert attn_type in self.SUPPORTED_ATTENTION_TYPES, \
            f"The attention_type {attn_type} you specified is not supported."
        self.attn_type = attn_type
        self.sharing_lookup_path = self.update_sharing_lookup_path(sharing_lookup_path, model_name)
        self.model_name = model_name
        self.pattern_threshold = pattern_threshold
        self.similarity_threshold = similarity_threshold
        self.fallback_threshold = fallback_threshold
        self.queryaware_threshold = queryaware_threshold
        self.block_size = block_size
        self.min_budget = min_budget
        self.max_budget = max_budget
        self.extra = dict(kwargs)

    @classmethod
    def _resolve_sharing_lookup_path(cls, model_key: str) -> str:
        if model_key not in SHARING_LOOKUP_REGISTRY:
            raise AssertionError(f"Unsupported model {model_key}. Known: {sorted(SHARING_LOOKUP_REGISTRY)}; "
                                 "pass sharing_lookup_path for any other model.")
        return os.path.join(PACKAGE_DIR, SHARING_LOOKUP_REGISTRY[model_key])

    @classmethod
    def update_sharing_lookup_path(cls, sharing_lookup_path: Optional[str], model_name: Optional[str]) -> str:
        if sharing_lookup_path is not None:
            return sharing_lookup_path
        if model_name is None:
            raise AssertionError("SharePrefill needs model_name (a registered model) or sharing_lookup_path.")
        return cls._resolve_sharing_lookup_path(model_name.split("/")[-1])

    @classmethod
    def get_available_attn_types(cls):
        return cls.SUPPORTED_ATTENTION_TYPES

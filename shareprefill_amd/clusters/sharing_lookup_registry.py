"""Model name -> head-cluster table shipped with the package (reference:
shareprefill/clusters/sharing_lookup_registry.py:15-19).  The table is the reference's own
Llama-3.1-8B-Instruct clustering, stored compactly in the same JSON schema."""

SHARING_LOOKUP_REGISTRY = {
    "Llama-3.1-8B-Instruct": "clusters/sharing_lookup/Llama-3.1-8B-Instruct_code_debug_hiera-40.0-2.json",
}

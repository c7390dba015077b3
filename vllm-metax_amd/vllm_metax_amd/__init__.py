"""MI355X (gfx950) int8 KV-cache attention path, drop-in for the vLLM-metax TRITON_ATTN /
TRITON_MLA backends on that path.

``register()`` mirrors the platform-plugin entry point of the reference
(vllm_metax/__init__.py:14-16); it only matters when upstream vLLM is installed.
"""
__version__ = "0.1.0"


def register():
    """vllm.platform_plugins entry point: registers the attention backends with upstream
    vLLM's registry (when importable) and returns nothing else to override."""
    from .platform import register_attention_backends

    register_attention_backends()
    return None

"""MI355X (gfx950) int8 KV-cache attention path, drop-in for the vLLM-metax TRITON_ATTN /
TRITON_MLA backends on that path.

``register()`` mirrors the platform-plugin entry point of the reference
(vllm_metax/__init__.py:14-16); it only matters when upstream vLLM is installed.
"""
__version__ = "0.1.0"


def register():
    """``vllm.platform_plugins`` entry point: the class path of the platform, as the reference's
    ``register()`` returns ``"vllm_metax.platform.MacaPlatform"`` (vllm_metax/__init__.py:14-16)."""
    from .platform import PLATFORM_PATH

    return PLATFORM_PATH


def register_out_of_tree():
    """``vllm.general_plugins`` entry point (the reference's runs its patches and registry module,
    vllm_metax/__init__.py:30-32): nothing is overwritten by default -- the platform routes the int8
    KV-cache dtypes to this build's backends and leaves every other dtype to upstream's."""
    from .platform import register_attention_backends

    register_attention_backends(replace_slots=False)

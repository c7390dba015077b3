"""Backend registration and selection for the int8 KV-cache path.

Mirrors what the reference's platform does for attention backends
(vllm_metax/platform.py:76-150 registration, :386-514 selection): class paths are registered under
the registry names they take over (TRITON_ATTN for the per-token-head int8 cache, TRITON_MLA for
the int8 latent cache), and a backend is picked by asking each candidate, in priority order, for
the reasons it cannot serve a configuration.
"""
from __future__ import annotations

import importlib

INT8_ATTN_PATH = "vllm_metax_amd.v1.attention.backends.int8_attn.Int8AttentionBackend"
INT8_MLA_PATH = "vllm_metax_amd.v1.attention.backends.mla.int8_mla.Int8MLABackend"

# registry name -> class path; the order is the selection priority within a kind
_BACKENDS = {
    "TRITON_ATTN": INT8_ATTN_PATH,
    "TRITON_MLA": INT8_MLA_PATH,
}


def _get_backend_priorities(use_mla: bool) -> list[str]:
    return ["TRITON_MLA"] if use_mla else ["TRITON_ATTN"]


def register_attention_backends() -> None:
    """Register both backends with upstream vLLM's registry when vLLM is importable (the two
    ``register_backend`` calls of vllm_metax/platform.py:119-138); a no-op otherwise."""
    try:  # pragma: no cover - upstream vLLM is not installed in the build container
        from vllm.v1.attention.backends.registry import AttentionBackendEnum, register_backend
    except Exception:  # noqa: BLE001
        return
    register_backend(backend=AttentionBackendEnum.TRITON_ATTN, class_path=INT8_ATTN_PATH)  # pragma: no cover
    register_backend(backend=AttentionBackendEnum.TRITON_MLA, class_path=INT8_MLA_PATH)  # pragma: no cover


def resolve_backend_class(name: str):
    module, _, cls = _BACKENDS[name].rpartition(".")
    return getattr(importlib.import_module(module), cls)


def get_valid_backends(use_mla: bool, **config):
    valid, invalid = [], {}
    for priority, name in enumerate(_get_backend_priorities(use_mla)):
        try:
            reasons = resolve_backend_class(name).validate_configuration(use_mla=use_mla, **config)
        except ImportError:
            reasons = ["ImportError"]
        if reasons:
            invalid[name] = (priority, reasons)
        else:
            valid.append((name, priority))
    return valid, invalid


def get_attn_backend_cls(selected_backend: str | None = None, use_mla: bool = False, **config) -> str:
    """Class path of the backend serving ``config`` (``head_size``, ``dtype``, ``kv_cache_dtype``,
    ``block_size``, ...).  A forced backend that is not valid raises ValueError with its reasons, and
    so does a configuration no backend serves, like the reference (vllm_metax/platform.py:430-446,
    471-476)."""
    if selected_backend is not None:
        if selected_backend not in _BACKENDS:
            raise ValueError(f"Selected backend {selected_backend} is not provided by this build")
        reasons = resolve_backend_class(selected_backend).validate_configuration(use_mla=use_mla, **config)
        if reasons:
            raise ValueError(f"Selected backend {selected_backend} is not valid for this configuration. "
                             f"Reason: {reasons}")
        return _BACKENDS[selected_backend]
    valid, invalid = get_valid_backends(use_mla, **config)
    if not valid:
        why = ", ".join(f"{n}: [{', '.join(r)}]" for n, (_, r) in invalid.items())
        raise ValueError(f"No valid attention backend found with {config}. Reasons: {{{why}}}.")
    return _BACKENDS[sorted(valid, key=lambda x: x[1])[0][0]]

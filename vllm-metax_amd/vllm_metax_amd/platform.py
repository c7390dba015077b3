"""Backend registration and selection for the int8 KV-cache path.

Mirrors what the reference's platform does for attention backends
(vllm_metax/platform.py:76-150 registration, :386-514 selection): a backend is picked by asking each
candidate, in priority order, for the reasons it cannot serve a configuration.  The two backends of
this build stand in the registry slots TRITON_ATTN (per-token-head int8 cache) and TRITON_MLA (int8
latent cache) -- but ONLY for those two KV-cache dtypes: ``Int8KVPlatform.get_attn_backend_cls``
routes a layer here when its ``kv_cache_dtype`` is one of them and hands every other dtype (auto,
bf16, per-tensor fp8 ...) to the platform it derives from, so a
deployment that mixes cache dtypes keeps upstream's own backends for the rest.  Overwriting the two
registry slots globally is possible (``register_attention_backends(replace_slots=True)``) and then
removes those dtypes from the slots.
"""
from __future__ import annotations

import importlib

from .kv_cache_interface import FP8_PER_TOKEN_HEAD, INT4_PER_TOKEN_HEAD, INT8_PER_TOKEN, INT8_PER_TOKEN_HEAD

PLATFORM_PATH = "vllm_metax_amd.platform.Int8KVPlatform"
INT8_KV_DTYPES = (INT8_PER_TOKEN_HEAD, FP8_PER_TOKEN_HEAD, INT4_PER_TOKEN_HEAD, INT8_PER_TOKEN)   # the inline-scale dtypes this build serves

INT8_ATTN_PATH = "vllm_metax_amd.v1.attention.backends.int8_attn.Int8AttentionBackend"
INT8_MLA_PATH = "vllm_metax_amd.v1.attention.backends.mla.int8_mla.Int8MLABackend"

# registry name -> class path; the order is the selection priority within a kind
_BACKENDS = {
    "TRITON_ATTN": INT8_ATTN_PATH,
    "TRITON_MLA": INT8_MLA_PATH,
}


def _get_backend_priorities(use_mla: bool) -> list[str]:
    return ["TRITON_MLA"] if use_mla else ["TRITON_ATTN"]


def register_attention_backends(replace_slots: bool = False) -> bool:
    """With ``replace_slots=True`` and upstream vLLM importable: the two ``register_backend`` calls of
    vllm_metax/platform.py:119-138, which put this build's classes into the TRITON_ATTN / TRITON_MLA
    slots for EVERY KV-cache dtype (the classes then refuse all but the int8 ones).  By default nothing
    is overwritten: selection goes through ``Int8KVPlatform.get_attn_backend_cls``.  Returns whether
    the registry was changed."""
    if not replace_slots:
        return False
    try:  # pragma: no cover - upstream vLLM is not installed in the build container
        from vllm.v1.attention.backends.registry import AttentionBackendEnum, register_backend
    except Exception:  # noqa: BLE001
        return False
    register_backend(backend=AttentionBackendEnum.TRITON_ATTN, class_path=INT8_ATTN_PATH)  # pragma: no cover
    register_backend(backend=AttentionBackendEnum.TRITON_MLA, class_path=INT8_MLA_PATH)  # pragma: no cover
    return True  # pragma: no cover


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


def _platform_base():
    """The platform this one refines: upstream's ROCm platform when vLLM is importable."""
    try:  # pragma: no cover - upstream vLLM is not installed in the build container
        from vllm.platforms.rocm import RocmPlatform  # type: ignore

        return RocmPlatform
    except Exception:  # noqa: BLE001
        return object


class Int8KVPlatform(_platform_base()):
    """What ``register()`` names, as vllm_metax.register() names MacaPlatform
    (vllm_metax/__init__.py:14-16, vllm_metax/platform.py:418-514): upstream's ROCm platform with one
    method refined -- layers whose KV cache is one of the int8 dtypes get this build's backends, all
    others get whatever the base platform selects."""

    @classmethod
    def get_attn_backend_cls(cls, selected_backend=None, attn_selector_config=None, num_heads=None, **kwargs) -> str:
        cfg = attn_selector_config
        as_dict = cfg._asdict() if hasattr(cfg, "_asdict") else dict(getattr(cfg, "__dict__", {}) or {})
        as_dict.update(kwargs)
        kv_dtype = as_dict.get("kv_cache_dtype")
        if kv_dtype in INT8_KV_DTYPES:
            name = getattr(selected_backend, "name", selected_backend)
            if name is not None and name not in _BACKENDS:
                raise ValueError(f"Selected backend {name} does not serve kv_cache_dtype {kv_dtype!r}; "
                                 f"this build serves it in the {sorted(_BACKENDS)} slots")
            use_mla = bool(as_dict.pop("use_mla", kv_dtype == INT8_PER_TOKEN))
            return get_attn_backend_cls(name, use_mla=use_mla, **as_dict)
        base = super()
        if hasattr(base, "get_attn_backend_cls"):  # pragma: no cover - needs upstream vLLM
            return base.get_attn_backend_cls(selected_backend, attn_selector_config, num_heads)
        raise ValueError(f"kv_cache_dtype {kv_dtype!r} is not served by this build (it serves {list(INT8_KV_DTYPES)}) "
                         "and no upstream platform is importable to hand the layer to")

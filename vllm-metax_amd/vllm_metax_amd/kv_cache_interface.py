"""KV-cache quantisation modes understood by this backend.

The reference imports ``KVQuantMode``, ``get_kv_quant_mode`` and
``kv_cache_uses_per_token_head_scales`` from upstream ``vllm.v1.kv_cache_interface``
(vllm_metax/v1/attention/backends/triton_attn.py:44-49) and only uses the members
restated here; when upstream vLLM is importable its definitions are used instead so
the enum identities match.
"""
from __future__ import annotations

import enum

try:  # pragma: no cover - upstream vLLM is not installed in the build container
    from vllm.v1.kv_cache_interface import (  # type: ignore
        KVQuantMode,
        get_kv_quant_mode,
        kv_cache_uses_per_token_head_scales,
    )
except Exception:  # noqa: BLE001

    class KVQuantMode(enum.IntEnum):
        NONE = 0
        FP8_PER_TENSOR = 1
        INT8_PER_TOKEN_HEAD = 2
        FP8_PER_TOKEN_HEAD = 3
        INT4_PER_TOKEN_HEAD = 4

        @property
        def is_per_token_head(self) -> bool:
            return self in (
                KVQuantMode.INT8_PER_TOKEN_HEAD,
                KVQuantMode.FP8_PER_TOKEN_HEAD,
                KVQuantMode.INT4_PER_TOKEN_HEAD,
            )

    _MODES = {
        "auto": KVQuantMode.NONE,
        "float16": KVQuantMode.NONE,
        "bfloat16": KVQuantMode.NONE,
        "fp8": KVQuantMode.FP8_PER_TENSOR,
        "fp8_e4m3": KVQuantMode.FP8_PER_TENSOR,
        "fp8_e5m2": KVQuantMode.FP8_PER_TENSOR,
        "int8_per_token_head": KVQuantMode.INT8_PER_TOKEN_HEAD,
        "fp8_per_token_head": KVQuantMode.FP8_PER_TOKEN_HEAD,
        "int4_per_token_head": KVQuantMode.INT4_PER_TOKEN_HEAD,
    }

    def get_kv_quant_mode(cache_dtype_str: str) -> "KVQuantMode":
        try:
            return _MODES[cache_dtype_str]
        except KeyError:
            raise ValueError(f"unknown kv cache dtype {cache_dtype_str!r}") from None

    def kv_cache_uses_per_token_head_scales(cache_dtype_str: str) -> bool:
        return get_kv_quant_mode(cache_dtype_str).is_per_token_head


INT8_PER_TOKEN_HEAD = "int8_per_token_head"
# the fp8 mode of the same inline-scale record layout (vllm_metax/v1/attention/backends/triton_attn.py:336-348)
FP8_PER_TOKEN_HEAD = "fp8_per_token_head"
# the int4 mode of the same layout: two codes per byte, head_size / 2 code bytes + the scale per half
# (vllm_metax/v1/attention/backends/triton_attn.py:332-346)
INT4_PER_TOKEN_HEAD = "int4_per_token_head"
# MLA latent cache with one fp32 scale per token (this build's addition; the
# reference's MLA backends stop at fp8, vllm_metax/v1/attention/backends/mla/triton_mla.py:94-100).
INT8_PER_TOKEN = "int8_per_token"

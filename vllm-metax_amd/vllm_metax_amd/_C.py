"""ctypes binding of libkvq_hip.so, the C-ABI library holding the gfx950 kernels.

There is no fallback: if the library is missing or an entry point returns an
error, a RuntimeError is raised (the reference's ops raise through
STD_TORCH_CHECK the same way, csrc/libtorch_stable/cache_kernels.cu:884-889).
"""
from __future__ import annotations

import ctypes
import os

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib")
LIB_PATH = os.path.join(_LIB_DIR, "libkvq_hip.so")

KVQ_F32, KVQ_BF16, KVQ_F16 = 0, 1, 2
KVQ_CODE_INT8, KVQ_CODE_FP8_E4M3, KVQ_CODE_INT4 = 0, 1, 2
ABI_VERSION = 19


class CacheGeom(ctypes.Structure):
    """Mirror of ``kvq_cache_geom`` (include/kvq.h)."""

    _fields_ = [
        ("k_off", ctypes.c_int64), ("v_off", ctypes.c_int64),
        ("ks_off", ctypes.c_int64), ("vs_off", ctypes.c_int64),
        ("stride_block", ctypes.c_int64), ("stride_slot", ctypes.c_int64),
        ("stride_head", ctypes.c_int64),
        ("num_kv_heads", ctypes.c_int32), ("head_size", ctypes.c_int32),
        ("block_size", ctypes.c_int32), ("code_type", ctypes.c_int32),
    ]


class MlaGeom(ctypes.Structure):
    """Mirror of ``kvq_mla_geom`` (include/kvq.h)."""

    _fields_ = [
        ("stride_block", ctypes.c_int64), ("stride_row", ctypes.c_int64),
        ("scale_off", ctypes.c_int64),
        ("kv_lora_rank", ctypes.c_int32), ("rope_dim", ctypes.c_int32),
        ("block_size", ctypes.c_int32), ("reserved", ctypes.c_int32),
    ]


_vp, _i, _i64, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t
_geom_p, _mla_p = ctypes.POINTER(CacheGeom), ctypes.POINTER(MlaGeom)

# name -> (restype, argtypes); every symbol include/kvq.h declares.
SIGNATURES = {
    "kvq_abi_version": (_i, []),
    "kvq_last_error": (ctypes.c_char_p, []),
    "kvq_device_num_cus": (_i, []),
    "kvq_set_batch_invariant": (_i, [_i]),
    "kvq_get_batch_invariant": (_i, []),
    "kvq_reshape_and_cache_int8": (_i, [_vp, _vp, _i, _i64, _i64, _i64, _i64, _vp, _geom_p, _vp, _i64, _f, _vp]),
    "kvq_paged_attn_workspace_bytes": (_sz, [_i, _i, _i]),
    "kvq_paged_attn_int8": (_i, [_vp, _i, _i64, _i64, _vp, _i, _i64, _i64, _vp, _geom_p, _vp, _i64, _vp, _vp,
                                 _i, _i, _i, _f, _i, _i, _f, _vp, _vp, _vp, _vp, _sz, _vp]),
    "kvq_paged_attn_int8_fused_write": (_i, [_vp, _i, _i64, _i64, _vp, _i, _i64, _i64, _vp, _vp, _i, _i64, _i64, _i64, _i64,
                                             _f, _vp, _geom_p, _vp, _i64, _vp, _vp, _i, _i, _f, _i, _f, _vp, _vp, _vp, _vp, _sz,
                                             _vp]),
    "kvq_paged_attn_split_prefill_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "kvq_paged_attn_int8_split_prefill": (_i, [_vp, _i, _i64, _i64, _vp, _i, _i64, _i64, _vp, _geom_p, _vp, _i64, _vp, _vp,
                                               _i, _i, _i, _f, _i, _i, _f, _vp, _vp, _vp, _i, _i, _vp, _sz, _vp]),
    "kvq_paged_attn_static_scratch_bytes": (_sz, []),
    "kvq_paged_attn_int8_static_scratch": (_i, [_vp, _i, _i64, _i64, _vp, _i, _i64, _i64, _vp, _geom_p, _vp, _i64, _vp,
                                                _vp, _i, _i, _i, _f, _i, _i, _f, _vp, _vp, _vp, _vp]),
    "kvq_paged_attn_v2_int8": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _i64, _i64, _vp, _geom_p, _vp, _i64, _vp,
                                    _i, _i, _f, _vp, _i, _i, _vp]),
    "kvq_splitk_reduce": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "kvq_swap_blocks": (_i, [_vp, _vp, _i64, _vp, _i64, _i64, _i64, _i, _vp]),
    "kvq_swap_blocks_batch": (_i, [_vp, _vp, _vp, _i64, _i, _vp]),
    "kvq_copy_blocks": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _vp]),
    "kvq_merge_attn_states": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i, _i, _i64, _vp]),
    "kvq_concat_and_cache_mla_int8": (_i, [_vp, _vp, _i, _i64, _i64, _vp, _mla_p, _vp, _i64, _f, _vp]),
    "kvq_gather_and_dequant_mla_int8": (_i, [_vp, _i, _i64, _vp, _mla_p, _vp, _i64, _vp, _vp, _vp, _i64, _vp]),
    "kvq_concat_and_cache_mla_rope_int8": (_i, [_vp, _vp, _i64, _i64, _i, _vp, _i64, _vp, _i64, _i, _vp, _i, _i, _i,
                                                _vp, _mla_p, _vp, _i64, _f, _vp]),
    "kvq_cp_gather_mla_int8": (_i, [_vp, _i64, _vp, _mla_p, _vp, _i64, _vp, _vp, _i, _i64, _vp]),
    "kvq_mla_decode_workspace_bytes": (_sz, [_i, _i, _i]),
    "kvq_mla_decode_int8": (_i, [_vp, _i, _vp, _vp, _i, _i64, _i64, _vp, _i64, _i64, _vp, _mla_p, _vp, _i64, _vp,
                                 _i, _i, _f, _vp, _sz, _vp]),
    "kvq_mla_decode_int8_fused_write": (_i, [_vp, _i, _vp, _vp, _i, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _i, _i64,
                                             _i64, _f, _vp, _mla_p, _vp, _i64, _vp, _i, _i, _f, _vp, _sz, _vp]),
    "kvq_mla_decode_absorb_int8": (_i, [_vp, _i, _vp, _vp, _i, _i64, _i64, _i, _vp, _i64, _i64, _vp, _i64, _i64, _vp,
                                        _mla_p, _vp, _i64, _vp, _i, _i, _f, _vp, _sz, _vp]),
    "kvq_rope_and_cache_int8": (_i, [_vp, _vp, _i64, _i64, _i, _vp, _i64, _i64, _vp, _i64, _i64, _i, _vp, _i, _i, _i, _vp,
                                     _geom_p, _vp, _i64, _f, _vp]),
    "kvq_concat_mla_q": (_i, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i, _i64, _i, _i, _i, _vp]),
    "kvq_mla_v_up_proj": (_i, [_vp, _i64, _i64, _vp, _i, _i64, _i64, _vp, _i64, _i64, _i, _i, _i, _i, _vp]),
    "kvq_mla_prefill_attn": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _i, _i,
                                  _i64, _i, _i, _i, _i, _f, _i, _vp, _i64, _i64, _vp, _vp]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise if it is absent or of another ABI version."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP kernels are not built "
            "(run `make -C vllm-metax_amd/csrc` or __graft_entry__.build()). "
            "There is no CPU fallback for this path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    got = lib.kvq_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libkvq_hip.so ABI version {got}, expected {ABI_VERSION}")
    # the switch the reference reads as envs.VLLM_BATCH_INVARIANT, taken from the same variable
    if os.environ.get("VLLM_BATCH_INVARIANT", "0").strip().lower() in ("1", "true", "yes", "on"):
        lib.kvq_set_batch_invariant(1)
    _lib = lib
    return lib


def check(status: int, op: str) -> None:
    if status != 0:
        msg = load().kvq_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{op} failed (status {status}): {msg}")

"""Cache tensor layout of the int8 KV cache with inline per-(token, head) scales.

Byte-for-byte the layout of the reference's TRITON_ATTN backend:

* logical shape ``(num_blocks, num_kv_heads, block_size, 2 * (head_size + 4))``
  int8 (vllm_metax/v1/attention/backends/triton_attn.py:318-348);
* physical order NHD ``(0, 2, 1, 3)`` or HND ``(0, 1, 2, 3)`` (:350-372);
* the content dim of one (head, slot) is
  ``[K codes | K scale fp32 | V codes | V scale fp32]``; ``key_cache`` /
  ``value_cache`` are ``kv_cache.transpose(1, 2).split(head_size + 4, -1)`` and the
  scales are fp32 ``as_strided`` views of shape ``(num_blocks, block_size,
  num_kv_heads)`` over the same storage (:418-479, 729-739).

Everything here is shape/stride algebra on torch views (no kernels).  The MLA
latent cache layout at the bottom is this build's own (the reference has no int8
MLA cache): per block, ``block_size`` rows of 576 codes, then ``block_size`` fp32
scales, which keeps every row 16-byte aligned and a block opaque-copyable.
"""
from __future__ import annotations

import os
from dataclasses import dataclass

import torch

from . import _C
from .kv_cache_interface import (
    FP8_PER_TOKEN_HEAD,
    INT4_PER_TOKEN_HEAD,
    INT8_PER_TOKEN,
    INT8_PER_TOKEN_HEAD,
    KVQuantMode,
    kv_cache_uses_per_token_head_scales,
)

SCALE_BYTES = 4  # one fp32 scale
# absmax floor of the quantiser (tests/kernels/quant_utils.py:194: eps=1e-10)
QUANT_EPS = 1e-10


def _explicit_kv_cache_layout() -> str | None:
    """The memory order a deployment has ASKED for, or None: the ``VLLM_KV_CACHE_LAYOUT`` environment
    variable, or upstream's programmatic override where upstream vLLM is importable."""
    layout = os.environ.get("VLLM_KV_CACHE_LAYOUT")
    if layout is None:
        try:  # pragma: no cover - upstream vLLM is not installed in the build container
            from vllm.v1.attention.backends import utils as upstream

            layout = getattr(upstream, "_KV_CACHE_LAYOUT_OVERRIDE", None)
        except Exception:  # noqa: BLE001
            layout = None
    if layout is None:
        return None
    layout = str(layout).upper()
    if layout not in ("NHD", "HND"):
        raise ValueError(f"Unknown cache layout: {layout}")
    return layout


# The order this backend allocates its cache in when nobody has asked for one.  On MI355X a kv head's
# records of a block lying back to back (HND) let the decode kernel stream whole aligned runs past the
# caches; token-major blocks (NHD) read 10 % slower.
DEFAULT_KV_CACHE_LAYOUT = "HND"


def get_kv_cache_layout() -> str:
    """Physical order of the per-token-head cache, "HND" or "NHD".

    The reference asks upstream ``get_kv_cache_layout()``
    (vllm_metax/v1/attention/backends/triton_attn.py:356), which reads the ``VLLM_KV_CACHE_LAYOUT``
    environment variable; an explicit setting is honoured here the same way.  With no setting the
    reference's backend gets upstream's default; this backend owns the static that answers
    (``get_kv_cache_stride_order``, :350-372) and answers ``DEFAULT_KV_CACHE_LAYOUT``, the order its
    kernels read fastest.  Both orders are served by every kernel."""
    return _explicit_kv_cache_layout() or DEFAULT_KV_CACHE_LAYOUT


def kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                   cache_dtype_str: str = INT8_PER_TOKEN_HEAD) -> tuple[int, ...]:
    """Logical cache shape (vllm_metax/v1/attention/backends/triton_attn.py:318-348)."""
    if block_size % 16 != 0:
        raise ValueError("Block size must be a multiple of 16.")
    if kv_cache_uses_per_token_head_scales(cache_dtype_str):
        if cache_dtype_str not in (INT8_PER_TOKEN_HEAD, FP8_PER_TOKEN_HEAD, INT4_PER_TOKEN_HEAD):
            raise NotImplementedError(f"kv cache dtype {cache_dtype_str!r}: {INT8_PER_TOKEN_HEAD!r}, "
                                      f"{FP8_PER_TOKEN_HEAD!r} and {INT4_PER_TOKEN_HEAD!r} are built")
        scale_pad = SCALE_BYTES // torch.int8.itemsize   # fp8 and packed int4 elements are one byte as well
        # INT4 packs two values per byte, so the data occupies only head_size // 2 bytes (:332-346)
        data_head_size = head_size // 2 if cache_dtype_str == INT4_PER_TOKEN_HEAD else head_size
        if cache_dtype_str == INT4_PER_TOKEN_HEAD and head_size % 8:
            raise ValueError("int4 codes need a head size that is a multiple of 8 (4-byte aligned records)")
        return (num_blocks, num_kv_heads, block_size, 2 * (data_head_size + scale_pad))
    return (num_blocks, num_kv_heads, block_size, 2 * head_size)


def kv_cache_stride_order(include_num_layers_dimension: bool = False, layout: str | None = None) -> tuple[int, ...]:
    """Permutation from the logical shape to memory order
    (vllm_metax/v1/attention/backends/triton_attn.py:350-372)."""
    layout = layout or get_kv_cache_layout()
    if layout == "NHD":
        return (1, 0, 3, 2, 4) if include_num_layers_dimension else (0, 2, 1, 3)
    if layout == "HND":
        return (1, 2, 0, 3, 4) if include_num_layers_dimension else (0, 1, 2, 3)
    raise ValueError(f"Unknown cache layout: {layout}")


def allocate_kv_cache(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                      device="cuda", layout: str | None = None, fill: int | None = 0,
                      cache_dtype_str: str = INT8_PER_TOKEN_HEAD) -> torch.Tensor:
    """Allocate the cache the way the model runner does: physical tensor in stride
    order, returned permuted back to the logical ``(nb, Hkv, bs, 2*(D+4))`` shape
    (``2*(D/2+4)`` for int4 codes)."""
    shape = kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size, cache_dtype_str)
    order = kv_cache_stride_order(layout=layout)
    phys_shape = tuple(shape[i] for i in order)
    phys = torch.empty(phys_shape, dtype=torch.int8, device=device)
    if fill is not None:
        phys.fill_(fill)
    inv = [order.index(i) for i in range(len(order))]
    return phys.permute(*inv)


def key_value_views(kv_cache: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(nb, bs, Hkv, D+4)`` int8 views of the K and V halves; the last four
    "elements" of each row are the scale bytes
    (vllm_metax/v1/attention/backends/triton_attn.py:729-739)."""
    padded = kv_cache.shape[-1] // 2
    k, v = kv_cache.transpose(1, 2).split(padded, dim=-1)
    return k, v


def scale_views(kv_cache: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 strided views ``(nb, bs, Hkv)`` over the inline scale bytes
    (vllm_metax/v1/attention/backends/triton_attn.py:418-479).  Does NOT fill them;
    the backend fills 1.0 once at first use like the reference (:470, 479)."""
    num_blocks, nkv, block_size, content = kv_cache.shape
    esz = kv_cache.element_size()
    if esz != 1:
        raise ValueError("int8 cache expected")
    padded = content // 2
    hs = padded - SCALE_BYTES

    def f32_units(nbytes: int) -> int:
        if nbytes % 4:
            raise ValueError("cache strides/offsets must be multiples of 4 bytes")
        return nbytes // 4

    sb, sh, ss, se = kv_cache.stride()
    if se != 1:
        raise ValueError("content dim of the cache must be contiguous")
    base = torch.tensor([], dtype=torch.float32, device=kv_cache.device).set_(kv_cache.untyped_storage())
    off0 = f32_units(kv_cache.storage_offset())
    size = (num_blocks, block_size, nkv)
    stride = (f32_units(sb), f32_units(ss), f32_units(sh))
    k_scale = torch.as_strided(base, size, stride, off0 + f32_units(hs))
    v_scale = torch.as_strided(base, size, stride, off0 + f32_units(padded + hs))
    return k_scale, v_scale


@dataclass(frozen=True)
class CacheGeometry:
    """Byte geometry handed to the C ABI (``kvq_cache_geom``), derived from the
    typed views the same way a torch op would read ``tensor.stride()``."""

    k_off: int
    v_off: int
    ks_off: int
    vs_off: int
    stride_block: int
    stride_slot: int
    stride_head: int
    num_kv_heads: int
    head_size: int
    block_size: int
    num_blocks: int
    base_ptr: int
    code_type: int = _C.KVQ_CODE_INT8   # what a code byte is: int8, or an e4m3fn bit pattern

    def with_code_type(self, code_type: int) -> "CacheGeometry":
        """The same bytes read as another kind of code.  Offsets and strides do not depend on it; the head
        size does for int4 codes, two of which share a byte."""
        if code_type == self.code_type:
            return self
        others = self.__dict__.get("_others")
        if others is None:
            others = {}
            object.__setattr__(self, "_others", others)
        got = others.get(code_type)
        if got is None:
            d = {k: v for k, v in self.__dict__.items() if not k.startswith("_")}
            d["code_type"] = code_type
            d["head_size"] = self.code_bytes * 2 if code_type == _C.KVQ_CODE_INT4 else self.code_bytes
            got = CacheGeometry(**d)
            others[code_type] = got
        return got

    @property
    def code_bytes(self) -> int:
        """Code bytes of one half (K or V) of a record."""
        return self.head_size // 2 if self.code_type == _C.KVQ_CODE_INT4 else self.head_size

    def as_struct(self) -> "_C.CacheGeom":
        """The ctypes struct, built once per geometry object (it is read-only for the library)."""
        st = self.__dict__.get("_struct")
        if st is None:
            st = _C.CacheGeom(self.k_off, self.v_off, self.ks_off, self.vs_off, self.stride_block,
                              self.stride_slot, self.stride_head, self.num_kv_heads, self.head_size,
                              self.block_size, self.code_type)
            object.__setattr__(self, "_struct", st)
        return st

    @property
    def record_bytes(self) -> int:
        return 2 * (self.code_bytes + SCALE_BYTES)


_ONE_BYTE_DTYPES = tuple(d for d in (torch.int8, torch.uint8, getattr(torch, "float8_e4m3fn", None)) if d is not None)


def code_type_of(kv_quant_mode) -> int:
    """``kvq_cache_geom.code_type`` of a KV quantisation mode."""
    if kv_quant_mode == KVQuantMode.INT8_PER_TOKEN_HEAD:
        return _C.KVQ_CODE_INT8
    if kv_quant_mode == KVQuantMode.FP8_PER_TOKEN_HEAD:
        return _C.KVQ_CODE_FP8_E4M3
    if kv_quant_mode == KVQuantMode.INT4_PER_TOKEN_HEAD:
        return _C.KVQ_CODE_INT4
    raise NotImplementedError(f"kv_quant_mode {kv_quant_mode!r}: the per-token-head modes (int8, fp8, int4) are built")


def geometry_from_views(key_cache: torch.Tensor, value_cache: torch.Tensor,
                        k_scale_cache: torch.Tensor, v_scale_cache: torch.Tensor,
                        code_type: int = _C.KVQ_CODE_INT8) -> CacheGeometry:
    """Validate the four views and reduce them to one base pointer + byte geometry.

    key_cache / value_cache: ``(nb, bs, Hkv, D+4)`` of a one-byte dtype (int8; uint8 or float8_e4m3fn
    for fp8 codes; ``D/2+4`` bytes for int4 codes); scale caches ``(nb, bs, Hkv)`` fp32 over the same
    storage, all four with identical block/slot/head byte strides."""
    if key_cache.dtype not in _ONE_BYTE_DTYPES or value_cache.dtype != key_cache.dtype:
        raise ValueError("key_cache/value_cache must share a one-byte dtype (int8, uint8 or float8_e4m3fn)")
    if k_scale_cache.dtype != torch.float32 or v_scale_cache.dtype != torch.float32:
        raise ValueError("scale caches must be float32")
    if key_cache.dim() != 4 or key_cache.shape != value_cache.shape:
        raise ValueError("key_cache/value_cache must be (num_blocks, block_size, num_kv_heads, head_size+4)")
    nb, bs, hkv, padded = key_cache.shape
    if tuple(k_scale_cache.shape) != (nb, bs, hkv) or tuple(v_scale_cache.shape) != (nb, bs, hkv):
        raise ValueError("scale caches must be (num_blocks, block_size, num_kv_heads)")
    if key_cache.stride(-1) != 1 or value_cache.stride() != key_cache.stride():
        raise ValueError("key_cache/value_cache must share strides with a contiguous last dim")
    sb, ss, sh, _ = key_cache.stride()
    for t in (k_scale_cache, v_scale_cache):
        if tuple(4 * s for s in t.stride()) != (sb, ss, sh):
            raise ValueError("scale caches must have the same block/slot/head byte strides as the code views")
    base = min(key_cache.data_ptr(), value_cache.data_ptr(), k_scale_cache.data_ptr(), v_scale_cache.data_ptr())
    geom = CacheGeometry(
        k_off=key_cache.data_ptr() - base, v_off=value_cache.data_ptr() - base,
        ks_off=k_scale_cache.data_ptr() - base, vs_off=v_scale_cache.data_ptr() - base,
        stride_block=sb, stride_slot=ss, stride_head=sh,
        num_kv_heads=hkv, head_size=(padded - SCALE_BYTES) * (2 if code_type == _C.KVQ_CODE_INT4 else 1),
        block_size=bs, num_blocks=nb, base_ptr=base, code_type=code_type,
    )
    if any(v % 4 for v in (geom.k_off, geom.v_off, geom.ks_off, geom.vs_off, sb, ss, sh, base)):
        raise ValueError("cache views must be 4-byte aligned")
    return geom


def geometry_from_cache(kv_cache: torch.Tensor) -> CacheGeometry:
    k, v = key_value_views(kv_cache)
    ks, vs = scale_views(kv_cache)
    return geometry_from_views(k, v, ks, vs)


# ---------------------------------------------------------------------------
# MLA latent cache (int8 codes + one fp32 scale per token)
# ---------------------------------------------------------------------------

def mla_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int = 1, head_size: int = 576,
                    cache_dtype_str: str = INT8_PER_TOKEN) -> tuple[int, ...]:
    """Rank and first two dims of MLACommonBackend.get_kv_cache_shape
    (vllm_metax/model_executor/layers/attention/mla_attention.py:1166-1174); the entry
    grows by the 4 scale bytes for the int8 latent cache."""
    if cache_dtype_str == INT8_PER_TOKEN:
        return (num_blocks, block_size, head_size + SCALE_BYTES)
    return (num_blocks, block_size, head_size)


def allocate_mla_cache(num_blocks: int, block_size: int, head_size: int = 576, device="cuda",
                       fill: int | None = 0) -> torch.Tensor:
    t = torch.empty(mla_cache_shape(num_blocks, block_size, 1, head_size), dtype=torch.int8, device=device)
    if fill is not None:
        t.fill_(fill)
    return t


def mla_cache_views(cache: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Typed views of the int8 latent cache ``(nb, bs, W+4)``: codes ``(nb, bs, W)`` int8
    (rows first) and scales ``(nb, bs)`` fp32 (scale region after the rows)."""
    if cache.dtype != torch.int8 or cache.dim() != 3 or not cache.is_contiguous():
        raise ValueError("MLA int8 cache must be a contiguous int8 (num_blocks, block_size, W+4) tensor")
    nb, bs, entry = cache.shape
    w = entry - SCALE_BYTES
    block_bytes = bs * entry
    if (bs * w) % 4 or block_bytes % 4 or cache.storage_offset() % 4:
        raise ValueError("MLA int8 cache blocks must be 4-byte aligned")
    codes = torch.as_strided(cache, (nb, bs, w), (block_bytes, w, 1), cache.storage_offset())
    base = torch.tensor([], dtype=torch.float32, device=cache.device).set_(cache.untyped_storage())
    scales = torch.as_strided(base, (nb, bs), (block_bytes // 4, 1), (cache.storage_offset() + bs * w) // 4)
    return codes, scales


@dataclass(frozen=True)
class MlaGeometry:
    """Byte geometry of the int8 latent cache handed to the C ABI (``kvq_mla_geom``); the codes are int8
    only, so there is no code type to carry."""

    stride_block: int
    stride_row: int
    scale_off: int
    kv_lora_rank: int
    rope_dim: int
    block_size: int
    num_blocks: int
    base_ptr: int

    def as_struct(self) -> "_C.MlaGeom":
        """The ctypes struct, built once per geometry object (it is read-only for the library)."""
        st = self.__dict__.get("_struct")
        if st is None:
            st = _C.MlaGeom(self.stride_block, self.stride_row, self.scale_off, self.kv_lora_rank,
                            self.rope_dim, self.block_size, 0)
            object.__setattr__(self, "_struct", st)
        return st


def mla_geometry(cache: torch.Tensor, kv_lora_rank: int) -> MlaGeometry:
    codes, scales = mla_cache_views(cache)
    nb, bs, w = codes.shape
    if not 0 < kv_lora_rank <= w:
        raise ValueError("kv_lora_rank out of range")
    return MlaGeometry(stride_block=codes.stride(0), stride_row=codes.stride(1),
                       scale_off=scales.data_ptr() - codes.data_ptr(), kv_lora_rank=kv_lora_rank,
                       rope_dim=w - kv_lora_rank, block_size=bs, num_blocks=nb, base_ptr=codes.data_ptr())

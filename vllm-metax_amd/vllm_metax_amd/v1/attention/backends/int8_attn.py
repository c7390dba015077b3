"""Attention backend for the int8 per-token-head KV cache on MI355X.

Host-side mirror of the reference's TRITON_ATTN backend for this path
(vllm_metax/v1/attention/backends/triton_attn.py): same class triple
(Backend / MetadataBuilder / Impl), same method names, argument meaning and error behaviour,
same cache tensor layout and scale views.  Where the reference calls upstream Triton kernels
(:688-725, :805-814) this calls the HIP kernels through ``_custom_ops``.  The classes are
duck-typed: they subclass upstream vLLM's base classes only when vLLM is importable, and read
from ``vllm_config`` / ``kv_cache_spec`` only the attributes the reference reads.
"""
from __future__ import annotations

import weakref
from dataclasses import dataclass
from typing import ClassVar

import torch

from .... import _custom_ops as ops
from ....kv_cache_interface import KVQuantMode, get_kv_quant_mode, kv_cache_uses_per_token_head_scales
from ....layout import (
    code_type_of,
    geometry_from_views,
    key_value_views,
    kv_cache_shape,
    kv_cache_stride_order,
    scale_views,
)

try:  # pragma: no cover - upstream vLLM is not installed in the build container
    from vllm.v1.attention.backend import AttentionCGSupport  # type: ignore
except Exception:  # noqa: BLE001
    import enum as _enum

    class AttentionCGSupport(_enum.Enum):
        """Stand-in for upstream's enum of the same name (what a builder promises to graph capture)."""

        ALWAYS = 3
        UNIFORM_BATCH = 2
        UNIFORM_SINGLE_TOKEN_DECODE = 1
        NEVER = 0

try:  # pragma: no cover - upstream vLLM is not installed in the build container
    from vllm.v1.attention.backend import (  # type: ignore
        AttentionBackend as _BackendBase,
        AttentionImpl as _ImplBase,
        AttentionMetadataBuilder as _BuilderBase,
        AttentionType,
        MultipleOf,
    )
except Exception:  # noqa: BLE001
    _BackendBase = object
    _ImplBase = object
    _BuilderBase = object

    class AttentionType:
        DECODER = "decoder"
        ENCODER = "encoder"
        ENCODER_ONLY = "encoder_only"
        ENCODER_DECODER = "encoder_decoder"

    @dataclass(frozen=True)
    class MultipleOf:
        base: int


@dataclass
class Int8AttentionMetadata:
    """Fields of TritonAttentionMetadata that this path reads
    (vllm_metax/v1/attention/backends/triton_attn.py:60-99), plus the pre-sized split-K workspace
    that takes the place of the reference's softmax_segm_* scratch (:155-176)."""

    num_actual_tokens: int
    max_query_len: int
    query_start_loc: torch.Tensor
    max_seq_len: int
    seq_lens: torch.Tensor
    block_table: torch.Tensor
    slot_mapping: torch.Tensor
    workspace: torch.Tensor | None
    causal: bool = True
    prefill_splits: int = 1      # context splits of the long query runs (the builder's proposal for this launch)
    use_cascade: bool = False
    common_prefix_len: int = 0
    # False when the builder KNOWS (from the host copy of query_start_loc) that no sequence has exactly one query
    # row: the attention call then skips its decode kernels
    has_decode_rows: bool = True


def _first_attr(obj, *names, default=None):
    for n in names:
        v = getattr(obj, n, None)
        if v is not None:
            return v
    return default


class Int8AttentionMetadataBuilder(_BuilderBase):
    """Counterpart of TritonAttentionMetadataBuilder
    (vllm_metax/v1/attention/backends/triton_attn.py:102-269): packs the common metadata and owns
    the scratch that ``forward`` uses, sized once so a captured decode step never allocates."""

    # the kernels read lengths and tables on the device and nothing is allocated per step (:103)
    _cudagraph_support: ClassVar[AttentionCGSupport] = AttentionCGSupport.ALWAYS

    def __init__(self, kv_cache_spec, layer_names, vllm_config, device):
        if _BuilderBase is not object:  # pragma: no cover
            super().__init__(kv_cache_spec, layer_names, vllm_config, device)
        self.kv_cache_spec = kv_cache_spec
        self.layer_names = layer_names
        self.vllm_config = vllm_config
        self.device = torch.device(device)
        self.block_size = kv_cache_spec.block_size
        model_config = getattr(vllm_config, "model_config", None)
        parallel_config = getattr(vllm_config, "parallel_config", None)
        if model_config is not None and hasattr(model_config, "get_num_attention_heads"):
            self.num_heads_q = model_config.get_num_attention_heads(parallel_config)
            self.num_heads_kv = model_config.get_num_kv_heads(parallel_config)
            self.headdim = model_config.get_head_size()
        else:
            self.num_heads_kv = kv_cache_spec.num_kv_heads
            self.headdim = kv_cache_spec.head_size
            self.num_heads_q = _first_attr(kv_cache_spec, "num_q_heads", "num_heads", default=self.num_heads_kv)
        sched = getattr(vllm_config, "scheduler_config", None)
        self.max_num_seqs = int(_first_attr(sched, "max_num_seqs", default=256)) if sched is not None else 256
        self._workspace: torch.Tensor | None = None

    # query rows x context splits whose partial states the workspace has room for (a launch is split only when its
    # long runs are few: a small prefill chunk of a long request)
    MAX_SPLIT_TOKENS: ClassVar[int] = 4096

    def _get_workspace(self) -> torch.Tensor | None:
        if self._workspace is None and self.device.type == "cuda":
            # the plain workspace + the partial states of MAX_SPLIT_TOKENS (rows x splits)
            nbytes = ops.split_prefill_workspace_bytes(self.max_num_seqs, self.num_heads_q, self.headdim,
                                                       self.MAX_SPLIT_TOKENS // 2, 2)
            self._workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=self.device)
        return self._workspace

    def build_for_cudagraph_capture(self, common_attn_metadata) -> Int8AttentionMetadata:
        md = self.build(0, common_attn_metadata)
        # same trick as the reference (:184-194): capture with length-1 sequences
        md.seq_lens.fill_(1)
        return md

    def build(self, common_prefix_len: int, common_attn_metadata, fast_build: bool = False) -> Int8AttentionMetadata:
        if common_prefix_len > 0:
            raise NotImplementedError("cascade attention is not supported (the reference disables it too)")
        c = common_attn_metadata
        if c.num_reqs > self.max_num_seqs:
            raise RuntimeError(f"batch of {c.num_reqs} sequences exceeds max_num_seqs={self.max_num_seqs}")
        has_decode_rows = True
        prefill_splits = 1
        qsl_cpu = getattr(c, "query_start_loc_cpu", None)
        if qsl_cpu is not None and c.max_query_len > 1 and qsl_cpu.numel() > 1:
            qlens = qsl_cpu[1:] - qsl_cpu[:-1]
            has_decode_rows = bool((qlens == 1).any())
            # a launch whose long runs make too few workgroups for the chip walks a long context in context splits;
            # the partial states are indexed by the query row, so every row of the batch counts against the room
            prefill_splits = ops.prefill_context_splits(qlens, int(c.max_seq_len), self.num_heads_q, self.num_heads_kv,
                                                        max_split_tokens=self.MAX_SPLIT_TOKENS)
            while prefill_splits > 1 and prefill_splits * int(c.num_actual_tokens) > self.MAX_SPLIT_TOKENS:
                prefill_splits -= 1
        return Int8AttentionMetadata(
            has_decode_rows=has_decode_rows,
            prefill_splits=prefill_splits,
            num_actual_tokens=c.num_actual_tokens,
            max_query_len=c.max_query_len,
            query_start_loc=c.query_start_loc,
            max_seq_len=c.max_seq_len,
            seq_lens=c.seq_lens,
            block_table=c.block_table_tensor,
            slot_mapping=c.slot_mapping,
            workspace=self._get_workspace(),
            causal=bool(getattr(c, "causal", True)),
        )


class Int8AttentionBackend(_BackendBase):
    """Capability flags and cache geometry, as MacaTritonAttentionBackend
    (vllm_metax/v1/attention/backends/triton_attn.py:272-410)."""

    supported_dtypes: ClassVar[list[torch.dtype]] = [torch.float16, torch.bfloat16, torch.float32]
    supported_kv_cache_dtypes: ClassVar[list[str]] = ["int8_per_token_head", "fp8_per_token_head", "int4_per_token_head"]
    forward_includes_kv_cache_update: bool = False

    @staticmethod
    def get_name() -> str:
        return "TRITON_ATTN"  # the registry slot this backend takes over

    @staticmethod
    def get_supported_kernel_block_sizes():
        return [MultipleOf(16)]

    @classmethod
    def supports_block_size(cls, block_size: int | None) -> bool:
        return block_size is None or block_size % 16 == 0

    @classmethod
    def supports_head_size(cls, head_size: int) -> bool:
        return head_size in (64, 128, 256)

    @classmethod
    def supports_kv_cache_dtype(cls, kv_cache_dtype: str | None) -> bool:
        return kv_cache_dtype in cls.supported_kv_cache_dtypes

    @classmethod
    def supports_dtype(cls, dtype: torch.dtype) -> bool:
        return dtype in cls.supported_dtypes

    @classmethod
    def supports_attn_type(cls, attn_type: str) -> bool:
        """Decoder self-attention and cross-attention, the two types that go through the cache; the reference
        refuses a quantised cache for the encoder types too (triton_attn.py:759-764)."""
        return attn_type in (AttentionType.DECODER, AttentionType.ENCODER_DECODER)

    @classmethod
    def supports_non_causal(cls) -> bool:
        return True

    @classmethod
    def supports_sliding_window(cls) -> bool:
        return True

    @classmethod
    def supports_sink(cls) -> bool:
        return True   # triton_attn.py:390-392

    @classmethod
    def supports_batch_invariance(cls) -> bool:
        """triton_attn.py:310-312.  Served by the library's batch-invariant mode (on when VLLM_BATCH_INVARIANT
        is set, or through _custom_ops.set_batch_invariant): decode sequences are then cut by their own length
        alone, and prefill rows never depend on their neighbours."""
        return True

    @classmethod
    def supports_compute_capability(cls, capability) -> bool:
        return True

    @classmethod
    def validate_configuration(cls, head_size=None, dtype=None, kv_cache_dtype=None, block_size=None,
                               use_mla=False, attn_type=AttentionType.DECODER, has_sink=False,
                               use_sparse=False, **_ignored) -> list[str]:
        """Reasons this backend cannot serve a configuration (empty list = valid); the selection
        loop of the reference keeps the first backend with no reasons
        (vllm_metax/platform.py:386-416, 418-514)."""
        reasons = []
        if use_mla:
            reasons.append("MLA not supported")
        if use_sparse:
            reasons.append("sparse attention not supported")
        if head_size is not None and not cls.supports_head_size(head_size):
            reasons.append("head_size not supported")
        if dtype is not None and not cls.supports_dtype(dtype):
            reasons.append("dtype not supported")
        if not cls.supports_kv_cache_dtype(kv_cache_dtype):
            reasons.append("kv_cache_dtype not supported")
        if not cls.supports_block_size(block_size):
            reasons.append("block_size not supported")
        if not cls.supports_attn_type(attn_type):
            reasons.append("attention type not supported")
        return reasons

    @staticmethod
    def get_impl_cls():
        return Int8AttentionImpl

    @staticmethod
    def get_builder_cls():
        return Int8AttentionMetadataBuilder

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                           cache_dtype_str: str = "int8_per_token_head") -> tuple[int, ...]:
        return kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size, cache_dtype_str)

    @staticmethod
    def get_kv_cache_stride_order(include_num_layers_dimension: bool = False) -> tuple[int, ...]:
        return kv_cache_stride_order(include_num_layers_dimension)

    @staticmethod
    def use_cascade_attention(*args, **kwargs) -> bool:
        return False


class Int8AttentionImpl(_ImplBase):
    """Counterpart of TritonAttentionImpl for the per-token-head int8 cache
    (vllm_metax/v1/attention/backends/triton_attn.py:413-848)."""

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: int,
                 alibi_slopes: list[float] | None = None, sliding_window: int | None = None,
                 kv_cache_dtype: str = "int8_per_token_head", logits_soft_cap: float | None = None,
                 attn_type: str = AttentionType.DECODER, kv_sharing_target_layer_name: str | None = None,
                 sinks: torch.Tensor | None = None, use_alibi_sqrt: bool = False, chunk_lookback: int = -1) -> None:
        unsupported = {
            "use_alibi_sqrt": bool(use_alibi_sqrt),
            "kv_sharing_target_layer_name": kv_sharing_target_layer_name is not None,
            "chunk_lookback": chunk_lookback not in (-1, None),
        }
        bad = [k for k, v in unsupported.items() if v]
        if bad:  # the way TritonMLAImpl refuses features it lacks (mla/triton_mla.py:177-190)
            raise NotImplementedError(f"Int8AttentionImpl does not support: {', '.join(bad)}")
        if attn_type not in (AttentionType.DECODER, AttentionType.ENCODER_DECODER):   # triton_attn.py:759-764
            raise NotImplementedError("quantized KV cache is not supported for encoder attention")
        if attn_type == AttentionType.ENCODER_DECODER and alibi_slopes is not None:
            raise NotImplementedError("ALiBi needs causal attention")
        if not kv_cache_uses_per_token_head_scales(kv_cache_dtype) or get_kv_quant_mode(kv_cache_dtype) not in (
                KVQuantMode.INT8_PER_TOKEN_HEAD, KVQuantMode.FP8_PER_TOKEN_HEAD, KVQuantMode.INT4_PER_TOKEN_HEAD):
            raise ValueError("Int8AttentionImpl needs kv_cache_dtype 'int8_per_token_head', 'fp8_per_token_head' or 'int4_per_token_head', "
                             f"got {kv_cache_dtype!r}")
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if sinks is not None and sinks.shape[0] != num_heads:   # the reference's check, triton_attn.py:548-554
            raise ValueError(f"Sinks must have the same number of heads as the number of heads in the layer. "
                             f"Sinks shape: {tuple(sinks.shape)}, num_heads: {num_heads}.")
        # the kernels read the sinks as float32; converted once (a parameter in the model's dtype otherwise)
        self.sinks = None if sinks is None else sinks.detach().to(torch.float32).contiguous()
        # ALiBi slopes as a float32 tensor, as the reference keeps them (triton_attn.py:504-506)
        if alibi_slopes is not None:
            alibi_slopes = torch.as_tensor(alibi_slopes, dtype=torch.float32).contiguous()
            if tuple(alibi_slopes.shape) != (num_heads,):
                raise ValueError(f"alibi_slopes must have one slope per head ({num_heads}), got {tuple(alibi_slopes.shape)}")
        self.alibi_slopes = alibi_slopes
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.num_kv_heads = num_kv_heads
        self.num_queries_per_kv = num_heads // num_kv_heads
        self.kv_cache_dtype = kv_cache_dtype
        self.attn_type = attn_type
        # decoder attention only: (W - 1, 0), as at triton_attn.py:507-512; soft cap 0 = none (:536-539)
        if sliding_window is not None and sliding_window < 1:
            raise ValueError(f"sliding_window must be >= 1, got {sliding_window}")
        self.sliding_window = (-1, -1) if sliding_window is None else (sliding_window - 1, 0)
        self.logits_soft_cap = float(logits_soft_cap or 0)
        self._kv_quant_mode = get_kv_quant_mode(kv_cache_dtype)
        self._is_per_token_head_quant = True
        # per-cache views and byte geometry, built when a cache tensor is first seen
        self._filled: dict = {}          # (storage id, offset, shape, strides) -> weak reference to the storage
        self._views_for = None
        self._views_storage = None
        self._key_cache = self._value_cache = None
        self._k_scale_cache = self._v_scale_cache = None
        self._geometry = None

    def fused_output_quant_supported(self, quant_key) -> bool:
        return False

    def fused_rope_kvcache_supported(self) -> bool:
        """The reference answers False and raises in the method below (triton_attn.py:833-848); here the rotary
        embedding and the cache update are one launch."""
        return True

    def do_rope_and_kv_cache_update(self, layer, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                    positions: torch.Tensor, cos_sin_cache: torch.Tensor, is_neox: bool,
                                    kv_cache: torch.Tensor, layer_slot_mapping: torch.Tensor) -> None:
        """Signature of triton_attn.py:836-848.  ``query`` / ``key`` ``[T, H * D]`` or ``[T, H, D]`` are rotated in
        place, the rotated ``key`` and ``value`` quantised into ``kv_cache``."""
        if self.attn_type in (AttentionType.ENCODER_ONLY, AttentionType.ENCODER):
            return
        key_cache, value_cache = self._pth_key_value_caches(kv_cache)
        n = query.shape[0]
        ops.rope_and_cache_per_token_head_quant(
            positions, query.view(n, self.num_heads, self.head_size), key.view(n, self.num_kv_heads, self.head_size),
            value.view(n, self.num_kv_heads, self.head_size), cos_sin_cache, is_neox, key_cache, value_cache,
            self._k_scale_cache, self._v_scale_cache, layer_slot_mapping, kv_quant_mode=self._kv_quant_mode,
            geometry=self._geometry)

    def _sinks_on(self, device):
        if self.sinks is not None and self.sinks.device != device:
            self.sinks = self.sinks.to(device)
        return self.sinks

    def _alibi_on(self, device):
        if self.alibi_slopes is not None and self.alibi_slopes.device != device:
            self.alibi_slopes = self.alibi_slopes.to(device)
        return self.alibi_slopes

    # -- cache views ---------------------------------------------------------------------------
    def _ensure_scale_caches(self, kv_cache: torch.Tensor) -> None:
        """fp32 strided views over the inline scale bytes, as
        vllm_metax/v1/attention/backends/triton_attn.py:418-479.  The reference builds them -- and
        fills the scales with 1.0 -- once per impl, at first use; an impl here may meet several cache
        tensors (tests, a re-bound cache).  Views are held for the cache in use only, so a cache that
        was replaced is not kept alive; which caches have had their scales filled is remembered by
        the identity of their storage through weak references, so coming back to a cache never wipes
        the scales written into it, and a new allocation that lands on a freed cache's address is
        filled like any new cache."""
        storage = kv_cache.untyped_storage()
        key = (storage._cdata, kv_cache.storage_offset(), tuple(kv_cache.shape), tuple(kv_cache.stride()))
        if self._views_for == key and self._views_storage is storage:
            return
        seen = self._filled.get(key)
        k_scale, v_scale = scale_views(kv_cache)
        if seen is None or seen() is not storage:
            k_scale.fill_(1.0)
            v_scale.fill_(1.0)
            filled = self._filled
            self._filled[key] = weakref.ref(storage, lambda _r, key=key: filled.pop(key, None))
        key_cache, value_cache = key_value_views(kv_cache)
        self._key_cache, self._value_cache, self._k_scale_cache, self._v_scale_cache = key_cache, value_cache, k_scale, v_scale
        self._geometry = geometry_from_views(key_cache, value_cache, k_scale, v_scale, code_type_of(self._kv_quant_mode))
        self._views_for, self._views_storage = key, storage

    def _pth_key_value_caches(self, kv_cache: torch.Tensor):
        """(nb, bs, Hkv, D+4) int8 views of the K and V halves (:729-739)."""
        self._ensure_scale_caches(kv_cache)
        return self._key_cache, self._value_cache

    # -- the two per-layer calls ---------------------------------------------------------------
    def do_kv_cache_update(self, layer, key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor,
                           slot_mapping: torch.Tensor) -> None:
        """Quantise-on-write of this step's tokens; mutates ``kv_cache`` in place (:788-815)."""
        key_cache, value_cache = self._pth_key_value_caches(kv_cache)
        ops.reshape_and_cache_flash_per_token_head_quant(
            key, value, key_cache, value_cache, self._k_scale_cache, self._v_scale_cache, slot_mapping,
            kv_quant_mode=self._kv_quant_mode, geometry=self._geometry)

    def do_rope_and_kv_cache_update(self, *args, **kwargs):
        raise NotImplementedError("fused rope + cache update is not built (the reference raises here too)")

    def forward(self, layer, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor,
                attn_metadata: Int8AttentionMetadata | None, output: torch.Tensor,
                output_scale: torch.Tensor | None = None, output_block_scale: torch.Tensor | None = None) -> torch.Tensor:
        """Paged attention over the int8 cache (:577-727).  ``key`` / ``value`` are not read: this
        step's tokens are read back from the cache, where ``do_kv_cache_update`` has put them.
        Writes ``output[:num_actual_tokens]``; rows beyond stay untouched."""
        if output_scale is not None or output_block_scale is not None:
            raise NotImplementedError("fused output quantization is not supported")
        if attn_metadata is None:  # profiling run
            return output.fill_(0)
        if attn_metadata.use_cascade:
            raise NotImplementedError("cascade attention is not supported")
        n = attn_metadata.num_actual_tokens
        key_cache, value_cache = self._pth_key_value_caches(kv_cache)
        q = query[:n].view(n, self.num_heads, self.head_size)
        out = output[:n].view(n, self.num_heads, self.head_size)
        ops.unified_attention(
            q=q, k=key_cache, v=value_cache, out=out, cu_seqlens_q=attn_metadata.query_start_loc,
            max_seqlen_q=attn_metadata.max_query_len, seqused_k=attn_metadata.seq_lens,
            max_seqlen_k=attn_metadata.max_seq_len, softmax_scale=self.scale, causal=attn_metadata.causal,
            window_size=self.sliding_window, block_table=attn_metadata.block_table, softcap=self.logits_soft_cap,
            kv_quant_mode=self._kv_quant_mode, k_scale_cache=self._k_scale_cache, v_scale_cache=self._v_scale_cache,
            workspace=attn_metadata.workspace, geometry=self._geometry,
            has_decode_rows=getattr(attn_metadata, "has_decode_rows", True), sinks=self._sinks_on(q.device),
            alibi_slopes=self._alibi_on(q.device), prefill_splits=getattr(attn_metadata, "prefill_splits", 1))
        return output


class Int8FusedUpdateAttentionImpl(Int8AttentionImpl):
    """The same layer with the KV cache update inside ``forward``: a decode-only step is ONE launch (the
    attention kernel quantises each sequence's new token into the cache before it streams the tile that holds
    it; the slot comes from the block table and the sequence length, and a row whose ``slot_mapping`` entry is
    negative -- cudagraph padding -- is not written, as in the write kernel); a step with prefill rows falls
    back to the two calls, in this order, inside ``forward``."""

    def forward(self, layer, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor,
                attn_metadata: Int8AttentionMetadata | None, output: torch.Tensor,
                output_scale: torch.Tensor | None = None, output_block_scale: torch.Tensor | None = None) -> torch.Tensor:
        if output_scale is not None or output_block_scale is not None:
            raise NotImplementedError("fused output quantization is not supported")
        if attn_metadata is None:  # profiling run
            return output.fill_(0)
        if attn_metadata.use_cascade:
            raise NotImplementedError("cascade attention is not supported")
        n = attn_metadata.num_actual_tokens
        num_seqs = attn_metadata.seq_lens.shape[0]
        if attn_metadata.max_query_len != 1 or n != num_seqs or key is None or value is None:
            if key is not None and value is not None:
                self.do_kv_cache_update(layer, key[:n], value[:n], kv_cache, attn_metadata.slot_mapping[:n])
            return super().forward(layer, query, key, value, kv_cache, attn_metadata, output)
        key_cache, value_cache = self._pth_key_value_caches(kv_cache)
        ops.decode_attention_with_cache_update(
            q=query[:n].view(n, self.num_heads, self.head_size),
            key=key[:n].view(n, self.num_kv_heads, self.head_size),
            value=value[:n].view(n, self.num_kv_heads, self.head_size),
            k=key_cache, v=value_cache, out=output[:n].view(n, self.num_heads, self.head_size),
            seqused_k=attn_metadata.seq_lens, max_seqlen_k=attn_metadata.max_seq_len, softmax_scale=self.scale,
            block_table=attn_metadata.block_table, k_scale_cache=self._k_scale_cache, v_scale_cache=self._v_scale_cache,
            window_size=self.sliding_window, softcap=self.logits_soft_cap, kv_quant_mode=self._kv_quant_mode,
            workspace=attn_metadata.workspace, geometry=self._geometry,
            slot_mapping=attn_metadata.slot_mapping[:n] if attn_metadata.slot_mapping is not None else None,
            sinks=self._sinks_on(query.device), alibi_slopes=self._alibi_on(query.device))
        return output


class Int8FusedUpdateAttentionBackend(Int8AttentionBackend):
    """``Int8AttentionBackend`` with ``forward_includes_kv_cache_update`` set (the reference's attribute of that
    name, vllm_metax/v1/attention/backends/triton_attn.py:296): the layer then does not call
    ``do_kv_cache_update`` and hands key and value to ``forward``."""

    forward_includes_kv_cache_update: bool = True

    @staticmethod
    def get_impl_cls():
        return Int8FusedUpdateAttentionImpl

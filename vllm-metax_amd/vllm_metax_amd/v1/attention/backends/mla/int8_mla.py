"""MLA backend over the int8 latent cache on MI355X.

Host-side mirror of the reference's TRITON_MLA backend
(vllm_metax/v1/attention/backends/mla/triton_mla.py): ``forward_mqa`` has the reference's
signature and returns ``(o, lse)``; the cache write keeps ``concat_and_cache_mla``'s argument
order; ``forward_mha`` is the prefill half of the MLA layer with its chunked context
(vllm_metax/model_executor/layers/attention/mla_attention.py:2298-2378).  The int8 latent entry (576 codes + one fp32 scale per token, rows first and the scale
region after them inside each block) is this build's: the reference's MLA backends stop at fp8
(:94-100).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import torch

from ..... import _custom_ops as ops
from .....kv_cache_interface import INT8_PER_TOKEN
from .....layout import mla_cache_shape, mla_geometry
from ..int8_attn import AttentionCGSupport, AttentionType, MultipleOf, _BackendBase, _BuilderBase, _first_attr
from .prefill import (Int8MLAPrefillBackend, Int8MLAPrefillMetadata, build_mla_chunked_context_metadata,
                      compute_prefill_context, determine_chunked_prefill_workspace_size)

try:  # pragma: no cover - upstream vLLM is not installed in the build container
    from vllm.v1.attention.backend import MLAAttentionImpl as _MLAImplBase  # type: ignore
except Exception:  # noqa: BLE001
    _MLAImplBase = object

# The number of KV splits (the reference's _compute_num_kv_splits, mla/triton_mla.py:42-55, and its one split
# under VLLM_BATCH_INVARIANT, :247-253) is chosen inside the library: by the batch and the device's CUs, or, in
# the batch-invariant mode (_custom_ops.set_batch_invariant), a fixed count that depends on nothing.


@dataclass
class Int8MLADecodeMetadata:
    """The decode half of the MLA metadata, fields of MLACommonDecodeMetadata that ``forward_mqa`` reads
    (vllm_metax/v1/attention/backends/mla/triton_mla.py:283-284)."""

    block_table: torch.Tensor
    seq_lens: torch.Tensor


@dataclass
class Int8MLAMetadata:
    """What the MLA layer and ``forward_mqa`` read of MLACommonMetadata
    (vllm_metax/model_executor/layers/attention/mla_attention.py:1384-1440): the split of the batch into
    decode requests (first, one token each) and prefill requests, and the decode half; plus the buffers
    the builder owns so that a decode step allocates nothing."""

    num_actual_tokens: int
    num_reqs: int
    max_query_len: int
    max_seq_len: int
    query_start_loc: torch.Tensor
    slot_mapping: torch.Tensor
    num_decodes: int
    num_decode_tokens: int
    num_prefills: int
    decode: Int8MLADecodeMetadata | None
    prefill: Int8MLAPrefillMetadata | None = None
    workspace: torch.Tensor | None = None   # split states + int8 query terms of the decode launch
    decode_out: torch.Tensor | None = None  # [max_num_seqs, H, kv_lora_rank]
    decode_lse: torch.Tensor | None = None  # [max_num_seqs, H] fp32


class Int8MLAMetadataBuilder(_BuilderBase):
    """Counterpart of TritonMLAMetadataBuilder (vllm_metax/v1/attention/backends/mla/triton_mla.py:57-88) and
    of the decode side of MLACommonMetadataBuilder.build (mla_attention.py:1753-1960): decode requests come
    first in the batch (``reorder_batch_threshold = 1``, mla_attention.py:1546-1551) and are split off on
    the host copy of the lengths, with no device synchronisation; the decode launch's scratch is reserved
    once, at the worst case (``max_num_seqs`` decode tokens), as ``_reserve_attn_logits_workspace`` does,
    so a step -- captured or not -- never allocates."""

    _cudagraph_support: ClassVar[AttentionCGSupport] = AttentionCGSupport.UNIFORM_SINGLE_TOKEN_DECODE
    reorder_batch_threshold: int = 1

    def __init__(self, kv_cache_spec, layer_names, vllm_config, device):
        if _BuilderBase is not object:  # pragma: no cover
            super().__init__(kv_cache_spec, layer_names, vllm_config, device)
        self.kv_cache_spec = kv_cache_spec
        self.layer_names = layer_names
        self.vllm_config = vllm_config
        self.device = torch.device(device)
        model_config = getattr(vllm_config, "model_config", None)
        parallel_config = getattr(vllm_config, "parallel_config", None)
        if model_config is not None and hasattr(model_config, "get_num_attention_heads"):
            self.num_heads = model_config.get_num_attention_heads(parallel_config)
        else:
            self.num_heads = _first_attr(kv_cache_spec, "num_q_heads", "num_heads", default=None)
        hf = getattr(getattr(model_config, "hf_text_config", None), "kv_lora_rank", None)
        self.kv_lora_rank = int(hf or _first_attr(kv_cache_spec, "kv_lora_rank", default=512))
        sched = getattr(vllm_config, "scheduler_config", None)
        self.max_num_seqs = int(_first_attr(sched, "max_num_seqs", default=256)) if sched is not None else 256
        self.dtype = _first_attr(model_config, "dtype", default=torch.bfloat16) if model_config is not None \
            else torch.bfloat16
        self._workspace = self._out = self._lse = None
        self._reserve_decode_buffers()
        # prefill side: the context workspace (mla_attention.py:1554-1582, 1668-1690) and the attention calls
        hf_cfg = getattr(model_config, "hf_text_config", None)
        self.qk_nope_head_dim = int(getattr(hf_cfg, "qk_nope_head_dim", 128) or 128)
        self.qk_rope_head_dim = int(getattr(hf_cfg, "qk_rope_head_dim", 64) or 64)
        self.v_head_dim = int(getattr(hf_cfg, "v_head_dim", 128) or 128)
        self.block_size = int(_first_attr(kv_cache_spec, "block_size", default=64))
        max_model_len = int(_first_attr(model_config, "max_model_len", default=0) or 0) if model_config is not None else 0
        self.chunked_prefill_workspace_size = int(
            _first_attr(vllm_config, "mla_chunked_prefill_workspace_size", default=0)
            or determine_chunked_prefill_workspace_size(max_model_len or 8192, self.max_num_seqs, self.block_size))
        self._chunked_prefill_workspace = None
        self._prefill_backend = None
        if self.num_heads is not None:
            scale = (self.qk_nope_head_dim + self.qk_rope_head_dim) ** -0.5
            self._prefill_backend = Int8MLAPrefillBackend(self.num_heads, scale, self.kv_lora_rank,
                                                          self.qk_nope_head_dim, self.qk_rope_head_dim,
                                                          self.v_head_dim, vllm_config)

    def _reserve_decode_buffers(self) -> None:
        if self.device.type != "cuda" or self.num_heads is None:
            return
        nbytes = ops.mla_decode_workspace_bytes(self.max_num_seqs, self.num_heads, self.kv_lora_rank)
        self._workspace = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=self.device)
        self._out = torch.empty((self.max_num_seqs, self.num_heads, self.kv_lora_rank), dtype=self.dtype,
                                device=self.device)
        self._lse = torch.empty((self.max_num_seqs, self.num_heads), dtype=torch.float32, device=self.device)

    def build_for_cudagraph_capture(self, common_attn_metadata) -> Int8MLAMetadata:
        md = self.build(0, common_attn_metadata)
        if md.decode is not None:
            md.decode.seq_lens.fill_(1)
        return md

    def build(self, common_prefix_len: int, common_attn_metadata, fast_build: bool = False) -> Int8MLAMetadata:
        c = common_attn_metadata
        if c.num_reqs > self.max_num_seqs:
            raise RuntimeError(f"batch of {c.num_reqs} sequences exceeds max_num_seqs={self.max_num_seqs}")
        qsl_cpu = getattr(c, "query_start_loc_cpu", None)
        if qsl_cpu is None:
            qsl_cpu = c.query_start_loc.cpu() if c.query_start_loc.is_cuda else c.query_start_loc
        qlens = (qsl_cpu[1:c.num_reqs + 1] - qsl_cpu[:c.num_reqs]).tolist()
        num_decodes = 0
        while num_decodes < len(qlens) and qlens[num_decodes] <= self.reorder_batch_threshold:
            num_decodes += 1
        if any(q <= self.reorder_batch_threshold for q in qlens[num_decodes:]):
            raise RuntimeError("decode requests must come first in the batch (reorder_batch_threshold = 1)")
        num_decode_tokens = int(qsl_cpu[num_decodes])
        decode = None
        if num_decodes > 0:
            decode = Int8MLADecodeMetadata(block_table=c.block_table_tensor[:num_decodes],
                                           seq_lens=c.seq_lens[:num_decodes])
        prefill = None
        if c.num_reqs > num_decodes:
            prefill = self._build_prefill(c, qsl_cpu, num_decodes)
        return Int8MLAMetadata(
            num_actual_tokens=c.num_actual_tokens, num_reqs=c.num_reqs, max_query_len=c.max_query_len,
            max_seq_len=c.max_seq_len, query_start_loc=c.query_start_loc, slot_mapping=c.slot_mapping,
            num_decodes=num_decodes, num_decode_tokens=num_decode_tokens, num_prefills=c.num_reqs - num_decodes,
            decode=decode, prefill=prefill, workspace=self._workspace, decode_out=self._out, decode_lse=self._lse)

    def _build_prefill(self, c, qsl_cpu: torch.Tensor, start: int) -> Int8MLAPrefillMetadata:
        """The prefill half of MLACommonMetadataBuilder.build (mla_attention.py:1784-1830): offsets relative
        to the first prefill token, context lengths from the host copy of the sequence lengths."""
        n = c.num_reqs
        seq_lens_cpu = _first_attr(c, "seq_lens_cpu_upper_bound", "seq_lens_cpu", default=None)
        if seq_lens_cpu is None:
            seq_lens_cpu = c.seq_lens.cpu()
        qlens = qsl_cpu[start + 1:n + 1] - qsl_cpu[start:n]
        context_lens = seq_lens_cpu[start:n].to(qlens.dtype) - qlens
        qsl_rel_cpu = (qsl_cpu[start:n + 1] - qsl_cpu[start]).to(torch.int32)
        qsl_rel = (c.query_start_loc[start:n + 1] - c.query_start_loc[start]).to(torch.int32)
        chunked = None
        if int(context_lens.max()) > 0:
            if self._chunked_prefill_workspace is None:
                self._chunked_prefill_workspace = torch.empty(
                    (self.chunked_prefill_workspace_size, self.kv_lora_rank + self.qk_rope_head_dim),
                    dtype=self.dtype, device=self.device)
            chunked = build_mla_chunked_context_metadata(
                context_lens_cpu=context_lens, prefill_query_start_loc_cpu=qsl_rel_cpu, num_prefills=n - start,
                chunked_prefill_workspace=self._chunked_prefill_workspace,
                chunked_prefill_workspace_size=self.chunked_prefill_workspace_size, block_size=self.block_size,
                align_chunk_to_block=True, device=self.device)
        md = Int8MLAPrefillMetadata(block_table=c.block_table_tensor[start:n], query_start_loc=qsl_rel,
                                    max_query_len=int(qlens.max()), chunked_context=chunked,
                                    prefill_backend=self._prefill_backend)
        if self._prefill_backend is not None:
            self._prefill_backend.prepare_metadata(md)
        return md


class Int8MLABackend(_BackendBase):
    supported_dtypes: ClassVar[list[torch.dtype]] = [torch.float16, torch.bfloat16]
    supported_kv_cache_dtypes: ClassVar[list[str]] = [INT8_PER_TOKEN]

    @staticmethod
    def get_name() -> str:
        return "TRITON_MLA"

    @staticmethod
    def get_supported_kernel_block_sizes():
        return [MultipleOf(16)]

    @classmethod
    def supports_block_size(cls, block_size: int | None) -> bool:
        return block_size is None or block_size % 16 == 0

    @classmethod
    def get_supported_head_sizes(cls) -> list[int]:
        return [576]

    @classmethod
    def supports_batch_invariance(cls) -> bool:
        """Served by the library's batch-invariant mode (VLLM_BATCH_INVARIANT, as mla/triton_mla.py:247-253 reads
        it): a fixed number of KV splits per sequence, merged in split order."""
        return True

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                           cache_dtype_str: str = INT8_PER_TOKEN) -> tuple[int, ...]:
        return mla_cache_shape(num_blocks, block_size, num_kv_heads, head_size, cache_dtype_str)

    @staticmethod
    def get_kv_cache_stride_order(include_num_layers_dimension: bool = False) -> tuple[int, ...]:
        return (1, 0, 2, 3) if include_num_layers_dimension else (0, 1, 2)

    @classmethod
    def validate_configuration(cls, head_size=None, dtype=None, kv_cache_dtype=None, block_size=None,
                               use_mla=True, attn_type=AttentionType.DECODER, use_sparse=False, **_ignored) -> list[str]:
        reasons = []
        if not use_mla:
            reasons.append("non-MLA not supported")
        if use_sparse:
            reasons.append("sparse attention not supported")
        if dtype is not None and dtype not in cls.supported_dtypes:
            reasons.append("dtype not supported")
        if kv_cache_dtype not in cls.supported_kv_cache_dtypes:
            reasons.append("kv_cache_dtype not supported")
        if not cls.supports_block_size(block_size):
            reasons.append("block_size not supported")
        if attn_type != AttentionType.DECODER:
            reasons.append("attention type not supported")
        return reasons

    @staticmethod
    def get_impl_cls():
        return Int8MLAImpl

    @staticmethod
    def get_builder_cls():
        return Int8MLAMetadataBuilder


class Int8MLAImpl(_MLAImplBase):
    """Decode half of TritonMLAImpl (vllm_metax/v1/attention/backends/mla/triton_mla.py:140-295)."""

    can_return_lse_for_decode: bool = True

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: int = 1,
                 alibi_slopes=None, sliding_window=None, kv_cache_dtype: str = INT8_PER_TOKEN,
                 logits_soft_cap=None, attn_type: str = AttentionType.DECODER,
                 kv_sharing_target_layer_name=None, kv_lora_rank: int = 512, qk_rope_head_dim: int = 64,
                 qk_nope_head_dim: int = 128, v_head_dim: int = 128, kv_b_proj=None, **mla_args) -> None:
        if any([alibi_slopes, sliding_window, logits_soft_cap]):
            raise NotImplementedError(
                "Int8MLAImpl does not support one of the following: alibi_slopes, sliding_window, logits_soft_cap")
        if attn_type != AttentionType.DECODER:
            raise NotImplementedError("Encoder self-attention and encoder/decoder cross-attention are not "
                                      "implemented for Int8MLAImpl")
        if kv_cache_dtype != INT8_PER_TOKEN:
            raise ValueError(f"Int8MLAImpl needs kv_cache_dtype {INT8_PER_TOKEN!r}, got {kv_cache_dtype!r}")
        self.num_heads = num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.kv_lora_rank = kv_lora_rank
        self.qk_rope_head_dim = qk_rope_head_dim
        self.qk_nope_head_dim = qk_nope_head_dim
        self.v_head_dim = v_head_dim
        self.kv_b_proj = kv_b_proj
        self.kv_cache_dtype = kv_cache_dtype
        self.supports_quant_query_input = False
        self._geometry = None
        self._geometry_for = None
        self._sm_count = None

    def _geom(self, cache: torch.Tensor):
        key = (cache.data_ptr(), tuple(cache.shape))
        if self._geometry_for != key:
            self._geometry = mla_geometry(cache, self.kv_lora_rank)
            self._geometry_for = key
        return self._geometry

    def do_kv_cache_update(self, kv_c_normed: torch.Tensor, k_pe: torch.Tensor, kv_cache: torch.Tensor,
                           slot_mapping: torch.Tensor, kv_cache_dtype: str | None = None, k_scale=None) -> None:
        """Quantise-on-write of the latent rows, call shape of the reference's MLA layer
        (vllm_metax/model_executor/layers/attention/mla_attention.py:633-640)."""
        ops.concat_and_cache_mla(kv_c_normed, k_pe.reshape(k_pe.shape[0], -1), kv_cache, slot_mapping,
                                 kv_cache_dtype or self.kv_cache_dtype, k_scale, geometry=self._geom(kv_cache))

    def forward_mqa(self, q, kv_c_and_k_pe_cache: torch.Tensor, attn_metadata, layer=None, new_rows=None):
        """``q`` [B, H, 576] or ``(ql_nope [B, H, 512], q_pe [B, H, 64])``; returns
        ``(o [B, H, kv_lora_rank], lse [B, H] float32)``, valid until the next decode call on the same
        metadata (see below).  ``new_rows`` = (kv_c_normed [B, R], k_pe [B, P]):
        the launch also writes the step's rows (see ``forward_mqa_with_cache_update``)."""
        assert kv_c_and_k_pe_cache.numel() > 0
        assert attn_metadata.decode is not None
        # a (ql_nope, q_pe) pair goes to the kernel as it is: the reference concatenates first
        # (vllm_metax/v1/attention/backends/mla/triton_mla.py:236-237)
        q0 = q[0] if type(q) is tuple else q
        B, H = q0.shape[0], q0.shape[1]
        # the builder's buffers when the metadata carries them (nothing is allocated then: the step can be
        # captured in a graph).  What is returned are views of them, and every layer of the KV-cache group
        # shares them through the same metadata: they are valid until the NEXT forward_mqa / decode_absorbed
        # call on this metadata -- the next layer's, in the same step.  A caller that keeps (o, lse) across
        # layers (a deferred merge) must copy them, or pass metadata without decode_out / decode_lse.
        o_buf, lse_buf = getattr(attn_metadata, "decode_out", None), getattr(attn_metadata, "decode_lse", None)
        if o_buf is not None and lse_buf is not None and o_buf.dtype == q0.dtype and o_buf.shape[0] >= B \
                and o_buf.shape[1] == H and o_buf.shape[2] == self.kv_lora_rank:
            o, lse = o_buf[:B], lse_buf[:B]
        else:
            o = torch.empty((B, H, self.kv_lora_rank), dtype=q0.dtype, device=q0.device)
            lse = torch.empty((B, H), dtype=torch.float32, device=q0.device)
        ops.mla_decode_int8(q, kv_c_and_k_pe_cache, o, lse, attn_metadata.decode.block_table,
                            attn_metadata.decode.seq_lens, self.scale, self.kv_lora_rank,
                            workspace=getattr(attn_metadata, "workspace", None),
                            geometry=self._geom(kv_c_and_k_pe_cache), new_rows=new_rows)
        return o, lse

    def forward_mqa_with_cache_update(self, q, kv_c_normed: torch.Tensor, k_pe: torch.Tensor,
                                      kv_c_and_k_pe_cache: torch.Tensor, attn_metadata, layer=None):
        """``do_kv_cache_update`` + ``forward_mqa`` of a decode-only batch (one new token per sequence, row i
        of ``kv_c_normed`` / ``k_pe`` at position ``seq_lens[i] - 1`` of sequence i) in one launch: the two
        calls the reference's MLA layer makes for such a batch
        (vllm_metax/model_executor/layers/attention/mla_attention.py:633-640, then forward_mqa,
        vllm_metax/v1/attention/backends/mla/triton_mla.py:226-295).  Same cache bytes, same result."""
        B = (q[0] if type(q) is tuple else q).shape[0]
        if kv_c_normed.shape[0] != B:
            raise RuntimeError("one new token per sequence: a batch with prefill tokens takes the two calls")
        return self.forward_mqa(q, kv_c_and_k_pe_cache, attn_metadata, layer,
                                new_rows=(kv_c_normed, k_pe.reshape(B, -1)))

    def _kv_up_proj(self, kv_c: torch.Tensor) -> torch.Tensor:
        if self.kv_b_proj is None:
            raise RuntimeError("forward_mha needs the layer's kv_b_proj (pass kv_b_proj= to the impl)")
        y = self.kv_b_proj(kv_c)
        y = y[0] if type(y) is tuple else y    # the reference's linear layers return (output, bias)
        return y.view(-1, self.num_heads, self.qk_nope_head_dim + self.v_head_dim)

    def forward_mha(self, q: torch.Tensor, kv_c_normed: torch.Tensor, k_pe: torch.Tensor,
                    kv_c_and_k_pe_cache: torch.Tensor, attn_metadata, k_scale=None,
                    output: torch.Tensor | None = None, output_scale=None) -> torch.Tensor:
        """Prefill tokens, signature of MLACommonImpl.forward_mha (mla_attention.py:2298-2378): ``q
        [T, H, nope + rope]``, ``kv_c_normed [T, kv_lora_rank]`` and ``k_pe [T, 1, rope]`` (or ``[T, rope]``)
        of the new tokens, ``output [T, H * v_head_dim]``.  The causal pass over the new tokens is merged
        with the attention over the cached context, which is read back from the int8 latent cache chunk by
        chunk (``compute_prefill_context``)."""
        prefill = attn_metadata.prefill
        assert prefill is not None and prefill.prefill_backend is not None
        if output_scale is not None:
            raise NotImplementedError("quantised attention output is not built")
        T = q.shape[0]
        if output is None:
            output = torch.empty((T, self.num_heads * self.v_head_dim), dtype=q.dtype, device=q.device)
        out3 = output.view(T, self.num_heads, self.v_head_dim)
        kv_nope = self._kv_up_proj(kv_c_normed)
        k_nope, v = kv_nope[..., :self.qk_nope_head_dim], kv_nope[..., self.qk_nope_head_dim:]
        k_pe2 = k_pe.reshape(T, -1)
        has_context = prefill.chunked_context is not None
        if not has_context:
            prefill.prefill_backend.run_prefill_new_tokens(q=q, k=(k_nope, k_pe2), v=v, return_softmax_lse=False,
                                                           out=out3)
            return output
        suffix_output, suffix_lse = prefill.prefill_backend.run_prefill_new_tokens(
            q=q, k=(k_nope, k_pe2), v=v, return_softmax_lse=True)
        context_output, context_lse = compute_prefill_context(
            q, kv_c_and_k_pe_cache, prefill, self._kv_up_proj, self.num_heads, self.kv_lora_rank,
            self.qk_nope_head_dim, self.v_head_dim, geometry=self._geom(kv_c_and_k_pe_cache))
        if not out3.is_contiguous():
            raise RuntimeError("output must be contiguous")
        ops.merge_attn_states(output=out3, prefix_output=context_output, prefix_lse=context_lse,
                              suffix_output=suffix_output, suffix_lse=suffix_lse,
                              prefill_tokens_with_context=prefill.chunked_context.prefill_tokens_with_context)
        return output


class Int8MLADecodeCaller:
    """The steps either side of ``forward_mqa`` in the reference's MLA layer
    (vllm_metax/model_executor/layers/attention/mla_attention.py:833-848, 857, 874, 902,
    1087-1110), for the plain (unquantised-weight) branch: Q absorption
    ``bmm(q_nope [N, B, P], W_UK_T [N, P, L])``, the decode, and the V up-projection
    ``bmm(o [N, B, L], W_UV [N, L, V])``.  The absorption runs inside the decode launch
    (``kvq_mla_decode_absorb_int8``): its product lands in the decode's int8 operand layout and is
    never stored in the activation type.  The up-projection is ``kvq_mla_v_up_proj``, a stream of the
    weights with the handful of decode rows as the MFMA's other operand.  fp32 activations (not a
    serving dtype) take the library GEMMs and the two-step path ``absorb_q`` + ``forward_mqa``."""

    def __init__(self, impl: Int8MLAImpl, W_UK_T: torch.Tensor, W_UV: torch.Tensor) -> None:
        N, P, L = W_UK_T.shape
        if N != impl.num_heads or L != impl.kv_lora_rank or W_UV.shape[0] != N or W_UV.shape[1] != L:
            raise ValueError("W_UK_T must be [num_heads, qk_nope_head_dim, kv_lora_rank] and W_UV "
                             "[num_heads, kv_lora_rank, v_head_dim]")
        self.impl = impl
        self.W_UK_T = W_UK_T
        self.W_UV = W_UV
        self.num_heads = N
        self.kv_lora_rank = L
        self.v_head_dim = W_UV.shape[2]

    def absorb_q(self, mqa_q_nope: torch.Tensor) -> torch.Tensor:
        """``[B, N, P]`` -> ``[B, N, L]`` as the library GEMM (a transposed view of the ``[N, B, L]``
        product): the separate first step of the reference, kept for fp32 and for comparison."""
        q = mqa_q_nope.transpose(0, 1)                       # (N, B, P)
        ql = q.new_empty((self.num_heads, q.shape[1], self.kv_lora_rank))
        torch.bmm(q, self.W_UK_T, out=ql)
        return ql.transpose(0, 1)

    def v_up_proj_library(self, x: torch.Tensor, out: torch.Tensor) -> None:
        """``x [B, N, L]`` -> ``out [B, N * V]`` as the library GEMM of the reference (strided views, no
        transposed copies): fp32 activations, shapes the kernel does not take, and comparison."""
        x = x.view(-1, self.num_heads, self.kv_lora_rank).transpose(0, 1)
        out = out.view(-1, self.num_heads, self.v_head_dim)
        torch.bmm(x, self.W_UV, out=out.transpose(0, 1))

    # Rows x heads up to which the weight stream (kvq_mla_v_up_proj) beats the library GEMM: measured through graph
    # replays at 128 heads, 5.9 against 8.8 us at 32 rows, 15.5 against 16.6 us at 256, 26.6 against 19.5 us at 512
    # (there the activations, not the weights, are the larger stream); at 16 heads it is ahead or level up to 1024.
    KERNEL_MAX_ROWS_X_HEADS = 256 * 128
    # Rows x heads up to which the absorption inside the decode launch is level with or ahead of the library GEMM
    # + decode (whole chain, 128 heads: 78.1 against 78.4 us at 64 rows, 116.9 against 116.2 us at 128, 124.9 against
    # 118.2 us at 256; 16 heads: 32.7 against 44.7 us at 64 rows, 107.6 against 110.2 us at 1024): the kernel writes
    # the int8 operands as 64-byte pieces of lines that two heads share, which a large batch of many heads pays for.
    ABSORB_MAX_ROWS_X_HEADS = 128 * 128

    def v_up_proj(self, x: torch.Tensor, out: torch.Tensor) -> None:
        """``x [B, N, L]`` -> ``out [B, N * V]``."""
        rows = x.numel() // (self.num_heads * self.kv_lora_rank)
        if x.dtype == torch.float32 or self.kv_lora_rank % 128 != 0 or self.v_head_dim % 128 != 0 \
                or rows * self.num_heads > self.KERNEL_MAX_ROWS_X_HEADS:
            self.v_up_proj_library(x, out)
            return
        ops.mla_v_up_proj(x.view(-1, self.num_heads, self.kv_lora_rank), self.W_UV,
                          out.view(-1, self.num_heads, self.v_head_dim))

    def decode_absorbed(self, mqa_q_nope: torch.Tensor, mqa_q_pe: torch.Tensor, kv_cache: torch.Tensor, attn_metadata):
        """Absorption + decode in one launch; returns ``(o [B, N, L], lse [B, N])`` like ``forward_mqa``
        (views of the builder's buffers when the metadata carries them: valid until the next decode call on
        this metadata, the next layer's included)."""
        impl = self.impl
        B = mqa_q_nope.shape[0]
        o_buf, lse_buf = getattr(attn_metadata, "decode_out", None), getattr(attn_metadata, "decode_lse", None)
        if o_buf is not None and lse_buf is not None and o_buf.dtype == mqa_q_nope.dtype and o_buf.shape[0] >= B \
                and o_buf.shape[1] == self.num_heads and o_buf.shape[2] == self.kv_lora_rank:
            o, lse = o_buf[:B], lse_buf[:B]
        else:
            o = torch.empty((B, self.num_heads, self.kv_lora_rank), dtype=mqa_q_nope.dtype, device=mqa_q_nope.device)
            lse = torch.empty((B, self.num_heads), dtype=torch.float32, device=mqa_q_nope.device)
        ops.mla_decode_absorb_int8(mqa_q_nope, self.W_UK_T, mqa_q_pe, kv_cache, o, lse, attn_metadata.decode.block_table,
                                   attn_metadata.decode.seq_lens, impl.scale, self.kv_lora_rank,
                                   workspace=getattr(attn_metadata, "workspace", None), geometry=impl._geom(kv_cache))
        return o, lse

    def forward_decode(self, mqa_q_nope: torch.Tensor, mqa_q_pe: torch.Tensor, kv_cache: torch.Tensor,
                       attn_metadata, out: torch.Tensor):
        """q_nope ``[B, N, P]``, q_pe ``[B, N, rope]`` (already rotated), writes ``out [B, N * V]``;
        returns the decode's ``lse [B, N]``."""
        if mqa_q_nope.dtype == torch.float32 or mqa_q_nope.shape[0] * self.num_heads > self.ABSORB_MAX_ROWS_X_HEADS:
            attn_out, lse = self.impl.forward_mqa((self.absorb_q(mqa_q_nope), mqa_q_pe), kv_cache, attn_metadata)
        else:
            attn_out, lse = self.decode_absorbed(mqa_q_nope, mqa_q_pe, kv_cache, attn_metadata)
        self.v_up_proj(attn_out, out)
        return lse

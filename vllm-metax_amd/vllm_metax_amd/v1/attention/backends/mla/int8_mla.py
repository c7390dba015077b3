"""MLA decode backend over the int8 latent cache on MI355X.

Host-side mirror of the reference's TRITON_MLA backend for the decode path
(vllm_metax/v1/attention/backends/mla/triton_mla.py): ``forward_mqa`` has the reference's
signature and returns ``(o, lse)``; the cache write keeps ``concat_and_cache_mla``'s argument
order.  The int8 latent entry (576 codes + one fp32 scale per token, rows first and the scale
region after them inside each block) is this build's: the reference's MLA backends stop at fp8
(:94-100).
"""
from __future__ import annotations

from typing import ClassVar

import torch

from ..... import _custom_ops as ops
from .....kv_cache_interface import INT8_PER_TOKEN
from .....layout import mla_cache_shape, mla_geometry
from ..int8_attn import AttentionType, MultipleOf

# num_kv_splits policy of the reference (vllm_metax/v1/attention/backends/mla/triton_mla.py:42-55)
_MIN_WORK_PER_SPLIT = 512
_SPLIT_OCCUPANCY_MULTIPLIER = 2


def _next_power_of_2(n: int) -> int:
    return 1 if n <= 1 else 1 << (n - 1).bit_length()


def _compute_num_kv_splits(max_seq_len: int, sm_count: int) -> int:
    ideal = _next_power_of_2(max(1, max_seq_len // _MIN_WORK_PER_SPLIT))
    return min(ideal, sm_count * _SPLIT_OCCUPANCY_MULTIPLIER)


class Int8MLABackend:
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


class Int8MLAImpl:
    """Decode half of TritonMLAImpl (vllm_metax/v1/attention/backends/mla/triton_mla.py:140-295)."""

    can_return_lse_for_decode: bool = True

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: int = 1,
                 alibi_slopes=None, sliding_window=None, kv_cache_dtype: str = INT8_PER_TOKEN,
                 logits_soft_cap=None, attn_type: str = AttentionType.DECODER,
                 kv_sharing_target_layer_name=None, kv_lora_rank: int = 512, qk_rope_head_dim: int = 64,
                 **mla_args) -> None:
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

    def forward_mqa(self, q, kv_c_and_k_pe_cache: torch.Tensor, attn_metadata, layer=None):
        """``q`` [B, H, 576] or ``(ql_nope [B, H, 512], q_pe [B, H, 64])``; returns
        ``(o [B, H, kv_lora_rank], lse [B, H] float32)``."""
        assert kv_c_and_k_pe_cache.numel() > 0
        assert attn_metadata.decode is not None
        # a (ql_nope, q_pe) pair goes to the kernel as it is: the reference concatenates first
        # (vllm_metax/v1/attention/backends/mla/triton_mla.py:236-237)
        q0 = q[0] if type(q) is tuple else q
        B, H = q0.shape[0], q0.shape[1]
        o = torch.empty((B, H, self.kv_lora_rank), dtype=q0.dtype, device=q0.device)
        lse = torch.empty((B, H), dtype=torch.float32, device=q0.device)
        ops.mla_decode_int8(q, kv_c_and_k_pe_cache, o, lse, attn_metadata.decode.block_table,
                            attn_metadata.decode.seq_lens, self.scale, self.kv_lora_rank,
                            workspace=getattr(attn_metadata, "workspace", None),
                            geometry=self._geom(kv_c_and_k_pe_cache))
        return o, lse


class Int8MLADecodeCaller:
    """The steps either side of ``forward_mqa`` in the reference's MLA layer
    (vllm_metax/model_executor/layers/attention/mla_attention.py:833-848, 857, 874, 902,
    1087-1110), for the plain (unquantised-weight) branch: Q absorption
    ``bmm(q_nope [N, B, P], W_UK_T [N, P, L])``, the decode, and the V up-projection
    ``bmm(o [N, B, L], W_UV [N, L, V])``.  The two products are library GEMMs, as they are there.
    What this path changes is the hand-off: the ``(ql_nope, q_pe)`` pair goes to the decode as the
    strided views the GEMM leaves -- neither the transposed copy nor the concatenation is made --
    and the decode's output feeds the second GEMM as a view as well."""

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
        """``[B, N, P]`` -> ``[B, N, L]`` (a transposed view of the ``[N, B, L]`` product)."""
        q = mqa_q_nope.transpose(0, 1)                       # (N, B, P)
        ql = q.new_empty((self.num_heads, q.shape[1], self.kv_lora_rank))
        torch.bmm(q, self.W_UK_T, out=ql)
        return ql.transpose(0, 1)

    def v_up_proj(self, x: torch.Tensor, out: torch.Tensor) -> None:
        """``x [B, N, L]`` -> ``out [B, N * V]``."""
        x = x.view(-1, self.num_heads, self.kv_lora_rank).transpose(0, 1)
        out = out.view(-1, self.num_heads, self.v_head_dim)
        torch.bmm(x, self.W_UV, out=out.transpose(0, 1))

    def forward_decode(self, mqa_q_nope: torch.Tensor, mqa_q_pe: torch.Tensor, kv_cache: torch.Tensor,
                       attn_metadata, out: torch.Tensor):
        """q_nope ``[B, N, P]``, q_pe ``[B, N, rope]`` (already rotated), writes ``out [B, N * V]``;
        returns the decode's ``lse [B, N]``."""
        ql_nope = self.absorb_q(mqa_q_nope)
        attn_out, lse = self.impl.forward_mqa((ql_nope, mqa_q_pe), kv_cache, attn_metadata)
        self.v_up_proj(attn_out, out)
        return lse


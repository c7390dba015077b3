"""Prefill half of the MLA layer over the int8 latent cache: chunked context.

Host-side mirror of what the reference's MLA layer does for prefill tokens whose sequences already have
context in the cache (vllm_metax/model_executor/layers/attention/mla_attention.py:1197-1232 the metadata,
:1352-1529 ``build_mla_chunked_context_metadata``, :1554-1582 the workspace size, :2017-2140
``_compute_prefill_context``, :2298-2378 ``forward_mha``) and of its prefill backend
(vllm_metax/v1/attention/backends/mla/prefill/base.py:114-176, flash_attn.py:176-221): the context is
walked in workspace-sized chunks -- gather + dequantise the chunk's latent rows, up-project them with
``kv_b_proj``, attend to them unmasked with the LSE kept, fold the chunk into the running state with the
LSE merge -- and the result is merged with the causal pass over the new tokens.

The arithmetic is in libkvq_hip.so (gather + dequantise, attention, merge); ``kv_b_proj`` stays the
library GEMM it is in the reference.  The attention kernel takes K in the two pieces the layer holds, so
the concatenated key of mla_attention.py:1995-2015 is never built.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..... import _custom_ops as ops


@dataclass
class ChunkedContextMetadata:
    """Fields of MLACommonPrefillMetadata.ChunkedContextMetadata (mla_attention.py:1201-1223) that the
    single-rank loop reads."""

    cu_seq_lens: torch.Tensor          # [num_chunks, num_prefills + 1] int32, device
    starts: torch.Tensor               # [num_chunks, num_prefills] int32, device
    seq_tot: list[int]                 # tokens gathered per chunk
    max_seq_lens: list[int]
    seq_lens: torch.Tensor             # [num_chunks, num_prefills] int32, host
    workspace: torch.Tensor            # [workspace_size, kv_lora_rank + rope_dim], model dtype
    token_to_seq: torch.Tensor         # [num_chunks, max tokens of a chunk] int32, device
    chunk_total_token: list[int]
    has_empty_context: list[bool]
    prefill_tokens_with_context: int


@dataclass
class Int8MLAPrefillMetadata:
    """MLACommonPrefillMetadata (mla_attention.py:1197-1232): prefill requests only, offsets from the
    first prefill token."""

    block_table: torch.Tensor
    query_start_loc: torch.Tensor
    max_query_len: int
    chunked_context: ChunkedContextMetadata | None = None
    prefill_backend: "Int8MLAPrefillBackend | None" = None


def determine_chunked_prefill_workspace_size(max_model_len: int, max_num_seqs: int, block_size: int) -> int:
    """Rows of the context workspace (mla_attention.py:1554-1582): eight full-length requests or four
    pages per request, at most 64k tokens, at least one page per request."""
    size = min(max(8 * max_model_len, 4 * max_num_seqs * block_size), 64 * 1024)
    return max(size, max_num_seqs * block_size)


def build_mla_chunked_context_metadata(*, context_lens_cpu: torch.Tensor, prefill_query_start_loc_cpu: torch.Tensor,
                                       num_prefills: int, chunked_prefill_workspace: torch.Tensor,
                                       chunked_prefill_workspace_size: int, block_size: int,
                                       align_chunk_to_block: bool = True,
                                       device: torch.device | str | None = None) -> ChunkedContextMetadata | None:
    """Split every prefill's context into chunks that fit the workspace together
    (mla_attention.py:1352-1529, single rank): each prefill with context gets an equal share of the
    workspace rows, rounded down to whole cache blocks; chunk ``i`` of prefill ``b`` covers context
    positions ``[i * share, min((i + 1) * share, context_len[b]))``.  ``None`` when no prefill has context."""
    ctx = context_lens_cpu.to(torch.int64).reshape(-1)[:num_prefills]
    max_ctx = int(ctx.max()) if num_prefills > 0 else 0
    if max_ctx <= 0:
        return None
    with_ctx = int((ctx > 0).sum())
    share = chunked_prefill_workspace_size // with_ctx
    if align_chunk_to_block:
        share = share // block_size * block_size
    if share <= 0:
        raise RuntimeError(f"context workspace of {chunked_prefill_workspace_size} rows is too small for "
                           f"{with_ctx} prefills with context at block size {block_size}")
    num_chunks = -(-max_ctx // share)
    starts = (torch.arange(num_chunks, dtype=torch.int64) * share)[:, None].expand(num_chunks, num_prefills)
    ends = torch.minimum(ctx[None, :], starts + share)
    lens = (ends - starts).clamp_(min=0)
    cu = torch.zeros(num_chunks, num_prefills + 1, dtype=torch.int64)
    torch.cumsum(lens, dim=1, out=cu[:, 1:])
    totals = cu[:, -1].tolist()
    token_to_seq = torch.zeros(num_chunks, max(totals), dtype=torch.int32)
    seq_ids = torch.arange(num_prefills, dtype=torch.int32)
    for i in range(num_chunks):
        token_to_seq[i, :totals[i]] = torch.repeat_interleave(seq_ids, lens[i])
    # rows past the last prefill that has context never need the merge; everything before it does (a row
    # without context in between carries lse = -inf and comes out as its suffix)
    last_with_ctx = int(torch.nonzero(ctx > 0).max())
    qsl = prefill_query_start_loc_cpu.reshape(-1)
    dev = device if device is not None else chunked_prefill_workspace.device
    md = ChunkedContextMetadata(
        cu_seq_lens=cu.to(torch.int32).to(dev, non_blocking=True),
        starts=starts.to(torch.int32).contiguous().to(dev, non_blocking=True),
        seq_tot=lens.sum(dim=1).tolist(), max_seq_lens=lens.max(dim=1).values.tolist(),
        seq_lens=lens.to(torch.int32), workspace=chunked_prefill_workspace,
        token_to_seq=token_to_seq.to(dev, non_blocking=True), chunk_total_token=totals,
        has_empty_context=(lens == 0).any(dim=1).tolist(),
        prefill_tokens_with_context=int(qsl[last_with_ctx + 1]))
    assert max(md.max_seq_lens) <= chunked_prefill_workspace_size
    return md


def _split_k(k, nope: int):
    """``(k_nope, k_pe)`` as given, or the two views of a concatenated ``[S, H, nope + rope]`` key (whose
    rope part is the same in every head, mla_attention.py:1995-2015)."""
    if type(k) is tuple:
        return k
    return k[..., :nope], (k[:, 0, nope:] if k.shape[-1] > nope else None)


class Int8MLAPrefillBackend:
    """The two attention calls of the MLA prefill (prefill/base.py:114-176, flash_attn.py:176-221), on
    ``kvq_mla_prefill_attn``.  ``k`` is ``(k_nope [S, H, nope], k_pe [S, rope] or [S, 1, rope])`` or the
    concatenated tensor."""

    def __init__(self, num_heads: int, scale: float, kv_lora_rank: int, qk_nope_head_dim: int,
                 qk_rope_head_dim: int, v_head_dim: int, vllm_config=None) -> None:
        self.num_heads = num_heads
        self.scale = float(scale)
        self.kv_lora_rank = kv_lora_rank
        self.qk_nope_head_dim = qk_nope_head_dim
        self.qk_rope_head_dim = qk_rope_head_dim
        self.v_head_dim = v_head_dim
        self.vllm_config = vllm_config
        self._prefill_metadata: Int8MLAPrefillMetadata | None = None

    @staticmethod
    def get_name() -> str:
        return "KVQ_HIP"

    def clone(self) -> "Int8MLAPrefillBackend":
        return self.__class__(self.num_heads, self.scale, self.kv_lora_rank, self.qk_nope_head_dim,
                              self.qk_rope_head_dim, self.v_head_dim, self.vllm_config)

    def prepare_metadata(self, prefill_metadata: Int8MLAPrefillMetadata) -> None:
        self._prefill_metadata = prefill_metadata

    def run_prefill_new_tokens(self, q: torch.Tensor, k, v: torch.Tensor, return_softmax_lse: bool,
                               out: torch.Tensor | None = None, output_scale=None):
        if output_scale is not None:
            raise NotImplementedError("quantised attention output is not built")
        md = self._prefill_metadata
        k_nope, k_pe = _split_k(k, self.qk_nope_head_dim)
        return ops.mla_prefill_attention(q, k_nope, k_pe, v, md.query_start_loc, md.query_start_loc, md.max_query_len,
                                         self.scale, causal=True, out=out, return_softmax_lse=return_softmax_lse)

    def run_prefill_context_chunk(self, chunk_idx: int, q: torch.Tensor, k, v: torch.Tensor):
        md = self._prefill_metadata
        k_nope, k_pe = _split_k(k, self.qk_nope_head_dim)
        return ops.mla_prefill_attention(q, k_nope, k_pe, v, md.query_start_loc,
                                         md.chunked_context.cu_seq_lens[chunk_idx], md.max_query_len, self.scale,
                                         causal=False, return_softmax_lse=True)


def compute_prefill_context(q: torch.Tensor, kv_c_and_k_pe_cache: torch.Tensor, prefill: Int8MLAPrefillMetadata,
                            kv_b_proj, num_heads: int, kv_lora_rank: int, qk_nope_head_dim: int, v_head_dim: int,
                            geometry=None):
    """The chunk loop of ``_compute_prefill_context`` (mla_attention.py:2017-2140) over the int8 latent
    cache; returns the context's ``(output [T, H, v_head_dim], lse [H, T])``."""
    cc = prefill.chunked_context
    backend = prefill.prefill_backend
    output = output_lse = merge_output = merge_lse = None
    for i in range(len(cc.seq_tot)):
        toks = cc.seq_tot[i]
        ops.gather_and_maybe_dequant_cache(
            src_cache=kv_c_and_k_pe_cache, dst=cc.workspace, block_table=prefill.block_table,
            cu_seq_lens=cc.cu_seq_lens[i], token_to_seq=cc.token_to_seq[i], num_tokens=cc.chunk_total_token[i],
            kv_cache_dtype="int8_per_token", seq_starts=cc.starts[i], kv_lora_rank=kv_lora_rank, geometry=geometry)
        rows = cc.workspace[:toks]
        kv_nope = kv_b_proj(rows[..., :kv_lora_rank])
        if type(kv_nope) is tuple:     # the linear layers of the reference return (output, bias)
            kv_nope = kv_nope[0]
        kv_nope = kv_nope.view(-1, num_heads, qk_nope_head_dim + v_head_dim)
        k_nope, v = kv_nope[..., :qk_nope_head_dim], kv_nope[..., qk_nope_head_dim:]
        k_pe = rows[..., kv_lora_rank:]
        # a prefill without rows in this chunk comes back with out = 0, lse = -inf from the kernel itself
        # (what mask_empty_context forces, mla_attention.py:2104-2110)
        attn_output, attn_lse = backend.run_prefill_context_chunk(chunk_idx=i, q=q, k=(k_nope, k_pe), v=v)
        if output is None:
            output, output_lse = attn_output, attn_lse
        else:
            if merge_output is None:
                merge_output, merge_lse = torch.empty_like(output), torch.empty_like(output_lse)
            ops.merge_attn_states(output=merge_output, output_lse=merge_lse, prefix_output=output,
                                  prefix_lse=output_lse, suffix_output=attn_output, suffix_lse=attn_lse)
            output, merge_output = merge_output, output
            output_lse, merge_lse = merge_lse, output_lse
    return output, output_lse

"""Python op layer: thin functions that validate torch tensors and call the C ABI.

Same convention as the reference's op layer (vllm_metax/_custom_ops.py:5-17,
137-166: a python function per op that forwards to the native library): ops return
``None``, mutate their output arguments in place, take strides from the tensors,
run on the current torch stream, and raise ``RuntimeError`` on bad arguments
(csrc/libtorch_stable/cache_kernels.cu:884-889).  torch is only the owner of device
memory and of the stream here; all arithmetic happens in libkvq_hip.so.
"""
from __future__ import annotations

import ctypes

import torch

from . import _C
from .kv_cache_interface import KVQuantMode
from .layout import QUANT_EPS, CacheGeometry, MlaGeometry, code_type_of, geometry_from_views, mla_geometry

_DTYPE_CODE = {torch.float32: _C.KVQ_F32, torch.bfloat16: _C.KVQ_BF16, torch.float16: _C.KVQ_F16}


def _dtype_code(t: torch.Tensor, what: str) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise RuntimeError(f"{what}: unsupported dtype {t.dtype}") from None


def _require_cuda(*tensors: torch.Tensor) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("int8 KV-cache ops need GPU tensors (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} vs {t.device}")
    return dev


class _on_device:
    """``torch.cuda.device(dev)`` that does nothing when ``dev`` is already current (the usual case on
    a per-step path; the context manager costs several microseconds of host time)."""

    __slots__ = ("_ctx",)

    def __init__(self, dev: torch.device):
        idx = dev.index if dev.index is not None else torch.cuda.current_device()
        self._ctx = None if idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)
        return False


# the raw handle of the current stream without building a torch.cuda.Stream object (4 us of host time per call,
# a quarter of a small decode step's)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev: torch.device) -> ctypes.c_void_p:
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(dev.index if dev.index is not None else torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _ptr(t) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_eps_cache: dict = {}


def eps_for_dtype(dtype: torch.dtype) -> float:
    """absmax floor as the reference's quantiser applies it: ``clamp(min=1e-10)`` in the
    SOURCE dtype, before the cast to fp32 (tests/kernels/quant_utils.py:212-213)."""
    got = _eps_cache.get(dtype)
    if got is None:
        got = float(torch.tensor(QUANT_EPS, dtype=torch.float64).to(dtype).to(torch.float32))
        _eps_cache[dtype] = got
    return got


def _check_sinks(sinks, num_q_heads: int, dev, what: str = "sinks") -> None:
    """Attention sinks (or ALiBi slopes) as the library takes them: contiguous float32 ``[num_q_heads]`` on the
    call's device."""
    if sinks is None:
        return
    if sinks.dtype != torch.float32 or not sinks.is_contiguous() or tuple(sinks.shape) != (num_q_heads,) \
            or sinks.device != dev:
        raise RuntimeError(f"{what} must be a contiguous float32 [num_q_heads] tensor on the device of q")


def device_num_cus() -> int:
    return int(_C.load().kvq_device_num_cus())


def set_batch_invariant(on: bool) -> bool:
    """Turn the library's batch-invariant mode on or off (process-wide; on at load time when the environment
    sets ``VLLM_BATCH_INVARIANT``, the variable the reference reads: mla/triton_mla.py:247-253).  While on, a
    decode row's bits depend on its own sequence only.  Workspaces must be sized AFTER the mode is set
    (``paged_attn_workspace_bytes`` / ``mla_decode_workspace_bytes`` return what the mode needs).  Returns the
    previous setting."""
    _ws_bytes_cache.clear()   # the remembered workspace sizes are those of the other mode
    return bool(_C.load().kvq_set_batch_invariant(1 if on else 0))


def batch_invariant() -> bool:
    return bool(_C.load().kvq_get_batch_invariant())


# ---------------------------------------------------------------------------------------------
# quantise-on-write
# ---------------------------------------------------------------------------------------------

def reshape_and_cache_flash_per_token_head_quant(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    k_scale_cache: torch.Tensor,
    v_scale_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    kv_quant_mode: KVQuantMode = KVQuantMode.INT8_PER_TOKEN_HEAD,
    geometry: CacheGeometry | None = None,
) -> None:
    """Drop-in for ``triton_reshape_and_cache_flash_per_token_head_quant`` as called at
    vllm_metax/v1/attention/backends/triton_attn.py:805-814.

    key/value ``[>= T, Hkv, D]``; key_cache/value_cache ``(nb, bs, Hkv, D+4)`` int8 views and
    k/v_scale_cache ``(nb, bs, Hkv)`` fp32 views of one cache; slot_mapping ``[T]`` int64
    (negative = padding, skipped).  ``geometry`` may carry the precomputed byte geometry of
    the four views so the per-step call does no view arithmetic.  ``kv_quant_mode``
    INT8_PER_TOKEN_HEAD (scale = absmax / 127, codes rint(x / scale)) or FP8_PER_TOKEN_HEAD
    (scale = absmax / 448, e4m3fn codes) -- the two one-byte modes of this record layout."""
    code_type = code_type_of(kv_quant_mode)   # int8, or the fp8 mode of the same record layout
    dev = _require_cuda(key, value, key_cache, value_cache, k_scale_cache, v_scale_cache, slot_mapping)
    geom = (geometry or geometry_from_views(key_cache, value_cache, k_scale_cache, v_scale_cache)).with_code_type(code_type)
    if key.dim() != 3 or value.shape != key.shape or key.dtype != value.dtype:
        raise RuntimeError("key/value must be [num_tokens, num_kv_heads, head_size] of one dtype")
    if key.shape[1] != geom.num_kv_heads or key.shape[2] != geom.head_size:
        raise RuntimeError(f"key shape {tuple(key.shape)} does not match cache (Hkv={geom.num_kv_heads}, D={geom.head_size})")
    if key.stride(2) != 1 or value.stride(2) != 1:
        raise RuntimeError("key/value head dim must be contiguous")
    if slot_mapping.dtype != torch.int64 or slot_mapping.dim() != 1 or not slot_mapping.is_contiguous():
        raise RuntimeError("slot_mapping must be a contiguous 1-D int64 tensor")
    num_tokens = slot_mapping.shape[0]
    if num_tokens > key.shape[0]:
        raise RuntimeError("slot_mapping is longer than key")
    lib = _C.load()
    g = geom.as_struct()
    with _on_device(dev):
        rc = lib.kvq_reshape_and_cache_int8(
            _ptr(key), _ptr(value), _dtype_code(key, "key"), key.stride(0), key.stride(1), value.stride(0),
            value.stride(1), ctypes.c_void_p(geom.base_ptr), ctypes.byref(g), _ptr(slot_mapping), num_tokens,
            eps_for_dtype(key.dtype), _stream(dev))
    _C.check(rc, "reshape_and_cache_flash_per_token_head_quant")


# name used at the reference's call site
triton_reshape_and_cache_flash_per_token_head_quant = reshape_and_cache_flash_per_token_head_quant


def rope_and_cache_per_token_head_quant(
    positions: torch.Tensor,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    cos_sin_cache: torch.Tensor,
    is_neox: bool,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    k_scale_cache: torch.Tensor,
    v_scale_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    kv_quant_mode: KVQuantMode = KVQuantMode.INT8_PER_TOKEN_HEAD,
    geometry: CacheGeometry | None = None,
) -> None:
    """Rotary embedding of ``query`` ``[T, Hq, D]`` and ``key`` ``[T, Hkv, D]`` (in place, their first ``rot_dim =
    cos_sin_cache.shape[1]`` dims) and the quantise-on-write of the rotated ``key`` and of ``value`` in ONE launch:
    the work of ``do_rope_and_kv_cache_update``, which the reference's backend declares and refuses
    (vllm_metax/v1/attention/backends/triton_attn.py:833-848).  Same results as the rotary embedding followed by
    ``reshape_and_cache_flash_per_token_head_quant``; tokens whose slot is negative are neither rotated nor
    written."""
    code_type = code_type_of(kv_quant_mode)
    dev = _require_cuda(positions, query, key, value, cos_sin_cache, key_cache, value_cache, k_scale_cache,
                        v_scale_cache, slot_mapping)
    geom = (geometry or geometry_from_views(key_cache, value_cache, k_scale_cache, v_scale_cache)).with_code_type(code_type)
    if query.dim() != 3 or key.dim() != 3 or value.dim() != 3 or not (query.dtype == key.dtype == value.dtype):
        raise RuntimeError("query [T, Hq, D], key and value [T, Hkv, D] must share one dtype")
    if key.shape != value.shape or key.shape[1] != geom.num_kv_heads or key.shape[2] != geom.head_size \
            or query.shape[2] != geom.head_size:
        raise RuntimeError(f"query / key / value shapes do not match the cache (Hkv={geom.num_kv_heads}, D={geom.head_size})")
    if query.stride(2) != 1 or key.stride(2) != 1 or value.stride(2) != 1:
        raise RuntimeError("query / key / value rows must be contiguous")
    if cos_sin_cache.dim() != 2 or not cos_sin_cache.is_contiguous():
        raise RuntimeError("cos_sin_cache must be a contiguous [max_position, rot_dim] tensor")
    rot = cos_sin_cache.shape[1]
    if rot % 2 or rot > geom.head_size:
        raise RuntimeError("rot_dim must be even and at most the head size")
    for name, t in (("positions", positions), ("slot_mapping", slot_mapping)):
        if t.dtype != torch.int64 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous int64")
    T = slot_mapping.shape[0]
    if positions.shape[0] < T or query.shape[0] < T or key.shape[0] < T:
        raise RuntimeError("slot_mapping is longer than positions / query / key")
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_rope_and_cache_int8(
            _ptr(positions), _ptr(query), query.stride(0), query.stride(1), query.shape[1], _ptr(key), key.stride(0),
            key.stride(1), _ptr(value), value.stride(0), value.stride(1), _dtype_code(key, "key"), _ptr(cos_sin_cache),
            _dtype_code(cos_sin_cache, "cos_sin_cache"), rot, 1 if is_neox else 0, ctypes.c_void_p(geom.base_ptr),
            ctypes.byref(g), _ptr(slot_mapping), T, eps_for_dtype(key.dtype), _stream(dev))
    _C.check(rc, "rope_and_cache_per_token_head_quant")


# ---------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------

_ws_bytes_cache: dict = {}


def paged_attn_workspace_bytes(max_num_seqs: int, num_q_heads: int, head_size: int,
                               device: torch.device | None = None) -> int:
    """Host query (depends on the device's CU count); answers are remembered per device.
    ``device`` defaults to the current one."""
    if device is None or device.index is None:
        idx = torch.cuda.current_device() if torch.cuda.is_available() else -1
    else:
        idx = device.index
    key = (idx, max_num_seqs, num_q_heads, head_size)
    got = _ws_bytes_cache.get(key)
    if got is None:
        if idx >= 0 and idx != torch.cuda.current_device():
            with torch.cuda.device(idx):
                got = int(_C.load().kvq_paged_attn_workspace_bytes(max_num_seqs, num_q_heads, head_size))
        else:
            got = int(_C.load().kvq_paged_attn_workspace_bytes(max_num_seqs, num_q_heads, head_size))
        _ws_bytes_cache[key] = got
    return got


_ws_cache: dict = {}
_ws_retired: list = []


def _default_workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """Grow-only per-device scratch for callers that did not bring their own (tests, eager use).
    The backends' metadata builders pre-size their own instead, so a captured step never lands here.
    A buffer that is outgrown is kept alive, not freed: a HIP graph captured earlier may still hold
    its address.  Growing while a capture is under way is refused (it would allocate inside the
    capture and leave the graph with a buffer no later call uses)."""
    cur = _ws_cache.get(dev)
    if cur is None or cur.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("the default workspace would have to grow during stream capture: pass a "
                               "pre-sized workspace (the metadata builders hold one)")
        if cur is not None:
            _ws_retired.append(cur)
        cur = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
        _ws_cache[dev] = cur
    return cur


def unified_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    max_seqlen_q: int,
    seqused_k: torch.Tensor,
    max_seqlen_k: int,
    softmax_scale: float,
    causal: bool,
    window_size=(-1, -1),
    block_table: torch.Tensor | None = None,
    softcap: float = 0.0,
    q_descale=None,
    k_descale=None,
    v_descale=None,
    alibi_slopes=None,
    use_alibi_sqrt: bool = False,
    sinks=None,
    output_scale=None,
    mm_prefix_range=None,
    kv_quant_mode: KVQuantMode = KVQuantMode.INT8_PER_TOKEN_HEAD,
    k_scale_cache: torch.Tensor | None = None,
    v_scale_cache: torch.Tensor | None = None,
    workspace: torch.Tensor | None = None,
    geometry: CacheGeometry | None = None,
    lse: torch.Tensor | None = None,
    static_scratch: bool = False,
    has_decode_rows: bool = True,
    prefill_splits: int = 1,
    **unused,
) -> None:
    """Drop-in for ``unified_attention`` as called at
    vllm_metax/v1/attention/backends/triton_attn.py:688-725 with an int8 per-token-head cache.

    q/out ``[N, Hq, D]``; k/v are the ``(nb, bs, Hkv, D+4)`` int8 cache views; ``seqused_k`` ``[B]``
    int32 context lengths; ``cu_seqlens_q`` ``[B+1]`` int32; ``block_table`` ``[B, max_blocks]``
    int32.  Extra keyword arguments of the reference's call that only steer its Triton launch
    (``seq_threshold_3D``, ``softmax_segm_*``, ``use_td`` ...) are accepted and ignored; features
    this path does not build raise ``NotImplementedError``.  ``window_size=(W - 1, 0)`` restricts a
    query to its last W keys; ``softcap > 0`` maps logits through ``softcap * tanh(x / softcap)``.
    ``static_scratch=True`` keeps the split-K states in the library's own fixed array instead of a
    workspace tensor (nothing is allocated; calls on one GPU must then not overlap in time).
    ``sinks`` ``[Hq]`` float32: attention sinks, one more logit per head with a zero value row (the reference
    passes them through, triton_attn.py:712).
    ``alibi_slopes`` ``[Hq]`` float32: the logit of query position p and key position j gets ``slope * (j - p)``
    added (triton_attn.py:699; causal attention only); the square-root form (``use_alibi_sqrt``) is not built.
    ``has_decode_rows=False`` is the caller's promise that no sequence of the batch has exactly one query row (a
    pure prefill batch): the decode kernel and its reduce are then not launched.
    ``prefill_splits`` (1..8): the context of the long query runs is cut into that many ranges, each a workgroup of
    its own, and merged (``prefill_context_splits`` proposes a value): for launches whose long runs make few
    workgroups on a long context, e.g. one request's small prefill chunk.  The workspace must then hold
    ``split_prefill_workspace_bytes(...)``; the default workspace is grown as needed."""
    code_type = code_type_of(kv_quant_mode)
    if output_scale is not None or mm_prefix_range is not None:
        raise NotImplementedError("fused output quantisation and mm-prefix ranges are not built")
    if use_alibi_sqrt:
        raise NotImplementedError("the square-root form of ALiBi is not built")
    if alibi_slopes is not None and not causal:
        raise NotImplementedError("ALiBi needs causal attention")
    softcap = float(softcap or 0.0)
    if softcap < 0:
        raise RuntimeError("softcap must be >= 0")
    # (left, right) as the reference passes it (triton_attn.py:507-512): (-1, -1) = none,
    # (W - 1, 0) = causal window of W keys ending at the query; two-sided windows are encoder-only
    left, right = (int(x) for x in window_size)
    if (left, right) == (-1, -1):
        window = 0
    elif left >= 0 and right == 0:
        if not causal:
            raise NotImplementedError("a sliding window needs causal attention")
        window = left + 1
    else:
        raise NotImplementedError(f"window_size {(left, right)}: only (-1, -1) and (W - 1, 0) are built")
    if q_descale is not None:
        raise NotImplementedError("quantised query input is not built")
    if unused.get("rswa_window") is not None or unused.get("chunk_lookback", -1) not in (-1, None):
        raise NotImplementedError("rswa / chunk_lookback are not built")
    if block_table is None or k_scale_cache is None or v_scale_cache is None:
        raise RuntimeError("block_table, k_scale_cache and v_scale_cache are required")
    dev = _require_cuda(q, k, v, out, cu_seqlens_q, seqused_k, block_table, k_scale_cache, v_scale_cache, workspace, lse)
    geom = (geometry or geometry_from_views(k, v, k_scale_cache, v_scale_cache)).with_code_type(code_type)
    if q.dim() != 3 or out.shape != q.shape or q.shape[2] != geom.head_size:
        raise RuntimeError("q/out must be [num_tokens, num_q_heads, head_size] matching the cache head size")
    if q.stride(2) != 1 or out.stride(2) != 1:
        raise RuntimeError("q/out head dim must be contiguous")
    num_seqs = seqused_k.shape[0]
    if seqused_k.dtype != torch.int32 or cu_seqlens_q.dtype != torch.int32 or block_table.dtype != torch.int32:
        raise RuntimeError("seqused_k, cu_seqlens_q and block_table must be int32")
    if cu_seqlens_q.shape[0] != num_seqs + 1 or block_table.shape[0] < num_seqs or block_table.stride(1) != 1:
        raise RuntimeError("cu_seqlens_q must have num_seqs+1 entries and block_table num_seqs contiguous rows")
    if not seqused_k.is_contiguous() or not cu_seqlens_q.is_contiguous():
        raise RuntimeError("seqused_k and cu_seqlens_q must be contiguous")
    if block_table.shape[1] * geom.block_size < int(max_seqlen_k):
        raise RuntimeError("block_table rows are too short for max_seqlen_k")
    if num_seqs == 0 or q.shape[0] == 0:
        return
    num_q_heads = q.shape[1]
    _check_sinks(sinks, num_q_heads, q.device)
    _check_sinks(alibi_slopes, num_q_heads, q.device, "alibi_slopes")
    lib = _C.load()
    if lse is not None and (lse.dtype != torch.float32 or not lse.is_contiguous()
                            or tuple(lse.shape) != (q.shape[0], num_q_heads)):
        raise RuntimeError("lse must be a contiguous float32 [num_tokens, num_q_heads] tensor")
    g = geom.as_struct()
    head = (_ptr(out), _dtype_code(out, "out"), out.stride(0), out.stride(1),
            _ptr(q), _dtype_code(q, "q"), q.stride(0), q.stride(1),
            ctypes.c_void_p(geom.base_ptr), ctypes.byref(g), _ptr(block_table), block_table.stride(0),
            _ptr(seqused_k), _ptr(cu_seqlens_q), num_seqs, num_q_heads, int(max_seqlen_q),
            float(softmax_scale), (1 if causal else 0) | (0 if has_decode_rows else 2), window, softcap,
            _ptr(sinks), _ptr(alibi_slopes), _ptr(lse))
    prefill_splits = int(prefill_splits)
    if not 1 <= prefill_splits <= 8:
        raise RuntimeError("prefill_splits must be 1..8")
    if static_scratch:
        with _on_device(dev):
            rc = lib.kvq_paged_attn_int8_static_scratch(*head, _stream(dev))
    elif prefill_splits > 1 and int(max_seqlen_q) > 1:
        need = split_prefill_workspace_bytes(num_seqs, num_q_heads, geom.head_size, q.shape[0], prefill_splits, dev)
        if workspace is None:
            workspace = _default_workspace(dev, need)
        with _on_device(dev):
            rc = lib.kvq_paged_attn_int8_split_prefill(*head, q.shape[0], prefill_splits, _ptr(workspace),
                                                       workspace.numel() * workspace.element_size(), _stream(dev))
    else:
        if workspace is None:
            workspace = _default_workspace(dev, paged_attn_workspace_bytes(num_seqs, num_q_heads, geom.head_size, dev))
        with _on_device(dev):
            rc = lib.kvq_paged_attn_int8(*head, _ptr(workspace), workspace.numel() * workspace.element_size(),
                                         _stream(dev))
    _C.check(rc, "unified_attention")


def split_prefill_workspace_bytes(max_num_seqs: int, num_q_heads: int, head_size: int, num_tokens: int,
                                  prefill_splits: int, device: torch.device | None = None) -> int:
    """Workspace of ``unified_attention(..., prefill_splits=n)``: the plain workspace plus the partial states of
    ``num_tokens`` query rows."""
    idx = torch.cuda.current_device() if device is None or device.index is None else device.index
    with torch.cuda.device(idx):
        return int(_C.load().kvq_paged_attn_split_prefill_workspace_bytes(max_num_seqs, num_q_heads, head_size,
                                                                         num_tokens, prefill_splits))


def prefill_context_splits(query_lens, max_seq_len: int, num_q_heads: int, num_kv_heads: int, num_cus: int = 256,
                           max_split_tokens: int = 4096) -> int:
    """How many context splits a launch should ask for, from what a metadata builder knows on the host: the query
    run lengths of the batch (``query_lens``: a list or CPU tensor; one-token runs do not count), the longest
    sequence, the head counts.  A run of q tokens makes ceil(q / (128 / group)) x Hkv workgroups of the
    workgroup-shared tile; when the launch's workgroups do not fill the chip's two per compute unit and the context
    is long, the context is cut so that they do -- as long as the partial states stay small (splits x run tokens
    <= ``max_split_tokens``)."""
    group = max(1, num_q_heads // max(1, num_kv_heads))
    lens = [int(x) for x in (query_lens.tolist() if hasattr(query_lens, "tolist") else query_lens)]
    runs = [x for x in lens if x > 1]
    if not runs or max(runs) * group < 64 or max_seq_len < 4096:
        return 1
    q_tokens = max(1, 128 // group)
    wgs = sum((x + q_tokens - 1) // q_tokens for x in runs) * num_kv_heads
    splits = min(8, (2 * num_cus) // max(1, wgs), max_split_tokens // max(1, sum(runs)), max_seq_len // 2048)
    return max(1, splits)


def decode_attention_with_cache_update(
    q: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    seqused_k: torch.Tensor,
    max_seqlen_k: int,
    softmax_scale: float,
    block_table: torch.Tensor,
    k_scale_cache: torch.Tensor,
    v_scale_cache: torch.Tensor,
    window_size=(-1, -1),
    softcap: float = 0.0,
    kv_quant_mode: KVQuantMode = KVQuantMode.INT8_PER_TOKEN_HEAD,
    workspace: torch.Tensor | None = None,
    geometry: CacheGeometry | None = None,
    lse: torch.Tensor | None = None,
    slot_mapping: torch.Tensor | None = None,
    sinks: torch.Tensor | None = None,
    alibi_slopes: torch.Tensor | None = None,
) -> None:
    """A decode step in one launch: the cache update of ``reshape_and_cache_flash_per_token_head_quant`` and the
    attention of ``unified_attention`` with one query row per sequence, for a backend whose ``forward`` includes
    the KV cache update (``forward_includes_kv_cache_update``, vllm_metax/v1/attention/backends/triton_attn.py:296).

    ``q``/``out`` ``[B, Hq, D]``; ``key``/``value`` ``[B, Hkv, D]``: row ``i`` is the token at position
    ``seqused_k[i] - 1`` of sequence ``i`` (the block table gives its slot); ``k``/``v`` and the scale views as in
    ``unified_attention``.  ``slot_mapping`` (int64 ``[B]``, optional) is the step's slot mapping: a row whose
    entry is negative is a padding row and is not written, as in the write kernel; the slot of every other row
    comes from the block table.  The cache ends up with the same bytes and ``out`` with the same values as the
    two calls give."""
    code_type = code_type_of(kv_quant_mode)
    softcap = float(softcap or 0.0)
    if softcap < 0:
        raise RuntimeError("softcap must be >= 0")
    left, right = (int(x) for x in window_size)
    if (left, right) == (-1, -1):
        window = 0
    elif left >= 0 and right == 0:
        window = left + 1
    else:
        raise NotImplementedError(f"window_size {(left, right)}: only (-1, -1) and (W - 1, 0) are built")
    dev = _require_cuda(q, key, value, k, v, out, seqused_k, block_table, k_scale_cache, v_scale_cache, workspace, lse)
    geom = (geometry or geometry_from_views(k, v, k_scale_cache, v_scale_cache)).with_code_type(code_type)
    num_seqs = seqused_k.shape[0]
    if q.dim() != 3 or out.shape != q.shape or q.shape[2] != geom.head_size or q.shape[0] != num_seqs:
        raise RuntimeError("q/out must be [num_seqs, num_q_heads, head_size] matching the cache head size")
    if q.stride(2) != 1 or out.stride(2) != 1:
        raise RuntimeError("q/out head dim must be contiguous")
    if key.dim() != 3 or value.shape != key.shape or key.dtype != value.dtype or key.shape[0] < num_seqs:
        raise RuntimeError("key/value must be [num_seqs, num_kv_heads, head_size] of one dtype")
    if key.shape[1] != geom.num_kv_heads or key.shape[2] != geom.head_size:
        raise RuntimeError(f"key shape {tuple(key.shape)} does not match cache (Hkv={geom.num_kv_heads}, D={geom.head_size})")
    if key.stride(2) != 1 or value.stride(2) != 1:
        raise RuntimeError("key/value head dim must be contiguous")
    if seqused_k.dtype != torch.int32 or block_table.dtype != torch.int32 or not seqused_k.is_contiguous():
        raise RuntimeError("seqused_k (contiguous) and block_table must be int32")
    if block_table.shape[0] < num_seqs or block_table.stride(1) != 1:
        raise RuntimeError("block_table needs num_seqs contiguous rows")
    if block_table.shape[1] * geom.block_size < int(max_seqlen_k):
        raise RuntimeError("block_table rows are too short for max_seqlen_k")
    if slot_mapping is not None:
        _require_cuda(slot_mapping)
        if slot_mapping.dtype != torch.int64 or slot_mapping.dim() != 1 or slot_mapping.shape[0] < num_seqs \
                or not slot_mapping.is_contiguous():
            raise RuntimeError("slot_mapping must be a contiguous int64 tensor with one entry per sequence")
    if num_seqs == 0:
        return
    num_q_heads = q.shape[1]
    if lse is not None and (lse.dtype != torch.float32 or not lse.is_contiguous()
                            or tuple(lse.shape) != (num_seqs, num_q_heads)):
        raise RuntimeError("lse must be a contiguous float32 [num_seqs, num_q_heads] tensor")
    _check_sinks(sinks, num_q_heads, q.device)
    _check_sinks(alibi_slopes, num_q_heads, q.device, "alibi_slopes")
    lib = _C.load()
    g = geom.as_struct()
    if workspace is None:
        workspace = _default_workspace(dev, paged_attn_workspace_bytes(num_seqs, num_q_heads, geom.head_size, dev))
    with _on_device(dev):
        rc = lib.kvq_paged_attn_int8_fused_write(
            _ptr(out), _dtype_code(out, "out"), out.stride(0), out.stride(1),
            _ptr(q), _dtype_code(q, "q"), q.stride(0), q.stride(1),
            _ptr(key), _ptr(value), _dtype_code(key, "key"), key.stride(0), key.stride(1), value.stride(0),
            value.stride(1), eps_for_dtype(key.dtype), ctypes.c_void_p(geom.base_ptr), ctypes.byref(g),
            _ptr(block_table), block_table.stride(0), _ptr(seqused_k), _ptr(slot_mapping), num_seqs, num_q_heads,
            float(softmax_scale), window, softcap, _ptr(sinks), _ptr(alibi_slopes), _ptr(lse), _ptr(workspace),
            workspace.numel() * workspace.element_size(), _stream(dev))
    _C.check(rc, "decode_attention_with_cache_update")


def paged_attention_v2(
    out: torch.Tensor,
    exp_sums: torch.Tensor,
    max_logits: torch.Tensor,
    tmp_out: torch.Tensor,
    query: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    num_kv_heads: int,
    scale: float,
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    block_size: int,
    max_seq_len: int,
    alibi_slopes=None,
    kv_cache_dtype: str = "int8_per_token_head",
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
    partition_size: int = 512,
    **unused,
) -> None:
    """Fixed-partition split-K decode, argument order of ``paged_attention_v2``
    (csrc/libtorch_stable/torch_bindings.cpp:631-641).  key_cache/value_cache are the int8 cache
    views and k_scale/v_scale the per-(token, head) fp32 scale views; exp_sums / max_logits
    ``[B, Hq, P]`` and tmp_out ``[B, Hq, P, D]`` are fp32, P = ceil(max_seq_len / partition_size).
    ``alibi_slopes`` ``[Hq]`` float32 as in the reference op: the key at position j gets
    ``slope * (j - seq_len + 1)`` on its scaled logit."""
    if kv_cache_dtype != "int8_per_token_head":
        raise NotImplementedError(f"kv_cache_dtype {kv_cache_dtype!r}: only int8_per_token_head is built")
    if k_scale is None or v_scale is None:
        raise RuntimeError("k_scale / v_scale (the per-token-head scale views) are required")
    dev = _require_cuda(out, exp_sums, max_logits, tmp_out, query, key_cache, value_cache, block_tables, seq_lens, k_scale, v_scale)
    geom = geometry_from_views(key_cache, value_cache, k_scale, v_scale)
    if geom.num_kv_heads != num_kv_heads or geom.block_size != block_size:
        raise RuntimeError("num_kv_heads / block_size do not match the cache views")
    B, Hq, D = query.shape
    P = (max_seq_len + partition_size - 1) // partition_size
    for t, shape, name in ((exp_sums, (B, Hq, P), "exp_sums"), (max_logits, (B, Hq, P), "max_logits"),
                           (tmp_out, (B, Hq, P, D), "tmp_out")):
        if t.dtype != torch.float32 or tuple(t.shape) != shape or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous float32 tensor of shape {shape}")
    if tuple(out.shape) != (B, Hq, D) or not out.is_contiguous() or query.stride(2) != 1:
        raise RuntimeError("out must be contiguous [B, Hq, D]; query head dim contiguous")
    if seq_lens.dtype != torch.int32 or block_tables.dtype != torch.int32 or block_tables.stride(1) != 1:
        raise RuntimeError("seq_lens and block_tables must be int32 (rows contiguous)")
    _check_sinks(alibi_slopes, Hq, query.device, "alibi_slopes")
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_paged_attn_v2_int8(
            _ptr(out), _dtype_code(out, "out"), _ptr(exp_sums), _ptr(max_logits), _ptr(tmp_out), _ptr(query),
            _dtype_code(query, "query"), query.stride(0), query.stride(1), ctypes.c_void_p(geom.base_ptr),
            ctypes.byref(g), _ptr(block_tables), block_tables.stride(0), _ptr(seq_lens), B, Hq, float(scale),
            _ptr(alibi_slopes), int(partition_size), int(P), _stream(dev))
    _C.check(rc, "paged_attention_v2")


def splitk_reduce(out: torch.Tensor, exp_sums: torch.Tensor, max_logits: torch.Tensor, tmp_out: torch.Tensor,
                  seq_lens: torch.Tensor, partition_size: int = 512, lse: torch.Tensor | None = None) -> None:
    """The reduce stage alone (csrc/libtorch_stable/attention/attention_kernels.cuh:556-661)."""
    dev = _require_cuda(out, exp_sums, max_logits, tmp_out, seq_lens, lse)
    B, Hq, P, D = tmp_out.shape
    for t, name in ((exp_sums, "exp_sums"), (max_logits, "max_logits"), (tmp_out, "tmp_out")):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous float32")
    if tuple(out.shape) != (B, Hq, D) or not out.is_contiguous() or seq_lens.dtype != torch.int32:
        raise RuntimeError("out must be contiguous [B, Hq, D] and seq_lens int32")
    with _on_device(dev):
        rc = _C.load().kvq_splitk_reduce(_ptr(out), _dtype_code(out, "out"), _ptr(lse), _ptr(exp_sums),
                                         _ptr(max_logits), _ptr(tmp_out), _ptr(seq_lens), B, Hq, D,
                                         int(partition_size), P, _stream(dev))
    _C.check(rc, "splitk_reduce")


def swap_blocks(src: torch.Tensor, dst: torch.Tensor, block_size_in_bytes: int, block_mapping: torch.Tensor) -> None:
    """``swap_blocks(Tensor src, Tensor! dst, int block_size_in_bytes, Tensor block_mapping)``
    (csrc/libtorch_stable/torch_bindings.cpp:816-818, cache_kernels.cu:33-77): dst block
    ``block_mapping[i, 1]`` = src block ``block_mapping[i, 0]``.  ``block_mapping`` is a CPU int64
    ``[n, 2]`` tensor (the reference refuses a GPU one, cache_kernels.cu:51-55); src / dst are cache
    tensors of the int8 layouts (GQA or MLA) on the GPU or in (pinned) host memory, at least one of
    them on the GPU, both on the same GPU if both are.  Asynchronous on the current stream."""
    if block_mapping.is_cuda:
        raise RuntimeError("block_mapping must be on CPU")
    if block_mapping.dtype != torch.int64 or block_mapping.dim() != 2 or block_mapping.shape[1] != 2:
        raise RuntimeError("block_mapping must be an int64 [n, 2] tensor")
    if src.is_cuda and dst.is_cuda:
        if src.device != dst.device:
            raise RuntimeError("src and dst must be on the same GPU")
        direction, dev = 0, src.device
    elif src.is_cuda and not dst.is_cuda:
        direction, dev = 1, src.device
    elif dst.is_cuda and not src.is_cuda:
        direction, dev = 2, dst.device
    else:
        raise RuntimeError("Invalid device combination")
    n = block_mapping.shape[0]
    if n == 0:
        return
    block_size_in_bytes = int(block_size_in_bytes)
    if int(block_mapping.min()) < 0:
        raise RuntimeError("block numbers must not be negative")
    for t, col, name in ((src, 0, "src"), (dst, 1, "dst")):
        top = int(block_mapping[:, col].max()) + 1
        if top * block_size_in_bytes > t.untyped_storage().nbytes() - t.storage_offset() * t.element_size():
            raise RuntimeError(f"block_mapping names block {top - 1} beyond the end of {name}")
    lib = _C.load()
    with _on_device(dev):
        rc = lib.kvq_swap_blocks(_ptr(src), _ptr(dst), block_size_in_bytes, _ptr(block_mapping), n,
                                 block_mapping.stride(0), block_mapping.stride(1), direction, _stream(dev))
    _C.check(rc, "swap_blocks")


def swap_blocks_batch(src_ptrs: torch.Tensor, dst_ptrs: torch.Tensor, sizes: torch.Tensor,
                      is_src_access_order_any: bool = False, all_on_device: bool = False) -> None:
    """``swap_blocks_batch(Tensor src_ptrs, Tensor dst_ptrs, Tensor sizes, bool
    is_src_access_order_any=False)`` (torch_bindings.cpp:821-823, cache_kernels.cu:79-178): ``n``
    independent copies given as CPU int64 tensors of raw addresses and byte counts, submitted
    together on the current stream.  ``is_src_access_order_any`` steers a driver hint of the
    reference's batched memcpy and changes no result; it is accepted and ignored.
    ``all_on_device=True`` promises that every address is memory of the current GPU: the batch then
    runs as one kernel launch per 64 entries instead of one copy call per entry."""
    for t, name in ((src_ptrs, "src_ptrs"), (dst_ptrs, "dst_ptrs"), (sizes, "sizes")):
        if t.is_cuda:
            raise RuntimeError(f"{name} must be on CPU")
        if t.dtype != torch.int64:
            raise RuntimeError(f"{name} must be int64")
        if not t.is_contiguous() or t.dim() != 1:
            raise RuntimeError(f"{name} must be a contiguous 1-D tensor")
    n = src_ptrs.shape[0]
    if dst_ptrs.shape[0] != n:
        raise RuntimeError("dst_ptrs length must match src_ptrs")
    if sizes.shape[0] != n:
        raise RuntimeError("sizes length must match src_ptrs")
    if n == 0:
        return
    if not torch.cuda.is_available():
        raise RuntimeError("swap_blocks_batch needs a GPU (there is no CPU path)")
    dev = torch.device("cuda", torch.cuda.current_device())
    lib = _C.load()
    rc = lib.kvq_swap_blocks_batch(_ptr(src_ptrs), _ptr(dst_ptrs), _ptr(sizes), n, 1 if all_on_device else 0,
                                   _stream(dev))
    _C.check(rc, "swap_blocks_batch")


def copy_blocks(kv_caches: list[torch.Tensor], block_mapping: torch.Tensor) -> None:
    """``copy_blocks`` / ``copy_blocks_mla`` over the int8 format (kernels
    csrc/libtorch_stable/cache_kernels.cu:184-232; tests/kernels/attention/test_cache.py:55-110,
    592-650): block ``dst`` of EVERY layer's cache becomes a copy of block ``src`` for every row
    ``(src, dst)`` of ``block_mapping`` (``[num_pairs, 2]`` int64, on the GPU, as in the
    reference's test).  A block of these layouts holds keys, values and scales, so one cache list
    replaces the reference's key / value lists.  All caches share shape and block stride."""
    if len(kv_caches) == 0:
        return
    dev = _require_cuda(*kv_caches, block_mapping)
    if block_mapping.dtype != torch.int64 or block_mapping.dim() != 2 or block_mapping.shape[1] != 2 \
            or not block_mapping.is_contiguous():
        raise RuntimeError("block_mapping must be a contiguous [num_pairs, 2] int64 tensor")
    first = kv_caches[0]
    block_bytes = first.stride(0) * first.element_size()
    for t in kv_caches:
        if t.shape != first.shape or t.stride() != first.stride() or t.dtype != first.dtype:
            raise RuntimeError("every layer's cache must have the same shape, strides and dtype")
    num_pairs = block_mapping.shape[0]
    if num_pairs == 0:
        return
    ptrs = torch.tensor([t.data_ptr() for t in kv_caches], dtype=torch.int64).to(dev)
    with _on_device(dev):
        rc = _C.load().kvq_copy_blocks(_ptr(ptrs), len(kv_caches), _ptr(block_mapping), num_pairs, block_bytes,
                                       first.shape[0], _stream(dev))
        # the pointer table must outlive the launch that reads it
        ptrs.record_stream(torch.cuda.current_stream(dev))
    _C.check(rc, "copy_blocks")


# the latent cache is one joint tensor per layer as well
copy_blocks_mla = copy_blocks


def merge_attn_states(output: torch.Tensor, prefix_output: torch.Tensor, prefix_lse: torch.Tensor,
                      suffix_output: torch.Tensor, suffix_lse: torch.Tensor,
                      output_lse: torch.Tensor | None = None, prefill_tokens_with_context: int | None = None) -> None:
    """LSE merge, signature of vllm_metax/v1/attention/ops/merge_attn_states.py:10-114.
    outputs ``[T, H, D]`` (one dtype, contiguous), lse ``[H, T]`` fp32."""
    dev = _require_cuda(output, prefix_output, prefix_lse, suffix_output, suffix_lse, output_lse)
    T, H, D = output.shape
    if prefix_output.shape != output.shape or suffix_output.shape != output.shape:
        raise RuntimeError("prefix/suffix/output shapes differ")
    if prefix_output.dtype != output.dtype or suffix_output.dtype != output.dtype:
        raise RuntimeError("prefix/suffix/output dtypes differ")
    for t in (output, prefix_output, suffix_output, prefix_lse, suffix_lse):
        if not t.is_contiguous():
            raise RuntimeError("merge_attn_states needs contiguous tensors")
    if prefix_lse.dtype != torch.float32 or suffix_lse.dtype != torch.float32 or tuple(prefix_lse.shape) != (H, T):
        raise RuntimeError("lse tensors must be float32 [num_heads, num_tokens]")
    n_prefix = T if prefill_tokens_with_context is None else int(prefill_tokens_with_context)
    with _on_device(dev):
        rc = _C.load().kvq_merge_attn_states(_ptr(output), _ptr(output_lse), _ptr(prefix_output), _ptr(prefix_lse),
                                             _ptr(suffix_output), _ptr(suffix_lse), _dtype_code(output, "output"),
                                             T, H, D, n_prefix, _stream(dev))
    _C.check(rc, "merge_attn_states")


# ---------------------------------------------------------------------------------------------
# MLA latent cache
# ---------------------------------------------------------------------------------------------

def concat_and_cache_mla(kv_c: torch.Tensor, k_pe: torch.Tensor, kv_cache: torch.Tensor,
                         slot_mapping: torch.Tensor, kv_cache_dtype: str = "int8_per_token",
                         scale: torch.Tensor | None = None, geometry: MlaGeometry | None = None) -> None:
    """Argument order of ``concat_and_cache_mla`` (csrc/libtorch_stable/torch_bindings.cpp:843-848).
    kv_c ``[T, R]``, k_pe ``[T, P]``; kv_cache is the int8 latent cache ``(nb, bs, R+P+4)``."""
    if kv_cache_dtype != "int8_per_token":
        raise NotImplementedError(f"kv_cache_dtype {kv_cache_dtype!r}: only int8_per_token is built")
    dev = _require_cuda(kv_c, k_pe, kv_cache, slot_mapping)
    geom = geometry or mla_geometry(kv_cache, kv_c.shape[-1])
    if kv_c.dim() != 2 or k_pe.dim() != 2 or kv_c.dtype != k_pe.dtype:
        raise RuntimeError("kv_c [T, R] and k_pe [T, P] must be 2-D of one dtype")
    if kv_c.shape[1] != geom.kv_lora_rank or k_pe.shape[1] != geom.rope_dim:
        raise RuntimeError("kv_c / k_pe widths do not match the cache entry")
    if kv_c.stride(1) != 1 or k_pe.stride(1) != 1:
        raise RuntimeError("kv_c / k_pe rows must be contiguous")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
        raise RuntimeError("slot_mapping must be contiguous int64")
    T = slot_mapping.shape[0]
    if T > kv_c.shape[0] or T > k_pe.shape[0]:
        raise RuntimeError("slot_mapping is longer than kv_c / k_pe")
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_concat_and_cache_mla_int8(_ptr(kv_c), _ptr(k_pe), _dtype_code(kv_c, "kv_c"),
                                                     kv_c.stride(0), k_pe.stride(0), ctypes.c_void_p(geom.base_ptr),
                                                     ctypes.byref(g), _ptr(slot_mapping), T,
                                                     eps_for_dtype(kv_c.dtype), _stream(dev))
    _C.check(rc, "concat_and_cache_mla")


def concat_and_cache_mla_rope_fused(positions: torch.Tensor, q_pe: torch.Tensor, k_pe: torch.Tensor,
                                    kv_c: torch.Tensor, cos_sin_cache: torch.Tensor, is_neox: bool,
                                    slot_mapping: torch.Tensor, kv_cache: torch.Tensor,
                                    kv_cache_dtype: str = "int8_per_token", kv_cache_scale: torch.Tensor | None = None,
                                    geometry: MlaGeometry | None = None) -> None:
    """Argument order of ``concat_and_cache_mla_rope_fused``
    (csrc/libtorch_stable/torch_bindings.cpp:851-862, cache_kernels_fused.cu:24-168): rotary
    embedding of ``q_pe`` ``[T, Hq, rot]`` and ``k_pe`` ``[T, rot]`` in place, then ``[kv_c | k_pe]`` into
    the int8 latent cache.  ``kv_cache_scale`` (the reference's per-tensor fp8 scale) is not used:
    every row carries its own scale."""
    if kv_cache_dtype != "int8_per_token":
        raise NotImplementedError(f"kv_cache_dtype {kv_cache_dtype!r}: only int8_per_token is built")
    dev = _require_cuda(positions, q_pe, k_pe, kv_c, cos_sin_cache, slot_mapping, kv_cache)
    geom = geometry or mla_geometry(kv_cache, kv_c.shape[-1])
    if q_pe.dim() != 3 or k_pe.dim() != 2 or kv_c.dim() != 2 or not (q_pe.dtype == k_pe.dtype == kv_c.dtype):
        raise RuntimeError("q_pe [T, Hq, rot], k_pe [T, rot] and kv_c [T, R] must share one dtype")
    rot = k_pe.shape[1]
    if q_pe.shape[2] != rot or rot != geom.rope_dim or kv_c.shape[1] != geom.kv_lora_rank:
        raise RuntimeError("q_pe / k_pe / kv_c widths do not match the cache entry")
    if cos_sin_cache.dim() != 2 or cos_sin_cache.shape[1] != rot or not cos_sin_cache.is_contiguous():
        raise RuntimeError("cos_sin_cache must be a contiguous [max_position, rot_dim] tensor")
    if q_pe.stride(2) != 1 or k_pe.stride(1) != 1 or kv_c.stride(1) != 1:
        raise RuntimeError("q_pe / k_pe / kv_c rows must be contiguous")
    for name, t in (("positions", positions), ("slot_mapping", slot_mapping)):
        if t.dtype != torch.int64 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous int64")
    T = slot_mapping.shape[0]
    if positions.shape[0] < T or q_pe.shape[0] < T or k_pe.shape[0] < T or kv_c.shape[0] < T:
        raise RuntimeError("slot_mapping is longer than positions / q_pe / k_pe / kv_c")
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_concat_and_cache_mla_rope_int8(
            _ptr(positions), _ptr(q_pe), q_pe.stride(0), q_pe.stride(1), q_pe.shape[1], _ptr(k_pe), k_pe.stride(0),
            _ptr(kv_c), kv_c.stride(0), _dtype_code(kv_c, "kv_c"), _ptr(cos_sin_cache),
            _dtype_code(cos_sin_cache, "cos_sin_cache"), rot, 1 if is_neox else 0, ctypes.c_void_p(geom.base_ptr),
            ctypes.byref(g), _ptr(slot_mapping), T, eps_for_dtype(kv_c.dtype), _stream(dev))
    _C.check(rc, "concat_and_cache_mla_rope_fused")


def gather_and_maybe_dequant_cache(src_cache: torch.Tensor, dst: torch.Tensor, block_table: torch.Tensor,
                                   cu_seq_lens: torch.Tensor, token_to_seq: torch.Tensor, num_tokens: int,
                                   kv_cache_dtype: str = "int8_per_token", scale: torch.Tensor | None = None,
                                   seq_starts: torch.Tensor | None = None, kv_lora_rank: int = 512,
                                   geometry: MlaGeometry | None = None) -> None:
    """Argument order of ``gather_and_maybe_dequant_cache``
    (csrc/libtorch_stable/cache_kernels.cu:1181-1247), for the int8 latent cache: ``dst[t] = code *
    row scale`` of the row that token ``t`` of sequence ``token_to_seq[t]`` names.  ``scale`` (the
    reference's per-tensor scale) is not used: every row carries its own."""
    if kv_cache_dtype != "int8_per_token":
        raise NotImplementedError(f"kv_cache_dtype {kv_cache_dtype!r}: only int8_per_token is built")
    dev = _require_cuda(src_cache, dst, block_table, cu_seq_lens, token_to_seq, seq_starts)
    geom = geometry or mla_geometry(src_cache, kv_lora_rank)
    W = geom.kv_lora_rank + geom.rope_dim
    if dst.dim() != 2 or dst.shape[1] != W or dst.stride(1) != 1 or dst.shape[0] < num_tokens:
        raise RuntimeError(f"dst must be [>= num_tokens, {W}] with a contiguous last dim")
    for name, t in (("block_table", block_table), ("cu_seq_lens", cu_seq_lens), ("token_to_seq", token_to_seq),
                    ("seq_starts", seq_starts)):
        if t is not None and t.dtype != torch.int32:
            raise RuntimeError(f"{name} must be int32")
    if block_table.stride(1) != 1 or not cu_seq_lens.is_contiguous() or not token_to_seq.is_contiguous():
        raise RuntimeError("block_table rows, cu_seq_lens and token_to_seq must be contiguous")
    if token_to_seq.numel() < num_tokens:
        raise RuntimeError("token_to_seq is shorter than num_tokens")
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_gather_and_dequant_mla_int8(
            _ptr(dst), _dtype_code(dst, "dst"), dst.stride(0), ctypes.c_void_p(geom.base_ptr), ctypes.byref(g),
            _ptr(block_table), block_table.stride(0), _ptr(cu_seq_lens), _ptr(token_to_seq), _ptr(seq_starts),
            int(num_tokens), _stream(dev))
    _C.check(rc, "gather_and_maybe_dequant_cache")


def cp_gather_cache(src_cache: torch.Tensor, dst: torch.Tensor, block_table: torch.Tensor, cu_seq_lens: torch.Tensor,
                    batch_size: int, seq_starts: torch.Tensor | None = None, kv_lora_rank: int = 512,
                    geometry: MlaGeometry | None = None) -> None:
    """Argument order of ``cp_gather_cache`` (csrc/libtorch_stable/cache_kernels.cu:1397-1462) over
    the int8 latent cache: ``dst`` ``[tot_tokens, W + 4]`` int8/uint8 receives, for every token of the
    ``batch_size`` sequences (rows ``cu_seq_lens[b] .. cu_seq_lens[b+1]-1``, cache positions
    shifted by ``seq_starts[b]`` when given), its ``W`` code bytes followed by the 4 bytes of its
    fp32 scale -- no dequantisation."""
    dev = _require_cuda(src_cache, dst, block_table, cu_seq_lens, seq_starts)
    geom = geometry or mla_geometry(src_cache, kv_lora_rank)
    W = geom.kv_lora_rank + geom.rope_dim
    if dst.dtype not in (torch.int8, torch.uint8) or dst.dim() != 2 or dst.shape[1] != W + 4 or dst.stride(1) != 1:
        raise RuntimeError(f"dst must be an int8 [tot_tokens, {W + 4}] tensor with a contiguous last dim")
    for name, t in (("block_table", block_table), ("cu_seq_lens", cu_seq_lens), ("seq_starts", seq_starts)):
        if t is not None and t.dtype != torch.int32:
            raise RuntimeError(f"{name} must be int32")
    if block_table.stride(1) != 1 or not cu_seq_lens.is_contiguous():
        raise RuntimeError("block_table rows and cu_seq_lens must be contiguous")
    if cu_seq_lens.numel() < batch_size + 1 or block_table.shape[0] < batch_size:
        raise RuntimeError("cu_seq_lens needs batch_size + 1 entries and block_table batch_size rows")
    if seq_starts is not None and (seq_starts.numel() < batch_size or not seq_starts.is_contiguous()):
        raise RuntimeError("seq_starts needs batch_size contiguous entries")
    if batch_size == 0 or dst.shape[0] == 0:
        return
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_cp_gather_mla_int8(
            _ptr(dst), dst.stride(0), ctypes.c_void_p(geom.base_ptr), ctypes.byref(g), _ptr(block_table),
            block_table.stride(0), _ptr(cu_seq_lens), _ptr(seq_starts), int(batch_size), dst.shape[0], _stream(dev))
    _C.check(rc, "cp_gather_cache")


def mla_decode_workspace_bytes(max_num_seqs: int, num_heads: int, kv_lora_rank: int) -> int:
    return int(_C.load().kvq_mla_decode_workspace_bytes(max_num_seqs, num_heads, kv_lora_rank))


def mla_decode_int8(q, kv_cache: torch.Tensor, o: torch.Tensor, lse: torch.Tensor | None,
                    block_table: torch.Tensor, seq_lens: torch.Tensor, sm_scale: float, kv_lora_rank: int,
                    workspace: torch.Tensor | None = None, geometry: MlaGeometry | None = None,
                    new_rows: tuple[torch.Tensor, torch.Tensor] | None = None) -> None:
    """MLA decode over the int8 latent cache: the job of ``decode_attention_fwd(..., is_mla=True)``
    (vllm_metax/v1/attention/ops/triton_decode_attention.py:763-825).  q ``[B, H, R+P]`` or the pair
    ``(ql_nope [B, H, R], q_pe [B, H, P])`` that ``forward_mqa`` may receive
    (vllm_metax/v1/attention/backends/mla/triton_mla.py:226-238; read as it is, no concatenation),
    o ``[B, H, R]``, lse ``[B, H]`` fp32 or None.  ``new_rows`` = (kv_c ``[B, R]``, k_pe ``[B, P]``): see
    :func:`mla_decode_with_cache_update`."""
    q_pe = None
    if type(q) is tuple:
        q, q_pe = q
    kv_c, k_pe = new_rows if new_rows is not None else (None, None)
    dev = _require_cuda(q, q_pe, kv_cache, o, lse, block_table, seq_lens, workspace, kv_c, k_pe)
    geom = geometry or mla_geometry(kv_cache, kv_lora_rank)
    B, H, W = q.shape
    if new_rows is not None:
        if kv_c.dim() != 2 or k_pe.dim() != 2 or kv_c.dtype != k_pe.dtype:
            raise RuntimeError("kv_c [B, R] and k_pe [B, P] must be 2-D of one dtype")
        if tuple(kv_c.shape) != (B, geom.kv_lora_rank) or tuple(k_pe.shape) != (B, geom.rope_dim):
            raise RuntimeError("kv_c / k_pe must hold one row per sequence, as wide as the cache entry")
        if kv_c.stride(1) != 1 or k_pe.stride(1) != 1:
            raise RuntimeError("kv_c / k_pe rows must be contiguous")
    if q_pe is None:
        if W != geom.kv_lora_rank + geom.rope_dim:
            raise RuntimeError("q must be [B, H, R+P]")
    else:
        if W != geom.kv_lora_rank or tuple(q_pe.shape) != (B, H, geom.rope_dim) or q_pe.dtype != q.dtype:
            raise RuntimeError("(ql_nope, q_pe) must be [B, H, R] and [B, H, P] of one dtype")
        if q_pe.stride(2) != 1:
            raise RuntimeError("q_pe head dim must be contiguous")
    if tuple(o.shape) != (B, H, geom.kv_lora_rank):
        raise RuntimeError("o must be [B, H, R]")
    if q.stride(2) != 1 or not o.is_contiguous():
        raise RuntimeError("q head dim must be contiguous and o contiguous")
    if seq_lens.dtype != torch.int32 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise RuntimeError("seq_lens and block_table must be int32")
    if lse is not None and (lse.dtype != torch.float32 or tuple(lse.shape) != (B, H) or not lse.is_contiguous()):
        raise RuntimeError("lse must be contiguous float32 [B, H]")
    need = mla_decode_workspace_bytes(B, H, geom.kv_lora_rank)
    if workspace is None:
        workspace = _default_workspace(dev, need)
    g = geom.as_struct()
    head = (_ptr(o), _dtype_code(o, "o"), _ptr(lse), _ptr(q), _dtype_code(q, "q"), q.stride(0), q.stride(1), _ptr(q_pe),
            q_pe.stride(0) if q_pe is not None else 0, q_pe.stride(1) if q_pe is not None else 0)
    with _on_device(dev):
        tail = (ctypes.c_void_p(geom.base_ptr), ctypes.byref(g), _ptr(block_table), block_table.stride(0),
                _ptr(seq_lens), B, H, float(sm_scale), _ptr(workspace),
                workspace.numel() * workspace.element_size(), _stream(dev))
        if new_rows is None:
            rc = _C.load().kvq_mla_decode_int8(*head, *tail)
        else:
            rc = _C.load().kvq_mla_decode_int8_fused_write(*head, _ptr(kv_c), _ptr(k_pe), _dtype_code(kv_c, "kv_c"),
                                                           kv_c.stride(0), k_pe.stride(0),
                                                           eps_for_dtype(kv_c.dtype), *tail)
    _C.check(rc, "mla_decode_int8" if new_rows is None else "mla_decode_int8_fused_write")


def mla_decode_with_cache_update(q, kv_c: torch.Tensor, k_pe: torch.Tensor, kv_cache: torch.Tensor, o: torch.Tensor,
                                 lse: torch.Tensor | None, block_table: torch.Tensor, seq_lens: torch.Tensor,
                                 sm_scale: float, kv_lora_rank: int, workspace: torch.Tensor | None = None,
                                 geometry: MlaGeometry | None = None) -> None:
    """One decode step of an MLA layer in one launch: ``concat_and_cache_mla(kv_c, k_pe, kv_cache, slot_mapping)``
    followed by :func:`mla_decode_int8`, for a batch that holds one new token per sequence (row i of kv_c / k_pe is
    the token at position ``seq_lens[i] - 1`` of sequence i; its slot comes from the block table, as
    ``slot_mapping`` would name it).  What ``do_kv_cache_update`` + ``forward_mqa`` do in two steps
    (vllm_metax/v1/attention/backends/mla/triton_mla.py:226-295); cache bytes and outputs are those of the two
    calls."""
    mla_decode_int8(q, kv_cache, o, lse, block_table, seq_lens, sm_scale, kv_lora_rank, workspace, geometry,
                    new_rows=(kv_c, k_pe))


def mla_decode_absorb_int8(q_nope: torch.Tensor, W_UK_T: torch.Tensor, q_pe: torch.Tensor, kv_cache: torch.Tensor,
                           o: torch.Tensor, lse: torch.Tensor | None, block_table: torch.Tensor,
                           seq_lens: torch.Tensor, sm_scale: float, kv_lora_rank: int,
                           workspace: torch.Tensor | None = None, geometry: MlaGeometry | None = None) -> None:
    """``mla_decode_int8`` with the absorption ``ql_nope = bmm(q_nope, W_UK_T)`` of the MLA layer
    (vllm_metax/model_executor/layers/attention/mla_attention.py:835-848) done inside the launch: q_nope
    ``[B, H, P]``, W_UK_T ``[H, P, R]``, q_pe ``[B, H, rope]`` (bf16 or fp16, one dtype); the product is
    written directly as the decode's int8 query operands.  o ``[B, H, R]``, lse ``[B, H]`` fp32 or None."""
    dev = _require_cuda(q_nope, W_UK_T, q_pe, kv_cache, o, lse, block_table, seq_lens, workspace)
    geom = geometry or mla_geometry(kv_cache, kv_lora_rank)
    B, H, P = q_nope.shape
    if tuple(W_UK_T.shape) != (H, P, geom.kv_lora_rank) or tuple(q_pe.shape) != (B, H, geom.rope_dim):
        raise RuntimeError("W_UK_T must be [H, P, R] and q_pe [B, H, rope]")
    if not (q_nope.dtype == W_UK_T.dtype == q_pe.dtype):
        raise RuntimeError("q_nope, W_UK_T and q_pe must share a dtype")
    if q_nope.stride(2) != 1 or W_UK_T.stride(2) != 1 or q_pe.stride(2) != 1:
        raise RuntimeError("last dims must be contiguous")
    if tuple(o.shape) != (B, H, geom.kv_lora_rank) or not o.is_contiguous():
        raise RuntimeError("o must be contiguous [B, H, R]")
    if seq_lens.dtype != torch.int32 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise RuntimeError("seq_lens and block_table must be int32")
    if lse is not None and (lse.dtype != torch.float32 or tuple(lse.shape) != (B, H) or not lse.is_contiguous()):
        raise RuntimeError("lse must be contiguous float32 [B, H]")
    if workspace is None:
        workspace = _default_workspace(dev, mla_decode_workspace_bytes(B, H, geom.kv_lora_rank))
    g = geom.as_struct()
    with _on_device(dev):
        rc = _C.load().kvq_mla_decode_absorb_int8(
            _ptr(o), _dtype_code(o, "o"), _ptr(lse), _ptr(q_nope), _dtype_code(q_nope, "q_nope"), q_nope.stride(0),
            q_nope.stride(1), P, _ptr(W_UK_T), W_UK_T.stride(0), W_UK_T.stride(1), _ptr(q_pe), q_pe.stride(0),
            q_pe.stride(1), ctypes.c_void_p(geom.base_ptr), ctypes.byref(g), _ptr(block_table), block_table.stride(0),
            _ptr(seq_lens), B, H, float(sm_scale), _ptr(workspace), workspace.numel() * workspace.element_size(),
            _stream(dev))
    _C.check(rc, "mla_decode_absorb_int8")


def mla_v_up_proj(x: torch.Tensor, W_UV: torch.Tensor, out: torch.Tensor) -> None:
    """``out[b, h, :] = x[b, h, :] @ W_UV[h]``: the V up-projection behind the MLA decode, the
    reference's ``_v_up_proj`` (vllm_metax/model_executor/layers/attention/mla_attention.py:1087-1109)
    for unquantised weights.  x ``[B, H, L]``, W_UV ``[H, L, V]``, out ``[B, H, V]`` or ``[B, H * V]``;
    bf16 or fp16, one dtype; L and V multiples of 128."""
    dev = _require_cuda(x, W_UV, out)
    if x.dim() != 3 or W_UV.dim() != 3:
        raise RuntimeError("mla_v_up_proj takes x [B, H, L] and W_UV [H, L, V]")
    B, H, L = x.shape
    V = W_UV.shape[2]
    if tuple(W_UV.shape) != (H, L, V):
        raise RuntimeError("W_UV must be [H, L, V]")
    if out.dim() == 2:
        if tuple(out.shape) != (B, H * V) or out.stride(1) != 1:
            raise RuntimeError("out must be [B, H * V] with a contiguous last dim")
        o_sb, o_sh = out.stride(0), V
    else:
        if tuple(out.shape) != (B, H, V) or out.stride(2) != 1:
            raise RuntimeError("out must be [B, H, V] with a contiguous last dim")
        o_sb, o_sh = out.stride(0), out.stride(1)
    if not (x.dtype == W_UV.dtype == out.dtype):
        raise RuntimeError("x, W_UV and out must share a dtype")
    if x.stride(2) != 1 or W_UV.stride(2) != 1:
        raise RuntimeError("last dims must be contiguous")
    if B == 0:
        return
    with _on_device(dev):
        rc = _C.load().kvq_mla_v_up_proj(_ptr(out), o_sb, o_sh, _ptr(x), _dtype_code(x, "x"), x.stride(0), x.stride(1),
                                         _ptr(W_UV), W_UV.stride(0), W_UV.stride(1), B, H, L, V, _stream(dev))
    _C.check(rc, "mla_v_up_proj")


def concat_mla_q(ql_nope: torch.Tensor, q_pe: torch.Tensor, q_out: torch.Tensor) -> None:
    """``q_out[..., :R] = ql_nope; q_out[..., R:] = q_pe``: the reference's ``ops.concat_mla_q``
    (csrc/libtorch_stable/cache_kernels.cu:1740-1783; call site
    vllm_metax/v1/attention/backends/mla/flashmla_sparse.py:1100).  ``[T, H, R]``, ``[T, H, P]`` ->
    ``[T, H, R+P]``, one dtype, last dims contiguous."""
    dev = _require_cuda(ql_nope, q_pe, q_out)
    if ql_nope.dim() != 3 or q_pe.dim() != 3 or q_out.dim() != 3:
        raise RuntimeError("concat_mla_q takes [num_tokens, num_heads, dim] tensors")
    T, H, R = ql_nope.shape
    P = q_pe.shape[2]
    if tuple(q_pe.shape[:2]) != (T, H) or tuple(q_out.shape) != (T, H, R + P):
        raise RuntimeError("q_pe must be [T, H, P] and q_out [T, H, R+P]")
    if not (ql_nope.dtype == q_pe.dtype == q_out.dtype):
        raise RuntimeError("ql_nope, q_pe and q_out must share a dtype")
    if ql_nope.stride(2) != 1 or q_pe.stride(2) != 1 or q_out.stride(2) != 1:
        raise RuntimeError("last dims must be contiguous")
    with _on_device(dev):
        rc = _C.load().kvq_concat_mla_q(_ptr(q_out), q_out.stride(0), q_out.stride(1), _ptr(ql_nope),
                                        ql_nope.stride(0), ql_nope.stride(1), _ptr(q_pe), q_pe.stride(0),
                                        q_pe.stride(1), _dtype_code(ql_nope, "ql_nope"), T, H, R, P, _stream(dev))
    _C.check(rc, "concat_mla_q")


def mla_prefill_attention(q: torch.Tensor, k_nope: torch.Tensor, k_pe: torch.Tensor | None, v: torch.Tensor,
                          cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, max_seqlen_q: int,
                          softmax_scale: float, causal: bool, out: torch.Tensor | None = None,
                          lse: torch.Tensor | None = None, return_softmax_lse: bool = False):
    """Varlen attention of the MLA prefill with the LSE the chunked-context merge needs: the role of
    ``flash_attn_varlen_func`` in vllm_metax/v1/attention/backends/mla/prefill/flash_attn.py:128-221 (keyword
    names kept), except that the key comes in the two pieces the layer holds -- ``k_nope [S, H, nope]`` and
    ``k_pe [S, rope]`` or ``[S, 1, rope]``, shared by the heads -- and ``v [S, H, v_dim]`` keeps its own
    head size.  ``q [T, H, nope + rope]``; returns ``out [T, H, v_dim]``, and ``(out, lse [H, T] fp32)`` with
    ``return_softmax_lse``.  ``out`` / ``lse`` may be passed in to avoid the allocation."""
    dev = _require_cuda(q, k_nope, k_pe, v, cu_seqlens_q, cu_seqlens_k, out, lse)
    if q.dim() != 3 or k_nope.dim() != 3 or v.dim() != 3:
        raise RuntimeError("q, k_nope and v must be [tokens, heads, dim]")
    T, H, Dqk = q.shape
    S, _, nope = k_nope.shape
    rope = Dqk - nope
    dv = v.shape[2]
    if k_pe is not None and k_pe.dim() == 3:
        if k_pe.shape[1] != 1:
            raise RuntimeError("k_pe must be shared by the heads: [S, rope] or [S, 1, rope]")
        k_pe = k_pe[:, 0]
    if rope < 0 or (rope > 0 and (k_pe is None or tuple(k_pe.shape) != (S, rope))):
        raise RuntimeError(f"k_pe must be [{S}, {rope}] for q of head size {Dqk} and k_nope of {nope}")
    if k_nope.shape[1] != H or tuple(v.shape[:2]) != (S, H):
        raise RuntimeError("k_nope and v must have q's head count and one row per key")
    for name, t in (("q", q), ("k_nope", k_nope), ("k_pe", k_pe), ("v", v)):
        if t is not None and (t.dtype != q.dtype or t.stride(-1) != 1):
            raise RuntimeError(f"{name}: one dtype and contiguous last dims are required")
    for name, t in (("cu_seqlens_q", cu_seqlens_q), ("cu_seqlens_k", cu_seqlens_k)):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous int32")
    B = cu_seqlens_q.numel() - 1
    if cu_seqlens_k.numel() != B + 1:
        raise RuntimeError("cu_seqlens_q and cu_seqlens_k must have the same length")
    if out is None:
        out = torch.empty(T, H, dv, dtype=q.dtype, device=dev)
    elif tuple(out.shape) != (T, H, dv) or out.dtype != q.dtype or out.stride(2) != 1:
        raise RuntimeError(f"out must be [{T}, {H}, {dv}] of q's dtype with a contiguous last dim")
    if lse is None and return_softmax_lse:
        lse = torch.empty(H, T, dtype=torch.float32, device=dev)
    if lse is not None and (tuple(lse.shape) != (H, T) or lse.dtype != torch.float32 or not lse.is_contiguous()):
        raise RuntimeError(f"lse must be contiguous float32 [{H}, {T}]")
    with _on_device(dev):
        rc = _C.load().kvq_mla_prefill_attn(
            _ptr(q), _dtype_code(q, "q"), q.stride(0), q.stride(1), _ptr(k_nope), k_nope.stride(0), k_nope.stride(1),
            _ptr(k_pe), k_pe.stride(0) if k_pe is not None else 0, _ptr(v), v.stride(0), v.stride(1),
            _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), B, int(max_seqlen_q), T, H, nope, rope, dv, float(softmax_scale),
            1 if causal else 0, _ptr(out), out.stride(0), out.stride(1), _ptr(lse), _stream(dev))
    _C.check(rc, "mla_prefill_attention")
    return (out, lse) if return_softmax_lse else out

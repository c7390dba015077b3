"""CPU oracle for the int8 KV-cache attention path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the product (``vllm_metax_amd``) never
does.  It wraps ``kvq_oracle.c`` (a plain-C restatement of the reference
algorithm, every function citing the reference file:line it follows) through
ctypes, and takes CPU torch tensors purely as typed memory.

``torch_ref.py`` next to this file restates the reference's tests/kernels
torch ops in their as-written numeric form; it is what the CPU baseline times
and what the C oracle is cross-checked against.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkvq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile kvq_oracle.c with gcc (a second or two)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE, "libkvq_oracle.so"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in (
            "kvq_oracle_quant_rows",
            "kvq_oracle_cache_write",
            "kvq_oracle_paged_attn",
            "kvq_oracle_paged_attn_partition",
            "kvq_oracle_splitk_reduce",
            "kvq_oracle_merge_attn_states",
            "kvq_oracle_mla_cache_write",
            "kvq_oracle_mla_decode",
            "kvq_oracle_num_threads",
        ):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().kvq_oracle_num_threads())


@dataclass(frozen=True)
class RecordLayout:
    """Byte geometry of the paged cache: where the K codes, V codes and the two
    fp32 scales of a (block, slot, head) record sit relative to the storage base."""

    k_off: int
    v_off: int
    ks_off: int
    vs_off: int
    stride_block: int
    stride_slot: int
    stride_head: int
    head_size: int
    block_size: int
    num_kv_heads: int

    @staticmethod
    def from_views(kv_cache, key_cache, value_cache, k_scale_cache, v_scale_cache, code_type: int = 0):
        """Derive the geometry from the typed views alone (data_ptr differences
        and strides), independent of how the views were constructed.

        key_cache/value_cache: (num_blocks, block_size, Hkv, D + 4) int8 views;
        scale caches: (num_blocks, block_size, Hkv) fp32 views."""
        base = kv_cache.data_ptr()
        nb, bs, hkv, padded = key_cache.shape
        assert key_cache.element_size() == 1 and k_scale_cache.dtype == torch.float32
        sb, ss, sh, se = key_cache.stride()
        assert se == 1
        assert tuple(4 * s for s in k_scale_cache.stride()) == (sb, ss, sh)
        assert tuple(4 * s for s in v_scale_cache.stride()) == (sb, ss, sh)
        assert value_cache.stride() == key_cache.stride()
        return RecordLayout(
            k_off=key_cache.data_ptr() - base,
            v_off=value_cache.data_ptr() - base,
            ks_off=k_scale_cache.data_ptr() - base,
            vs_off=v_scale_cache.data_ptr() - base,
            stride_block=sb,
            stride_slot=ss,
            stride_head=sh,
            head_size=(padded - 4) * (2 if code_type == 2 else 1),   # int4: two codes per byte
            block_size=bs,
            num_kv_heads=hkv,
        )


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _f32c(t):
    assert t.device.type == "cpu"
    return t.detach().to(torch.float32).contiguous()


def _i32c(t):
    return t.detach().to("cpu", torch.int32).contiguous()


def _i64(v):
    return ctypes.c_int64(int(v))


def _check(rc, name):
    if rc != 0:
        raise RuntimeError(f"{name} failed with status {rc}")


def eps_for(dtype: torch.dtype, eps: float = 1e-10) -> float:
    """The absmax floor as the reference's op sees it: ``clamp(min=eps)`` is applied
    in the SOURCE dtype before the cast to fp32 (tests/kernels/quant_utils.py:212-213)."""
    return float(torch.tensor(eps, dtype=torch.float64).to(dtype).to(torch.float32))


def quant_rows(x: torch.Tensor, eps: float | None = None):
    """x [..., D] (fp32/bf16/fp16, CPU) -> (codes int8 [..., D], scales fp32 [...])."""
    if eps is None:
        eps = eps_for(x.dtype)
    xf = _f32c(x)
    D = xf.shape[-1]
    rows = xf.numel() // D
    codes = torch.empty(xf.shape, dtype=torch.int8)
    scales = torch.empty(xf.shape[:-1], dtype=torch.float32)
    _check(
        lib().kvq_oracle_quant_rows(_p(xf), _i64(rows), _i64(D), ctypes.c_float(eps), _p(codes), _p(scales)),
        "kvq_oracle_quant_rows",
    )
    return codes, scales


CODE_INT8, CODE_FP8, CODE_INT4 = 0, 1, 2


def quant_rows_int4(x: torch.Tensor, eps: float | None = None):
    """x [..., D] (CPU) -> (packed codes uint8 [..., D/2], scales fp32 [...]): scale = max(absmax, eps) / 7,
    code = clamp(rint(x / scale), -8, 7) as a 4-bit two's-complement number, the even dim in the low nibble."""
    if eps is None:
        eps = eps_for(x.dtype)
    xf = _f32c(x)
    D = xf.shape[-1]
    rows = xf.numel() // D
    codes = torch.empty(xf.shape[:-1] + (D // 2,), dtype=torch.uint8)
    scales = torch.empty(xf.shape[:-1], dtype=torch.float32)
    lib().kvq_oracle_quant_rows_int4.restype = ctypes.c_int
    _check(
        lib().kvq_oracle_quant_rows_int4(_p(xf), _i64(rows), _i64(D), ctypes.c_float(eps), _p(codes), _p(scales)),
        "kvq_oracle_quant_rows_int4",
    )
    return codes, scales


def unpack_int4(codes: torch.Tensor) -> torch.Tensor:
    """Packed int4 codes uint8 [..., D/2] -> their values int8 [..., D] (pure torch, for the tests)."""
    c = codes.to(torch.int16)
    lo, hi = c & 15, (c >> 4) & 15
    both = torch.stack((lo, hi), dim=-1).reshape(codes.shape[:-1] + (codes.shape[-1] * 2,))
    return torch.where(both >= 8, both - 16, both).to(torch.int8)


def quant_rows_fp8(x: torch.Tensor, eps: float | None = None):
    """x [..., D] (CPU) -> (codes uint8 [..., D] holding e4m3fn bit patterns, scales fp32 [...]):
    scale = max(absmax, eps) / 448, code = nearest e4m3fn to x / scale (ties to even)."""
    if eps is None:
        eps = eps_for(x.dtype)
    xf = _f32c(x)
    D = xf.shape[-1]
    rows = xf.numel() // D
    codes = torch.empty(xf.shape, dtype=torch.uint8)
    scales = torch.empty(xf.shape[:-1], dtype=torch.float32)
    _check(
        lib().kvq_oracle_quant_rows_fp8(_p(xf), _i64(rows), _i64(D), ctypes.c_float(eps), _p(codes), _p(scales)),
        "kvq_oracle_quant_rows_fp8",
    )
    return codes, scales


def e4m3fn_table() -> torch.Tensor:
    """The 256 values of the e4m3fn byte (0x7f / 0xff, the format's NaN, read as +-480 and never produced)."""
    fn = lib().kvq_oracle_e4m3fn_value
    fn.restype = ctypes.c_float
    return torch.tensor([fn(ctypes.c_int(i)) for i in range(256)], dtype=torch.float32)


def cache_write(key, value, kv_cache, lay: RecordLayout, slot_mapping, eps: float | None = None,
                code_type: int = CODE_INT8):
    """Quantise key/value [T', Hkv, D] into kv_cache (CPU int8 storage) in place."""
    if eps is None:
        eps = eps_for(key.dtype)
    kf, vf = _f32c(key), _f32c(value)
    sm = slot_mapping.detach().to("cpu", torch.int64).contiguous()
    T = sm.shape[0]
    assert kf.shape[0] >= T and kf.shape[1] == lay.num_kv_heads and kf.shape[2] == lay.head_size
    _check(
        lib().kvq_oracle_cache_write_ex(
            _p(kf), _p(vf), _p(kv_cache),
            _i64(lay.k_off), _i64(lay.v_off), _i64(lay.ks_off), _i64(lay.vs_off),
            _i64(lay.stride_block), _i64(lay.stride_slot), _i64(lay.stride_head),
            _p(sm), _i64(T), ctypes.c_int(lay.num_kv_heads), ctypes.c_int(lay.head_size),
            ctypes.c_int(lay.block_size), ctypes.c_float(eps), ctypes.c_int(code_type),
        ),
        "kvq_oracle_cache_write_ex",
    )


def paged_attn(q, kv_cache, lay: RecordLayout, block_table, seq_lens, cu_seqlens_q,
               scale: float, causal: bool = True, return_lse: bool = False, sliding_window: int = 0,
               soft_cap: float = 0.0, code_type: int = CODE_INT8, sinks=None, alibi_slopes=None):
    """q [N, Hq, D] -> out fp32 [N, Hq, D] (and lse fp32 [N, Hq]).  sliding_window > 0: a query sees its
    last `sliding_window` keys (itself included); soft_cap > 0: logits -> cap * tanh(logit / cap);
    sinks [Hq]: one more logit per head with a zero value row (attention sinks); alibi_slopes [Hq]: the logit
    of query position p and key position j gets slope * (j - p) added."""
    qf = _f32c(q)
    sk = _f32c(sinks) if sinks is not None else None
    al = _f32c(alibi_slopes) if alibi_slopes is not None else None
    N, Hq, D = qf.shape
    bt, sl, cu = _i32c(block_table), _i32c(seq_lens), _i32c(cu_seqlens_q)
    B = sl.shape[0]
    out = torch.empty((N, Hq, D), dtype=torch.float32)
    lse = torch.empty((N, Hq), dtype=torch.float32) if return_lse else None
    _check(
        lib().kvq_oracle_paged_attn_ex4(
            _p(out), _p(lse), _p(qf), _p(kv_cache),
            _i64(lay.k_off), _i64(lay.v_off), _i64(lay.ks_off), _i64(lay.vs_off),
            _i64(lay.stride_block), _i64(lay.stride_slot), _i64(lay.stride_head),
            _p(bt), _i64(bt.stride(0)), _p(sl), _p(cu),
            ctypes.c_int(B), ctypes.c_int(Hq), ctypes.c_int(lay.num_kv_heads), ctypes.c_int(D),
            ctypes.c_int(lay.block_size), ctypes.c_float(scale), ctypes.c_int(1 if causal else 0),
            ctypes.c_int(int(sliding_window or 0)), ctypes.c_float(float(soft_cap or 0.0)),
            ctypes.c_int(code_type), _p(sk), _p(al),
        ),
        "kvq_oracle_paged_attn_ex4",
    )
    return (out, lse) if return_lse else out


def paged_attn_partition(q, kv_cache, lay: RecordLayout, block_table, seq_lens, scale: float,
                         partition_size: int, max_parts: int):
    """Decode rows only.  Returns (tmp_out [B,Hq,P,D], max_logits [B,Hq,P], exp_sums [B,Hq,P])."""
    qf = _f32c(q)
    B, Hq, D = qf.shape
    bt, sl = _i32c(block_table), _i32c(seq_lens)
    tmp = torch.zeros((B, Hq, max_parts, D), dtype=torch.float32)
    ml = torch.zeros((B, Hq, max_parts), dtype=torch.float32)
    es = torch.zeros((B, Hq, max_parts), dtype=torch.float32)
    _check(
        lib().kvq_oracle_paged_attn_partition(
            _p(tmp), _p(ml), _p(es), _p(qf), _p(kv_cache),
            _i64(lay.k_off), _i64(lay.v_off), _i64(lay.ks_off), _i64(lay.vs_off),
            _i64(lay.stride_block), _i64(lay.stride_slot), _i64(lay.stride_head),
            _p(bt), _i64(bt.stride(0)), _p(sl),
            ctypes.c_int(B), ctypes.c_int(Hq), ctypes.c_int(lay.num_kv_heads), ctypes.c_int(D),
            ctypes.c_int(lay.block_size), ctypes.c_float(scale), ctypes.c_int(partition_size),
            ctypes.c_int(max_parts),
        ),
        "kvq_oracle_paged_attn_partition",
    )
    return tmp, ml, es


def splitk_reduce(tmp_out, max_logits, exp_sums, seq_lens, partition_size: int, return_lse: bool = False):
    tmp, ml, es = _f32c(tmp_out), _f32c(max_logits), _f32c(exp_sums)
    B, Hq, P, D = tmp.shape
    sl = _i32c(seq_lens)
    out = torch.empty((B, Hq, D), dtype=torch.float32)
    lse = torch.empty((B, Hq), dtype=torch.float32) if return_lse else None
    _check(
        lib().kvq_oracle_splitk_reduce(
            _p(out), _p(lse), _p(tmp), _p(ml), _p(es), _p(sl),
            ctypes.c_int(B), ctypes.c_int(Hq), ctypes.c_int(D), ctypes.c_int(partition_size), ctypes.c_int(P),
        ),
        "kvq_oracle_splitk_reduce",
    )
    return (out, lse) if return_lse else out


def merge_attn_states(prefix_output, prefix_lse, suffix_output, suffix_lse, prefix_num_tokens=None):
    """outputs [T, H, D]; lse [H, T].  Returns (output fp32, output_lse fp32)."""
    po, so = _f32c(prefix_output), _f32c(suffix_output)
    pl, sl = _f32c(prefix_lse), _f32c(suffix_lse)
    T, H, D = po.shape
    if prefix_num_tokens is None:
        prefix_num_tokens = T
    out = torch.empty((T, H, D), dtype=torch.float32)
    lse = torch.empty((H, T), dtype=torch.float32)
    _check(
        lib().kvq_oracle_merge_attn_states(
            _p(out), _p(lse), _p(po), _p(pl), _p(so), _p(sl),
            _i64(T), ctypes.c_int(H), ctypes.c_int(D), _i64(prefix_num_tokens),
        ),
        "kvq_oracle_merge_attn_states",
    )
    return out, lse


@dataclass(frozen=True)
class MlaLayout:
    """Byte geometry of the int8 latent cache: code rows and the per-token fp32
    scale region of a block."""

    stride_block: int
    stride_row: int
    scale_off: int
    block_size: int
    kv_lora_rank: int
    rope_dim: int

    @staticmethod
    def from_views(cache, codes_view, scales_view, kv_lora_rank):
        base = cache.data_ptr()
        nb, bs, W = codes_view.shape
        assert codes_view.data_ptr() == base and codes_view.stride(2) == 1
        assert scales_view.stride(1) == 1 and 4 * scales_view.stride(0) == codes_view.stride(0)
        return MlaLayout(
            stride_block=codes_view.stride(0),
            stride_row=codes_view.stride(1),
            scale_off=scales_view.data_ptr() - base,
            block_size=bs,
            kv_lora_rank=kv_lora_rank,
            rope_dim=W - kv_lora_rank,
        )


def mla_cache_write(kv_c, k_pe, cache, lay: MlaLayout, slot_mapping, eps: float | None = None):
    if eps is None:
        eps = eps_for(kv_c.dtype)
    a, b = _f32c(kv_c), _f32c(k_pe)
    sm = slot_mapping.detach().to("cpu", torch.int64).contiguous()
    _check(
        lib().kvq_oracle_mla_cache_write(
            _p(a), _p(b), _p(cache), _i64(lay.stride_block), _i64(lay.stride_row), _i64(lay.scale_off),
            _p(sm), _i64(sm.shape[0]), ctypes.c_int(lay.kv_lora_rank), ctypes.c_int(lay.rope_dim),
            ctypes.c_int(lay.block_size), ctypes.c_float(eps),
        ),
        "kvq_oracle_mla_cache_write",
    )


def rope_rotate(x, positions, cos_sin_cache, is_neox: bool):
    """Rotary embedding as the reference's fused kernel applies it
    (csrc/libtorch_stable/cache_kernels_fused.cu:55-84 for q_pe, :90-117 for k_pe), restated with
    torch ops in the tensor's own dtype: cos / sin are cast to it first, every product and every
    sum is rounded to it on its own (the reference's ``qk_t`` operators; for float32 that means no
    fused multiply-add; which rounding a 16-bit type's operators perform is spelled out below).  ``x`` ``[T, ..., rot_dim]``; ``cos_sin_cache`` ``[max_position, rot_dim]``
    = ``rot_dim/2`` cosines then ``rot_dim/2`` sines per position.  Pair i is ``(i, rot_dim/2 + i)``
    when ``is_neox`` else ``(2i, 2i + 1)``.  Returns a new tensor."""
    rot = x.shape[-1]
    embed = rot // 2
    cs = cos_sin_cache[positions.long()].to(x.dtype)                  # [T, rot]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [embed]
    cos, sin = cs[:, :embed].reshape(shape), cs[:, embed:].reshape(shape)
    if is_neox:
        xs, ys = x[..., :embed], x[..., embed:]
    else:
        xs, ys = x[..., 0::2], x[..., 1::2]
    if x.dtype == torch.float16:
        # native half operators: every result is the exact one rounded ONCE to fp16.  The exact
        # products and sums of fp16 numbers fit a double; numpy converts double -> half directly.
        import numpy as np

        def once(t):
            return torch.from_numpy(t.astype(np.float16))

        d = lambda t: t.double().numpy()
        xo = once(d(once(d(xs) * d(cos))) - d(once(d(ys) * d(sin))))
        yo = once(d(once(d(ys) * d(cos))) + d(once(d(xs) * d(sin))))
    else:
        # bfloat16: torch's operators go through float and round after every operation, like the
        # bf16 operators of hip_bf16.h that the reference's ROCm branch uses (:13-16); float32: plain
        xo = xs * cos - ys * sin
        yo = ys * cos + xs * sin
    out = torch.empty_like(x)
    if is_neox:
        out[..., :embed], out[..., embed:] = xo, yo
    else:
        out[..., 0::2], out[..., 1::2] = xo, yo
    return out


def mla_rope_cache_write(positions, q_pe, k_pe, kv_c, cos_sin_cache, is_neox: bool, cache, lay: MlaLayout,
                         slot_mapping, eps: float | None = None):
    """``concat_and_cache_mla_rope_fused`` (csrc/libtorch_stable/cache_kernels_fused.cu:24-168) over
    the int8 latent cache: rotates ``q_pe`` ``[T, Hq, rot]`` and ``k_pe`` ``[T, rot]`` IN PLACE for the
    tokens whose slot is >= 0 (padded tokens are skipped before anything is touched, :42-46) and
    writes ``[kv_c | rotated k_pe]`` through the latent quantiser."""
    live = slot_mapping >= 0
    q_pe[live] = rope_rotate(q_pe[live], positions[live], cos_sin_cache, is_neox)
    k_pe[live] = rope_rotate(k_pe[live], positions[live], cos_sin_cache, is_neox)
    mla_cache_write(kv_c, k_pe, cache, lay, slot_mapping, eps)


def mla_decode(q, cache, lay: MlaLayout, block_table, seq_lens, scale: float):
    """q [B, H, R+P] -> (out fp32 [B, H, R], lse fp32 [B, H])."""
    qf = _f32c(q)
    B, H, W = qf.shape
    assert W == lay.kv_lora_rank + lay.rope_dim
    bt, sl = _i32c(block_table), _i32c(seq_lens)
    out = torch.empty((B, H, lay.kv_lora_rank), dtype=torch.float32)
    lse = torch.empty((B, H), dtype=torch.float32)
    _check(
        lib().kvq_oracle_mla_decode(
            _p(out), _p(lse), _p(qf), _p(cache), _i64(lay.stride_block), _i64(lay.stride_row),
            _i64(lay.scale_off), _p(bt), _i64(bt.stride(0)), _p(sl),
            ctypes.c_int(B), ctypes.c_int(H), ctypes.c_int(lay.kv_lora_rank), ctypes.c_int(lay.rope_dim),
            ctypes.c_int(lay.block_size), ctypes.c_float(scale),
        ),
        "kvq_oracle_mla_decode",
    )
    return out, lse


def mla_gather_dequant(cache, lay: MlaLayout, block_table, cu_seq_lens, token_to_seq, num_tokens, seq_starts=None):
    """int8 latent cache -> fp32 [num_tokens, R+P] rows (code * row scale)."""
    bt, cu, t2s = _i32c(block_table), _i32c(cu_seq_lens), _i32c(token_to_seq)
    ss = _i32c(seq_starts) if seq_starts is not None else None
    W = lay.kv_lora_rank + lay.rope_dim
    dst = torch.zeros((num_tokens, W), dtype=torch.float32)
    _check(
        lib().kvq_oracle_mla_gather_dequant(
            _p(dst), _i64(W), _p(cache), _i64(lay.stride_block), _i64(lay.stride_row), _i64(lay.scale_off),
            _p(bt), _i64(bt.stride(0)), _p(cu), _p(t2s), _p(ss) if ss is not None else None,
            ctypes.c_int(num_tokens), ctypes.c_int(W), ctypes.c_int(lay.block_size),
        ),
        "kvq_oracle_mla_gather_dequant",
    )
    return dst

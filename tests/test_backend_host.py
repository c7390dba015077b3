"""Host-side logic of the backend mirror: capability flags, cache geometry, selection, error
behaviour, and that the C-ABI library loads and exports every symbol include/kvq.h declares.
No GPU needed."""
import os
import re
import types

import pytest
import torch

from vllm_metax_amd import _C, platform as P
from vllm_metax_amd.kv_cache_interface import KVQuantMode, get_kv_quant_mode, kv_cache_uses_per_token_head_scales
from vllm_metax_amd.v1.attention.backends.int8_attn import (
    AttentionType, Int8AttentionBackend, Int8AttentionImpl, Int8AttentionMetadataBuilder, MultipleOf)
from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLABackend, Int8MLAImpl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "kvq.h")).read()
    declared = set(re.findall(r"KVQ_API\s+[\w\s\*]+?\b(kvq_\w+)\s*\(", header))
    assert declared == set(_C.SIGNATURES), declared ^ set(_C.SIGNATURES)
    lib = _C.load()                                   # raises if a symbol is missing
    assert lib.kvq_abi_version() == _C.ABI_VERSION
    for name in declared:
        assert hasattr(lib, name)


def test_quant_modes():
    assert get_kv_quant_mode("int8_per_token_head") == KVQuantMode.INT8_PER_TOKEN_HEAD
    assert kv_cache_uses_per_token_head_scales("int8_per_token_head")
    assert not kv_cache_uses_per_token_head_scales("auto")
    with pytest.raises(ValueError):
        get_kv_quant_mode("int3")


def test_backend_statics_match_the_reference_surface():
    B = Int8AttentionBackend
    assert B.get_name() == "TRITON_ATTN" and B.forward_includes_kv_cache_update is False
    assert "int8_per_token_head" in B.supported_kv_cache_dtypes
    assert B.get_supported_kernel_block_sizes() == [MultipleOf(16)]
    assert B.supports_block_size(None) and B.supports_block_size(48) and not B.supports_block_size(24)
    assert B.get_kv_cache_shape(40000, 16, 8, 128, "int8_per_token_head") == (40000, 8, 16, 264)
    with pytest.raises(ValueError):
        B.get_kv_cache_shape(10, 8, 8, 128)
    # no setting: the order the decode kernel streams (a head's records of a block back to back)
    os.environ.pop("VLLM_KV_CACHE_LAYOUT", None)
    assert B.get_kv_cache_stride_order() == (0, 1, 2, 3)
    assert B.get_kv_cache_stride_order(include_num_layers_dimension=True) == (1, 2, 0, 3, 4)
    # an explicit setting is honoured either way (vllm_metax/v1/attention/backends/triton_attn.py:350-372)
    for asked, order, order5 in (("NHD", (0, 2, 1, 3), (1, 0, 3, 2, 4)), ("HND", (0, 1, 2, 3), (1, 2, 0, 3, 4)),
                                 ("nhd", (0, 2, 1, 3), (1, 0, 3, 2, 4))):
        os.environ["VLLM_KV_CACHE_LAYOUT"] = asked
        try:
            assert B.get_kv_cache_stride_order() == order
            assert B.get_kv_cache_stride_order(include_num_layers_dimension=True) == order5
        finally:
            os.environ.pop("VLLM_KV_CACHE_LAYOUT")
    os.environ["VLLM_KV_CACHE_LAYOUT"] = "DHN"
    try:
        with pytest.raises(ValueError):
            B.get_kv_cache_stride_order()
    finally:
        os.environ.pop("VLLM_KV_CACHE_LAYOUT")
    assert B.use_cascade_attention() is False
    assert B.get_impl_cls() is Int8AttentionImpl and B.get_builder_cls() is Int8AttentionMetadataBuilder
    M = Int8MLABackend
    assert M.get_name() == "TRITON_MLA"
    assert M.get_kv_cache_shape(100, 64, 1, 576) == (100, 64, 580)
    assert M.get_kv_cache_stride_order() == (0, 1, 2) and M.get_kv_cache_stride_order(True) == (1, 0, 2, 3)


def test_selection_and_reasons():
    ok = dict(kv_cache_dtype="int8_per_token_head", head_size=128, dtype=torch.bfloat16, block_size=16)
    assert P.get_attn_backend_cls(**ok) == P.INT8_ATTN_PATH
    assert P.get_attn_backend_cls("TRITON_ATTN", **ok) == P.INT8_ATTN_PATH
    assert P.get_attn_backend_cls(use_mla=True, kv_cache_dtype="int8_per_token", dtype=torch.bfloat16,
                                  block_size=64) == P.INT8_MLA_PATH
    assert Int8AttentionBackend.validate_configuration(**ok) == []
    assert Int8AttentionBackend.validate_configuration(**{**ok, "kv_cache_dtype": "fp8"}) == ["kv_cache_dtype not supported"]
    assert Int8AttentionBackend.validate_configuration(**{**ok, "block_size": 24}) == ["block_size not supported"]
    with pytest.raises(ValueError, match="not valid for this configuration"):
        P.get_attn_backend_cls("TRITON_ATTN", **{**ok, "head_size": 80})
    with pytest.raises(ValueError, match="No valid attention backend"):
        P.get_attn_backend_cls(**{**ok, "kv_cache_dtype": "auto"})
    with pytest.raises(ValueError):
        P.get_attn_backend_cls("FLASH_ATTN", **ok)
    assert P.register_attention_backends() is False    # nothing is overwritten by default
    assert P.register_attention_backends(replace_slots=True) is False   # no upstream vLLM here: a no-op


def test_register_returns_the_platform_and_the_platform_routes_by_kv_dtype():
    """register() names the platform class, as the reference's does (vllm_metax/__init__.py:14-16); the platform
    sends int8 KV dtypes to this build's backends and refuses to swallow the others."""
    import importlib

    import vllm_metax_amd

    path = vllm_metax_amd.register()
    assert path == P.PLATFORM_PATH
    module, _, cls = path.rpartition(".")
    plat = getattr(importlib.import_module(module), cls)
    sel = types.SimpleNamespace(kv_cache_dtype="int8_per_token_head", head_size=128, dtype=torch.bfloat16, block_size=16)
    assert plat.get_attn_backend_cls(None, sel, 32) == P.INT8_ATTN_PATH
    mla = types.SimpleNamespace(kv_cache_dtype="int8_per_token", dtype=torch.bfloat16, block_size=64, use_mla=True)
    assert plat.get_attn_backend_cls(None, mla, 128) == P.INT8_MLA_PATH
    with pytest.raises(ValueError, match="does not serve kv_cache_dtype"):
        plat.get_attn_backend_cls("FLASH_ATTN", sel, 32)
    with pytest.raises(ValueError, match="not served by this build"):          # no upstream platform to hand it to here
        plat.get_attn_backend_cls(None, types.SimpleNamespace(kv_cache_dtype="auto"), 32)
    vllm_metax_amd.register_out_of_tree()
    toml = open(os.path.join(ROOT, "vllm-metax_amd", "pyproject.toml")).read()
    assert 'vllm.platform_plugins' in toml and '"vllm_metax_amd:register"' in toml
    assert 'vllm.general_plugins' in toml and '"vllm_metax_amd:register_out_of_tree"' in toml


def test_mla_builder_splits_decodes_first_and_needs_no_gpu():
    from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLAMetadataBuilder

    assert Int8MLABackend.get_builder_cls() is Int8MLAMetadataBuilder
    assert Int8MLAMetadataBuilder._cudagraph_support.name == "UNIFORM_SINGLE_TOKEN_DECODE"
    assert Int8AttentionMetadataBuilder._cudagraph_support.name == "ALWAYS"
    spec = types.SimpleNamespace(block_size=64, num_kv_heads=1, head_size=576, num_heads=16)
    cfg = types.SimpleNamespace(scheduler_config=types.SimpleNamespace(max_num_seqs=4))
    b = Int8MLAMetadataBuilder(spec, ["l0"], cfg, "cpu")
    c = types.SimpleNamespace(num_reqs=3, num_actual_tokens=7, max_query_len=5, max_seq_len=90,
                              query_start_loc=torch.tensor([0, 1, 2, 7], dtype=torch.int32),
                              seq_lens=torch.tensor([9, 4, 90], dtype=torch.int32),
                              block_table_tensor=torch.zeros((3, 2), dtype=torch.int32),
                              slot_mapping=torch.arange(7))
    md = b.build(0, c)
    assert (md.num_decodes, md.num_decode_tokens, md.num_prefills) == (2, 2, 1)
    assert md.decode.seq_lens.tolist() == [9, 4] and md.decode.block_table.shape == (2, 2)
    assert md.workspace is None and md.decode_out is None      # no GPU: nothing reserved
    c.query_start_loc = torch.tensor([0, 5, 6, 7], dtype=torch.int32)           # a decode after a prefill
    with pytest.raises(RuntimeError, match="decode requests must come first"):
        b.build(0, c)


def test_impl_fills_scale_views_once_per_cache_tensor():
    impl = Int8AttentionImpl(8, 128, 0.09, 2)
    from vllm_metax_amd import layout as L

    a = L.allocate_kv_cache(4, 16, 2, 128, device="cpu")
    b = L.allocate_kv_cache(4, 16, 2, 128, device="cpu")
    impl._ensure_scale_caches(a)
    ks, vs = L.scale_views(a)
    assert bool((ks == 1).all()) and bool((vs == 1).all())
    ks.fill_(0.5)                                              # scales a write has stored
    impl._ensure_scale_caches(b)
    impl._ensure_scale_caches(a)                               # back on A: must not be wiped
    assert bool((L.scale_views(a)[0] == 0.5).all())
    impl._ensure_scale_caches(a.view(a.shape))                 # another tensor object over the same cache
    assert bool((L.scale_views(a)[0] == 0.5).all())


def test_impl_does_not_pin_replaced_caches_and_refills_a_new_cache_at_a_reused_address():
    import gc
    import weakref

    from vllm_metax_amd import layout as L

    impl = Int8AttentionImpl(8, 128, 0.09, 2)
    a = L.allocate_kv_cache(4, 16, 2, 128, device="cpu")
    b = L.allocate_kv_cache(4, 16, 2, 128, device="cpu")
    impl._ensure_scale_caches(a)
    dead = weakref.ref(a.untyped_storage())
    addr = a.data_ptr()
    impl._ensure_scale_caches(b)                               # the impl moves on to another cache ...
    del a
    gc.collect()
    assert dead() is None                                      # ... and the first one is free to go
    assert len(impl._filled) == 1
    # allocations of the freed size until one lands on the freed address (the allocator usually hands it
    # straight back); whichever address it gets, a cache never seen before must come out with scales 1.0
    for _ in range(16):
        c = L.allocate_kv_cache(4, 16, 2, 128, device="cpu", fill=None)
        L.scale_views(c)[0].fill_(7.0)
        L.scale_views(c)[1].fill_(7.0)
        same = c.data_ptr() == addr
        impl._ensure_scale_caches(c)
        ks, vs = L.scale_views(c)
        assert bool((ks == 1).all()) and bool((vs == 1).all())
        if same:
            break


def test_impl_constructor_errors():
    mk = lambda **kw: Int8AttentionImpl(32, 128, 0.088, 8, **kw)
    impl = mk()
    assert impl.num_queries_per_kv == 4 and impl.fused_rope_kvcache_supported() is True   # built here; the reference answers False
    for kw in (dict(use_alibi_sqrt=True), dict(attn_type=AttentionType.ENCODER_ONLY)):
        with pytest.raises(NotImplementedError):
            mk(**kw)
    # cross-attention goes through the cache like decoder self-attention (triton_attn.py:394-402, 796-799)
    assert mk(attn_type=AttentionType.ENCODER_DECODER).attn_type == AttentionType.ENCODER_DECODER
    assert Int8AttentionBackend.supports_attn_type(AttentionType.ENCODER_DECODER)
    assert not Int8AttentionBackend.supports_attn_type(AttentionType.ENCODER)
    # ALiBi slopes: a float32 tensor with one slope per head, as the reference keeps them (triton_attn.py:504-506)
    al = mk(alibi_slopes=[0.5] * 32).alibi_slopes
    assert al.dtype == torch.float32 and tuple(al.shape) == (32,) and mk().alibi_slopes is None
    with pytest.raises(ValueError):
        mk(alibi_slopes=[0.5] * 8)
    # attention sinks: one per q head, kept as float32 (triton_attn.py:548-554)
    assert mk(sinks=torch.zeros(32, dtype=torch.bfloat16)).sinks.dtype == torch.float32
    with pytest.raises(ValueError):
        mk(sinks=torch.zeros(8))
    # the reference's mapping of the two knobs (triton_attn.py:507-512, 536-539)
    assert impl.sliding_window == (-1, -1) and impl.logits_soft_cap == 0
    w = mk(sliding_window=128, logits_soft_cap=30.0)
    assert w.sliding_window == (127, 0) and w.logits_soft_cap == 30.0
    with pytest.raises(ValueError):
        mk(sliding_window=0)
    with pytest.raises(ValueError):
        mk(kv_cache_dtype="auto")
    with pytest.raises(NotImplementedError):
        impl.do_rope_and_kv_cache_update()
    out = torch.ones(3, 32 * 128)
    assert impl.forward(None, None, None, None, None, None, out) is out and bool((out == 0).all())   # profiling run
    with pytest.raises(NotImplementedError):
        impl.forward(None, None, None, None, None, types.SimpleNamespace(), out, output_scale=torch.ones(1))
    with pytest.raises(NotImplementedError):
        Int8MLAImpl(128, 576, 0.07, sliding_window=4)
    with pytest.raises(ValueError):
        Int8MLAImpl(128, 576, 0.07, kv_cache_dtype="fp8")


def test_backends_serve_batch_invariance_and_the_switch_is_the_librarys():
    """triton_attn.py:310-312; the mode itself is a process-wide switch of the library (no GPU needed to flip it)."""
    assert Int8AttentionBackend.supports_batch_invariance() is True
    assert Int8MLABackend.supports_batch_invariance() is True
    lib = _C.load()
    before = lib.kvq_set_batch_invariant(1)
    assert lib.kvq_get_batch_invariant() == 1 and lib.kvq_set_batch_invariant(0) == 1
    assert lib.kvq_get_batch_invariant() == 0
    lib.kvq_set_batch_invariant(before)


def test_builder_packs_metadata_without_touching_the_gpu():
    spec = types.SimpleNamespace(block_size=16, num_kv_heads=8, head_size=128, num_q_heads=32)
    cfg = types.SimpleNamespace(scheduler_config=types.SimpleNamespace(max_num_seqs=4))
    b = Int8AttentionMetadataBuilder(spec, ["l0"], cfg, "cpu")
    c = types.SimpleNamespace(num_reqs=2, num_actual_tokens=2, max_query_len=1, max_seq_len=9,
                              query_start_loc=torch.tensor([0, 1, 2], dtype=torch.int32),
                              seq_lens=torch.tensor([9, 4], dtype=torch.int32),
                              block_table_tensor=torch.zeros((2, 1), dtype=torch.int32),
                              slot_mapping=torch.tensor([8, 19]), causal=True)
    md = b.build(0, c)
    assert md.num_actual_tokens == 2 and md.workspace is None and md.use_cascade is False
    assert b.build_for_cudagraph_capture(c).seq_lens.tolist() == [1, 1]
    assert md.has_decode_rows is True
    # the host copy of query_start_loc tells a pure prefill batch from a mixed one
    c2 = types.SimpleNamespace(**{**c.__dict__, "max_query_len": 7, "num_actual_tokens": 10,
                                  "query_start_loc_cpu": torch.tensor([0, 3, 10], dtype=torch.int32)})
    assert b.build(0, c2).has_decode_rows is False
    c2.query_start_loc_cpu = torch.tensor([0, 1, 8], dtype=torch.int32)
    assert b.build(0, c2).has_decode_rows is True
    with pytest.raises(NotImplementedError):
        b.build(4, c)
    c.num_reqs = 5
    with pytest.raises(RuntimeError):
        b.build(0, c)


def test_ops_refuse_cpu_tensors_and_bad_shapes_before_touching_the_library():
    """There is no CPU path: every op raises RuntimeError on host tensors (the product must fail
    loudly, never fall back), and shape / dtype mistakes are reported by the wrappers themselves."""
    import pytest
    import torch

    from vllm_metax_amd import _custom_ops as ops
    from vllm_metax_amd import layout as L

    a = torch.zeros((2, 4, 512), dtype=torch.bfloat16)
    b = torch.zeros((2, 4, 64), dtype=torch.bfloat16)
    out = torch.zeros((2, 4, 576), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.concat_mla_q(a, b, out)
    kv = L.allocate_kv_cache(4, 16, 2, 64, device="cpu")
    with pytest.raises(RuntimeError):
        ops.copy_blocks([kv], torch.zeros((1, 2), dtype=torch.int64))
    ops.copy_blocks([], torch.zeros((1, 2), dtype=torch.int64))          # nothing to do: no library call
    cache = L.allocate_mla_cache(2, 64, 576, device="cpu")
    o = torch.zeros((2, 4, 512), dtype=torch.bfloat16)
    bt = torch.zeros((2, 1), dtype=torch.int32)
    sl = torch.ones(2, dtype=torch.int32)
    with pytest.raises(RuntimeError):
        ops.mla_decode_int8((a, b), cache, o, None, bt, sl, 0.1, 512)
    with pytest.raises(RuntimeError):
        ops.mla_decode_int8(out, cache, o, None, bt, sl, 0.1, 512)


def test_c_abi_rejects_bad_arguments_of_the_newer_entry_points_without_a_gpu():
    """Argument checks run before anything is launched: the entry points return KVQ_EINVAL (-22) and leave a
    message, also on a machine without a GPU."""
    import ctypes

    lib = _C.load()
    g = _C.CacheGeom(0, 132, 128, 260, 16 * 8 * 264, 8 * 264, 264, 8, 128, 16, _C.KVQ_CODE_INT8)
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)   # any non-NULL address: nothing is dereferenced on the host
    # rope + write: NULL pointers, an odd rotary width, a rotary width beyond the head size, an unknown code type
    assert lib.kvq_rope_and_cache_int8(null, one, 0, 0, 32, one, 0, 0, one, 0, 0, _C.KVQ_BF16, one, _C.KVQ_BF16, 64, 1,
                                       one, ctypes.byref(g), one, 4, 0.0, null) == -22
    assert b"NULL" in lib.kvq_last_error()
    for rot in (63, 130):
        assert lib.kvq_rope_and_cache_int8(one, one, 0, 0, 32, one, 0, 0, one, 0, 0, _C.KVQ_BF16, one, _C.KVQ_BF16, rot,
                                           1, one, ctypes.byref(g), one, 4, 0.0, null) == -22
        assert b"rot_dim" in lib.kvq_last_error()
    bad = _C.CacheGeom(0, 132, 128, 260, 16 * 8 * 264, 8 * 264, 264, 8, 128, 16, 7)
    assert lib.kvq_rope_and_cache_int8(one, one, 0, 0, 32, one, 0, 0, one, 0, 0, _C.KVQ_BF16, one, _C.KVQ_BF16, 64, 1,
                                       one, ctypes.byref(bad), one, 4, 0.0, null) == -22
    assert b"code_type" in lib.kvq_last_error()
    assert lib.kvq_rope_and_cache_int8(one, one, 0, 0, 32, one, 0, 0, one, 0, 0, _C.KVQ_BF16, one, _C.KVQ_BF16, 64, 1,
                                       one, ctypes.byref(g), one, 0, 0.0, null) == 0      # no tokens: nothing to do
    # an int4 geometry whose record is not [D/2 codes | scale | D/2 codes | scale] is refused by the attention entry
    g4 = _C.CacheGeom(0, 132, 128, 260, 16 * 8 * 264, 8 * 264, 264, 8, 128, 16, _C.KVQ_CODE_INT4)
    rc = lib.kvq_paged_attn_int8(one, _C.KVQ_BF16, 4096, 128, one, _C.KVQ_BF16, 4096, 128, one, ctypes.byref(g4), one, 8,
                                 one, null, 2, 32, 1, 0.1, 1, 0, 0.0, null, null, null, one, 1 << 20, null)
    assert rc == -22 and b"record" in lib.kvq_last_error()
    # an unknown flag in `causal`
    rc = lib.kvq_paged_attn_int8(one, _C.KVQ_BF16, 4096, 128, one, _C.KVQ_BF16, 4096, 128, one, ctypes.byref(g), one, 8,
                                 one, null, 2, 32, 1, 0.1, 9, 0, 0.0, null, null, null, one, 1 << 20, null)
    assert rc == -22 and b"flag" in lib.kvq_last_error()


def test_mla_prefill_entry_checks_scale_and_strides_without_a_gpu():
    """The kernel takes row maxima before scaling and addresses a tile's rows with 32-bit offsets: a scale that is
    not positive and a token stride of 2^24 elements or more are refused before anything is launched."""
    import ctypes

    lib = _C.load()
    p = ctypes.c_void_p(256)    # any non-NULL, 16-byte aligned address: nothing is dereferenced on the host
    null = ctypes.c_void_p(0)

    def call(scale=0.1, kn_stride=128 * 128, v_stride=128 * 128):
        return lib.kvq_mla_prefill_attn(p, _C.KVQ_BF16, 128 * 192, 192, p, kn_stride, 128, p, 64, p, v_stride, 128, p, p,
                                        1, 64, 64, 128, 128, 64, 128, scale, 1, p, 128 * 128, 128, null, null)

    for bad in (0.0, -0.1, float("inf"), float("nan")):
        assert call(scale=bad) == -22 and b"scale" in lib.kvq_last_error()
    assert call(kn_stride=1 << 24) == -22 and b"stride" in lib.kvq_last_error()
    assert call(v_stride=1 << 24) == -22 and b"stride" in lib.kvq_last_error()


def test_context_split_proposal_follows_the_launch_shape():
    """prefill_context_splits: what a metadata builder asks for from the host copy of the query lengths."""
    from vllm_metax_amd._custom_ops import prefill_context_splits as f
    # one request's small chunk on a long context: 512 tokens x 8 kv heads = 128 workgroups on 256 CUs
    assert f([512], 32768, 32, 8) == 4
    assert f([512] + [1] * 60, 32768, 32, 8) == 4          # decode rows do not count
    assert f([256], 32768, 32, 8) == 8
    assert f([2048], 32768, 32, 8) == 1                    # fills the chip as it is
    assert f([512], 2048, 32, 8) == 1                      # a short context is walked quickly anyway
    assert f([1] * 64, 32768, 32, 8) == 1                  # decode only
    assert f([4] * 64, 32768, 32, 8) == 1                  # short runs: the other kernel
    assert f([2048], 131072, 32, 8, max_split_tokens=4096) == 1
    assert f([1024], 131072, 32, 8, max_split_tokens=4096) == 2    # 256 workgroups: two ranges fill the chip's 512 places
    assert f(torch.tensor([300, 1, 1]), 8192, 28, 4) == 4          # the context allows one split per 2048 tokens

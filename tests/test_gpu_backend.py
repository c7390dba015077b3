"""The backend mirror end to end on the GPU, the way the reference's backend tests drive an impl
without a model runner (tests/v1/attention/test_attention_backends.py:74-183): hand-built paged
cache and metadata, a mock layer, ``do_kv_cache_update`` then ``forward``, compared with the oracle
run on the same tokens (the new tokens are quantised first and read back from the cache)."""
import math
import types

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L
from vllm_metax_amd.v1.attention.backends.int8_attn import Int8AttentionBackend, Int8FusedUpdateAttentionBackend

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("backend", [Int8AttentionBackend, Int8FusedUpdateAttentionBackend],
                         ids=["two_calls", "forward_includes_kv_cache_update"])
@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_decode_step_through_the_backend(gpu_device, layout, backend, monkeypatch):
    """With ``forward_includes_kv_cache_update`` the layer skips ``do_kv_cache_update`` and ``forward`` writes the
    step's tokens itself (one launch for a decode step); cache bytes and output are the same either way."""
    monkeypatch.setenv("VLLM_KV_CACHE_LAYOUT", layout)
    dev = gpu_device
    hq, hkv, d, bs, nb = 32, 8, 128, 16, 200
    ctx = [257, 31, 1024, 5]                       # lengths INCLUDING this step's token
    B = len(ctx)
    g = torch.Generator().manual_seed(7)
    shape = Int8AttentionBackend.get_kv_cache_shape(nb, bs, hkv, d, "int8_per_token_head")
    order = Int8AttentionBackend.get_kv_cache_stride_order()
    phys = torch.zeros(tuple(shape[i] for i in order), dtype=torch.int8, device=dev)
    kv_cache = phys.permute(*[order.index(i) for i in range(4)])      # what the model runner hands over
    kv_cpu, views, lay = T.cpu_cache(nb, bs, hkv, d, layout)
    views[2].fill_(1.0)                            # the impl fills the scale views with 1.0 at first use
    views[3].fill_(1.0)
    bt = T.make_block_tables(ctx, bs, nb, g)
    impl = backend.get_impl_cls()(hq, d, 1 / math.sqrt(d), hkv, kv_cache_dtype="int8_per_token_head")
    spec = types.SimpleNamespace(block_size=bs, num_kv_heads=hkv, head_size=d, num_q_heads=hq)
    cfg = types.SimpleNamespace(scheduler_config=types.SimpleNamespace(max_num_seqs=16))
    builder = Int8AttentionBackend.get_builder_cls()(spec, ["layer.0"], cfg, dev)
    layer = types.SimpleNamespace(_k_scale=torch.ones(1, device=dev), _v_scale=torch.ones(1, device=dev))
    # prefill the context (all but the last token) through the backend's own cache update
    slots = T.slots_for(bt, ctx, bs)
    for i, c in enumerate(ctx):
        if c > 1:
            k = torch.randn((c - 1, hkv, d), generator=g).to(torch.bfloat16)
            v = torch.randn((c - 1, hkv, d), generator=g).to(torch.bfloat16)
            impl.do_kv_cache_update(layer, k.to(dev), v.to(dev), kv_cache, slots[i][:-1].to(dev))
            oracle.cache_write(k, v, T.storage_bytes(kv_cpu), lay, slots[i][:-1])
    # the decode step: one new token per sequence, padded batch (2 padding rows, slot -1)
    pad = 2
    k_new = torch.randn((B + pad, hkv, d), generator=g).to(torch.bfloat16)
    v_new = torch.randn((B + pad, hkv, d), generator=g).to(torch.bfloat16)
    q = torch.randn((B + pad, hq * d), generator=g).to(torch.bfloat16)
    slot_new = torch.tensor([int(s[-1]) for s in slots] + [-1] * pad, dtype=torch.int64)
    common = types.SimpleNamespace(
        num_reqs=B, num_actual_tokens=B, max_query_len=1, max_seq_len=max(ctx),
        query_start_loc=torch.arange(B + 1, dtype=torch.int32, device=dev),
        seq_lens=torch.tensor(ctx, dtype=torch.int32, device=dev), block_table_tensor=bt.to(dev),
        slot_mapping=slot_new.to(dev), causal=True)
    md = builder.build(0, common)
    if not backend.forward_includes_kv_cache_update:
        impl.do_kv_cache_update(layer, k_new.to(dev), v_new.to(dev), kv_cache, md.slot_mapping)
    out = torch.full((B + pad, hq * d), 7.0, dtype=torch.bfloat16, device=dev)
    ret = impl.forward(layer, q.to(dev), k_new.to(dev), v_new.to(dev), kv_cache, md, out)
    torch.cuda.synchronize()
    assert ret is out and bool((out[B:] == 7.0).all()), "rows beyond num_actual_tokens must stay untouched"
    oracle.cache_write(k_new, v_new, T.storage_bytes(kv_cpu), lay, slot_new)
    assert torch.equal(T.storage_bytes(kv_cache).cpu(), T.storage_bytes(kv_cpu)), "cache bytes differ"
    want = oracle.paged_attn(q[:B].view(B, hq, d), T.storage_bytes(kv_cpu), lay, bt,
                             torch.tensor(ctx, dtype=torch.int32), torch.arange(B + 1, dtype=torch.int32),
                             1 / math.sqrt(d))
    T.assert_close_attn(out[:B].view(B, hq, d), want, what=f"backend decode {layout}")


def test_impl_keeps_the_scales_of_a_cache_it_comes_back_to(gpu_device):
    """One impl, two cache tensors: write to A, touch B, attend on A.  The scale views are filled with 1.0
    only the first time a tensor is seen, so A's stored scales survive the visit to B."""
    dev = gpu_device
    hq, hkv, d, bs, nb = 8, 2, 128, 16, 12
    ctx = [70, 33]
    B = len(ctx)
    g = torch.Generator().manual_seed(3)
    impl = Int8AttentionBackend.get_impl_cls()(hq, d, 0.09, hkv, kv_cache_dtype="int8_per_token_head")
    kv_a = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD")
    kv_b = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD")
    kv_cpu, views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    views[2].fill_(1.0)
    views[3].fill_(1.0)
    bt = T.make_block_tables(ctx, bs, nb, g)
    slots = T.slots_for(bt, ctx, bs)
    layer = types.SimpleNamespace()
    for i, c in enumerate(ctx):
        k = torch.randn((c, hkv, d), generator=g).to(torch.bfloat16)
        v = torch.randn((c, hkv, d), generator=g).to(torch.bfloat16)
        impl.do_kv_cache_update(layer, k.to(dev), v.to(dev), kv_a, slots[i].to(dev))
        oracle.cache_write(k, v, T.storage_bytes(kv_cpu), lay, slots[i])
    junk = torch.randn((5, hkv, d), generator=g).to(torch.bfloat16).to(dev)
    impl.do_kv_cache_update(layer, junk, junk, kv_b, torch.arange(5, dtype=torch.int64, device=dev))   # touch B
    q = torch.randn((B, hq * d), generator=g).to(torch.bfloat16)
    md = types.SimpleNamespace(num_actual_tokens=B, max_query_len=1, max_seq_len=max(ctx), use_cascade=False,
                               query_start_loc=torch.arange(B + 1, dtype=torch.int32, device=dev),
                               seq_lens=torch.tensor(ctx, dtype=torch.int32, device=dev), causal=True,
                               block_table=bt.to(dev), workspace=None)
    out = torch.zeros((B, hq * d), dtype=torch.bfloat16, device=dev)
    impl.forward(layer, q.to(dev), None, None, kv_a, md, out)                                            # back on A
    torch.cuda.synchronize()
    assert torch.equal(T.storage_bytes(kv_a).cpu(), T.storage_bytes(kv_cpu)), "A's bytes changed by the visit to B"
    want = oracle.paged_attn(q.view(B, hq, d), T.storage_bytes(kv_cpu), lay, bt, torch.tensor(ctx, dtype=torch.int32),
                             torch.arange(B + 1, dtype=torch.int32), 0.09)
    T.assert_close_attn(out.view(B, hq, d), want, what="attend on A after touching B")


def test_small_chunk_on_a_long_context_goes_through_context_splits(gpu_device):
    """A step with one request's 160-token prefill chunk on 9000 cached tokens and two decode rows: the builder
    proposes context splits from the host copy of query_start_loc, reserves their room in its workspace, and the
    layer's forward gives the oracle's rows."""
    dev = gpu_device
    hq, hkv, d, bs, nb = 32, 8, 128, 16, 700
    ctx = [9160, 300, 41]
    qls = [160, 1, 1]
    B = len(ctx)
    g = torch.Generator().manual_seed(11)
    kv_cache = L.allocate_kv_cache(nb, bs, hkv, d, device=dev)
    layout = "HND" if Int8AttentionBackend.get_kv_cache_stride_order() != (0, 1, 2, 3) else "NHD"
    kv_cpu, views, lay = T.cpu_cache(nb, bs, hkv, d, layout)
    views[2].fill_(1.0)
    views[3].fill_(1.0)
    bt = T.make_block_tables(ctx, bs, nb, g)
    impl = Int8AttentionBackend.get_impl_cls()(hq, d, 1 / math.sqrt(d), hkv, kv_cache_dtype="int8_per_token_head")
    spec = types.SimpleNamespace(block_size=bs, num_kv_heads=hkv, head_size=d, num_q_heads=hq)
    cfg = types.SimpleNamespace(scheduler_config=types.SimpleNamespace(max_num_seqs=16))
    builder = Int8AttentionBackend.get_builder_cls()(spec, ["layer.0"], cfg, dev)
    layer = types.SimpleNamespace()
    slots = T.slots_for(bt, ctx, bs)
    for i, c in enumerate(ctx):
        k = torch.randn((c, hkv, d), generator=g).to(torch.bfloat16)
        v = torch.randn((c, hkv, d), generator=g).to(torch.bfloat16)
        impl.do_kv_cache_update(layer, k.to(dev), v.to(dev), kv_cache, slots[i].to(dev))
        oracle.cache_write(k, v, T.storage_bytes(kv_cpu), lay, slots[i])
    n = sum(qls)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    common = types.SimpleNamespace(
        num_reqs=B, num_actual_tokens=n, max_query_len=max(qls), max_seq_len=max(ctx), query_start_loc=cu.to(dev),
        query_start_loc_cpu=cu, seq_lens=torch.tensor(ctx, dtype=torch.int32, device=dev),
        block_table_tensor=bt.to(dev), slot_mapping=torch.zeros(n, dtype=torch.int64, device=dev), causal=True)
    md = builder.build(0, common)
    assert md.prefill_splits == 4 and md.has_decode_rows          # 5 query blocks x 8 kv heads; 9160 // 2048 = 4
    assert md.workspace.numel() >= ops.split_prefill_workspace_bytes(16, hq, d, n, md.prefill_splits)
    q = torch.randn((n, hq * d), generator=g).to(torch.bfloat16)
    out = torch.zeros((n, hq * d), dtype=torch.bfloat16, device=dev)
    impl.forward(layer, q.to(dev), None, None, kv_cache, md, out)
    torch.cuda.synchronize()
    want = oracle.paged_attn(q.view(n, hq, d), T.storage_bytes(kv_cpu), lay, bt, torch.tensor(ctx, dtype=torch.int32),
                             cu, 1 / math.sqrt(d))
    T.assert_close_attn(out.view(n, hq, d), want, what="chunk on a long context through the backend")

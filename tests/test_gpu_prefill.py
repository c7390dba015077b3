"""GPU parity of chunked prefill and mixed decode + prefill batches over the int8 cache, through
the C ABI's varlen entry point, against the oracle (causal attention of a query run of q_len
tokens that ends at the sequence end; the run's own K/V are already in the cache, as in the
unified attention op the reference calls, vllm_metax/v1/attention/backends/triton_attn.py:688-725,
and in its test oracle, tests/kernels/attention/test_triton_unified_attention.py:26-78)."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def build(ctx_lens, q_lens, hq, hkv, d, bs, layout="NHD", seed=0, q_dtype=torch.bfloat16, outlier=False):
    g = torch.Generator().manual_seed(seed)
    nb = sum((c + bs - 1) // bs for c in ctx_lens) + 5
    kv, views, lay = T.cpu_cache(nb, bs, hkv, d, layout)
    T.storage_bytes(kv).fill_(0xFF)                    # NaN scales wherever nothing is written
    bt = T.make_block_tables(ctx_lens, bs, nb, g)
    mk = (lambda c: T.outlier_sources((c, hkv, d), g, torch.bfloat16)) if outlier else \
         (lambda c: torch.randn((c, hkv, d), generator=g).to(torch.bfloat16))
    T.fill_cache_from_sources(kv, lay, bt, ctx_lens, bs, [mk(c) for c in ctx_lens], [mk(c) for c in ctx_lens])
    q = torch.randn((sum(q_lens), hq, d), generator=g).to(q_dtype)
    sl = torch.tensor(ctx_lens, dtype=torch.int32)
    cu = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
    return kv, lay, bt, q, sl, cu


def run(dev, kv_cpu, layout, bt, q, sl, cu, max_q, scale, out_dtype=None, want_lse=False, causal=True):
    kv = T.to_device_cache(kv_cpu, dev, layout)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    out = torch.full(q.shape, float("nan"), dtype=out_dtype or q.dtype, device=dev)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev) if want_lse else None
    ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max_q, sl.to(dev), int(sl.max()), scale, causal,
                          block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse)
    torch.cuda.synchronize()
    return (out, lse) if want_lse else out


@pytest.mark.parametrize("hq,hkv,d,bs", [
    (28, 4, 128, 16),     # Qwen2-7B: 7 q heads per kv head (columns do not fill the MFMA tile evenly)
    (32, 8, 128, 16),     # Llama-3-8B
    (8, 8, 64, 32),       # no grouping
    (16, 1, 128, 16),     # 16 q heads on one kv head
    (4, 2, 256, 16),
])
def test_mixed_batch_matches_oracle(gpu_device, hq, hkv, d, bs):
    ctx = [700, 33, 129, 64, 257, 5]
    qls = [1, 33, 100, 1, 17, 5]      # decode rows, a pure prefill, chunks with context, a short full run
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, bs, seed=hq + d)
    scale = 1 / math.sqrt(d)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True)
    got, lse = run(gpu_device, kv, "NHD", bt, q, sl, cu, max(qls), scale, want_lse=True)
    T.assert_close_attn(got, want, what=f"mixed batch {hq}/{hkv} d{d}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("q_dtype,out_dtype", [(torch.float32, torch.float32), (torch.float16, torch.float16),
                                               (torch.bfloat16, torch.float32)])
def test_prefill_dtypes_and_layouts(gpu_device, layout, q_dtype, out_dtype):
    ctx, qls = [300, 48], [64, 48]
    kv, lay, bt, q, sl, cu = build(ctx, qls, 8, 2, 128, 16, layout=layout, seed=4, q_dtype=q_dtype)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, 0.09)
    got = run(gpu_device, kv, layout, bt, q, sl, cu, 64, 0.09, out_dtype=out_dtype)
    tol = dict(atol=4e-3, rtol=4e-3) if out_dtype == torch.float32 else {}
    T.assert_close_attn(got, want, what="prefill dtypes", **tol)


def test_long_chunk_with_outliers(gpu_device):
    """A 2048-token chunk on top of 1000 context tokens, 1 % outlier channels (x20)."""
    ctx, qls = [3048], [2048]
    kv, lay, bt, q, sl, cu = build(ctx, qls, 8, 2, 128, 16, seed=9, outlier=True)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, 0.0884)
    got = run(gpu_device, kv, "NHD", bt, q, sl, cu, 2048, 0.0884, out_dtype=torch.float32)
    T.assert_close_attn(got, want, atol=2e-2, rtol=1e-2, what="long chunk")


def test_causality_first_token_sees_only_itself_and_context(gpu_device):
    """Changing the K/V records of later tokens of a run must not change earlier rows."""
    ctx, qls = [96], [40]
    kv, lay, bt, q, sl, cu = build(ctx, qls, 8, 2, 128, 16, seed=12)
    dev = gpu_device
    a = run(dev, kv, "NHD", bt, q, sl, cu, 40, 0.1, out_dtype=torch.float32)
    # scramble the records of the last 10 tokens of the sequence
    slots = T.slots_for(bt, ctx, 16)[0][-10:]
    g = torch.Generator().manual_seed(1)
    oracle.cache_write(torch.randn((10, 2, 128), generator=g).to(torch.bfloat16) * 3,
                       torch.randn((10, 2, 128), generator=g).to(torch.bfloat16) * 3, T.storage_bytes(kv), lay, slots)
    b = run(dev, kv, "NHD", bt, q, sl, cu, 40, 0.1, out_dtype=torch.float32)
    assert torch.equal(a[:30].cpu(), b[:30].cpu()), "rows before the changed tokens moved"
    assert not torch.equal(a[30:].cpu(), b[30:].cpu())


def test_prefill_golden_mixed_batch(gpu_device):
    import os
    G = torch.load(os.path.join(os.path.dirname(__file__), "golden", "kvq_golden_small.pt"), weights_only=True)
    dev = gpu_device
    hq, hkv, d, bs, nb = (int(G[k]) for k in ("hq", "hkv", "d", "bs", "nb"))
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD")
    T.storage_bytes(kv).copy_(G["cache_bytes"].to(dev))
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    out = torch.empty(G["q"].shape, dtype=torch.float32, device=dev)
    lse = torch.empty(G["q"].shape[:2], dtype=torch.float32, device=dev)
    ops.unified_attention(G["q"].to(dev), k, v, out, G["cu"].to(dev), 5, G["ctx"].to(dev), int(G["ctx"].max()),
                          float(G["scale"]), True, block_table=G["block_table"].to(dev), k_scale_cache=ks,
                          v_scale_cache=vs, lse=lse)
    torch.cuda.synchronize()
    T.assert_close_attn(out, G["out"], atol=2e-3, rtol=2e-3, what="golden mixed batch")
    torch.testing.assert_close(lse.cpu(), G["lse"], atol=5e-3, rtol=1e-3)


def test_backend_forward_mixed_batch(gpu_device, monkeypatch):
    """Through the backend mirror: builder metadata -> do_kv_cache_update of the runs' own tokens ->
    forward, on a batch holding a decode row, a pure prefill and a chunk with context."""
    import types

    from vllm_metax_amd.v1.attention.backends.int8_attn import Int8AttentionBackend

    monkeypatch.setenv("VLLM_KV_CACHE_LAYOUT", "NHD")
    dev = gpu_device
    hq, hkv, d, bs, nb = 8, 2, 128, 16, 24
    ctx, qls = [50, 20, 90], [1, 20, 7]
    B = len(ctx)
    g = torch.Generator().manual_seed(31)
    shape = Int8AttentionBackend.get_kv_cache_shape(nb, bs, hkv, d, "int8_per_token_head")
    order = Int8AttentionBackend.get_kv_cache_stride_order()
    phys = torch.zeros(tuple(shape[i] for i in order), dtype=torch.int8, device=dev)
    kv_cache = phys.permute(*[order.index(i) for i in range(4)])
    kv_cpu, views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    views[2].fill_(1.0)
    views[3].fill_(1.0)
    bt = T.make_block_tables(ctx, bs, nb, g)
    impl = Int8AttentionBackend.get_impl_cls()(hq, d, 0.0884, hkv, kv_cache_dtype="int8_per_token_head")
    spec = types.SimpleNamespace(block_size=bs, num_kv_heads=hkv, head_size=d, num_q_heads=hq)
    cfg = types.SimpleNamespace(scheduler_config=types.SimpleNamespace(max_num_seqs=16))
    builder = Int8AttentionBackend.get_builder_cls()(spec, ["layer.0"], cfg, dev)
    layer = types.SimpleNamespace(_k_scale=torch.ones(1, device=dev), _v_scale=torch.ones(1, device=dev))
    slots = T.slots_for(bt, ctx, bs)
    ksrc = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    vsrc = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    for i, c in enumerate(ctx):                      # earlier steps: everything before the run
        n = c - qls[i]
        if n > 0:
            impl.do_kv_cache_update(layer, ksrc[i][:n].to(dev), vsrc[i][:n].to(dev), kv_cache, slots[i][:n].to(dev))
        oracle.cache_write(ksrc[i], vsrc[i], T.storage_bytes(kv_cpu), lay, slots[i])
    new_k = torch.cat([ksrc[i][ctx[i] - qls[i]:] for i in range(B)])
    new_v = torch.cat([vsrc[i][ctx[i] - qls[i]:] for i in range(B)])
    new_slots = torch.cat([slots[i][ctx[i] - qls[i]:] for i in range(B)])
    n_tok = sum(qls)
    q = torch.randn((n_tok, hq * d), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    common = types.SimpleNamespace(
        num_reqs=B, num_actual_tokens=n_tok, max_query_len=max(qls), max_seq_len=max(ctx),
        query_start_loc=cu.to(dev), seq_lens=torch.tensor(ctx, dtype=torch.int32, device=dev),
        block_table_tensor=bt.to(dev), slot_mapping=new_slots.to(dev), causal=True)
    md = builder.build(0, common)
    impl.do_kv_cache_update(layer, new_k.to(dev), new_v.to(dev), kv_cache, md.slot_mapping)
    out = torch.zeros((n_tok, hq * d), dtype=torch.bfloat16, device=dev)
    impl.forward(layer, q.to(dev), new_k.to(dev), new_v.to(dev), kv_cache, md, out)
    torch.cuda.synchronize()
    assert torch.equal(T.storage_bytes(kv_cache).cpu(), T.storage_bytes(kv_cpu)), "cache bytes differ"
    want = oracle.paged_attn(q.view(n_tok, hq, d), T.storage_bytes(kv_cpu), lay, bt,
                             torch.tensor(ctx, dtype=torch.int32), cu, 0.0884)
    T.assert_close_attn(out.view(n_tok, hq, d), want, what="backend forward, mixed batch")


@pytest.mark.parametrize("step", [0.2, 2.0])
def test_prefill_logits_that_keep_rising(gpu_device, step):
    """Keys whose logits grow along the sequence by ``step`` (log2 units) per 32-token tile: the
    prefill tile's reference maximum may lag the true one by up to 2^8 before it moves.  A 300-token
    chunk on 1500 cached tokens (workgroup-shared tile) plus short runs."""
    hq, hkv, d, bs = 8, 2, 128, 16
    ctx, qls = [1800, 400, 90], [300, 40, 1]
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, bs, seed=12)
    g = torch.Generator().manual_seed(13)
    u = torch.randn(d, generator=g)
    u = u / u.norm()
    ks = [0.3 * torch.randn((c, hkv, d), generator=g) + (torch.arange(c) / 32.0 * step * 0.6931)[:, None, None] * u for c in ctx]
    vs = [torch.randn((c, hkv, d), generator=g) for c in ctx]
    T.fill_cache_from_sources(kv, lay, bt, ctx, bs, [k.to(torch.bfloat16) for k in ks], [v.to(torch.bfloat16) for v in vs])
    q = (0.3 * q.float() + u).to(torch.bfloat16)          # unit projection on the ramp direction
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, 1.0, return_lse=True)
    got, lse = run(gpu_device, kv, "NHD", bt, q, sl, cu, max(qls), 1.0, want_lse=True)
    T.assert_close_attn(got, want, what=f"prefill, rising logits {step}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=2e-2, rtol=1e-3)


def test_prefill_huge_value_scales(gpu_device):
    """V rows in the thousands in every other tile: scales above 1, for which the tile moves its
    reference maximum eagerly (p * scale must stay inside fp16)."""
    hq, hkv, d, bs = 8, 2, 128, 16
    ctx, qls = [1200, 64], [500, 64]
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, bs, seed=14)
    g = torch.Generator().manual_seed(15)
    ks = [torch.randn((c, hkv, d), generator=g) for c in ctx]
    vs = [torch.randn((c, hkv, d), generator=g) * (((torch.arange(c) // 32) % 2 == 1).float() * 1999.0 + 1.0)[:, None, None]
          for c in ctx]
    T.fill_cache_from_sources(kv, lay, bt, ctx, bs, [k.to(torch.bfloat16) for k in ks], [v.to(torch.bfloat16) for v in vs])
    scale = 1 / math.sqrt(d)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run(gpu_device, kv, "NHD", bt, q, sl, cu, max(qls), scale, out_dtype=torch.float32)
    assert torch.isfinite(got).all()
    T.assert_close_attn(got, want, atol=2e-2 * 2000, rtol=1e-2, what="prefill, huge value scales")


def test_pure_prefill_batch_with_the_no_decode_rows_promise(gpu_device):
    """has_decode_rows=False (KVQ_ATTN_NO_DECODE_ROWS): the decode kernels are skipped; a batch without one-row
    sequences gives the same bits either way, for both prefill tiles."""
    dev = gpu_device
    for hq, hkv, qls in ((32, 8, [300, 64, 2048]), (8, 8, [5, 33, 2])):
        ctx = [q + extra for q, extra in zip(qls, [700, 0, 133])]
        kv_cpu, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, 128, 16, seed=21)
        kv = T.to_device_cache(kv_cpu, dev, "NHD")
        k, v = L.key_value_views(kv)
        ks, vs = L.scale_views(kv)
        outs = []
        for promise in (True, False):
            out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
            lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
            ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), int(sl.max()), 0.0884, True,
                                  block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse,
                                  has_decode_rows=promise)
            torch.cuda.synchronize()
            outs.append((out.cpu(), lse.cpu()))
        assert torch.equal(outs[0][0].view(torch.int16), outs[1][0].view(torch.int16)) and torch.equal(outs[0][1], outs[1][1])
        want = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, 0.0884)
        T.assert_close_attn(outs[1][0], want, what="pure prefill batch")


@pytest.mark.parametrize("hq,hkv,d,layout", [(32, 8, 128, "HND"), (28, 4, 128, "NHD"), (8, 2, 64, "HND"), (4, 2, 256, "NHD")])
def test_non_causal_rows_see_every_key(gpu_device, hq, hkv, d, layout):
    """causal=False, the cross-attention form of the reference's call (`causal=attn_metadata.causal`,
    vllm_metax/v1/attention/backends/triton_attn.py:698; AttentionType.ENCODER_DECODER goes through the cached
    path, :394-402): every query row of a run attends all `seq_len` keys, whatever its place in the run -- decode
    rows, short runs (the per-wave tile), long runs (the workgroup-shared tile), output and lse against the oracle,
    and every row of a run of copies of one query gets the same bits."""
    ctx = [700, 33, 1500, 64, 257, 5, 900]
    qls = [1, 33, 300, 1, 17, 5, 70]
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, 16, layout=layout, seed=hq + d + 1)
    # the last run: copies of one query row
    q[int(cu[-2]):] = q[int(cu[-2])].clone()
    scale = 1 / math.sqrt(d)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, causal=False, return_lse=True)
    causal = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, causal=True)
    assert not torch.allclose(want, causal, atol=5e-2)
    got, lse = run(gpu_device, kv, layout, bt, q, sl, cu, max(qls), scale, want_lse=True, causal=False)
    T.assert_close_attn(got, want, what=f"non-causal {hq}/{hkv} d{d}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)
    tail = got[int(cu[-2]):].cpu()
    assert torch.equal(tail.view(torch.int16), tail[:1].expand_as(tail).contiguous().view(torch.int16))


@pytest.mark.parametrize("hq,hkv,d,layout,qmax", [(32, 8, 128, "HND", 4), (32, 8, 128, "NHD", 8), (28, 4, 128, "HND", 2),
                                                  (8, 8, 64, "HND", 16), (16, 2, 256, "NHD", 2), (16, 1, 128, "HND", 1)])
def test_short_runs_on_long_contexts_spread_over_a_workgroup(gpu_device, hq, hkv, d, layout, qmax):
    """A speculative-decoding step: every sequence brings a few query tokens (1 + k) on a long context.  With few
    items per launch the short-run kernel spreads an item's tiles over the waves of a workgroup and folds their
    states; contexts shorter than the waves' stride (waves without a tile), one-token sequences next to them (the
    decode kernel's) and a sliding window are in the batch.  Output and lse against the oracle."""
    ctx = [9000, 37, 2500, 300, 64, 5000, 1, 700]
    qls = [min(c, q) for c, q in zip(ctx, [qmax, 2, qmax, 1, 3, qmax, 1, 2])]
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, 16, layout=layout, seed=hq + qmax)
    scale = 1 / math.sqrt(d)
    for window in (0, 1000):
        want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True,
                                           sliding_window=window)
        dev = gpu_device
        kvd = T.to_device_cache(kv, dev, layout)
        k, v = L.key_value_views(kvd)
        ks, vs = L.scale_views(kvd)
        out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=dev)
        lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), int(sl.max()), scale, True,
                              window_size=(window - 1, 0) if window else (-1, -1), block_table=bt.to(dev),
                              k_scale_cache=ks, v_scale_cache=vs, lse=lse)
        torch.cuda.synchronize()
        T.assert_close_attn(out, want, what=f"short runs {hq}/{hkv} d{d} q<={qmax} window {window}")
        torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


def test_many_short_runs_take_one_wave_per_item(gpu_device):
    """Beyond a few thousand items per launch an item stays with one wave (300 sequences x 8 kv heads here): the
    same rows as the oracle's, also when the batch is cut in three launches that spread their items over
    workgroups."""
    hq, hkv, d = 32, 8, 128
    g = torch.Generator().manual_seed(17)
    n = 300
    ctx = torch.randint(20, 400, (n,), generator=g).tolist()
    qls = [min(c, int(x)) for c, x in zip(ctx, torch.randint(1, 5, (n,), generator=g).tolist())]
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, 16, layout="HND", seed=3)
    scale = 1 / math.sqrt(d)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run(gpu_device, kv, "HND", bt, q, sl, cu, max(qls), scale)
    T.assert_close_attn(got, want, what="300 short runs, one wave per item")
    parts = []
    for lo_, hi_ in ((0, 100), (100, 200), (200, 300)):
        qq = q[int(cu[lo_]):int(cu[hi_])]
        cc = (cu[lo_:hi_ + 1] - cu[lo_]).contiguous()
        parts.append(run(gpu_device, kv, "HND", bt[lo_:hi_].contiguous(), qq, sl[lo_:hi_].contiguous(), cc, max(qls), scale))
    T.assert_close_attn(torch.cat(parts), want, what="the same runs in three launches")


@pytest.mark.parametrize("hq,hkv,d,layout,code", [(32, 8, 128, "HND", "int8"), (28, 4, 128, "NHD", "int8"),
                                                  (8, 2, 64, "HND", "fp8"), (16, 8, 128, "HND", "int4")])
@pytest.mark.parametrize("window,cap,extras", [(0, 0.0, False), (1500, 30.0, True)])
def test_context_splits_of_long_runs(gpu_device, hq, hkv, d, layout, code, window, cap, extras):
    """kvq_paged_attn_int8_split_prefill: the context of the long query runs in 2..8 ranges, merged afterwards.  A
    small chunk on a long context, a run that starts its sequence, a decode row and a short run (both served as in
    the plain call) in one batch; ranges without a visible tile (window, causal limit); sinks and ALiBi on top.
    Output and lse against the oracle for every split count, and within 1e-2 of the plain call."""
    from vllm_metax_amd.kv_cache_interface import KVQuantMode
    ct = {"int8": oracle.CODE_INT8, "fp8": oracle.CODE_FP8, "int4": oracle.CODE_INT4}[code]
    mode = {"int8": KVQuantMode.INT8_PER_TOKEN_HEAD, "fp8": KVQuantMode.FP8_PER_TOKEN_HEAD,
            "int4": KVQuantMode.INT4_PER_TOKEN_HEAD}[code]
    dev = gpu_device
    bs = 16
    ctx = [6000, 700, 200, 64, 3000]
    qls = [200, 1, 200, 3, 77]
    g = torch.Generator().manual_seed(hq + d + window)
    nb = sum((c + bs - 1) // bs for c in ctx) + 5
    kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, layout, code_type=ct)
    bt = T.make_block_tables(ctx, bs, nb, g)
    ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    vs_ = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    T.fill_cache_from_sources(kv_cpu, lay, bt, ctx, bs, ks, vs_, code_type=ct)
    q = torch.randn((sum(qls), hq, d), generator=g).to(torch.bfloat16)
    sl = torch.tensor(ctx, dtype=torch.int32)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    sinks = (torch.randn(hq, generator=g) * 2).float() if extras else None
    slopes = torch.tensor([2.0 ** (-8.0 * (i + 1) / hq) for i in range(hq)], dtype=torch.float32) if extras else None
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, scale, return_lse=True,
                                       sliding_window=window, soft_cap=cap, code_type=ct, sinks=sinks, alibi_slopes=slopes)
    kv = T.to_device_cache(kv_cpu, dev, layout, code_type=ct)
    k, v = L.key_value_views(kv)
    ksc, vsc = L.scale_views(kv)
    plain = None
    for splits in (1, 2, 3, 5, 8):
        out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), max(ctx), scale, True,
                              window_size=(window - 1, 0) if window else (-1, -1), softcap=cap, block_table=bt.to(dev),
                              k_scale_cache=ksc, v_scale_cache=vsc, kv_quant_mode=mode, lse=lse,
                              sinks=None if sinks is None else sinks.to(dev),
                              alibi_slopes=None if slopes is None else slopes.to(dev), prefill_splits=splits)
        torch.cuda.synchronize()
        T.assert_close_attn(out, want, what=f"{splits} context splits, {code}")
        torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)
        if plain is None:
            plain = out.float().cpu()
        else:
            torch.testing.assert_close(out.float().cpu(), plain, atol=1e-2, rtol=1e-2)


def test_context_splits_need_their_workspace(gpu_device):
    dev = gpu_device
    kv = L.allocate_kv_cache(40, 16, 2, 128, device=dev)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    q = torch.zeros((64, 8, 128), dtype=torch.bfloat16, device=dev)
    cu = torch.tensor([0, 64], dtype=torch.int32, device=dev)
    sl = torch.tensor([500], dtype=torch.int32, device=dev)
    bt = torch.arange(32, dtype=torch.int32, device=dev).view(1, 32)
    small = torch.empty(ops.paged_attn_workspace_bytes(1, 8, 128), dtype=torch.uint8, device=dev)
    need = ops.split_prefill_workspace_bytes(1, 8, 128, 64, 4)
    assert need >= small.numel() + 64 * 8 * 4 * 130 * 4
    with pytest.raises(RuntimeError, match="workspace"):
        ops.unified_attention(q, k, v, torch.empty_like(q), cu, 64, sl, 500, 0.1, True, block_table=bt,
                              k_scale_cache=ks, v_scale_cache=vs, workspace=small, prefill_splits=4)
    with pytest.raises(RuntimeError):
        ops.unified_attention(q, k, v, torch.empty_like(q), cu, 64, sl, 500, 0.1, True, block_table=bt,
                              k_scale_cache=ks, v_scale_cache=vs, prefill_splits=9)

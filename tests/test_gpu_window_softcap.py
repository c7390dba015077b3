"""GPU parity of the sliding window and the logits soft cap of the varlen entry point against the
oracle: decode rows (split-K tile line that starts at the window's first tile), short query runs
(one wave per work item) and long ones (the workgroup-shared tile).  The reference's own grid for
these two knobs is sliding_window in (None, 256) x soft_cap in (None, 50.0),
tests/kernels/attention/test_triton_unified_attention.py:87-89; it passes them on as
window_size = (sliding_window - 1, 0) and softcap, :118, :173-175."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from test_gpu_prefill import build
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def run(dev, kv_cpu, bt, q, sl, cu, max_q, scale, window, cap, want_lse=False, out_dtype=None, layout="NHD"):
    kv = T.to_device_cache(kv_cpu, dev, layout)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    out = torch.full(q.shape, float("nan"), dtype=out_dtype or q.dtype, device=dev)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev) if want_lse else None
    ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max_q, sl.to(dev), int(sl.max()), scale, True,
                          window_size=(window - 1, 0) if window else (-1, -1), softcap=cap or 0.0,
                          block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse)
    torch.cuda.synchronize()
    return (out, lse) if want_lse else out


def check(dev, ctx, qls, hq, hkv, d, bs, window, cap, seed, scale=None, q_dtype=torch.bfloat16, what="", layout="NHD"):
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, bs, seed=seed, q_dtype=q_dtype, layout=layout)
    scale = scale if scale is not None else 1 / math.sqrt(d)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True,
                                       sliding_window=window or 0, soft_cap=cap or 0.0)
    got, lse = run(dev, kv, bt, q, sl, cu, max(qls), scale, window, cap, want_lse=True, layout=layout)
    T.assert_close_attn(got, want, what=f"{what} window={window} cap={cap} {layout}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("layout", ["NHD", "HND"])   # HND without a cap: the streamed run loads, first tile peeled
@pytest.mark.parametrize("window", [None, 1, 31, 32, 33, 256, 5000])
@pytest.mark.parametrize("cap", [None, 50.0])
def test_decode_rows(gpu_device, window, cap, layout):
    """Windows that start inside the first tile, on a tile edge, deep inside a long sequence (so
    that most tiles never enter the tile line) and beyond every sequence (no effect)."""
    if window is None and cap is None:
        pytest.skip("covered by the plain decode tests")
    ctx = [1, 31, 32, 33, 257, 1000, 4097, 300, 64]
    check(gpu_device, ctx, [1] * len(ctx), 32, 8, 128, 16, window, cap, seed=3, what="decode", layout=layout)


@pytest.mark.parametrize("hq,hkv,d,bs", [(28, 4, 128, 16), (8, 8, 64, 32), (4, 2, 256, 16), (16, 1, 128, 16)])
def test_decode_head_shapes(gpu_device, hq, hkv, d, bs):
    ctx = [700, 5, 129, 2048]
    check(gpu_device, ctx, [1] * len(ctx), hq, hkv, d, bs, 256, 30.0, seed=hq + d, what=f"decode {hq}/{hkv} d{d}")


def test_decode_many_sequences_long_window(gpu_device):
    """More sequences than a wave scans at once, each a few tiles of window inside a long context:
    the tile line is built from the windows, not from the sequence lengths."""
    g = torch.Generator().manual_seed(1)
    ctx = torch.randint(200, 1500, (70,), generator=g).tolist()
    check(gpu_device, ctx, [1] * len(ctx), 8, 2, 128, 16, 100, None, seed=11, what="decode b70")


@pytest.mark.parametrize("window", [None, 1, 20, 64, 256, 3000])
@pytest.mark.parametrize("cap", [None, 50.0])
def test_mixed_batch(gpu_device, window, cap):
    """Decode rows, short query runs and a long chunk in one call (Llama-3-8B head shape)."""
    if window is None and cap is None:
        pytest.skip("covered by the plain prefill tests")
    ctx = [700, 33, 129, 64, 257, 5, 900]
    qls = [1, 33, 100, 1, 17, 5, 600]
    check(gpu_device, ctx, qls, 32, 8, 128, 16, window, cap, seed=5, what="mixed")


@pytest.mark.parametrize("hq,hkv,d,bs", [(28, 4, 128, 16), (8, 8, 64, 32), (4, 2, 256, 16), (16, 1, 128, 16)])
def test_prefill_head_shapes(gpu_device, hq, hkv, d, bs):
    ctx = [700, 129, 300]
    qls = [400, 100, 3]
    check(gpu_device, ctx, qls, hq, hkv, d, bs, 96, 30.0, seed=hq + d + 1, what=f"prefill {hq}/{hkv} d{d}")


def test_long_chunk_short_window(gpu_device):
    """A 2048-token chunk over 1000 context tokens with a 128-token window: every workgroup starts
    far into the sequence and most of its tiles straddle a window edge of some column."""
    check(gpu_device, [3048], [2048], 8, 2, 128, 16, 128, None, seed=9, what="long chunk")
    check(gpu_device, [3048], [2048], 8, 2, 128, 16, 1000, 50.0, seed=9, what="long chunk")


@pytest.mark.parametrize("q_dtype", [torch.float16, torch.float32])
def test_query_dtypes(gpu_device, q_dtype):
    check(gpu_device, [500, 77, 260], [1, 77, 130], 8, 2, 128, 16, 64, 20.0, seed=2, q_dtype=q_dtype, what=str(q_dtype))


def test_window_of_one_returns_the_last_value_row(gpu_device):
    """Closed form: with a window of one key, every output row is that key's dequantised V."""
    ctx, qls = [130, 77], [1, 40]
    kv, lay, bt, q, sl, cu = build(ctx, qls, 8, 2, 128, 16, seed=8)
    got = run(gpu_device, kv, bt, q, sl, cu, max(qls), 0.1, 1, None, out_dtype=torch.float32).cpu()
    _, v_views = L.key_value_views(kv)                                # (nb, bs, Hkv, D+4) int8 on the CPU
    _, vs = L.scale_views(kv)
    v_deq = v_views[..., :128].to(torch.float32) * vs[..., None]      # (nb, bs, Hkv, D)
    row = 0
    for s, (c, ql) in enumerate(zip(ctx, qls)):
        for r in range(ql):
            pos = c - ql + r
            want = v_deq[int(bt[s, pos // 16]), pos % 16].repeat_interleave(4, dim=0)   # [Hq, D]
            torch.testing.assert_close(got[row], want, atol=2e-3, rtol=2e-3)
            row += 1


def test_large_cap_is_the_identity_and_huge_window_too(gpu_device):
    """A cap far above every logit and a window >= every length leave the result of the plain call
    (property).  The cap is accurate relative to the logit for every cap (a series near zero, the
    exponential form elsewhere), so a cap of 1e6 on logits below 10 is the identity to fp32 rounding."""
    ctx, qls = [700, 129, 64], [1, 100, 1]
    kv, lay, bt, q, sl, cu = build(ctx, qls, 8, 2, 128, 16, seed=6)
    plain = run(gpu_device, kv, bt, q, sl, cu, 100, 0.09, None, None, out_dtype=torch.float32)
    wide = run(gpu_device, kv, bt, q, sl, cu, 100, 0.09, 100000, None, out_dtype=torch.float32)
    assert torch.equal(plain, wide)
    for cap in (1e6, 1e3):
        capped = run(gpu_device, kv, bt, q, sl, cu, 100, 0.09, None, cap, out_dtype=torch.float32)
        # (the capped call runs the kernels' other instantiation: same algebra, its own rounding)
        torch.testing.assert_close(capped, plain, atol=2e-3, rtol=2e-3)


def test_rejected_arguments(gpu_device):
    kv, lay, bt, q, sl, cu = build([64], [1], 8, 2, 128, 16, seed=0)
    dev = gpu_device
    kvd = T.to_device_cache(kv, dev, "NHD")
    k, v = L.key_value_views(kvd)
    ks, vs = L.scale_views(kvd)
    out = torch.empty_like(q, device=dev)
    common = dict(block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs)
    with pytest.raises(NotImplementedError):      # two-sided (encoder) window
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), 1, sl.to(dev), 64, 0.1, True, window_size=(7, 7), **common)
    with pytest.raises(NotImplementedError):      # window without causal
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), 1, sl.to(dev), 64, 0.1, False, window_size=(7, 0), **common)
    with pytest.raises(RuntimeError):
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), 1, sl.to(dev), 64, 0.1, True, softcap=-1.0, **common)


@pytest.mark.parametrize("hq,hkv,d,layout,code", [(32, 8, 128, "HND", "int8"), (28, 4, 128, "NHD", "int8"),
                                                  (8, 2, 64, "HND", "fp8"), (4, 1, 256, "NHD", "int4"),
                                                  (16, 8, 128, "HND", "int4")])
@pytest.mark.parametrize("window,cap", [(0, 0.0), (200, 25.0)])
def test_attention_sinks_decode_prefill_and_mixed(gpu_device, hq, hkv, d, layout, code, window, cap):
    """Attention sinks (the `sinks` argument the reference passes to unified_attention, triton_attn.py:712): decode
    rows through every merge path (unsplit, a few cuts, dozens of cuts), both prefill tiles and the fused write,
    output and lse against the oracle; the batch-invariant cutting as well."""
    import oracle
    from vllm_metax_amd.kv_cache_interface import KVQuantMode
    ct = {"int8": oracle.CODE_INT8, "fp8": oracle.CODE_FP8, "int4": oracle.CODE_INT4}[code]
    mode = {"int8": KVQuantMode.INT8_PER_TOKEN_HEAD, "fp8": KVQuantMode.FP8_PER_TOKEN_HEAD,
            "int4": KVQuantMode.INT4_PER_TOKEN_HEAD}[code]
    dev = gpu_device
    bs = 16
    g = torch.Generator().manual_seed(hq * 7 + d + window)
    sinks = (torch.randn(hq, generator=g) * 2).float()
    scale = 1 / math.sqrt(d)
    for ctx, qls in (([1000, 3, 517, 64, 9000, 33], [1] * 6),          # decode rows: whole sequences and cut ones
                     ([40000, 700], [1, 1]),                           # a handful of sequences, dozens of cuts
                     ([900, 2300, 33, 257], [300, 1, 33, 2])):         # both prefill tiles beside a decode row
        nb = sum((c + bs - 1) // bs for c in ctx) + 5
        kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, layout, code_type=ct)
        bt = T.make_block_tables(ctx, bs, nb, g)
        ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
        vs_ = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
        T.fill_cache_from_sources(kv_cpu, lay, bt, ctx, bs, ks, vs_, code_type=ct)
        q = torch.randn((sum(qls), hq, d), generator=g).to(torch.bfloat16)
        sl = torch.tensor(ctx, dtype=torch.int32)
        cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
        want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, scale, return_lse=True,
                                           sliding_window=window, soft_cap=cap, code_type=ct, sinks=sinks)
        kv = T.to_device_cache(kv_cpu, dev, layout, code_type=ct)
        k, v = L.key_value_views(kv)
        ksc, vsc = L.scale_views(kv)
        for invariant in (False, True):
            before = ops.set_batch_invariant(invariant)
            try:
                out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
                lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
                ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), max(ctx), scale, True,
                                      window_size=(window - 1, 0) if window else (-1, -1), softcap=cap,
                                      block_table=bt.to(dev), k_scale_cache=ksc, v_scale_cache=vsc, kv_quant_mode=mode,
                                      lse=lse, sinks=sinks.to(dev))
                torch.cuda.synchronize()
            finally:
                ops.set_batch_invariant(before)
            T.assert_close_attn(out, want, what=f"sinks {code} ctx {ctx} invariant={invariant}")
            torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)
        if max(qls) == 1:   # the one-launch step: same rows (the new token rewrites the last record with its own bytes)
            out2 = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
            ops.decode_attention_with_cache_update(q.to(dev), ks_last(ks).to(dev), ks_last(vs_).to(dev), k, v, out2,
                                                   sl.to(dev), max(ctx), scale, bt.to(dev), ksc, vsc,
                                                   window_size=(window - 1, 0) if window else (-1, -1), softcap=cap,
                                                   kv_quant_mode=mode, sinks=sinks.to(dev))
            torch.cuda.synchronize()
            T.assert_close_attn(out2, want, what=f"sinks fused write {code}")


def ks_last(rows):
    """The last token's row of every sequence, [B, Hkv, D]."""
    return torch.stack([r[-1] for r in rows])


@pytest.mark.parametrize("hq,hkv,d,layout,code", [(32, 8, 128, "HND", "int8"), (28, 4, 128, "NHD", "int8"),
                                                  (8, 2, 64, "HND", "fp8"), (4, 1, 256, "NHD", "int4"),
                                                  (16, 8, 128, "HND", "int4"), (16, 1, 128, "HND", "int8")])
@pytest.mark.parametrize("window,cap,with_sinks", [(0, 0.0, False), (200, 25.0, True)])
def test_alibi_decode_prefill_and_mixed(gpu_device, hq, hkv, d, layout, code, window, cap, with_sinks):
    """ALiBi (alibi_slopes of the reference's attention op, triton_attn.py:504-506, 699; the bias of
    tests/kernels/attention/test_attention.py:109-117): decode rows whole and cut, both prefill tiles, a mixed
    batch and the one-launch decode step, alone and on top of window + soft cap + sinks, output and lse against
    the oracle; the batch-invariant cutting as well."""
    import oracle
    from vllm_metax_amd.kv_cache_interface import KVQuantMode
    ct = {"int8": oracle.CODE_INT8, "fp8": oracle.CODE_FP8, "int4": oracle.CODE_INT4}[code]
    mode = {"int8": KVQuantMode.INT8_PER_TOKEN_HEAD, "fp8": KVQuantMode.FP8_PER_TOKEN_HEAD,
            "int4": KVQuantMode.INT4_PER_TOKEN_HEAD}[code]
    dev = gpu_device
    bs = 16
    g = torch.Generator().manual_seed(hq * 11 + d + window)
    # the usual geometric slopes, and a steep and a zero one
    slopes = torch.tensor([2.0 ** (-8.0 * (i + 1) / hq) for i in range(hq)], dtype=torch.float32)
    slopes[0], slopes[-1] = 1.5, 0.0
    sinks = (torch.randn(hq, generator=g) * 2).float() if with_sinks else None
    scale = 1 / math.sqrt(d)
    for ctx, qls in (([1000, 3, 517, 64, 9000, 33], [1] * 6),          # decode rows: whole sequences and cut ones
                     ([40000, 700], [1, 1]),                           # a handful of sequences, dozens of cuts
                     ([900, 2300, 33, 257], [300, 1, 33, 2]),          # both prefill tiles beside a decode row
                     ([700, 1500], [700, 1100])):                      # long runs: the workgroup-shared tile
        nb = sum((c + bs - 1) // bs for c in ctx) + 5
        kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, layout, code_type=ct)
        bt = T.make_block_tables(ctx, bs, nb, g)
        ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
        vs_ = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
        T.fill_cache_from_sources(kv_cpu, lay, bt, ctx, bs, ks, vs_, code_type=ct)
        q = torch.randn((sum(qls), hq, d), generator=g).to(torch.bfloat16)
        sl = torch.tensor(ctx, dtype=torch.int32)
        cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
        want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, scale, return_lse=True,
                                           sliding_window=window, soft_cap=cap, code_type=ct, sinks=sinks,
                                           alibi_slopes=slopes)
        plain = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, scale, sliding_window=window,
                                  soft_cap=cap, code_type=ct, sinks=sinks)
        assert not torch.allclose(want, plain, atol=5e-2)      # the bias matters in this case
        kv = T.to_device_cache(kv_cpu, dev, layout, code_type=ct)
        k, v = L.key_value_views(kv)
        ksc, vsc = L.scale_views(kv)
        sk = sinks.to(dev) if with_sinks else None
        for invariant in (False, True):
            before = ops.set_batch_invariant(invariant)
            try:
                out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
                lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
                ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), max(ctx), scale, True,
                                      window_size=(window - 1, 0) if window else (-1, -1), softcap=cap,
                                      block_table=bt.to(dev), k_scale_cache=ksc, v_scale_cache=vsc, kv_quant_mode=mode,
                                      lse=lse, sinks=sk, alibi_slopes=slopes.to(dev))
                torch.cuda.synchronize()
            finally:
                ops.set_batch_invariant(before)
            T.assert_close_attn(out, want, what=f"alibi {code} ctx {ctx} invariant={invariant}")
            torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)
        if max(qls) == 1:   # the one-launch step: same rows (the new token rewrites the last record with its own bytes)
            out2 = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
            ops.decode_attention_with_cache_update(q.to(dev), ks_last(ks).to(dev), ks_last(vs_).to(dev), k, v, out2,
                                                   sl.to(dev), max(ctx), scale, bt.to(dev), ksc, vsc,
                                                   window_size=(window - 1, 0) if window else (-1, -1), softcap=cap,
                                                   kv_quant_mode=mode, sinks=sk, alibi_slopes=slopes.to(dev))
            torch.cuda.synchronize()
            T.assert_close_attn(out2, want, what=f"alibi fused write {code}")


def test_alibi_is_refused_without_causal_and_in_its_sqrt_form(gpu_device):
    dev = gpu_device
    kv = L.allocate_kv_cache(4, 16, 2, 64, device=dev)
    k, v = L.key_value_views(kv)
    ksc, vsc = L.scale_views(kv)
    q = torch.zeros((1, 4, 64), dtype=torch.bfloat16, device=dev)
    args = (q, k, v, torch.empty_like(q), torch.tensor([0, 1], dtype=torch.int32, device=dev), 1,
            torch.tensor([5], dtype=torch.int32, device=dev), 5, 0.1)
    kw = dict(block_table=torch.zeros((1, 1), dtype=torch.int32, device=dev), k_scale_cache=ksc, v_scale_cache=vsc)
    sl = torch.ones(4, device=dev)
    with pytest.raises(NotImplementedError):
        ops.unified_attention(*args, False, alibi_slopes=sl, **kw)
    with pytest.raises(NotImplementedError):
        ops.unified_attention(*args, True, alibi_slopes=sl, use_alibi_sqrt=True, **kw)
    with pytest.raises(RuntimeError):
        ops.unified_attention(*args, True, alibi_slopes=torch.ones(3, device=dev), **kw)

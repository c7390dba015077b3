"""The library's batch-invariant mode (the switch the reference reads as envs.VLLM_BATCH_INVARIANT:
vllm_metax/v1/attention/backends/mla/triton_mla.py:247-253, triton_attn.py:310-312), through the C ABI: with
the mode on, the BITS of a sequence's output row and log-sum-exp must not depend on what else the batch holds,
where the sequence stands in it, or how large it is -- and the results must still match the oracle."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from test_gpu_decode import build_case
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu

# one span, a few spans, the 32-span cap (> 16384 tokens), an empty sequence, a one-token one
LENS = [20000, 513, 40, 5000, 1024, 8192, 3, 0, 16400, 700, 1, 2049]


@pytest.fixture
def invariant_mode():
    before = ops.set_batch_invariant(True)
    assert ops.batch_invariant()
    yield
    ops.set_batch_invariant(before)
    assert ops.batch_invariant() == before


def _sub_batches(n):
    """Index lists: every sequence alone, the whole batch, the batch reversed, and two mixed subsets."""
    alone = [[i] for i in range(n)]
    return alone + [list(range(n)), list(range(n))[::-1], list(range(0, n, 2)), [5, 0, 9, 8, 3] if n > 9 else [0]]


def _gqa_rows(dev, kv, bt, q, sl, idx, scale, window=0, fused=None, out_dtype=torch.bfloat16):
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    ii = torch.tensor(idx)
    qb, btb, slb = q[ii].contiguous().to(dev), bt[ii].contiguous().to(dev), sl[ii].contiguous().to(dev)
    out = torch.full(qb.shape, float("nan"), dtype=out_dtype, device=dev)
    lse = torch.full(qb.shape[:2], float("nan"), dtype=torch.float32, device=dev)
    kw = dict(window_size=(window - 1, 0)) if window else {}
    if fused is not None:
        nk, nv = fused
        ops.decode_attention_with_cache_update(qb, nk[ii].contiguous().to(dev), nv[ii].contiguous().to(dev), k, v, out,
                                               slb, int(slb.max()), scale, btb, ks, vs, lse=lse, **kw)
    else:
        cu = torch.arange(len(idx) + 1, dtype=torch.int32, device=dev)
        ops.unified_attention(qb, k, v, out, cu, 1, slb, int(slb.max()), scale, True, block_table=btb,
                              k_scale_cache=ks, v_scale_cache=vs, lse=lse, **kw)
    torch.cuda.synchronize()
    return out.cpu(), lse.cpu()


@pytest.mark.parametrize("hq,hkv,d,layout,window", [
    (32, 8, 128, "HND", 0),
    (32, 8, 128, "NHD", 0),
    (28, 4, 128, "HND", 0),      # two waves per kv head: their states are folded in the workgroup
    (16, 2, 64, "NHD", 0),
    (8, 1, 256, "HND", 0),
    (32, 8, 128, "HND", 4096),   # sliding window: the spans are those of the window's tiles
])
def test_gqa_decode_rows_do_not_depend_on_the_batch(gpu_device, invariant_mode, hq, hkv, d, layout, window):
    dev = gpu_device
    bs = 16
    kv_cpu, lay, bt, q, sl, _ = build_case(LENS, hq, hkv, d, bs, layout, 7, poison=False)
    kv = T.to_device_cache(kv_cpu, dev, layout)
    scale = 1 / math.sqrt(d)
    ref = {}
    for idx in _sub_batches(len(LENS)):
        out, lse = _gqa_rows(dev, kv, bt, q, sl, idx, scale, window)
        for j, i in enumerate(idx):
            if i not in ref:
                ref[i] = (out[j].clone(), lse[j].clone())
                continue
            assert torch.equal(out[j].view(torch.int16), ref[i][0].view(torch.int16)), \
                f"row of sequence {i} (len {LENS[i]}) changed its bits in batch {idx}"
            assert torch.equal(lse[j].view(torch.int32), ref[i][1].view(torch.int32)), \
                f"lse of sequence {i} (len {LENS[i]}) changed its bits in batch {idx}"
    # and the mode's results are the right ones
    sub = [1, 2, 3, 6, 7, 8, 9, 10]
    ii = torch.tensor(sub)
    cu = torch.arange(len(sub) + 1, dtype=torch.int32)
    want, want_lse = oracle.paged_attn(q[ii], T.storage_bytes(kv_cpu), lay, bt[ii], sl[ii], cu, scale, return_lse=True,
                                       **({"sliding_window": window} if window else {}))
    got = torch.stack([ref[i][0] for i in sub])
    got_lse = torch.stack([ref[i][1] for i in sub])
    live = sl[ii] > 0
    T.assert_close_attn(got[live], want[live], what="batch-invariant decode vs oracle")
    torch.testing.assert_close(got_lse[live], want_lse[live], atol=5e-3, rtol=1e-3)
    assert torch.equal(got[~live].float(), torch.zeros_like(got[~live].float()))


def test_gqa_workspace_query_follows_the_mode(gpu_device):
    before = ops.set_batch_invariant(False)
    try:
        plain = ops.paged_attn_workspace_bytes(64, 32, 128)
        ops.set_batch_invariant(True)
        fixed = ops.paged_attn_workspace_bytes(64, 32, 128)
        assert fixed > plain     # 32 span states per sequence against one per workgroup + one per sequence
        assert ops.mla_decode_workspace_bytes(256, 128, 512) >= 8 * 256 * 128 * (512 * 2 + 4)
    finally:
        ops.set_batch_invariant(before)


def test_gqa_fused_write_rows_do_not_depend_on_the_batch(gpu_device, invariant_mode):
    """The one-launch step (decode + write of the new token) in the mode: same bits alone and in a batch, and the
    same bits as write-then-attend."""
    dev = gpu_device
    hq, hkv, d, bs = 32, 8, 128, 16
    lens = [l for l in LENS if l > 0]
    kv_cpu, lay, bt, q, sl, _ = build_case(lens, hq, hkv, d, bs, "HND", 11, poison=False)
    g = torch.Generator().manual_seed(3)
    nk = torch.randn((len(lens), hkv, d), generator=g).to(torch.bfloat16)
    nv = torch.randn((len(lens), hkv, d), generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    kv = T.to_device_cache(kv_cpu, dev, "HND")
    whole, whole_lse = _gqa_rows(dev, kv, bt, q, sl, list(range(len(lens))), scale, fused=(nk, nv))
    # the cache now holds the new tokens: the two-call path reads the same records
    two, two_lse = _gqa_rows(dev, kv, bt, q, sl, list(range(len(lens))), scale)
    assert torch.equal(whole.view(torch.int16), two.view(torch.int16))
    assert torch.equal(whole_lse, two_lse)
    for i in (0, 3, 8):
        kv1 = T.to_device_cache(kv_cpu, dev, "HND")
        one, one_lse = _gqa_rows(dev, kv1, bt, q, sl, [i], scale, fused=(nk, nv))
        assert torch.equal(one[0].view(torch.int16), whole[i].view(torch.int16))
        assert torch.equal(one_lse[0], whole_lse[i])


def test_mixed_batch_rows_do_not_depend_on_the_batch(gpu_device, invariant_mode):
    """Decode rows next to prefill chunks, and a prefill chunk next to other sequences."""
    dev = gpu_device
    hq, hkv, d, bs = 28, 4, 128, 16
    lens = [700, 3000, 96, 5000, 130, 2048]
    qls = [1, 200, 96, 1, 1, 33]
    kv_cpu, lay, bt, _, sl, _ = build_case(lens, hq, hkv, d, bs, "HND", 5, poison=False)
    kv = T.to_device_cache(kv_cpu, dev, "HND")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    g = torch.Generator().manual_seed(9)
    qs = [torch.randn((n, hq, d), generator=g).to(torch.bfloat16) for n in qls]
    scale = 1 / math.sqrt(d)

    def run(idx):
        q = torch.cat([qs[i] for i in idx]).to(dev)
        cu = torch.tensor([0] + torch.tensor([qls[i] for i in idx]).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        ii = torch.tensor(idx)
        out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
        ops.unified_attention(q, k, v, out, cu, max(qls[i] for i in idx), sl[ii].to(dev), int(sl[ii].max()), scale,
                              True, block_table=bt[ii].contiguous().to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse)
        torch.cuda.synchronize()
        cu = cu.cpu()
        return {i: (out[int(cu[j]):int(cu[j + 1])].cpu(), lse[int(cu[j]):int(cu[j + 1])].cpu()) for j, i in enumerate(idx)}

    ref = run(list(range(len(lens))))
    for idx in ([0], [1], [2], [3], [5], [3, 1, 0], [5, 4, 3, 2, 1, 0]):
        got = run(idx)
        for i in idx:
            assert torch.equal(got[i][0].view(torch.int16), ref[i][0].view(torch.int16)), f"sequence {i} in batch {idx}"
            assert torch.equal(got[i][1], ref[i][1]), f"lse of sequence {i} in batch {idx}"


@pytest.mark.parametrize("heads", [128, 16, 40])
def test_mla_decode_rows_do_not_depend_on_the_batch(gpu_device, invariant_mode, heads):
    dev = gpu_device
    R = 512
    lens = [4096, 77, 513, 0, 1, 2500, 64, 9000]
    bs = 64
    cache, lay, bt, sl = T.build_mla_cache(lens, bs, 13)
    g = torch.Generator().manual_seed(2)
    q = (torch.randn((len(lens), heads, 576), generator=g) * 0.5).to(torch.bfloat16)
    scale = (128 + 64) ** -0.5
    cache_d = cache.to(dev)

    def run(idx):
        ii = torch.tensor(idx)
        o = torch.full((len(idx), heads, R), float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full((len(idx), heads), float("nan"), dtype=torch.float32, device=dev)
        ops.mla_decode_int8(q[ii].contiguous().to(dev), cache_d, o, lse, bt[ii].contiguous().to(dev),
                            sl[ii].contiguous().to(dev), scale, R)
        torch.cuda.synchronize()
        return o.cpu(), lse.cpu()

    ref = {}
    batches = [[i] for i in range(len(lens))] + [list(range(len(lens))), list(range(len(lens)))[::-1], [5, 0, 7],
                                                  list(range(len(lens))) * 5]   # 40 rows: beyond the CU-filling count
    for idx in batches:
        o, lse = run(idx)
        for j, i in enumerate(idx):
            if i not in ref:
                ref[i] = (o[j].clone(), lse[j].clone())
                continue
            assert torch.equal(o[j].view(torch.int16), ref[i][0].view(torch.int16)), f"sequence {i} (len {lens[i]}) in {idx}"
            assert torch.equal(lse[j].view(torch.int32), ref[i][1].view(torch.int32)), f"lse of sequence {i} in {idx}"
    want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
    got = torch.stack([ref[i][0] for i in range(len(lens))])
    got_lse = torch.stack([ref[i][1] for i in range(len(lens))])
    live = sl > 0
    T.assert_close_attn(got[live], want[live], what="batch-invariant mla decode vs oracle")
    torch.testing.assert_close(got_lse[live], want_lse[live], atol=5e-3, rtol=1e-3)


def test_short_runs_and_context_splits_keep_their_bits_in_the_mode(gpu_device, invariant_mode):
    """Short query runs alone (a launch with few items) and among 300 sequences (a launch with many), and a long run
    with and without a proposal of context splits: the mode keeps one way of cutting, so the bits do not move."""
    dev = gpu_device
    hq, hkv, d, bs = 32, 8, 128, 16
    g = torch.Generator().manual_seed(4)
    n = 300
    ctx = [3000, 900] + torch.randint(20, 200, (n - 2,), generator=g).tolist()
    qls = [3, 150] + torch.randint(1, 4, (n - 2,), generator=g).tolist()
    qls = [min(c, x) for c, x in zip(ctx, qls)]
    kv_cpu, lay, bt, _, sl, _ = build_case(ctx, hq, hkv, d, bs, "HND", 6, poison=False)
    kv = T.to_device_cache(kv_cpu, dev, "HND")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    qs = [torch.randn((x, hq, d), generator=g).to(torch.bfloat16) for x in qls]
    scale = 1 / math.sqrt(d)

    def run(idx, splits=1):
        q = torch.cat([qs[i] for i in idx]).to(dev)
        cu = torch.tensor([0] + torch.tensor([qls[i] for i in idx]).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        ii = torch.tensor(idx)
        out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
        ops.unified_attention(q, k, v, out, cu, max(qls[i] for i in idx), sl[ii].to(dev), int(sl[ii].max()), scale, True,
                              block_table=bt[ii].contiguous().to(dev), k_scale_cache=ks, v_scale_cache=vs,
                              prefill_splits=splits)
        torch.cuda.synchronize()
        cu = cu.cpu()
        return {i: out[int(cu[j]):int(cu[j + 1])].cpu() for j, i in enumerate(idx)}

    whole = run(list(range(n)))
    for idx, splits in (([0], 1), ([1], 1), ([1], 4), ([0, 1, 5], 2), (list(range(0, n, 3)), 1)):
        got = run(idx, splits)
        for i in idx:
            assert torch.equal(got[i].view(torch.int16), whole[i].view(torch.int16)), f"sequence {i} in batch {idx[:4]} x{splits}"

"""GPU parity of paged decode attention over the int8 cache (balanced split-K kernel + reduce and
the fixed-partition entry point), through the C ABI, against the oracle: atol 2e-2 / rtol 1e-2 on
bf16 outputs (the north-star tolerance), tighter on fp32 outputs."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def build_case(ctx_lens, hq, hkv, d, bs, layout, seed, num_blocks=None, poison=True, outlier=False,
               q_std=1.0, q_dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    nb = num_blocks or (sum((c + bs - 1) // bs for c in ctx_lens) + 5)
    kv, views, lay = T.cpu_cache(nb, bs, hkv, d, layout)
    if poison:
        T.storage_bytes(kv).fill_(0xFF)     # NaN scales / -1 codes wherever nothing is written
    bt = T.make_block_tables(ctx_lens, bs, nb, g)
    mk = (lambda c: T.outlier_sources((c, hkv, d), g, torch.bfloat16)) if outlier else \
         (lambda c: torch.randn((c, hkv, d), generator=g).to(torch.bfloat16))
    ks = [mk(c) for c in ctx_lens]
    vs = [mk(c) for c in ctx_lens]
    T.fill_cache_from_sources(kv, lay, bt, ctx_lens, bs, ks, vs)
    q = (torch.randn((len(ctx_lens), hq, d), generator=g) * q_std).to(q_dtype)
    sl = torch.tensor(ctx_lens, dtype=torch.int32)
    cu = torch.arange(len(ctx_lens) + 1, dtype=torch.int32)
    return kv, lay, bt, q, sl, cu


def run_unified(dev, kv_cpu, layout, bt, q, sl, cu, scale, out_dtype=torch.bfloat16, want_lse=False):
    kv = T.to_device_cache(kv_cpu, dev, layout)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    out = torch.full(q.shape, float("nan"), dtype=out_dtype, device=dev)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev) if want_lse else None
    ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), 1, sl.to(dev), int(sl.max()), scale, True,
                          block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse)
    torch.cuda.synchronize()
    return (out, lse) if want_lse else out


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_config1_shape(gpu_device, layout):
    """32 q heads / 8 kv heads, head 128, block 16, batch 4, ctx 512 each, 128-block pool."""
    ctx = [512] * 4
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, layout, 0, num_blocks=129)
    scale = 1 / math.sqrt(128)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True)
    got, lse = run_unified(gpu_device, kv, layout, bt, q, sl, cu, scale, want_lse=True)
    T.assert_close_attn(got, want, what="config 1")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=2e-3, rtol=1e-3)


def test_config1_as_worded_fp32_sources_written_on_the_gpu(gpu_device):
    """The first configuration to the letter: K / V sources are fp32 N(0, 1), quantised per token and head by
    the write kernel itself (bit-exact against the oracle's cache), block tables a seeded permutation of the
    128-block pool, Q bf16, output bf16 [4, 32, 128]."""
    dev = gpu_device
    hq, hkv, d, bs, nb = 32, 8, 128, 16, 128
    ctx = [512] * 4
    g = torch.Generator().manual_seed(0)
    bt = torch.randperm(nb, generator=g).to(torch.int32).view(4, 32)
    kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    for i, slots in enumerate(T.slots_for(bt, ctx, bs)):
        key = torch.randn((ctx[i], hkv, d), generator=g, dtype=torch.float32)
        val = torch.randn((ctx[i], hkv, d), generator=g, dtype=torch.float32)
        oracle.cache_write(key, val, T.storage_bytes(kv_cpu), lay, slots)
        ops.reshape_and_cache_flash_per_token_head_quant(key.to(dev), val.to(dev), k, v, ks, vs, slots.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(T.storage_bytes(kv).cpu(), T.storage_bytes(kv_cpu)), "quantised cache differs from the oracle"
    q = torch.randn((4, hq, d), generator=g).to(torch.bfloat16)
    sl = torch.tensor(ctx, dtype=torch.int32)
    cu = torch.arange(5, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
    ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), 1, sl.to(dev), 512, scale, True, block_table=bt.to(dev),
                          k_scale_cache=ks, v_scale_cache=vs)
    torch.cuda.synchronize()
    want = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, scale)
    assert out.shape == (4, 32, 128) and out.dtype == torch.bfloat16
    T.assert_close_attn(out, want, what="config 1 as worded")


@pytest.mark.parametrize("ctx", [[1], [31, 32, 33], [15, 16, 17, 1, 2], [1000, 3, 517, 64, 4097], [700] * 70])
def test_ragged_lengths_fp32_out(gpu_device, ctx):
    """Ragged and tiny contexts, sequence boundaries falling inside workgroup ranges, more
    sequences than one wave scans at once; fp32 output isolates kernel error from bf16 rounding."""
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "NHD", len(ctx))
    scale = 1 / math.sqrt(128)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run_unified(gpu_device, kv, "NHD", bt, q, sl, cu, scale, out_dtype=torch.float32)
    T.assert_close_attn(got, want, atol=2e-3, rtol=2e-3, what=f"ctx={ctx[:5]}")


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("hkv", [1, 2, 8])
def test_hundreds_of_short_sequences(gpu_device, hkv, layout):
    """300 sequences of 0 .. 200 tokens with prefill rows in between: the sequence scans run in
    batches of several 64-sequence chunks, a workgroup's share crosses many sequence boundaries
    (or, with one kv head, the work line is so short that not every workgroup gets a share), and
    empty sequences must come out as zeros with lse = -inf."""
    g = torch.Generator().manual_seed(hkv)
    ctx = torch.randint(0, 201, (300,), generator=g).tolist()
    qls = [1] * 300
    for i in range(7, 300, 41):            # a few rows of another kind: short query runs
        qls[i] = min(3, max(ctx[i], 1))
        ctx[i] = max(ctx[i], qls[i])
    from test_gpu_prefill import build
    kv, lay, bt, q, sl, cu = build([max(c, 1) for c in ctx], qls, 2 * hkv, hkv, 128, 16, seed=hkv, layout=layout)
    sl = torch.tensor(ctx, dtype=torch.int32)   # the true lengths, zeros included
    scale = 1 / math.sqrt(128)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True)
    kvd = T.to_device_cache(kv, gpu_device, layout)
    k, v = L.key_value_views(kvd)
    ks, vs = L.scale_views(kvd)
    out = torch.full(q.shape, float("nan"), dtype=torch.float32, device=gpu_device)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=gpu_device)
    ops.unified_attention(q.to(gpu_device), k, v, out, cu.to(gpu_device), max(qls), sl.to(gpu_device), max(ctx), scale,
                          True, block_table=bt.to(gpu_device), k_scale_cache=ks, v_scale_cache=vs, lse=lse)
    torch.cuda.synchronize()
    T.assert_close_attn(out, want, atol=2e-3, rtol=2e-3, what=f"300 sequences, hkv={hkv}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("where", [0, 77, 139])
@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 2)])
def test_one_long_sequence_among_many_short(gpu_device, hq, hkv, where):
    """140 sequences of a few dozen tokens and one of 30000: the batch is large enough for the
    reduce that runs one block per share of the work line, and the long sequence alone covers
    far more than sixteen shares, so its partial results are merged by the long-span path of that
    kernel, whether it comes first, in the middle or last."""
    g = torch.Generator().manual_seed(hq + where)
    ctx = torch.randint(1, 97, (140,), generator=g).tolist()
    ctx[where] = 30000
    qls = [1] * 140
    from test_gpu_prefill import build
    kv, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, 128, 16, seed=where + 1)
    scale = 1 / math.sqrt(128)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True)
    kvd = T.to_device_cache(kv, gpu_device, "NHD")
    k, v = L.key_value_views(kvd)
    ks, vs = L.scale_views(kvd)
    out = torch.full(q.shape, float("nan"), dtype=torch.float32, device=gpu_device)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=gpu_device)
    ops.unified_attention(q.to(gpu_device), k, v, out, cu.to(gpu_device), 1, sl.to(gpu_device), max(ctx), scale,
                          True, block_table=bt.to(gpu_device), k_scale_cache=ks, v_scale_cache=vs, lse=lse)
    torch.cuda.synchronize()
    T.assert_close_attn(out, want, atol=2e-3, rtol=2e-3, what=f"long sequence at {where}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("hq,hkv,d,bs", [(28, 4, 128, 16), (8, 8, 128, 16), (16, 1, 128, 32), (8, 2, 64, 16),
                                         (4, 2, 256, 16), (32, 16, 128, 64),
                                         # head counts of the reference's paged-attention grid
                                         # (tests/kernels/attention/test_attention.py:31-47) at the built head sizes
                                         (40, 40, 128, 16), (64, 8, 128, 32), (40, 40, 256, 32), (64, 8, 64, 16),
                                         # kv head counts that leave the last workgroup partly empty (its
                                         # spare waves exit before the stream loop's rendezvous)
                                         (24, 12, 128, 16), (6, 3, 64, 16), (10, 5, 128, 32)])
@pytest.mark.parametrize("layout", ["NHD", "HND"])   # HND: the streamed run loads (head sizes 64 and 128)
def test_head_and_block_shapes(gpu_device, hq, hkv, d, bs, layout):
    ctx = [200, 77, 1025, 48]
    kv, lay, bt, q, sl, cu = build_case(ctx, hq, hkv, d, bs, layout, hq + d)
    scale = d ** -0.5
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run_unified(gpu_device, kv, layout, bt, q, sl, cu, scale)
    T.assert_close_attn(got, want, what=f"hq={hq} hkv={hkv} d={d} bs={bs} {layout}")


@pytest.mark.parametrize("q_dtype", [torch.float16, torch.float32])
def test_query_dtypes(gpu_device, q_dtype):
    ctx = [130, 700]
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "NHD", 21, q_dtype=q_dtype)
    scale = 128 ** -0.5
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run_unified(gpu_device, kv, "NHD", bt, q, sl, cu, scale, out_dtype=q_dtype)
    T.assert_close_attn(got, want, atol=5e-3, rtol=5e-3, what=f"q dtype {q_dtype}")


def test_outlier_heavy_sources_and_peaked_softmax(gpu_device):
    """1 % of channels x20 (stresses the scales) and a large |q| (nearly one-hot softmax)."""
    ctx = [3000, 513]
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "NHD", 9, outlier=True, q_std=3.0)
    scale = 1 / math.sqrt(128)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run_unified(gpu_device, kv, "NHD", bt, q, sl, cu, scale)
    T.assert_close_attn(got, want, what="outliers")


def test_empty_sequence_and_untouched_padding_rows(gpu_device):
    ctx = [40, 0, 9]
    kv, lay, bt, q, sl, cu = build_case([40, 1, 9], 8, 2, 128, 16, "NHD", 10)
    sl = torch.tensor(ctx, dtype=torch.int32)
    scale = 0.1
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run_unified(gpu_device, kv, "NHD", bt, q, sl, cu, scale)
    assert (got[1] == 0).all()
    T.assert_close_attn(got, want, what="empty sequence")


def test_fixed_partitions_v2_contract(gpu_device):
    """512-token partitions: tmp_out / max_logits / exp_sums per partition match the oracle's
    stage 1, and the reduce matches unsplit attention."""
    dev = gpu_device
    ctx = [1500, 512, 513, 30, 2048]
    hq, hkv, d, bs = 32, 8, 128, 16
    kv_cpu, lay, bt, q, sl, cu = build_case(ctx, hq, hkv, d, bs, "NHD", 12)
    scale = d ** -0.5
    P = (max(ctx) + 511) // 512
    kv = T.to_device_cache(kv_cpu, dev, "NHD")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    B = len(ctx)
    out = torch.empty((B, hq, d), dtype=torch.bfloat16, device=dev)
    es = torch.zeros((B, hq, P), dtype=torch.float32, device=dev)
    ml = torch.zeros((B, hq, P), dtype=torch.float32, device=dev)
    tmp = torch.zeros((B, hq, P, d), dtype=torch.float32, device=dev)
    ops.paged_attention_v2(out, es, ml, tmp, q.to(dev), k, v, hkv, scale, bt.to(dev), sl.to(dev), bs, max(ctx),
                           k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    base = T.storage_bytes(kv_cpu)
    wtmp, wml, wes = oracle.paged_attn_partition(q, base, lay, bt, sl, scale, 512, P)
    for i, c in enumerate(ctx):
        n = (c + 511) // 512
        T.assert_close_attn(tmp[i, :, :n], wtmp[i, :, :n], atol=2e-3, rtol=2e-3, what="tmp_out")
        torch.testing.assert_close(ml[i, :, :n].cpu(), wml[i, :, :n], atol=2e-3, rtol=1e-3)
        torch.testing.assert_close(es[i, :, :n].cpu(), wes[i, :, :n], atol=1e-3, rtol=5e-3)
    want = oracle.paged_attn(q, base, lay, bt, sl, cu, scale)
    T.assert_close_attn(out, want, what="v2 reduce")
    # the reduce entry point alone, on the oracle's stage-1 output, with lse
    out2 = torch.empty((B, hq, d), dtype=torch.float32, device=dev)
    lse = torch.empty((B, hq), dtype=torch.float32, device=dev)
    ops.splitk_reduce(out2, wes.to(dev), wml.to(dev), wtmp.to(dev), sl.to(dev), 512, lse=lse)
    w2, wl2 = oracle.splitk_reduce(wtmp, wml, wes, sl, 512, return_lse=True)
    torch.testing.assert_close(out2.cpu(), w2, atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(lse.cpu(), wl2, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (4, 1, 256)])
def test_fixed_partitions_v2_with_alibi(gpu_device, hq, hkv, d):
    """alibi_slopes of paged_attention_v2 (csrc/libtorch_stable/torch_bindings.cpp:631-641; the bias
    alibi_slopes * (position - seq_len + 1) of tests/kernels/attention/test_attention.py:109-117): the reduced
    output matches the oracle's biased attention, and the per-partition tmp_out / max_logits / exp_sums are a
    consistent stage 1 -- the oracle's reduce over them gives the same rows and the biased lse."""
    dev = gpu_device
    ctx = [1500, 512, 513, 30, 2048]
    bs = 16
    kv_cpu, lay, bt, q, sl, cu = build_case(ctx, hq, hkv, d, bs, "HND", 21)
    scale = d ** -0.5
    slopes = torch.tensor([2.0 ** (-8.0 * (i + 1) / hq) for i in range(hq)], dtype=torch.float32)
    slopes[0] = 1.0
    P = (max(ctx) + 511) // 512
    kv = T.to_device_cache(kv_cpu, dev, "HND")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    B = len(ctx)
    out = torch.empty((B, hq, d), dtype=torch.bfloat16, device=dev)
    es = torch.zeros((B, hq, P), dtype=torch.float32, device=dev)
    ml = torch.zeros((B, hq, P), dtype=torch.float32, device=dev)
    tmp = torch.zeros((B, hq, P, d), dtype=torch.float32, device=dev)
    ops.paged_attention_v2(out, es, ml, tmp, q.to(dev), k, v, hkv, scale, bt.to(dev), sl.to(dev), bs, max(ctx),
                           alibi_slopes=slopes.to(dev), k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    base = T.storage_bytes(kv_cpu)
    want, want_lse = oracle.paged_attn(q, base, lay, bt, sl, cu, scale, alibi_slopes=slopes, return_lse=True)
    plain = oracle.paged_attn(q, base, lay, bt, sl, cu, scale)
    assert not torch.allclose(want, plain, atol=5e-2)
    T.assert_close_attn(out, want, what="v2 with alibi")
    red, red_lse = oracle.splitk_reduce(tmp.cpu(), ml.cpu(), es.cpu(), sl, 512, return_lse=True)
    T.assert_close_attn(red, want, atol=2e-3, rtol=2e-3, what="v2 stage 1 with alibi, reduced by the oracle")
    torch.testing.assert_close(red_lse, want_lse, atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("q_lens", [[1, 1, 1], [1, 5, 129]])
def test_block_size_does_not_change_the_result(gpu_device, q_lens):
    """The same tokens paged with 16-, 32-, 64- and 128-token blocks give bit-identical outputs (the
    page-size self-consistency check of tests/kernels/attention/test_triton_decode_attention.py:12-90),
    for decode rows and for the reference's mixed batch (query, context) = (1, 1328), (5, 18), (129, 463)
    (tests/kernels/attention/test_triton_unified_attention.py:81-83)."""
    dev = gpu_device
    ctx = [1328, 18, 463]
    hq, hkv, d = 32, 8, 128
    g = torch.Generator().manual_seed(77)
    ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    vs = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    q = torch.randn((sum(q_lens), hq, d), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
    sl = torch.tensor(ctx, dtype=torch.int32)
    outs = []
    for bs in (16, 32, 64, 128):
        nb = sum((c + bs - 1) // bs for c in ctx) + 3
        kv, views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
        T.storage_bytes(kv).fill_(0xFF)
        bt = T.make_block_tables(ctx, bs, nb, torch.Generator().manual_seed(bs))
        T.fill_cache_from_sources(kv, lay, bt, ctx, bs, ks, vs)
        kvd = T.to_device_cache(kv, dev, "NHD")
        k, v = L.key_value_views(kvd)
        ksc, vsc = L.scale_views(kvd)
        out = torch.full(q.shape, float("nan"), dtype=torch.float32, device=dev)
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(q_lens), sl.to(dev), max(ctx), 0.0884, True,
                              block_table=bt.to(dev), k_scale_cache=ksc, v_scale_cache=vsc)
        torch.cuda.synchronize()
        outs.append(out.cpu())
        if bs == 16:
            want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, 0.0884)
            T.assert_close_attn(out, want, atol=4e-3, rtol=4e-3, what="reference mixed batch")
    for o in outs[1:]:
        assert torch.equal(o, outs[0]), "block size changed the result"


def test_block_permutation_invariance_on_device(gpu_device):
    dev = gpu_device
    ctx = [333, 1200]
    kv_cpu, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "NHD", 13, poison=False)
    scale = 0.09
    a = run_unified(dev, kv_cpu, "NHD", bt, q, sl, cu, scale, out_dtype=torch.float32)
    nb = kv_cpu.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1))
    kv2, _, _ = T.cpu_cache(nb, 16, 8, 128, "NHD")
    T.storage_bytes(kv2).view(nb, -1)[perm] = T.storage_bytes(kv_cpu).view(nb, -1)
    b = run_unified(dev, kv2, "NHD", perm[bt.long()].to(torch.int32), q, sl, cu, scale, out_dtype=torch.float32)
    assert torch.equal(a, b)


@pytest.mark.parametrize("vmag,ctx,rel", [(1e-3, 8192, 1e-3), (1e-2, 8192, 1e-3), (3000.0, 512, 2e-3), (6500.0, 512, 2e-3)])
def test_value_magnitudes_far_from_one(gpu_device, vmag, ctx, rel):
    """The weights reach the P~.V product as fp16 numbers p * v_scale * 2^8.  Tiny values spread thinly over a
    long uniform context (p ~ 1/8192: P~ is subnormal in fp16) and rows near the documented limit of the
    V scale (255.8, i.e. absmax 32 500: 6500 x the 4.6 sigma of 64k draws is ~30 000) must still match the
    oracle RELATIVE to the result's magnitude, not just within the absolute tolerance."""
    g = torch.Generator().manual_seed(5)
    hq, hkv, d, bs = 8, 2, 128, 16
    ctx_lens = [ctx, ctx // 3]
    nb = sum((c + bs - 1) // bs for c in ctx_lens) + 5
    kv, views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    bt = T.make_block_tables(ctx_lens, bs, nb, g)
    ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx_lens]
    vs = [(torch.randn((c, hkv, d), generator=g) * vmag).to(torch.bfloat16) for c in ctx_lens]
    T.fill_cache_from_sources(kv, lay, bt, ctx_lens, bs, ks, vs)
    q = (torch.randn((2, hq, d), generator=g) * (0.0 if vmag < 1 else 1.0)).to(torch.bfloat16)   # q = 0: uniform weights
    sl = torch.tensor(ctx_lens, dtype=torch.int32)
    cu = torch.arange(3, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    got = run_unified(gpu_device, kv, "NHD", bt, q, sl, cu, scale, out_dtype=torch.float32)
    mag = float(want.abs().max())
    assert float((got.cpu() - want).abs().max()) <= rel * mag, (float((got.cpu() - want).abs().max()), mag)

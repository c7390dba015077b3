"""The BASELINE configurations at their full sizes on the GPU.  The oracle cannot run whole
batches of this size in seconds, so each case is checked (a) against the oracle on a few of its
sequences, gathered out of the big cache into a small one, and (b) through properties that do not
depend on size: two independently partitioned kernels agree (balanced split-K vs fixed 512-token
partitions + reduce; 8 vs 64 MLA splits), rows of a long causal chunk equal a short run over a
truncated sequence, and re-quantising a dequantised row reproduces its codes."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def _tables(ctx, bs, pool, g):
    need = [(c + bs - 1) // bs for c in ctx]
    perm = torch.randperm(pool - 1, generator=g)[: sum(need)] + 1
    bt = torch.zeros((len(ctx), max(need)), dtype=torch.int32)
    o = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[o:o + n].to(torch.int32)
        o += n
    return bt


def _fill_gqa(dev, ctx, bt, hkv, d, bs, pool, outlier=False, layout="NHD"):
    """Cache filled on the GPU through the quantise-on-write kernel (bit-exactness of that kernel
    is its own test); sources N(0,1) bf16, optionally with 1 % of the channels scaled x20."""
    kv = L.allocate_kv_cache(pool, bs, hkv, d, device=dev, layout=layout, fill=0)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    ks.fill_(1.0)
    vs.fill_(1.0)
    bt_d = bt.to(dev)
    torch.manual_seed(1234)
    gain_k = torch.ones(hkv * d, device=dev)
    gain_v = torch.ones(hkv * d, device=dev)
    if outlier:
        n = max(1, round(0.01 * hkv * d))
        gain_k[torch.randperm(hkv * d, device=dev)[:n]] = 20.0
        gain_v[torch.randperm(hkv * d, device=dev)[:n]] = 20.0
    for i, c in enumerate(ctx):
        pos = torch.arange(c, device=dev)
        slots = bt_d[i, pos // bs].to(torch.int64) * bs + pos % bs
        for s0 in range(0, c, 32768):
            n = min(32768, c - s0)
            ksrc = (torch.randn((n, hkv * d), device=dev) * gain_k).view(n, hkv, d).to(torch.bfloat16)
            vsrc = (torch.randn((n, hkv * d), device=dev) * gain_v).view(n, hkv, d).to(torch.bfloat16)
            ops.reshape_and_cache_flash_per_token_head_quant(ksrc, vsrc, k, v, ks, vs, slots[s0:s0 + n])
    return kv, k, v, ks, vs


def _gather_to_cpu(kv, bt, seqs, ctx, hkv, d, bs, layout="NHD"):
    """The blocks of the chosen sequences as a small CPU cache with a renumbered block table."""
    per = [(ctx[i] + bs - 1) // bs for i in seqs]
    cpu, _views, lay = T.cpu_cache(sum(per) + 1, bs, hkv, d, layout)
    big = T.storage_bytes(kv).view(kv.shape[0], -1)
    small = T.storage_bytes(cpu).view(sum(per) + 1, -1)
    bt2 = torch.zeros((len(seqs), max(per)), dtype=torch.int32)
    o = 1
    for j, i in enumerate(seqs):
        ids = bt[i, : per[j]].long()
        small[o:o + per[j]] = big[ids.to(kv.device)].cpu()
        bt2[j, : per[j]] = torch.arange(o, o + per[j], dtype=torch.int32)
        o += per[j]
    return cpu, lay, bt2


def _decode_both_ways(dev, q, k, v, ks, vs, bt, ctx, hq, hkv, d, bs, scale):
    B = len(ctx)
    sl = torch.tensor(ctx, dtype=torch.int32, device=dev)
    cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
    a = torch.empty((B, hq, d), dtype=torch.float32, device=dev)
    lse = torch.empty((B, hq), dtype=torch.float32, device=dev)
    ops.unified_attention(q, k, v, a, cu, 1, sl, max(ctx), scale, True, block_table=bt.to(dev), k_scale_cache=ks,
                          v_scale_cache=vs, lse=lse)
    P = (max(ctx) + 511) // 512
    b = torch.empty((B, hq, d), dtype=torch.float32, device=dev)
    es = torch.empty((B, hq, P), dtype=torch.float32, device=dev)
    ml = torch.empty((B, hq, P), dtype=torch.float32, device=dev)
    tmp = torch.empty((B, hq, P, d), dtype=torch.float32, device=dev)
    ops.paged_attention_v2(b, es, ml, tmp, q, k, v, hkv, scale, bt.to(dev), sl, bs, max(ctx), k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    return a, b, lse


@pytest.mark.parametrize("layout", ["NHD", "HND"])   # HND: the streamed run loads of the decode kernel
def test_config2_llama3_8b_b64_ctx1k_8k(gpu_device, layout):
    dev = gpu_device
    hq, hkv, d, bs, pool = 32, 8, 128, 16, 40000
    g = torch.Generator().manual_seed(0)
    ctx = torch.randint(1024, 8193, (64,), generator=g).tolist()
    bt = _tables(ctx, bs, pool, g)
    kv, k, v, ks, vs = _fill_gqa(dev, ctx, bt, hkv, d, bs, pool, layout=layout)
    q = torch.randn((64, hq, d), device=dev).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    a, b, lse = _decode_both_ways(dev, q, k, v, ks, vs, bt, ctx, hq, hkv, d, bs, scale)
    assert torch.isfinite(a).all()
    T.assert_close_attn(a, b, atol=2e-3, rtol=2e-3, what="balanced split-K vs 512-token partitions")
    # every sequence of the batch against the oracle, sixteen at a time (their blocks gathered to the host)
    for s0 in range(0, 64, 16):
        seqs = list(range(s0, s0 + 16))
        cpu, lay, bt2 = _gather_to_cpu(kv, bt, seqs, ctx, hkv, d, bs, layout)
        sl2 = torch.tensor([ctx[i] for i in seqs], dtype=torch.int32)
        want, want_lse = oracle.paged_attn(q[seqs].cpu(), T.storage_bytes(cpu), lay, bt2, sl2,
                                           torch.arange(17, dtype=torch.int32), scale, return_lse=True)
        T.assert_close_attn(a[seqs], want, atol=4e-3, rtol=4e-3, what=f"config 2 vs oracle, sequences {s0}..")
        torch.testing.assert_close(lse[seqs].cpu(), want_lse, atol=5e-3, rtol=1e-3)
        del cpu
    # re-quantising the dequantised newest row of every sequence reproduces its codes
    last = torch.tensor([int(bt[i, (c - 1) // bs]) * bs + (c - 1) % bs for i, c in enumerate(ctx)], device=dev)
    kc_before = k.reshape(-1, hkv, d + 4)[last][..., :d].clone()
    vc_before = v.reshape(-1, hkv, d + 4)[last][..., :d].clone()
    kk = kc_before.float() * ks.reshape(-1, hkv)[last][..., None]
    vv = vc_before.float() * vs.reshape(-1, hkv)[last][..., None]
    ops.reshape_and_cache_flash_per_token_head_quant(kk, vv, k, v, ks, vs, last)
    torch.cuda.synchronize()
    assert torch.equal(k.reshape(-1, hkv, d + 4)[last][..., :d], kc_before)
    assert torch.equal(v.reshape(-1, hkv, d + 4)[last][..., :d], vc_before)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_config3_long_context_split_k(gpu_device, layout):
    dev = gpu_device
    hq, hkv, d, bs, pool = 32, 8, 128, 16, 66000
    g = torch.Generator().manual_seed(0)
    ctx = torch.randint(32768, 131073, (8,), generator=g).tolist()
    bt = _tables(ctx, bs, pool, g)
    kv, k, v, ks, vs = _fill_gqa(dev, ctx, bt, hkv, d, bs, pool, outlier=True, layout=layout)
    q = torch.randn((8, hq, d), device=dev).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    a, b, lse = _decode_both_ways(dev, q, k, v, ks, vs, bt, ctx, hq, hkv, d, bs, scale)
    assert torch.isfinite(a).all()
    T.assert_close_attn(a, b, atol=2e-3 * 20, rtol=2e-3, what="balanced split-K vs 512-token partitions")
    # every sequence of the batch against the oracle, two at a time (their blocks gathered to the host)
    for pair in ([0, 1], [2, 3], [4, 5], [6, 7]):
        cpu, lay, bt2 = _gather_to_cpu(kv, bt, pair, ctx, hkv, d, bs, layout)
        want, want_lse = oracle.paged_attn(q[pair].cpu(), T.storage_bytes(cpu), lay, bt2,
                                           torch.tensor([ctx[i] for i in pair], dtype=torch.int32),
                                           torch.arange(3, dtype=torch.int32), scale, return_lse=True)
        T.assert_close_attn(a[pair], want, atol=2e-2, rtol=1e-2, what=f"config 3 vs oracle, sequences {pair}")
        torch.testing.assert_close(lse[pair].cpu(), want_lse, atol=2e-2, rtol=1e-3)
        del cpu


def test_config4_mla_b32_ctx4096(gpu_device):
    dev = gpu_device
    R, P, H, bs, B, c = 512, 64, 128, 64, 32, 4096
    g = torch.Generator().manual_seed(0)
    nb = B * (c // bs) + 8
    ctx = [c] * B
    bt = _tables(ctx, bs, nb, g)
    cache = L.allocate_mla_cache(nb, bs, R + P, device=dev)
    bt_d = bt.to(dev)
    torch.manual_seed(5)
    for i in range(B):
        pos = torch.arange(c, device=dev)
        slots = bt_d[i, pos // bs].to(torch.int64) * bs + pos % bs
        ops.concat_and_cache_mla(torch.randn((c, R), device=dev).to(torch.bfloat16),
                                 torch.randn((c, P), device=dev).to(torch.bfloat16), cache, slots)
    q = (torch.randn((B, H, R + P), device=dev) * 0.5).to(torch.bfloat16)
    sl = torch.tensor(ctx, dtype=torch.int32, device=dev)
    scale = 192 ** -0.5
    o = torch.empty((B, H, R), dtype=torch.float32, device=dev)
    lse = torch.empty((B, H), dtype=torch.float32, device=dev)
    ops.mla_decode_int8(q, cache, o, lse, bt_d, sl, scale, R)
    # split-count invariance: a sequence on its own runs with 64 splits instead of 8
    for i in (0, 17):
        o1 = torch.empty((1, H, R), dtype=torch.float32, device=dev)
        l1 = torch.empty((1, H), dtype=torch.float32, device=dev)
        ops.mla_decode_int8(q[i:i + 1], cache, o1, l1, bt_d[i:i + 1], sl[i:i + 1], scale, R)
        torch.cuda.synchronize()
        T.assert_close_attn(o[i:i + 1], o1, atol=2e-3, rtol=2e-3, what="8 vs 64 splits")
        torch.testing.assert_close(lse[i:i + 1], l1, atol=1e-3, rtol=1e-4)
    # oracle on two sequences, gathered into a small cache
    seqs = [3, 31]
    n = c // bs
    small = L.allocate_mla_cache(2 * n + 1, bs, R + P, device="cpu")
    bt2 = torch.zeros((2, n), dtype=torch.int32)
    for j, i in enumerate(seqs):
        small[1 + j * n: 1 + (j + 1) * n] = cache[bt[i, :n].long().to(dev)].cpu()
        bt2[j] = torch.arange(1 + j * n, 1 + (j + 1) * n, dtype=torch.int32)
    codes, scales = L.mla_cache_views(small)
    lay = oracle.MlaLayout.from_views(small, codes, scales, R)
    want, want_lse = oracle.mla_decode(q[seqs].cpu(), small, lay, bt2, torch.tensor([c, c], dtype=torch.int32), scale)
    T.assert_close_attn(o[seqs], want, atol=4e-3, rtol=4e-3, what="config 4 vs oracle")
    torch.testing.assert_close(lse[seqs].cpu(), want_lse, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_config5_mixed_prefill_and_decode(gpu_device, layout):
    dev = gpu_device
    hq, hkv, d, bs, pool = 28, 4, 128, 16, 12000
    g = torch.Generator().manual_seed(0)
    dctx = torch.randint(512, 4097, (60,), generator=g).tolist()
    ctx = [2048, 4096, 6144, 8192] + dctx            # lengths including the run's own tokens
    qls = [2048] * 4 + [1] * 60
    bt = _tables(ctx, bs, pool, g)
    kv, k, v, ks, vs = _fill_gqa(dev, ctx, bt, hkv, d, bs, pool, layout=layout)
    n_tok = sum(qls)
    q = torch.randn((n_tok, hq, d), device=dev).to(torch.bfloat16)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    sl = torch.tensor(ctx, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    out = torch.full((n_tok, hq, d), float("nan"), dtype=torch.float32, device=dev)
    ops.unified_attention(q, k, v, out, cu.to(dev), 2048, sl.to(dev), max(ctx), scale, True, block_table=bt.to(dev),
                          k_scale_cache=ks, v_scale_cache=vs)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    # rows [r0, r0+32) of a causal chunk are a 32-token run over the sequence truncated after them
    cases = [(0, 0), (1, 1000), (3, 2016), (2, 37)]
    for i, r0 in cases:
        trunc = ctx[i] - qls[i] + r0 + 32
        cpu, lay, bt2 = _gather_to_cpu(kv, bt, [i], [trunc if j == i else c for j, c in enumerate(ctx)], hkv, d, bs, layout)
        rows = slice(int(cu[i]) + r0, int(cu[i]) + r0 + 32)
        want = oracle.paged_attn(q[rows].cpu(), T.storage_bytes(cpu), lay, bt2, torch.tensor([trunc], dtype=torch.int32),
                                 torch.tensor([0, 32], dtype=torch.int32), scale)
        T.assert_close_attn(out[rows], want, atol=4e-3, rtol=4e-3, what=f"chunk {i} rows {r0}..")
    # decode rows of the same call
    seqs = [4, 33, 63]
    cpu, lay, bt2 = _gather_to_cpu(kv, bt, seqs, ctx, hkv, d, bs, layout)
    rows = [int(cu[i]) for i in seqs]
    want = oracle.paged_attn(q[rows].cpu(), T.storage_bytes(cpu), lay, bt2, torch.tensor([ctx[i] for i in seqs], dtype=torch.int32),
                             torch.arange(4, dtype=torch.int32), scale)
    T.assert_close_attn(out[rows], want, atol=4e-3, rtol=4e-3, what="decode rows of the mixed batch")

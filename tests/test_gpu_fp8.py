"""GPU parity of the fp8 (e4m3fn) per-token-head mode of the inline-scale record layout, through the C ABI:
the write kernel's bytes equal the oracle's bit for bit, decode rows and mixed batches lie within the
attention tolerance (atol 2e-2 / rtol 1e-2) of the oracle run on the same fp8 cache, and the backend mirror
serves ``kv_cache_dtype="fp8_per_token_head"`` end to end."""
import math
import types

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L
from vllm_metax_amd.kv_cache_interface import KVQuantMode
from vllm_metax_amd.v1.attention.backends.int8_attn import Int8AttentionBackend

pytestmark = pytest.mark.gpu
FP8 = KVQuantMode.FP8_PER_TOKEN_HEAD


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_write_is_bit_exact(gpu_device, layout, dtype):
    dev = gpu_device
    hkv, d, bs, nb, n = 8, 128, 16, 40, 300
    g = torch.Generator().manual_seed(31)
    key = (torch.randn((n + 3, hkv, d), generator=g) * 2).to(dtype)
    val = T.outlier_sources((n + 3, hkv, d), g, dtype)
    key[::7] = 0                                                    # zero rows: scale floor, codes 0
    slots = torch.randperm(nb * bs, generator=g)[:n].to(torch.int64)
    slots[torch.rand(n, generator=g) < 0.1] = -1
    kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, layout, fill=0x11)
    oracle.cache_write(key, val, T.storage_bytes(kv_cpu), lay, slots, code_type=oracle.CODE_FP8)
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout=layout, fill=0x11)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    ops.reshape_and_cache_flash_per_token_head_quant(key.to(dev), val.to(dev), k, v, ks, vs, slots.to(dev),
                                                     kv_quant_mode=FP8)
    torch.cuda.synchronize()
    got, want = T.storage_bytes(kv).cpu(), T.storage_bytes(kv_cpu)
    assert torch.equal(got, want), f"{(got != want).sum().item()} bytes differ"


def test_write_other_head_sizes_and_ties(gpu_device):
    dev = gpu_device
    for hkv, d, bs in ((2, 64, 32), (1, 256, 16), (3, 80, 16)):
        g = torch.Generator().manual_seed(d)
        key = torch.randn((50, hkv, d), generator=g).to(torch.bfloat16)
        val = torch.randn((50, hkv, d), generator=g).to(torch.bfloat16)
        # exact midpoints between neighbouring codes in a row whose absmax is 448 (scale 1): ties to even
        tab = oracle.e4m3fn_table()[:0x7f]
        mid = ((tab[:-1] + tab[1:]) / 2)[-(min(d, 127) - 1):]
        val = val.to(torch.float32)
        val[0, 0] = 0
        val[0, 0, :mid.numel()] = mid
        val[0, 0, d - 1] = 448.0
        key = key.to(torch.float32)
        slots = torch.arange(50, dtype=torch.int64)
        kv_cpu, _, lay = T.cpu_cache(8, bs, hkv, d, "NHD")
        oracle.cache_write(key, val, T.storage_bytes(kv_cpu), lay, slots, code_type=oracle.CODE_FP8)
        kv = L.allocate_kv_cache(8, bs, hkv, d, device=dev, layout="NHD")
        k, v = L.key_value_views(kv)
        ks, vs = L.scale_views(kv)
        ops.reshape_and_cache_flash_per_token_head_quant(key.to(dev), val.to(dev), k, v, ks, vs, slots.to(dev),
                                                         kv_quant_mode=FP8)
        torch.cuda.synchronize()
        assert torch.equal(T.storage_bytes(kv).cpu(), T.storage_bytes(kv_cpu)), f"hkv={hkv} d={d}"


def _fp8_case(ctx, qls, hq, hkv, d, bs, seed, layout="NHD", outlier=False):
    g = torch.Generator().manual_seed(seed)
    nb = sum((c + bs - 1) // bs for c in ctx) + 5
    kv, _, lay = T.cpu_cache(nb, bs, hkv, d, layout)
    T.storage_bytes(kv).fill_(0xFF)                                  # NaN scales / NaN codes wherever nothing is written
    bt = T.make_block_tables(ctx, bs, nb, g)
    mk = (lambda c: T.outlier_sources((c, hkv, d), g, torch.bfloat16)) if outlier else \
         (lambda c: torch.randn((c, hkv, d), generator=g).to(torch.bfloat16))
    base = T.storage_bytes(kv)
    for i, slots in enumerate(T.slots_for(bt, ctx, bs)):
        if slots.numel():
            oracle.cache_write(mk(ctx[i]), mk(ctx[i]), base, lay, slots, code_type=oracle.CODE_FP8)
    q = torch.randn((sum(qls), hq, d), generator=g).to(torch.bfloat16)
    sl = torch.tensor(ctx, dtype=torch.int32)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    return kv, lay, bt, q, sl, cu


def _attend(dev, kv_cpu, layout, bt, q, sl, cu, max_q, scale, out_dtype=torch.bfloat16, lse=False):
    kv = T.to_device_cache(kv_cpu, dev, layout)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    out = torch.full(q.shape, float("nan"), dtype=out_dtype, device=dev)
    l = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev) if lse else None
    ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max_q, sl.to(dev), int(sl.max()), scale, True,
                          block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, kv_quant_mode=FP8, lse=l)
    torch.cuda.synchronize()
    return (out, l) if lse else out


@pytest.mark.parametrize("hq,hkv,d,bs,layout", [(32, 8, 128, 16, "NHD"), (32, 8, 128, 16, "HND"), (28, 4, 128, 16, "NHD"),
                                                (16, 1, 128, 32, "NHD"), (8, 2, 64, 16, "NHD"), (4, 2, 256, 16, "NHD")])
def test_decode_matches_oracle(gpu_device, hq, hkv, d, bs, layout):
    ctx = [1000, 3, 517, 64, 4097, 33]
    kv, lay, bt, q, sl, cu = _fp8_case(ctx, [1] * len(ctx), hq, hkv, d, bs, seed=hq + d, layout=layout)
    scale = 1 / math.sqrt(d)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True,
                                       code_type=oracle.CODE_FP8)
    got, lse = _attend(gpu_device, kv, layout, bt, q, sl, cu, 1, scale, lse=True)
    T.assert_close_attn(got, want, what=f"fp8 decode {hq}/{hkv} d{d} {layout}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


def test_decode_outliers_fp32_out(gpu_device):
    """Outlier-heavy sources (large scales, many subnormal codes) with an fp32 output: kernel error alone."""
    ctx = [3000, 513]
    kv, lay, bt, q, sl, cu = _fp8_case(ctx, [1, 1], 32, 8, 128, 16, seed=9, outlier=True)
    scale = 1 / math.sqrt(128)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, code_type=oracle.CODE_FP8)
    got = _attend(gpu_device, kv, "NHD", bt, q, sl, cu, 1, scale, out_dtype=torch.float32)
    T.assert_close_attn(got, want, atol=4e-3, rtol=4e-3, what="fp8 decode outliers")


def test_mixed_batch_matches_oracle(gpu_device):
    ctx = [700, 33, 129, 64, 257, 5]
    qls = [1, 33, 100, 1, 17, 5]
    kv, lay, bt, q, sl, cu = _fp8_case(ctx, qls, 32, 8, 128, 16, seed=5)
    scale = 1 / math.sqrt(128)
    want = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, code_type=oracle.CODE_FP8)
    got = _attend(gpu_device, kv, "NHD", bt, q, sl, cu, max(qls), scale)
    T.assert_close_attn(got, want, what="fp8 mixed batch")


@pytest.mark.parametrize("hq,hkv,d,qls,window,cap", [
    (32, 8, 128, [300, 1, 64, 2048], 0, 0.0),      # long chunks: the workgroup-shared fp16 tile expands fp8 codes
    (28, 4, 128, [257, 33, 1, 700], 0, 0.0),       # 7 q heads per kv head
    (16, 8, 64, [500, 100, 1, 90], 0, 0.0),
    (32, 8, 128, [300, 1, 64, 900], 128, 0.0),     # its window / soft-cap instantiation
    (32, 8, 128, [300, 1, 64, 900], 0, 30.0),
    (8, 8, 128, [40, 1, 63, 17], 0, 0.0),          # fewer than 64 columns: the per-wave tile
])
def test_prefill_chunks_both_tiles(gpu_device, hq, hkv, d, qls, window, cap):
    """fp8 codes through both prefill kernels, outlier-heavy sources (large scales, many subnormal codes)."""
    ctx = [q + extra for q, extra in zip(qls, [700, 2000, 0, 133])]
    kv, lay, bt, q, sl, cu = _fp8_case(ctx, qls, hq, hkv, d, 16, seed=hq + d + window, outlier=True)
    scale = 1 / math.sqrt(d)
    want, want_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True,
                                       sliding_window=window, soft_cap=cap, code_type=oracle.CODE_FP8)
    dev = gpu_device
    kvd = T.to_device_cache(kv, dev, "NHD")
    k, v = L.key_value_views(kvd)
    ks, vs = L.scale_views(kvd)
    out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
    ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), int(sl.max()), scale, True,
                          window_size=(window - 1, 0) if window else (-1, -1), softcap=cap, block_table=bt.to(dev),
                          k_scale_cache=ks, v_scale_cache=vs, kv_quant_mode=FP8, lse=lse)
    torch.cuda.synchronize()
    T.assert_close_attn(out, want, what=f"fp8 prefill {hq}/{hkv} d{d} window {window} cap {cap}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


def test_backend_serves_fp8_per_token_head(gpu_device):
    dev = gpu_device
    hq, hkv, d, bs, nb = 32, 8, 128, 16, 60
    ctx = [257, 31, 5]
    B = len(ctx)
    g = torch.Generator().manual_seed(17)
    assert Int8AttentionBackend.validate_configuration(kv_cache_dtype="fp8_per_token_head", head_size=d,
                                                       dtype=torch.bfloat16, block_size=bs) == []
    shape = Int8AttentionBackend.get_kv_cache_shape(nb, bs, hkv, d, "fp8_per_token_head")
    assert shape == (nb, hkv, bs, 2 * (d + 4))
    kv_cache = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD")
    kv_cpu, views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    views[2].fill_(1.0)
    views[3].fill_(1.0)
    bt = T.make_block_tables(ctx, bs, nb, g)
    impl = Int8AttentionBackend.get_impl_cls()(hq, d, 1 / math.sqrt(d), hkv, kv_cache_dtype="fp8_per_token_head")
    layer = types.SimpleNamespace()
    slots = T.slots_for(bt, ctx, bs)
    for i, c in enumerate(ctx):
        k = torch.randn((c, hkv, d), generator=g).to(torch.bfloat16)
        v = torch.randn((c, hkv, d), generator=g).to(torch.bfloat16)
        impl.do_kv_cache_update(layer, k.to(dev), v.to(dev), kv_cache, slots[i].to(dev))
        oracle.cache_write(k, v, T.storage_bytes(kv_cpu), lay, slots[i], code_type=oracle.CODE_FP8)
    torch.cuda.synchronize()
    assert torch.equal(T.storage_bytes(kv_cache).cpu(), T.storage_bytes(kv_cpu)), "cache bytes differ"
    q = torch.randn((B, hq * d), generator=g).to(torch.bfloat16)
    md = types.SimpleNamespace(num_actual_tokens=B, max_query_len=1, max_seq_len=max(ctx), use_cascade=False,
                               query_start_loc=torch.arange(B + 1, dtype=torch.int32, device=dev),
                               seq_lens=torch.tensor(ctx, dtype=torch.int32, device=dev), causal=True,
                               block_table=bt.to(dev), workspace=None)
    out = torch.zeros((B, hq * d), dtype=torch.bfloat16, device=dev)
    impl.forward(layer, q.to(dev), None, None, kv_cache, md, out)
    torch.cuda.synchronize()
    want = oracle.paged_attn(q.view(B, hq, d), T.storage_bytes(kv_cpu), lay, bt, torch.tensor(ctx, dtype=torch.int32),
                             torch.arange(B + 1, dtype=torch.int32), 1 / math.sqrt(d), code_type=oracle.CODE_FP8)
    T.assert_close_attn(out.view(B, hq, d), want, what="backend fp8")

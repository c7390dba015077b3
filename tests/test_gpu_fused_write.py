"""GPU parity of the decode step that writes its new tokens inside the attention launch
(kvq_paged_attn_int8_fused_write) against the two calls it replaces -- the cache update
(vllm_metax/v1/attention/backends/triton_attn.py:788-840) followed by the attention over the updated
cache (triton_attn.py:688-725): the cache must hold the same bytes afterwards and the output the same
values, and both are checked against the oracle too."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from test_gpu_decode import build_case
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L
from vllm_metax_amd.kv_cache_interface import KVQuantMode

pytestmark = pytest.mark.gpu


def _last_slots(bt, ctx, bs):
    return torch.tensor([int(bt[i, (c - 1) // bs]) * bs + (c - 1) % bs if c > 0 else -1 for i, c in enumerate(ctx)],
                        dtype=torch.int64)


def _both_ways(dev, kv_cpu, layout, bt, q, sl, ctx, key, value, scale, mode=KVQuantMode.INT8_PER_TOKEN_HEAD,
               window=(-1, -1), softcap=0.0, out_dtype=torch.bfloat16, padding=()):
    """`padding`: rows whose slot mapping entry is -1 (cudagraph padding): neither way may write them."""
    bs = L.key_value_views(T.to_device_cache(kv_cpu, dev, layout))[0].shape[1]
    slots = _last_slots(bt, ctx, bs)
    for i in padding:
        slots[i] = -1
    res = []
    for fused in (False, True):
        kv = T.to_device_cache(kv_cpu, dev, layout)
        k, v = L.key_value_views(kv)
        ks, vs = L.scale_views(kv)
        out = torch.full(q.shape, float("nan"), dtype=out_dtype, device=dev)
        lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
        common = dict(block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse, softcap=softcap,
                      window_size=window, kv_quant_mode=mode)
        if fused:
            ops.decode_attention_with_cache_update(q.to(dev), key.to(dev), value.to(dev), k, v, out, sl.to(dev),
                                                   int(sl.max()), scale, **common,
                                                   slot_mapping=slots.to(dev) if padding else None)
        else:
            ops.reshape_and_cache_flash_per_token_head_quant(key.to(dev), value.to(dev), k, v, ks, vs,
                                                             slots.to(dev), kv_quant_mode=mode)
            cu = torch.arange(len(ctx) + 1, dtype=torch.int32, device=dev)
            ops.unified_attention(q.to(dev), k, v, out, cu, 1, sl.to(dev), int(sl.max()), scale, True, **common)
        torch.cuda.synchronize()
        res.append((T.storage_bytes(kv).cpu(), out.cpu(), lse.cpu()))
    return res


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("hq,hkv,d,bs,ctx", [
    (32, 8, 128, 16, [512, 17, 16, 1, 33, 4096, 1000]),     # lengths that end at the first / last slot of a block
    (28, 4, 128, 16, [300, 64, 65, 2049]),                  # two waves per kv head
    (16, 2, 128, 32, [100, 31, 32, 33, 900]),
    (16, 1, 128, 16, [777, 1, 48]),                         # one kv head: eight waves share it
    (32, 8, 64, 16, [200, 1, 1500]),
    (16, 8, 256, 16, [260, 15, 1024]),
    (32, 8, 128, 16, [0, 40, 0, 1]),                        # empty sequences next to live ones
])
def test_fused_write_equals_write_then_attention(gpu_device, layout, hq, hkv, d, bs, ctx):
    kv, lay, bt, q, sl, cu = build_case(ctx, hq, hkv, d, bs, layout, seed=hq + hkv + d + bs, poison=False)
    g = torch.Generator().manual_seed(5)
    key = torch.randn((len(ctx), hkv, d), generator=g).to(torch.bfloat16)
    value = (torch.randn((len(ctx), hkv, d), generator=g) * 3).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    (cache_a, out_a, lse_a), (cache_b, out_b, lse_b) = _both_ways(gpu_device, kv, layout, bt, q, sl, ctx, key, value, scale)
    assert torch.equal(cache_a, cache_b), "the fused write left other bytes in the cache than the write kernel"
    assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16)), "outputs differ"
    assert torch.equal(lse_a.view(torch.int32), lse_b.view(torch.int32)), "lse differs"
    # and against the oracle: its cache write, then its attention
    ref = T.storage_bytes(kv).clone()
    live = [i for i, c in enumerate(ctx) if c > 0]
    oracle.cache_write(key[live], value[live], ref, lay, _last_slots(bt, ctx, bs)[live])
    assert torch.equal(cache_b, ref), "the fused write's cache differs from the oracle's"
    want = oracle.paged_attn(q, ref, lay, bt, sl, cu, scale)
    rows = torch.tensor(live)
    T.assert_close_attn(out_b[rows], want[rows], what="fused write + decode")


@pytest.mark.parametrize("hkv", [8, 2])
def test_fused_write_skips_padding_rows(gpu_device, hkv):
    """Rows whose slot_mapping entry is negative are padding (cache_kernels.cu:322-326): their sequence length
    may still be positive, and the cache bytes at their last position must stay what they were."""
    ctx = [300, 48, 1000, 17, 64]
    kv, lay, bt, q, sl, cu = build_case(ctx, 16, hkv, 128, 16, "HND", seed=21, poison=False)
    g = torch.Generator().manual_seed(4)
    key = torch.randn((len(ctx), hkv, 128), generator=g).to(torch.bfloat16)
    value = torch.randn((len(ctx), hkv, 128), generator=g).to(torch.bfloat16)
    before = T.storage_bytes(kv).clone()
    (cache_a, out_a, _), (cache_b, out_b, _) = _both_ways(gpu_device, kv, "HND", bt, q, sl, ctx, key, value, 0.088,
                                                          padding=(1, 4))
    assert torch.equal(cache_a, cache_b), "a padding row was written (or a live one was not)"
    assert not torch.equal(cache_b, before)
    assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_fused_write_source_types(gpu_device, dtype):
    ctx = [333, 16, 1, 2000]
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "HND", seed=3, poison=False)
    g = torch.Generator().manual_seed(9)
    key = torch.randn((4, 8, 128), generator=g).to(dtype)
    value = torch.randn((4, 8, 128), generator=g).to(dtype)
    key[1, 3] = 0          # an all-zero row: scale floor / zero scale for fp16
    (cache_a, out_a, _), (cache_b, out_b, _) = _both_ways(gpu_device, kv, "HND", bt, q, sl, ctx, key, value, 0.088)
    assert torch.equal(cache_a, cache_b)
    assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16))


def test_fused_write_fp8_codes_window_and_softcap(gpu_device):
    ctx = [700, 130, 4000]
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "HND", seed=11, poison=False)
    g = torch.Generator().manual_seed(2)
    key = torch.randn((3, 8, 128), generator=g).to(torch.bfloat16)
    value = torch.randn((3, 8, 128), generator=g).to(torch.bfloat16)
    for mode, window, cap in [(KVQuantMode.FP8_PER_TOKEN_HEAD, (-1, -1), 0.0),
                              (KVQuantMode.INT8_PER_TOKEN_HEAD, (255, 0), 0.0),
                              (KVQuantMode.INT8_PER_TOKEN_HEAD, (-1, -1), 30.0)]:
        (cache_a, out_a, _), (cache_b, out_b, _) = _both_ways(gpu_device, kv, "HND", bt, q, sl, ctx, key, value, 0.088,
                                                              mode=mode, window=window, softcap=cap)
        assert torch.equal(cache_a, cache_b), (mode, window, cap)
        assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16)), (mode, window, cap)


def test_fused_write_strided_sources_and_full_size(gpu_device):
    """The C2 shape; key / value are the two halves of one projection output (row stride 2 * Hkv * D)."""
    dev = gpu_device
    g = torch.Generator().manual_seed(0)
    ctx = torch.randint(1024, 8193, (64,), generator=g).tolist()
    kv, lay, bt, q, sl, cu = build_case(ctx, 32, 8, 128, 16, "HND", seed=1, poison=False)
    kvproj = torch.randn((64, 2, 8, 128), generator=g).to(torch.bfloat16)
    key, value = kvproj[:, 0], kvproj[:, 1]
    (cache_a, out_a, _), (cache_b, out_b, _) = _both_ways(dev, kv, "HND", bt, q, sl, ctx, key, value, 0.088)
    assert torch.equal(cache_a, cache_b)
    assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16))


# ---------------------------------------------------------------------------------------------
# MLA: kvq_mla_decode_int8_fused_write against concat_and_cache_mla + mla_decode_int8
# (vllm_metax/v1/attention/backends/mla/triton_mla.py:226-295 does the two in two steps)
# ---------------------------------------------------------------------------------------------
R, P = 512, 64


def _mla_both_ways(dev, cache_cpu, bt, sl, ctx, bs, q, kv_c, k_pe, scale):
    res = []
    for fused in (False, True):
        cache = cache_cpu.clone().to(dev)
        B, H, _ = q.shape
        o = torch.full((B, H, R), float("nan"), dtype=q.dtype, device=dev)
        lse = torch.full((B, H), float("nan"), dtype=torch.float32, device=dev)
        if fused:
            ops.mla_decode_with_cache_update(q.to(dev), kv_c.to(dev), k_pe.to(dev), cache, o, lse, bt.to(dev),
                                             sl.to(dev), scale, R)
        else:
            ops.concat_and_cache_mla(kv_c.to(dev), k_pe.to(dev), cache, _last_slots(bt, ctx, bs).to(dev))
            ops.mla_decode_int8(q.to(dev), cache, o, lse, bt.to(dev), sl.to(dev), scale, R)
        torch.cuda.synchronize()
        res.append((T.storage_bytes(cache).cpu(), o.cpu(), lse.cpu()))
    return res


def _same_bits(a, b):
    return torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


@pytest.mark.parametrize("bs,heads,ctx", [
    (64, 128, [300, 1, 64, 2049, 65, 33, 32]),      # many splits per sequence: the row is written before the tiles
    (16, 16, [17, 33, 511, 1, 16, 32, 64, 97]),     # one head tile; lengths that end at the first / last row of a tile
    (64, 20, [5, 0, 95, 1000, 31, 0, 32]),          # empty sequences next to live ones; part-filled 128-head block
    (64, 160, [70, 300, 33, 129]),                  # two 128-head blocks write the same row
    (16, 5, [5, 95, 1000, 31, 32, 4097]),
    (32, 8, [16384, 16385]),                        # one head tile, 64 splits
    (16, 16, [700, 701, 672, 673, 641, 400] * 44),  # one split per sequence: a wave has many tiles, the row is written late
    (16, 16, [2000, 2017, 1985, 3000] * 18),        # four splits of 16 tiles and more
    (32, 128, [2048, 4096, 4065, 3000] * 9),        # 128 heads, 36 sequences: long splits, the row is written late
])
def test_mla_fused_write_equals_write_then_decode(gpu_device, bs, heads, ctx):
    cache, lay, bt, sl = T.build_mla_cache(ctx, bs, seed=bs + heads, dtype=torch.bfloat16, poison=False)
    g = torch.Generator().manual_seed(13)
    B = len(ctx)
    q = torch.randn((B, heads, R + P), generator=g).to(torch.bfloat16)
    kv_c = (torch.randn((B, R), generator=g) * 2).to(torch.bfloat16)
    k_pe = (torch.randn((B, P), generator=g) * 2).to(torch.bfloat16)
    scale = (128 + 64) ** -0.5
    (cache_a, out_a, lse_a), (cache_b, out_b, lse_b) = _mla_both_ways(gpu_device, cache, bt, sl, ctx, bs, q, kv_c, k_pe, scale)
    assert torch.equal(cache_a, cache_b), "the fused write left other bytes in the cache than the write kernel"
    live = torch.tensor([i for i, c in enumerate(ctx) if c > 0])
    assert _same_bits(out_a[live], out_b[live]), "outputs differ"
    assert _same_bits(lse_a[live], lse_b[live]), "lse differs"
    # the cache against the oracle's write, and (where the oracle is quick) the output against its decode
    ref = cache.clone()
    oracle.mla_cache_write(kv_c[live], k_pe[live], ref, lay, _last_slots(bt, ctx, bs)[live])
    assert torch.equal(cache_b, T.storage_bytes(ref)), "the fused write's cache differs from the oracle's"
    if sum(ctx) * heads <= 1 << 20:
        want, want_lse = oracle.mla_decode(q, ref, lay, bt, sl, scale)
        T.assert_close_attn(out_b[live], want[live], what="mla fused write + decode")
        torch.testing.assert_close(lse_b[live], want_lse[live], atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("heads", [16, 128])
def test_mla_fused_write_source_types_and_strides(gpu_device, dtype, heads):
    """fp16 / fp32 rows (the query has the rows' type), an all-zero row, kv_c and k_pe as two slices of one
    projection output (row stride R + P)."""
    ctx = [333, 16, 1, 2000, 3000, 777] * 8
    bs = 16
    cache, lay, bt, sl = T.build_mla_cache(ctx, bs, seed=3, dtype=torch.bfloat16, poison=False)
    g = torch.Generator().manual_seed(9)
    B = len(ctx)
    q = torch.randn((B, heads, R + P), generator=g).to(dtype)
    proj = torch.randn((B, R + P), generator=g).to(dtype)
    proj[1] = 0
    kv_c, k_pe = proj[:, :R], proj[:, R:]
    (cache_a, out_a, lse_a), (cache_b, out_b, lse_b) = _mla_both_ways(gpu_device, cache, bt, sl, ctx, bs, q, kv_c, k_pe, 0.072)
    assert torch.equal(cache_a, cache_b)
    assert _same_bits(out_a, out_b) and _same_bits(lse_a, lse_b)


def test_mla_fused_write_rejects_bad_arguments(gpu_device):
    dev = gpu_device
    cache, lay, bt, sl = T.build_mla_cache([40, 50], 16, seed=1, poison=False)
    q = torch.zeros((2, 16, R + P), dtype=torch.bfloat16, device=dev)
    o = torch.zeros((2, 16, R), dtype=torch.bfloat16, device=dev)
    kv_c = torch.zeros((2, R), dtype=torch.bfloat16, device=dev)
    k_pe = torch.zeros((2, P), dtype=torch.bfloat16, device=dev)
    args = (cache.to(dev), o, None, bt.to(dev), sl.to(dev), 0.1, R)
    with pytest.raises(RuntimeError, match="one row per sequence"):
        ops.mla_decode_with_cache_update(q, kv_c[:1], k_pe, *args)
    with pytest.raises(RuntimeError, match="one dtype"):
        ops.mla_decode_with_cache_update(q, kv_c, k_pe.float(), *args)
    with pytest.raises(RuntimeError, match="4-byte aligned"):
        ops.mla_decode_with_cache_update(q, torch.zeros((2, R + 1), dtype=torch.bfloat16, device=dev)[:, 1:], k_pe, *args)

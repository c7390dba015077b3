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
               window=(-1, -1), softcap=0.0, out_dtype=torch.bfloat16):
    bs = L.key_value_views(T.to_device_cache(kv_cpu, dev, layout))[0].shape[1]
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
                                                   int(sl.max()), scale, **common)
        else:
            ops.reshape_and_cache_flash_per_token_head_quant(key.to(dev), value.to(dev), k, v, ks, vs,
                                                             _last_slots(bt, ctx, bs).to(dev), kv_quant_mode=mode)
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

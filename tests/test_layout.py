"""Closed-form checks of the cache layout algebra (shape, stride order, inline scale views)."""
import pytest
import torch

from vllm_metax_amd import layout as L


def test_shape_and_stride_order():
    assert L.kv_cache_shape(40000, 16, 8, 128, "int8_per_token_head") == (40000, 8, 16, 264)
    assert L.kv_cache_shape(10, 32, 4, 64, "auto") == (10, 4, 32, 128)
    with pytest.raises(ValueError):
        L.kv_cache_shape(10, 24, 4, 64)
    assert L.kv_cache_stride_order(layout="NHD") == (0, 2, 1, 3)
    assert L.kv_cache_stride_order(layout="HND") == (0, 1, 2, 3)
    assert L.kv_cache_stride_order(True, layout="NHD") == (1, 0, 3, 2, 4)
    assert L.kv_cache_stride_order(True, layout="HND") == (1, 2, 0, 3, 4)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_views_reproduce_record_bytes(layout):
    nb, bs, hkv, d = 5, 16, 3, 128
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device="cpu", layout=layout)
    assert kv.shape == (nb, hkv, bs, 2 * (d + 4))
    if layout == "NHD":
        assert kv.stride() == (bs * hkv * 264, 264, hkv * 264, 1)
    else:
        assert kv.stride() == (hkv * bs * 264, bs * 264, 264, 1)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    assert k.shape == (nb, bs, hkv, d + 4) and ks.shape == (nb, bs, hkv)
    g = torch.Generator().manual_seed(0)
    kc = torch.randint(-128, 128, (nb, bs, hkv, d), generator=g, dtype=torch.int8)
    vc = torch.randint(-128, 128, (nb, bs, hkv, d), generator=g, dtype=torch.int8)
    ksv = torch.rand((nb, bs, hkv), generator=g) + 0.5
    vsv = torch.rand((nb, bs, hkv), generator=g) + 0.5
    k[..., :d] = kc
    v[..., :d] = vc
    ks.copy_(ksv)
    vs.copy_(vsv)
    # re-read the raw storage record by record: [K | ks | V | vs]
    raw = torch.tensor([], dtype=torch.uint8).set_(kv.untyped_storage())
    geom = L.geometry_from_cache(kv)
    assert (geom.k_off, geom.ks_off, geom.v_off, geom.vs_off) == (0, d, d + 4, 2 * d + 4)
    for b, s, h in [(0, 0, 0), (4, 15, 2), (2, 7, 1)]:
        o = b * geom.stride_block + s * geom.stride_slot + h * geom.stride_head
        rec = raw[o:o + 264]
        assert torch.equal(rec[:d].view(torch.int8), kc[b, s, h])
        assert rec[d:d + 4].view(torch.float32).item() == ksv[b, s, h].item()
        assert torch.equal(rec[d + 4:2 * d + 4].view(torch.int8), vc[b, s, h])
        assert rec[2 * d + 4:].view(torch.float32).item() == vsv[b, s, h].item()
    # a block is one opaque contiguous byte range in both orders (swap/copy_blocks friendly)
    assert geom.stride_block == hkv * bs * 264


def test_mla_views():
    nb, bs = 3, 64
    c = L.allocate_mla_cache(nb, bs, 576, device="cpu")
    assert c.shape == (nb, bs, 580)
    codes, scales = L.mla_cache_views(c)
    assert codes.shape == (nb, bs, 576) and scales.shape == (nb, bs)
    codes[1, 5, :] = 7
    scales[1, 5] = 0.25
    raw = c.reshape(nb, -1).view(torch.uint8)
    assert (raw[1, 5 * 576:6 * 576] == 7).all()
    assert raw[1, bs * 576 + 5 * 4: bs * 576 + 6 * 4].view(torch.float32).item() == 0.25
    g = L.mla_geometry(c, 512)
    assert (g.stride_block, g.stride_row, g.scale_off, g.rope_dim) == (bs * 580, 576, bs * 576, 64)
    assert g.stride_block % 16 == 0 and g.stride_row % 16 == 0

"""The committed golden fixture (tests/golden/kvq_golden_small.pt, written by
tests/golden/make_golden.py): the oracle still reproduces it (CPU), and the HIP kernels reproduce
it through the C ABI (GPU) -- bit-exact for cache bytes, within tolerance for attention."""
import os

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import layout as L

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kvq_golden_small.pt")


@pytest.fixture(scope="module")
def G():
    return torch.load(PATH, weights_only=True)


def _layout(G, layout="NHD"):
    kv, views, lay = T.cpu_cache(int(G["nb"]), int(G["bs"]), int(G["hkv"]), int(G["d"]), layout)
    return kv, views, lay


def test_oracle_reproduces_golden(G):
    kv, views, lay = _layout(G)
    hkv, d = int(G["hkv"]), int(G["d"])
    oracle.cache_write(G["key"], G["value"], T.storage_bytes(kv), lay, G["slots"])
    assert torch.equal(T.storage_bytes(kv), G["cache_bytes"])
    out, lse = oracle.paged_attn(G["q"], G["cache_bytes"], lay, G["block_table"], G["ctx"], G["cu"],
                                 float(G["scale"]), return_lse=True)
    assert torch.equal(out, G["out"]) and torch.equal(lse, G["lse"])
    mc = L.allocate_mla_cache(int(G["mla_nb"]), int(G["mla_bs"]), 576, device="cpu")
    codes, scales = L.mla_cache_views(mc)
    mlay = oracle.MlaLayout.from_views(mc, codes, scales, 512)
    oracle.mla_cache_write(G["mla_kv_c"], G["mla_k_pe"], mc, mlay, G["mla_slots"])
    assert torch.equal(mc, G["mla_cache"])
    mout, mlse = oracle.mla_decode(G["mla_q"], mc, mlay, G["mla_block_table"], G["mla_ctx"], 192 ** -0.5)
    assert torch.equal(mout, G["mla_out"]) and torch.equal(mlse, G["mla_lse"])


@pytest.mark.gpu
def test_kernels_reproduce_golden(G, gpu_device):
    from vllm_metax_amd import _custom_ops as ops

    dev = gpu_device
    hq, hkv, d, bs, nb = (int(G[k]) for k in ("hq", "hkv", "d", "bs", "nb"))
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    ops.reshape_and_cache_flash_per_token_head_quant(G["key"].to(dev), G["value"].to(dev), k, v, ks, vs, G["slots"].to(dev))
    torch.cuda.synchronize()
    assert torch.equal(T.storage_bytes(kv).cpu(), G["cache_bytes"]), "quantised cache differs from the golden bytes"
    # decode rows of the mixed batch (rows 0, 1.., 6): as a decode-only batch
    qd = G["q"][[0, 1, 6]].contiguous().to(dev)
    out = torch.empty((3, hq, d), dtype=torch.float32, device=dev)
    cu = torch.arange(4, dtype=torch.int32, device=dev)
    ops.unified_attention(qd, k, v, out, cu, 1, G["ctx"].to(dev), int(G["ctx"].max()), float(G["scale"]), True,
                          block_table=G["block_table"].to(dev), k_scale_cache=ks, v_scale_cache=vs)
    torch.cuda.synchronize()
    T.assert_close_attn(out, G["part_reduced"], atol=2e-3, rtol=2e-3, what="golden decode")
    # the fixture's whole mixed batch (decode rows and a prefill chunk through the one varlen entry point),
    # output rows and log-sum-exp
    qm = G["q"].to(dev)
    outm = torch.empty(tuple(G["q"].shape), dtype=torch.float32, device=dev)
    lsem = torch.empty(tuple(G["q"].shape[:2]), dtype=torch.float32, device=dev)
    ops.unified_attention(qm, k, v, outm, G["cu"].to(dev), int(G["qlens"].max()), G["ctx"].to(dev), int(G["ctx"].max()),
                          float(G["scale"]), True, block_table=G["block_table"].to(dev), k_scale_cache=ks,
                          v_scale_cache=vs, lse=lsem)
    torch.cuda.synchronize()
    T.assert_close_attn(outm, G["out"], atol=4e-3, rtol=4e-3, what="golden mixed batch")
    torch.testing.assert_close(lsem.cpu(), G["lse"], atol=5e-3, rtol=1e-3)
    mc = L.allocate_mla_cache(int(G["mla_nb"]), int(G["mla_bs"]), 576, device=dev)
    ops.concat_and_cache_mla(G["mla_kv_c"].to(dev), G["mla_k_pe"].to(dev), mc, G["mla_slots"].to(dev))
    torch.cuda.synchronize()
    assert torch.equal(mc.cpu(), G["mla_cache"]), "MLA latent cache differs from the golden bytes"
    # MLA decode over the latent cache just written: output and log-sum-exp of the fixture
    mq = G["mla_q"].to(dev)
    mo = torch.empty(tuple(G["mla_out"].shape), dtype=torch.float32, device=dev)
    mlse = torch.empty(tuple(G["mla_lse"].shape), dtype=torch.float32, device=dev)
    ops.mla_decode_int8(mq, mc, mo, mlse, G["mla_block_table"].to(dev), G["mla_ctx"].to(dev), 192 ** -0.5, 512)
    torch.cuda.synchronize()
    T.assert_close_attn(mo, G["mla_out"], atol=4e-3, rtol=4e-3, what="golden mla decode")
    torch.testing.assert_close(mlse.cpu(), G["mla_lse"], atol=5e-3, rtol=1e-3)

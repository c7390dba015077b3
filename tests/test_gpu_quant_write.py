"""GPU parity of the quantise-on-write kernel: the cache bytes (codes AND fp32 scales AND every
untouched byte) must equal the oracle's, bit for bit, through the C ABI."""
import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def _run_case(dev, layout, dtype, hkv, d, bs, nb, num_tokens, pad, seed, kind="normal"):
    g = torch.Generator().manual_seed(seed)
    if kind == "outlier":
        key = T.outlier_sources((num_tokens + pad, hkv, d), g, dtype)
        val = T.outlier_sources((num_tokens + pad, hkv, d), g, dtype)
    else:
        key = torch.randn((num_tokens + pad, hkv, d), generator=g).to(dtype)
        val = torch.randn((num_tokens + pad, hkv, d), generator=g).to(dtype)
    if kind == "zeros":
        key[::3] = 0
        val[1::3] = 0
    slots = torch.randperm(nb * bs, generator=g)[:num_tokens].to(torch.int64)
    slots[torch.rand(num_tokens, generator=g) < 0.1] = -1          # padding tokens
    kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, layout, fill=0x11)
    oracle.cache_write(key, val, T.storage_bytes(kv_cpu), lay, slots)

    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout=layout, fill=0x11)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    ops.reshape_and_cache_flash_per_token_head_quant(key.to(dev), val.to(dev), k, v, ks, vs, slots.to(dev))
    torch.cuda.synchronize()
    got = T.storage_bytes(kv).cpu()
    want = T.storage_bytes(kv_cpu)
    if not torch.equal(got, want):
        bad = (got != want).nonzero().flatten()
        raise AssertionError(f"{bad.numel()} bytes differ, first at {bad[:8].tolist()}")


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_bit_exact_llama_shape(gpu_device, layout, dtype):
    _run_case(gpu_device, layout, dtype, hkv=8, d=128, bs=16, nb=64, num_tokens=300, pad=5, seed=1)


@pytest.mark.parametrize("hkv,d,bs", [(4, 128, 16), (1, 64, 32), (2, 256, 16), (3, 80, 16)])
def test_bit_exact_other_shapes(gpu_device, hkv, d, bs):
    _run_case(gpu_device, "NHD", torch.bfloat16, hkv, d, bs, nb=20, num_tokens=100, pad=0, seed=2)


@pytest.mark.parametrize("kind", ["outlier", "zeros"])
def test_bit_exact_outliers_and_zero_rows(gpu_device, kind):
    _run_case(gpu_device, "NHD", torch.bfloat16, 8, 128, 16, nb=40, num_tokens=256, pad=0, seed=3, kind=kind)
    _run_case(gpu_device, "HND", torch.float32, 8, 128, 16, nb=40, num_tokens=256, pad=0, seed=4, kind=kind)


def test_ties_on_device(gpu_device):
    """x / scale = k + 0.5 exactly: half-to-even on the device too."""
    dev = gpu_device
    kv = L.allocate_kv_cache(2, 16, 1, 128, device=dev, layout="NHD")
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    row = torch.tensor([127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 126.5, -126.5] + [0.0] * 118)
    key = row.reshape(1, 1, 128).to(dev)
    ops.reshape_and_cache_flash_per_token_head_quant(key, key.clone(), k, v, ks, vs, torch.tensor([3], device=dev))
    torch.cuda.synchronize()
    assert ks[0, 3, 0].item() == 1.0
    assert k[0, 3, 0, :10].cpu().tolist() == [127, 0, 2, 2, 4, 0, -2, -2, 126, -126]


def test_full_size_roundtrip_property(gpu_device):
    """At the Qwen2-7B mixed-batch write size (8252 tokens, 4 kv heads): every written record
    satisfies |code*scale - x| <= scale/2 and scale == absmax/127, unwritten records untouched."""
    dev = gpu_device
    Tn, hkv, d, bs = 8252, 4, 128, 16
    nb = (Tn + bs - 1) // bs + 8
    g = torch.Generator().manual_seed(5)
    key = torch.randn((Tn, hkv, d), generator=g).to(torch.bfloat16).to(dev)
    val = torch.randn((Tn, hkv, d), generator=g).to(torch.bfloat16).to(dev)
    slots = torch.randperm(nb * bs, generator=g)[:Tn].to(dev)
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="NHD", fill=0)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    ops.reshape_and_cache_flash_per_token_head_quant(key, val, k, v, ks, vs, slots)
    torch.cuda.synchronize()
    kc = k.reshape(-1, hkv, d + 4)[slots][..., :d].float()
    sc = ks.reshape(-1, hkv)[slots]
    # expected scale on the CPU: torch's GPU kernel turns "/ 127.0" into a multiply by a reciprocal
    want_sc = key.float().abs().amax(-1).cpu() / 127.0
    assert bool(torch.equal(sc.cpu(), want_sc))
    err = (kc.double().cpu() * sc.double().cpu()[..., None] - key.double().cpu()).abs()
    # half a step, plus the fp32 rounding of the quotient itself (|q| <= 127, ulp 2^-17 at that size)
    excess = (err - 0.5 * sc.double().cpu()[..., None] * (1 + 1e-4)).max().item()
    assert excess <= 0, excess
    written = torch.zeros(nb * bs, dtype=torch.bool, device=dev)
    written[slots] = True
    assert bool((k.reshape(-1, hkv, d + 4)[~written] == 0).all()) and bool((v.reshape(-1, hkv, d + 4)[~written] == 0).all())


def test_errors_are_loud(gpu_device):
    dev = gpu_device
    kv = L.allocate_kv_cache(2, 16, 2, 128, device=dev)
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    key = torch.zeros((4, 2, 128), device=dev, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.reshape_and_cache_flash_per_token_head_quant(key, key, k, v, ks, vs, torch.zeros(4, device=dev, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        ops.reshape_and_cache_flash_per_token_head_quant(key[:, :1], key[:, :1], k, v, ks, vs,
                                                         torch.zeros(4, device=dev, dtype=torch.int64))
    with pytest.raises(RuntimeError):
        ops.reshape_and_cache_flash_per_token_head_quant(key.cpu(), key.cpu(), k, v, ks, vs,
                                                         torch.zeros(4, dtype=torch.int64))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("hq,hkv,d,rot,mode", [
    (32, 8, 128, 128, "int8"), (28, 4, 128, 64, "int8"), (8, 2, 64, 64, "fp8"), (4, 1, 256, 128, "int4"),
    (6, 3, 80, 32, "int8"),
])
def test_fused_rope_and_write_is_rotate_then_write(gpu_device, dtype, is_neox, hq, hkv, d, rot, mode):
    """do_rope_and_kv_cache_update in one launch (the reference declares it and raises,
    vllm_metax/v1/attention/backends/triton_attn.py:833-848): query and key rotated in place bit for bit as the
    oracle's statement of the reference's rotary arithmetic rotates them, cache bytes equal to the oracle's write of
    the rotated key and the value; padded tokens untouched."""
    import oracle
    from vllm_metax_amd.kv_cache_interface import KVQuantMode

    dev = gpu_device
    code = {"int8": oracle.CODE_INT8, "fp8": oracle.CODE_FP8, "int4": oracle.CODE_INT4}[mode]
    qmode = {"int8": KVQuantMode.INT8_PER_TOKEN_HEAD, "fp8": KVQuantMode.FP8_PER_TOKEN_HEAD,
             "int4": KVQuantMode.INT4_PER_TOKEN_HEAD}[mode]
    dstr = {"int8": "int8_per_token_head", "fp8": "fp8_per_token_head", "int4": "int4_per_token_head"}[mode]
    bs, nb, n = 16, 12, 70
    g = torch.Generator().manual_seed(hq + d + rot)
    q = torch.randn((n, hq, d), generator=g).to(dtype)
    k = (torch.randn((n, hkv, d), generator=g) * 2).to(dtype)
    v = torch.randn((n, hkv, d), generator=g).to(dtype)
    positions = torch.randint(0, 500, (n,), generator=g, dtype=torch.int64)
    ang = torch.rand((500, rot // 2), generator=g, dtype=torch.float64) * 6.283
    cos_sin = torch.cat([ang.cos(), ang.sin()], dim=1).to(dtype)
    slots = torch.randperm(nb * bs, generator=g)[:n].to(torch.int64)
    slots[torch.rand(n, generator=g) < 0.15] = -1
    live = slots >= 0
    # the oracle: rotate the live tokens' first `rot` dims, then write
    q_want, k_want = q.clone(), k.clone()
    q_want[live, :, :rot] = oracle.rope_rotate(q[live][..., :rot].contiguous(), positions[live], cos_sin, is_neox)
    k_want[live, :, :rot] = oracle.rope_rotate(k[live][..., :rot].contiguous(), positions[live], cos_sin, is_neox)
    kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, "HND", fill=0x22, code_type=code)
    oracle.cache_write(k_want, v, T.storage_bytes(kv_cpu), lay, slots, code_type=code)
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout="HND", fill=0x22, cache_dtype_str=dstr)
    kc, vc = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    ops.rope_and_cache_per_token_head_quant(positions.to(dev), qd, kd, vd, cos_sin.to(dev), is_neox, kc, vc, ks, vs,
                                            slots.to(dev), kv_quant_mode=qmode)
    torch.cuda.synchronize()
    assert torch.equal(qd.cpu(), q_want), "rotated query differs"
    assert torch.equal(kd.cpu(), k_want), "rotated key differs"
    assert torch.equal(vd.cpu(), v)
    got, want = T.storage_bytes(kv).cpu(), T.storage_bytes(kv_cpu)
    assert torch.equal(got, want), f"{(got != want).sum().item()} cache bytes differ"

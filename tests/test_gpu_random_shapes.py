"""Randomised parity sweeps on the GPU, through the C ABI, against the oracle: shapes, lengths, dtypes, memory
orders and options drawn from a seeded generator, so that combinations nobody wrote down by hand are covered too
(the hand-written cases follow the reference's own parametrisations,
tests/kernels/attention/test_triton_unified_attention.py and test_mla_decode_cpu.py).  Every case is fully
determined by its number; a failure names it."""
import math
import random

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L
from vllm_metax_amd.kv_cache_interface import KVQuantMode

pytestmark = pytest.mark.gpu

_LENGTHS = [0, 1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65]


def _draw_paged(case):
    rng = random.Random(9176 * case + 11)
    d = rng.choice([64, 128, 128, 128, 256])
    hkv = rng.choice([1, 2, 4, 8, 8])
    group = rng.choice([1, 2, 4, 7, 8]) if hkv < 8 else rng.choice([1, 2, 4])
    cfg = dict(d=d, hkv=hkv, hq=hkv * group, bs=rng.choice([16, 16, 32, 64, 128]), layout=rng.choice(["NHD", "HND"]),
               fp8=rng.random() < 0.2, window=rng.choice([0, 0, 0, 17, 64, 300]), cap=rng.choice([0.0, 0.0, 0.0, 20.0]),
               qdt=rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32]),
               vmag=rng.choice([0.1, 1.0, 5.0]))
    cfg["odt"] = rng.choice([cfg["qdt"], torch.bfloat16, torch.float32])
    decode_only = rng.random() < 0.5
    ctx, qls = [], []
    for _ in range(rng.randint(1, 10)):
        c = rng.choice(_LENGTHS + [rng.randint(1, 200), rng.randint(1, 1500), rng.randint(1, 3000)])
        ql = 1 if (decode_only or c == 0) else rng.choice([1, 1, min(c, rng.randint(2, 40)), min(c, rng.randint(2, 300)), c])
        ctx.append(c)
        qls.append(ql)
    if sum(ctx) == 0:
        ctx[0] = 5
    cfg.update(ctx=ctx, qls=qls)
    # later additions draw last, so that the cases above keep the shapes they always had
    cfg["int4"] = (not cfg["fp8"]) and rng.random() < 0.25
    cfg["sinks"] = rng.random() < 0.25
    cfg["invariant"] = rng.random() < 0.15
    cfg["alibi"] = rng.random() < 0.2
    return cfg


@pytest.mark.parametrize("block", range(12))
def test_paged_attention_random_cases(gpu_device, block):
    dev = gpu_device
    for case in range(12 * block, 12 * block + 12):
        c = _draw_paged(case)
        what = f"case {case}: {c}"
        ctx, qls, bs, hkv, d = c["ctx"], c["qls"], c["bs"], c["hkv"], c["d"]
        g = torch.Generator().manual_seed(case)
        nb = sum((n + bs - 1) // bs for n in ctx) + 5
        code = oracle.CODE_FP8 if c["fp8"] else (oracle.CODE_INT4 if c["int4"] else oracle.CODE_INT8)
        kv, views, lay = T.cpu_cache(nb, bs, hkv, d, c["layout"], code_type=code)
        base = T.storage_bytes(kv)
        base.fill_(0xFF)                                     # NaN scales wherever nothing is written
        bt = T.make_block_tables(ctx, bs, nb, g)
        for i, slots in enumerate(T.slots_for(bt, ctx, bs)):
            if slots.numel() > 0:
                ksrc = torch.randn((ctx[i], hkv, d), generator=g).to(torch.bfloat16)
                vsrc = (torch.randn((ctx[i], hkv, d), generator=g) * c["vmag"]).to(torch.bfloat16)
                oracle.cache_write(ksrc, vsrc, base, lay, slots, code_type=code)
        q = torch.randn((sum(qls), c["hq"], d), generator=g).to(c["qdt"])
        sl = torch.tensor(ctx, dtype=torch.int32)
        cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
        scale = 1 / math.sqrt(d)
        sinks = (torch.randn(c["hq"], generator=g) * 2).float() if c["sinks"] else None
        # ALiBi slopes between 2^-8 and 2 (drawn after everything else, so that the other cases keep their data)
        slopes = torch.exp2(torch.rand(c["hq"], generator=g) * 9 - 8).float() if c["alibi"] else None
        want, want_lse = oracle.paged_attn(q, base, lay, bt, sl, cu, scale, return_lse=True,
                                           sliding_window=c["window"], soft_cap=c["cap"], code_type=code, sinks=sinks,
                                           alibi_slopes=slopes)
        kvd = T.to_device_cache(kv, dev, c["layout"], code_type=code)
        k, v = L.key_value_views(kvd)
        ks, vs = L.scale_views(kvd)
        out = torch.full(q.shape, float("nan"), dtype=c["odt"], device=dev)
        lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
        mode = KVQuantMode.FP8_PER_TOKEN_HEAD if c["fp8"] else (
            KVQuantMode.INT4_PER_TOKEN_HEAD if c["int4"] else KVQuantMode.INT8_PER_TOKEN_HEAD)
        before = ops.set_batch_invariant(c["invariant"])
        try:
            ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), max(qls), sl.to(dev), int(sl.max()), scale, True,
                                  window_size=(c["window"] - 1, 0) if c["window"] else (-1, -1), softcap=c["cap"],
                                  block_table=bt.to(dev), k_scale_cache=ks, v_scale_cache=vs, lse=lse,
                                  kv_quant_mode=mode, sinks=None if sinks is None else sinks.to(dev),
                                  alibi_slopes=None if slopes is None else slopes.to(dev))
            torch.cuda.synchronize()
        finally:
            ops.set_batch_invariant(before)
        live = torch.tensor([ctx[i] > 0 for i in range(len(ctx)) for _ in range(qls[i])])
        T.assert_close_attn(out[live], want[live], what=what)        # atol 2e-2, rtol 1e-2
        torch.testing.assert_close(lse.cpu()[live], want_lse[live], atol=5e-3, rtol=1e-3, msg=what)
        if (~live).any():
            assert torch.equal(out.float().cpu()[~live], torch.zeros_like(want[~live])), what


def _draw_mla(case):
    rng = random.Random(5501 * case + 3)
    heads = rng.choice([1, 5, 8, 16, 16, 17, 32, 64, 128, 128, 160])
    ctx = [rng.choice(_LENGTHS + [rng.randint(1, 300), rng.randint(1, 2500), rng.randint(1, 6000)])
           for _ in range(rng.choice([1, 2, 3, 6, 12, 40]))]
    if sum(ctx) == 0:
        ctx[0] = 7
    return dict(heads=heads, bs=rng.choice([16, 32, 64, 128]), ctx=ctx, fused=rng.random() < 0.5,
                qdt=rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32]),
                split_q=rng.random() < 0.3)


@pytest.mark.parametrize("block", range(6))
def test_mla_decode_random_cases(gpu_device, block):
    """MLA decode, half of the cases with the step's new rows written inside the launch (the oracle then writes the
    rows first)."""
    dev = gpu_device
    R, P = 512, 64
    for case in range(8 * block, 8 * block + 8):
        c = _draw_mla(case)
        what = f"case {case}: {c}"
        ctx, bs, H = c["ctx"], c["bs"], c["heads"]
        cache, lay, bt, sl = T.build_mla_cache(ctx, bs, seed=case, dtype=torch.bfloat16, poison=False)
        g = torch.Generator().manual_seed(1000 + case)
        B = len(ctx)
        q = torch.randn((B, H, R + P), generator=g).to(c["qdt"])
        scale = (128 + 64) ** -0.5
        cache_d = cache.clone().to(dev)
        o = torch.full((B, H, R), float("nan"), dtype=c["qdt"], device=dev)
        lse = torch.full((B, H), float("nan"), dtype=torch.float32, device=dev)
        qd = q.to(dev)
        q_arg = (qd[..., :R], qd[..., R:]) if c["split_q"] else qd
        live = torch.tensor([n > 0 for n in ctx])
        if c["fused"]:
            kv_c = (torch.randn((B, R), generator=g) * 2).to(c["qdt"])
            k_pe = (torch.randn((B, P), generator=g) * 2).to(c["qdt"])
            slots = torch.tensor([int(bt[i, (n - 1) // bs]) * bs + (n - 1) % bs if n > 0 else -1 for i, n in enumerate(ctx)])
            oracle.mla_cache_write(kv_c[live], k_pe[live], cache, lay, slots[live])
            ops.mla_decode_with_cache_update(q_arg, kv_c.to(dev), k_pe.to(dev), cache_d, o, lse, bt.to(dev), sl.to(dev), scale, R)
        else:
            ops.mla_decode_int8(q_arg, cache_d, o, lse, bt.to(dev), sl.to(dev), scale, R)
        torch.cuda.synchronize()
        assert torch.equal(T.storage_bytes(cache_d).cpu(), T.storage_bytes(cache)), what
        want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
        if c["qdt"] == torch.float32:
            T.assert_close_attn(o[live], want[live], atol=2e-2, rtol=1e-2, what=what)
        else:
            T.assert_close_attn(o[live], want[live], what=what)
        torch.testing.assert_close(lse.cpu()[live], want_lse[live], atol=5e-3, rtol=1e-3, msg=what)
        if (~live).any():
            assert torch.equal(o.float().cpu()[~live], torch.zeros_like(want[~live])), what


def _draw_write(case):
    rng = random.Random(7717 * case + 5)
    return dict(hkv=rng.choice([1, 2, 3, 4, 8, 16]), d=rng.choice([64, 80, 96, 112, 128, 128, 256]),
                bs=rng.choice([16, 32, 64]), layout=rng.choice(["NHD", "HND"]),
                dtype=rng.choice([torch.bfloat16, torch.float16, torch.float32]), fp8=rng.random() < 0.25,
                tokens=rng.choice([1, 2, 63, 64, 65, rng.randint(1, 400), rng.randint(1, 3000)]),
                mag=rng.choice([1e-12, 1e-6, 1e-3, 1.0, 1.0, 30.0, 3000.0]), zero_rows=rng.random() < 0.3,
                strided=rng.random() < 0.3)


@pytest.mark.parametrize("block", range(6))
def test_cache_write_random_cases_bit_exact(gpu_device, block):
    """Quantise-on-write: every byte of the cache (codes, scales, untouched slots) equals the oracle's, for shapes,
    source types, magnitudes (down to rows below the scale floor) and slot patterns drawn at random; MLA rows too."""
    dev = gpu_device
    for case in range(10 * block, 10 * block + 10):
        c = _draw_write(case)
        what = f"case {case}: {c}"
        g = torch.Generator().manual_seed(case)
        hkv, d, bs, n = c["hkv"], c["d"], c["bs"], c["tokens"]
        nb = (n + bs - 1) // bs + 3
        src = (torch.randn((n, 2, hkv, d), generator=g) * c["mag"]).to(c["dtype"])
        if c["zero_rows"]:
            src[::3, 0] = 0
            src[1::4, 1, hkv - 1] = 0
        if c["strided"]:
            key, val = src[:, 0], src[:, 1]                  # the two halves of one projection output
        else:
            key, val = src[:, 0].contiguous(), src[:, 1].contiguous()
        slots = torch.randperm(nb * bs, generator=g)[:n].to(torch.int64)
        slots[torch.rand(n, generator=g) < 0.1] = -1
        code = oracle.CODE_FP8 if c["fp8"] else oracle.CODE_INT8
        kv_cpu, _, lay = T.cpu_cache(nb, bs, hkv, d, c["layout"], fill=0x11)
        oracle.cache_write(key, val, T.storage_bytes(kv_cpu), lay, slots, code_type=code)
        kv = L.allocate_kv_cache(nb, bs, hkv, d, device=dev, layout=c["layout"], fill=0x11)
        k, v = L.key_value_views(kv)
        ks, vs = L.scale_views(kv)
        srcd = src.to(dev)
        kd, vd = (srcd[:, 0], srcd[:, 1]) if c["strided"] else (srcd[:, 0].contiguous(), srcd[:, 1].contiguous())
        mode = KVQuantMode.FP8_PER_TOKEN_HEAD if c["fp8"] else KVQuantMode.INT8_PER_TOKEN_HEAD
        ops.reshape_and_cache_flash_per_token_head_quant(kd, vd, k, v, ks, vs, slots.to(dev), kv_quant_mode=mode)
        torch.cuda.synchronize()
        assert torch.equal(T.storage_bytes(kv).cpu(), T.storage_bytes(kv_cpu)), what
        # the MLA latent row of the same case: [kv_c | k_pe], one scale per row
        R, P = 512, 64
        rows = (torch.randn((n, R + P), generator=g) * c["mag"]).to(c["dtype"])
        if c["zero_rows"]:
            rows[::5] = 0
        cache_cpu = L.allocate_mla_cache(nb, bs, R + P, device="cpu", fill=0x11)
        codes, scales = L.mla_cache_views(cache_cpu)
        mlay = oracle.MlaLayout.from_views(cache_cpu, codes, scales, R)
        oracle.mla_cache_write(rows[:, :R], rows[:, R:], cache_cpu, mlay, slots)
        cache = L.allocate_mla_cache(nb, bs, R + P, device=dev, fill=0x11)
        rd = rows.to(dev)
        if c["strided"]:
            ops.concat_and_cache_mla(rd[:, :R], rd[:, R:], cache, slots.to(dev))
        else:
            ops.concat_and_cache_mla(rd[:, :R].contiguous(), rd[:, R:].contiguous(), cache, slots.to(dev))
        torch.cuda.synchronize()
        assert torch.equal(T.storage_bytes(cache).cpu(), T.storage_bytes(cache_cpu)), what + " (MLA rows)"

"""GPU parity of the LSE merge kernel and of the MLA latent quantise-on-write, through the C ABI."""
import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,heads,d", [(613, 8, 128), (37, 5, 64), (256, 16, 512)])
def test_merge_attn_states(gpu_device, dtype, tokens, heads, d):
    dev = gpu_device
    g = torch.Generator().manual_seed(tokens + heads)
    po = torch.randn((tokens, heads, d), generator=g).to(dtype)
    so = torch.randn((tokens, heads, d), generator=g).to(dtype)
    pl = torch.randn((heads, tokens), generator=g) * 5
    sl = torch.randn((heads, tokens), generator=g) * 5
    sel = torch.rand((heads, tokens), generator=g)
    pl[sel < 0.05] = float("inf")                      # the reference's test injects +inf LSEs
    sl[(sel > 0.05) & (sel < 0.10)] = float("inf")
    pl[(sel > 0.10) & (sel < 0.12)] = float("-inf")
    both = (sel > 0.12) & (sel < 0.14)
    pl[both] = float("-inf")
    sl[both] = float("-inf")
    want, want_lse = oracle.merge_attn_states(po, pl, so, sl)
    out = torch.empty_like(po, device=dev)
    lse = torch.empty((heads, tokens), dtype=torch.float32, device=dev)
    ops.merge_attn_states(out, po.to(dev), pl.to(dev), so.to(dev), sl.to(dev), output_lse=lse)
    torch.cuda.synchronize()
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=1e-3, rtol=1e-2)
    torch.testing.assert_close(out.float().cpu(), want, **tol)
    torch.testing.assert_close(lse.cpu(), want_lse, atol=1e-5, rtol=1e-5)
    # rows at or beyond the prefix count copy the suffix bit for bit
    out2 = torch.empty_like(po, device=dev)
    ops.merge_attn_states(out2, po.to(dev), pl.to(dev), so.to(dev), sl.to(dev), prefill_tokens_with_context=10)
    torch.cuda.synchronize()
    assert torch.equal(out2[10:].cpu(), so[10:]) and torch.equal(out2[:10].cpu(), out[:10].cpu())


def test_merge_is_the_splitk_algebra(gpu_device):
    """Merging the two halves of a context reproduces attention over the whole context."""
    dev = gpu_device
    g = torch.Generator().manual_seed(3)
    Tn, H, D, n = 5, 4, 64, 200
    q = torch.randn((Tn, H, D), generator=g)
    k = torch.randn((n, H, D), generator=g)
    v = torch.randn((n, H, D), generator=g)
    def attend(ks, vs):
        s = torch.einsum("thd,nhd->htn", q, ks) * 0.125
        return torch.einsum("htn,nhd->thd", torch.softmax(s, -1), vs).contiguous(), torch.logsumexp(s, -1).contiguous()
    o1, l1 = attend(k[:77], v[:77])
    o2, l2 = attend(k[77:], v[77:])
    full, lf = attend(k, v)
    out = torch.empty((Tn, H, D), device=dev)
    lse = torch.empty((H, Tn), device=dev)
    ops.merge_attn_states(out, o1.to(dev), l1.contiguous().to(dev), o2.to(dev), l2.contiguous().to(dev), output_lse=lse)
    torch.testing.assert_close(out.cpu(), full, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(lse.cpu(), lf, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("bs", [16, 64])
def test_mla_cache_write_bit_exact(gpu_device, dtype, bs):
    dev = gpu_device
    R, P, nb, Tn = 512, 64, 9, 150
    g = torch.Generator().manual_seed(bs)
    kv_c = torch.randn((Tn + 3, R), generator=g).to(dtype)
    k_pe = (torch.randn((Tn + 3, P), generator=g) * 4).to(dtype)
    kv_c[7] = 0
    k_pe[7] = 0                                                # an all-zero row
    slots = torch.randperm(nb * bs, generator=g)[:Tn].to(torch.int64)
    slots[::17] = -1
    cpu = L.allocate_mla_cache(nb, bs, R + P, device="cpu", fill=0x33)
    codes, scales = L.mla_cache_views(cpu)
    lay = oracle.MlaLayout.from_views(cpu, codes, scales, R)
    oracle.mla_cache_write(kv_c, k_pe, cpu, lay, slots)
    gpu = L.allocate_mla_cache(nb, bs, R + P, device=dev, fill=0x33)
    ops.concat_and_cache_mla(kv_c.to(dev), k_pe.to(dev), gpu, slots.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(gpu.cpu(), cpu), "latent cache bytes differ from the oracle"


def test_mla_write_errors(gpu_device):
    dev = gpu_device
    cache = L.allocate_mla_cache(2, 16, 576, device=dev)
    kv_c = torch.zeros((4, 512), device=dev, dtype=torch.bfloat16)
    k_pe = torch.zeros((4, 64), device=dev, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        ops.concat_and_cache_mla(kv_c, k_pe[:, :32], cache, torch.zeros(4, device=dev, dtype=torch.int64))
    with pytest.raises(NotImplementedError):
        ops.concat_and_cache_mla(kv_c, k_pe, cache, torch.zeros(4, device=dev, dtype=torch.int64), kv_cache_dtype="fp8")


@pytest.mark.parametrize("dst_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("use_starts", [False, True])
def test_mla_gather_and_dequant_bit_exact(gpu_device, dst_dtype, use_starts):
    """Gather + dequantise for the chunked-context prefill: bit-exact against the oracle's
    code * scale (one fp32 rounding, then one rounding to the output type), rows beyond a sequence's
    end and beyond num_tokens untouched, and a round trip through the write."""
    dev = gpu_device
    R, P, bs, nb = 512, 64, 64, 12
    g = torch.Generator().manual_seed(17)
    ctx = [130, 64, 300]
    bt = T.make_block_tables(ctx, bs, nb, g)
    cpu = L.allocate_mla_cache(nb, bs, R + P, device="cpu", fill=0x33)
    codes, scales = L.mla_cache_views(cpu)
    lay = oracle.MlaLayout.from_views(cpu, codes, scales, R)
    rows = []
    for i, slots in enumerate(T.slots_for(bt, ctx, bs)):
        kv_c = torch.randn((ctx[i], R), generator=g).to(torch.bfloat16)
        k_pe = torch.randn((ctx[i], P), generator=g).to(torch.bfloat16)
        oracle.mla_cache_write(kv_c, k_pe, cpu, lay, slots)
        rows.append(torch.cat([kv_c, k_pe], -1).float())
    # a chunk of every sequence: seq_starts[b] .. seq_starts[b] + chunk[b]
    starts = [40, 0, 250] if use_starts else [0, 0, 0]
    chunk = [70, 64, 50] if use_starts else ctx
    cu = torch.tensor([0] + torch.tensor(chunk).cumsum(0).tolist(), dtype=torch.int32)
    n = int(cu[-1])
    t2s = torch.repeat_interleave(torch.arange(3, dtype=torch.int32), torch.tensor(chunk))
    ss = torch.tensor(starts, dtype=torch.int32) if use_starts else None
    want = oracle.mla_gather_dequant(cpu, lay, bt, cu, t2s, n, ss)
    dst = torch.full((n + 3, R + P), 7.0, dtype=dst_dtype, device=dev)
    ops.gather_and_maybe_dequant_cache(cpu.to(dev), dst, bt.to(dev), cu.to(dev), t2s.to(dev), n,
                                       seq_starts=ss.to(dev) if ss is not None else None)
    torch.cuda.synchronize()
    assert torch.equal(dst[:n].cpu(), want.to(dst_dtype)), "gathered rows differ from the oracle"
    assert bool((dst[n:] == 7.0).all()), "rows beyond num_tokens were written"
    # the gathered rows are the written rows up to the quantisation step
    src = torch.cat([rows[b][starts[b]:starts[b] + chunk[b]] for b in range(3)])
    amax = src.abs().amax(-1, keepdim=True)
    assert bool(((want - src).abs() <= amax / 127 * 0.5 * (1 + 1e-4)).all())


@pytest.mark.parametrize("use_starts", [False, True])
def test_mla_cp_gather_bit_exact(gpu_device, use_starts):
    """cp_gather_cache over the int8 latent cache (pattern of the reference's
    tests/kernels/attention/test_cache.py:706-863 gather tests): every destination row is the
    token's 576 code bytes followed by its 4 scale bytes, found with a plain python walk over the
    block table; chunk starts that are no multiple of the block size; rows past the last sequence
    untouched; and the rows dequantise to exactly what gather_and_maybe_dequant_cache returns."""
    dev = gpu_device
    R, P, bs, nb = 512, 64, 64, 12
    W = R + P
    g = torch.Generator().manual_seed(23)
    ctx = [130, 64, 300]
    bt = T.make_block_tables(ctx, bs, nb, g)
    cpu = L.allocate_mla_cache(nb, bs, W, device="cpu", fill=0x33)
    codes, scales = L.mla_cache_views(cpu)
    lay = oracle.MlaLayout.from_views(cpu, codes, scales, R)
    for i, slots in enumerate(T.slots_for(bt, ctx, bs)):
        oracle.mla_cache_write(torch.randn((ctx[i], R), generator=g).to(torch.bfloat16),
                               torch.randn((ctx[i], P), generator=g).to(torch.bfloat16), cpu, lay, slots)
    starts = [41, 0, 250] if use_starts else [0, 0, 0]
    chunk = [70, 64, 50] if use_starts else ctx
    cu = torch.tensor([0] + torch.tensor(chunk).cumsum(0).tolist(), dtype=torch.int32)
    n = int(cu[-1])
    want = torch.empty((n, W + 4), dtype=torch.int8)
    t = 0
    for b in range(3):
        for p in range(starts[b], starts[b] + chunk[b]):
            blk, off = int(bt[b, p // bs]), p % bs
            want[t, :W] = codes[blk, off]
            want[t, W:] = scales[blk, off].reshape(1).view(torch.int8)
            t += 1
    ss = torch.tensor(starts, dtype=torch.int32).to(dev) if use_starts else None
    dst = torch.full((n + 5, W + 4), 9, dtype=torch.int8, device=dev)
    cache_d = cpu.to(dev)
    ops.cp_gather_cache(cache_d, dst, bt.to(dev), cu.to(dev), 3, seq_starts=ss)
    torch.cuda.synchronize()
    assert torch.equal(dst[:n].cpu(), want), "gathered rows differ from the python walk"
    assert bool((dst[n:] == 9).all()), "rows past the last sequence were written"
    # the same rows, dequantised by the other gather
    t2s = torch.repeat_interleave(torch.arange(3, dtype=torch.int32), torch.tensor(chunk)).to(dev)
    deq = torch.empty((n, W), dtype=torch.float32, device=dev)
    ops.gather_and_maybe_dequant_cache(cache_d, deq, bt.to(dev), cu.to(dev), t2s, n, seq_starts=ss)
    torch.cuda.synchronize()
    row_scale = dst[:n, W:].contiguous().view(torch.float32)            # [n, 1]
    assert torch.equal(dst[:n, :W].float() * row_scale, deq)


def _cos_sin(max_pos, rot, dtype=torch.float32, base=10000.0):
    inv = 1.0 / (base ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.cat([ang.cos(), ang.sin()], -1).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("cs_same_dtype", [False, True])
def test_mla_rope_fused_write_bit_exact(gpu_device, dtype, is_neox, cs_same_dtype):
    """concat_and_cache_mla_rope_fused over the int8 latent cache: rotated q_pe and k_pe (in place),
    codes and scales all bit-identical to the oracle (the reference kernel's arithmetic restated with
    per-operation rounding in the activation dtype); padded tokens untouched; q_pe given as a strided
    slice of a wider tensor, as the caller's fused q projection leaves it."""
    dev = gpu_device
    R, P, bs, nb, H = 512, 64, 64, 6, 16
    g = torch.Generator().manual_seed(31 + is_neox)
    T_ = 150
    cs = _cos_sin(4096, P, dtype if cs_same_dtype else torch.float32)
    pos = torch.randint(0, 4096, (T_,), generator=g)
    q_full = torch.randn((T_, H, 128 + P), generator=g).to(dtype)     # [nope | pe] per head
    k_pe = torch.randn((T_, P), generator=g).to(dtype)
    kv_c = (torch.randn((T_, R), generator=g) * 3).to(dtype)
    slots = torch.randperm(nb * bs, generator=g)[:T_].to(torch.int64)
    slots[[3, 77, 149]] = -1
    cpu = L.allocate_mla_cache(nb, bs, R + P, device="cpu", fill=0x22)
    lay = oracle.MlaLayout.from_views(cpu, *L.mla_cache_views(cpu), R)
    want_q, want_k = q_full[..., 128:].clone(), k_pe.clone()
    oracle.mla_rope_cache_write(pos, want_q, want_k, kv_c, cs, is_neox, cpu, lay, slots)

    cache_d = L.allocate_mla_cache(nb, bs, R + P, device=dev, fill=0x22)
    q_d = q_full.to(dev)
    k_d = k_pe.to(dev)
    ops.concat_and_cache_mla_rope_fused(pos.to(dev), q_d[..., 128:], k_d, kv_c.to(dev), cs.to(dev), is_neox,
                                        slots.to(dev), cache_d)
    torch.cuda.synchronize()
    assert torch.equal(q_d[..., 128:].cpu(), want_q), "rotated q_pe differs"
    assert torch.equal(q_d[..., :128].cpu(), q_full[..., :128]), "the nope part of q was touched"
    assert torch.equal(k_d.cpu(), want_k), "rotated k_pe differs"
    assert torch.equal(cache_d.cpu(), cpu), "cache bytes (codes / scales) differ"
    # the fused op is rotation followed by the plain latent write
    cache2 = L.allocate_mla_cache(nb, bs, R + P, device=dev, fill=0x22)
    ops.concat_and_cache_mla(kv_c.to(dev), k_d, cache2, slots.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(cache2, cache_d)

"""GPU parity of the MLA decode over the int8 latent cache, through the C ABI, against the oracle
(fp32 + lse contract of the reference's tests/kernels/attention/test_mla_decode_cpu.py:14-41 on the
dequantised latent rows)."""
import os

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu

R, P = 512, 64
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kvq_golden_small.pt")


_build = T.build_mla_cache


def _run(q, cache, bt, sl, scale, out_dtype=None, want_lse=True):
    dev = "cuda:0"
    B, H, _ = q.shape
    o = torch.full((B, H, R), float("nan"), dtype=out_dtype or q.dtype, device=dev)
    lse = torch.full((B, H), float("nan"), dtype=torch.float32, device=dev) if want_lse else None
    ops.mla_decode_int8(q.to(dev), cache.to(dev), o, lse, bt.to(dev), sl.to(dev), scale, R)
    torch.cuda.synchronize()
    return o, lse


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bs,heads,ctx", [
    (64, 128, [300, 1, 64, 2049]),
    (16, 16, [17, 33, 511]),
    (32, 128, [4096]),
    (64, 20, [5, 0, 95, 1000, 31, 32]),
    (64, 160, [70, 300, 33]),          # a second 128-head group with only two of its eight 16-head blocks
    (64, 5, [5, 0, 95, 1000, 31, 32, 4097]),   # one head tile, partly filled; splits with fewer tiles than waves
    (16, 16, [700] * 70),              # one head tile, more sequences than compute units / 4: one split each
    (32, 8, [16384]),                  # one head tile, one long sequence: 64 splits
])
def test_mla_decode_matches_oracle(gpu_device, dtype, bs, heads, ctx):
    cache, lay, bt, sl = _build(ctx, bs, seed=bs + heads, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(7)
    q = torch.randn((len(ctx), heads, R + P), generator=g).to(dtype)
    scale = (128 + 64) ** -0.5
    want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
    got, lse = _run(q, cache, bt, sl, scale)
    if dtype == torch.float32:
        T.assert_close_attn(got, want, atol=4e-3, rtol=4e-3, what="mla decode fp32")   # fp16 operand rounding
    else:
        T.assert_close_attn(got, want, what="mla decode")
    live = sl > 0
    torch.testing.assert_close(lse.cpu()[live], want_lse[live], atol=5e-3, rtol=1e-3)
    if (~live).any():
        assert torch.equal(got.float().cpu()[~live], torch.zeros_like(want[~live]))
        assert torch.isinf(lse.cpu()[~live]).all() and (lse.cpu()[~live] < 0).all()


def test_mla_decode_peaked_softmax_and_large_values(gpu_device):
    """Logits with a large spread (one dominant token) and latent rows with large magnitudes."""
    ctx = [700, 129]
    cache, lay, bt, sl = _build(ctx, 64, seed=11, amp=8.0)
    g = torch.Generator().manual_seed(5)
    q = (torch.randn((2, 128, R + P), generator=g) * 2).to(torch.bfloat16)
    scale = 0.3
    want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
    got, lse = _run(q, cache, bt, sl, scale)
    T.assert_close_attn(got, want, atol=2e-2 * 8, rtol=1e-2, what="mla decode, peaked")  # atol scaled with |V|
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-2, rtol=1e-3)


@pytest.mark.parametrize("step", [0.1, 0.4, 3.0])
def test_mla_decode_logits_that_keep_rising(gpu_device, step):
    """Every head's logits grow along the sequence (a shared direction whose weight ramps up), by
    ``step`` (log2 units) per 32-token tile: the softmax's reference maximum may lag the true one by
    up to 2^8 before it moves, so a slow rise keeps it lagging for many tiles, a fast one moves it in
    most tiles.  16 tiles per split (32 sequences x 8 splits x 512 tokens)."""
    B, H, c = 32, 16, 4096
    u = torch.randn(R, generator=torch.Generator().manual_seed(1))
    u = u / u.norm()

    def ramp(kv_c, k_pe):
        n = kv_c.shape[0]
        w = torch.arange(n, dtype=torch.float32) / 32.0 * step          # log2 units by token
        return 0.3 * kv_c + w[:, None] * u[None, :] * 0.6931, 0.3 * k_pe   # q.u = 1 below, scale = 1

    cache, lay, bt, sl = _build([c] * B, 64, seed=21, rows_fn=ramp)
    g = torch.Generator().manual_seed(4)
    q = torch.randn((B, H, R + P), generator=g) * 0.3
    q[:, :, :R] += u                                    # unit projection on the ramp direction
    q = q.to(torch.bfloat16)
    want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, 1.0)
    got, lse = _run(q, cache, bt, sl, 1.0)
    vmax = float(want.abs().max())
    T.assert_close_attn(got, want, atol=2e-2 * max(1.0, vmax), rtol=1e-2, what=f"mla decode, rising logits {step}")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=2e-2, rtol=1e-3)


def test_mla_decode_huge_value_scales(gpu_device):
    """Latent rows in the thousands: per-token scales above 1, where p * scale of a lagging
    reference maximum could leave the fp16 range, so the kernel moves the maximum eagerly in such
    tiles.  Some sequences mix ordinary and huge rows tile by tile."""
    B, H = 16, 32

    def huge_every_other_tile(kv_c, k_pe):
        n = kv_c.shape[0]
        big = ((torch.arange(n) // 32) % 2 == 1).float() * 1999.0 + 1.0
        return kv_c * big[:, None], k_pe * big[:, None]

    cache, lay, bt, sl = _build([2048] * B, 64, seed=33, rows_fn=huge_every_other_tile)
    g = torch.Generator().manual_seed(6)
    q = (torch.randn((B, H, R + P), generator=g) * 0.01).to(torch.bfloat16)
    scale = 0.005
    want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
    got, lse = _run(q, cache, bt, sl, scale, out_dtype=torch.float32)
    assert torch.isfinite(got).all()
    T.assert_close_attn(got, want, atol=2e-2 * 2000, rtol=1e-2, what="mla decode, huge value scales")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=2e-2, rtol=1e-3)


def test_mla_decode_strided_q_and_no_lse(gpu_device):
    ctx = [100, 260]
    cache, lay, bt, sl = _build(ctx, 64, seed=3)
    g = torch.Generator().manual_seed(9)
    big = torch.randn((2, 16, 2 * (R + P)), generator=g).to(torch.bfloat16)
    q = big[:, :, : R + P]                       # head stride 1152, last dim contiguous
    want, _ = oracle.mla_decode(q, cache, lay, bt, sl, 0.07)
    dev = gpu_device
    o = torch.empty((2, 16, R), dtype=torch.bfloat16, device=dev)
    ops.mla_decode_int8(big.to(dev)[:, :, : R + P], cache.to(dev), o, None, bt.to(dev), sl.to(dev), 0.07, R)
    torch.cuda.synchronize()
    T.assert_close_attn(o, want, what="mla decode, strided q")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_mla_decode_takes_the_query_in_two_parts(gpu_device, dtype):
    """forward_mqa may receive (ql_nope, q_pe) (vllm_metax/v1/attention/backends/mla/triton_mla.py:226-238,
    where the reference concatenates them): the kernel reads the two parts where they lie, and the
    result is bit-identical to the call on the concatenated tensor.  The parts are strided views."""
    ctx = [300, 64, 1000]
    cache, lay, bt, sl = _build(ctx, 64, seed=17)
    g = torch.Generator().manual_seed(3)
    H = 48
    nope_store = torch.randn((3, H, R + 32), generator=g).to(dtype)      # rows wider than the part they hold
    pe_store = torch.randn((3, 2 * H, P), generator=g).to(dtype)         # every other head row is used
    dev = gpu_device
    ql_nope = nope_store.to(dev)[:, :, :R]
    q_pe = pe_store.to(dev)[:, ::2, :]
    joined = torch.cat([ql_nope, q_pe], dim=-1)
    kv = cache.to(dev)
    outs = []
    for q in (joined, (ql_nope, q_pe)):
        o = torch.full((3, H, R), float("nan"), dtype=dtype, device=dev)
        lse = torch.full((3, H), float("nan"), dtype=torch.float32, device=dev)
        ops.mla_decode_int8(q, kv, o, lse, bt.to(dev), sl.to(dev), 0.07, R)
        torch.cuda.synchronize()
        outs.append((o.cpu(), lse.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    want, _ = oracle.mla_decode(joined.cpu(), cache, lay, bt, sl, 0.07)
    tol = dict(atol=4e-3, rtol=4e-3) if dtype == torch.float32 else {}
    T.assert_close_attn(outs[1][0], want, what="mla decode, two-part query", **tol)
    with pytest.raises(RuntimeError):
        ops.mla_decode_int8((ql_nope, q_pe[:, :, :32]), kv, o, lse, bt.to(dev), sl.to(dev), 0.07, R)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_concat_mla_q(gpu_device, dtype):
    """ops.concat_mla_q(ql_nope, q_pe, q_out) == torch.cat((ql_nope, q_pe), dim=-1), which it replaces
    (csrc/libtorch_stable/cache_kernels.cu:1738-1739); strided inputs and output, bytes must match."""
    dev = gpu_device
    g = torch.Generator().manual_seed(8)
    for T_, H in [(1, 128), (37, 16), (300, 5), (0, 8)]:
        a = torch.randn((T_, H, R + 64), generator=g).to(dtype).to(dev)[:, :, 64:]
        b = torch.randn((T_, 2 * H, P), generator=g).to(dtype).to(dev)[:, 1::2, :]
        out_store = torch.full((T_, H, R + P + 16), 7.0, dtype=dtype, device=dev)
        out = out_store[:, :, : R + P]
        ops.concat_mla_q(a, b, out)
        torch.cuda.synchronize()
        assert torch.equal(out, torch.cat((a, b), dim=-1))
        assert bool((out_store[:, :, R + P:] == 7.0).all())          # nothing written past the rows
    with pytest.raises(RuntimeError):
        ops.concat_mla_q(a, b, out_store)                              # wrong output width
    with pytest.raises(RuntimeError):
        ops.concat_mla_q(a, b.float() if dtype != torch.float32 else b.half(), out)


@pytest.mark.parametrize("heads,nseq,dtype", [
    (128, 260, torch.bfloat16),     # one split per sequence: the decode kernel stores the result itself, no reduce
    (160, 130, torch.float16),      # two 128-head blocks per sequence, the second partly filled
    (20, 257, torch.float32),
    (16, 300, torch.bfloat16),      # the one-head-tile kernel
    (5, 256, torch.float32),
])
def test_mla_decode_one_split_per_sequence(gpu_device, heads, nseq, dtype):
    g = torch.Generator().manual_seed(heads + nseq)
    ctx = torch.randint(1, 200, (nseq,), generator=g).tolist()
    ctx[3] = 0
    ctx[nseq - 1] = 0                # empty sequences: zeros and lse = -inf, written by the decode kernel too
    ctx[7] = 33
    cache, lay, bt, sl = _build(ctx, 16, seed=nseq, dtype=torch.bfloat16)
    q = torch.randn((nseq, heads, R + P), generator=g).to(dtype)
    scale = (128 + 64) ** -0.5
    want, want_lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
    got, lse = _run(q, cache, bt, sl, scale)
    live = sl > 0
    if dtype == torch.float32:
        T.assert_close_attn(got[live], want[live], atol=4e-3, rtol=4e-3, what="mla decode, one split, fp32")
    else:
        T.assert_close_attn(got[live], want[live], what="mla decode, one split")
    torch.testing.assert_close(lse.cpu()[live], want_lse[live], atol=5e-3, rtol=1e-3)
    assert torch.equal(got.float().cpu()[~live], torch.zeros_like(want[~live]))
    assert torch.isinf(lse.cpu()[~live]).all() and (lse.cpu()[~live] < 0).all()


def test_mla_decode_golden(gpu_device):
    G = torch.load(GOLDEN, weights_only=True)
    cache = G["mla_cache"]
    got, lse = _run(G["mla_q"], cache, G["mla_block_table"], G["mla_ctx"], 192 ** -0.5)
    tol = dict(atol=4e-3, rtol=4e-3) if G["mla_q"].dtype == torch.float32 else {}
    T.assert_close_attn(got, G["mla_out"], what="golden mla decode", **tol)
    torch.testing.assert_close(lse.cpu(), G["mla_lse"], atol=5e-3, rtol=1e-3)


def test_mla_backend_forward_mqa(gpu_device):
    from types import SimpleNamespace

    from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLAImpl

    dev = gpu_device
    ctx = [77, 513]
    bs = 64
    g = torch.Generator().manual_seed(21)
    H = 16
    impl = Int8MLAImpl(num_heads=H, head_size=R + P, scale=0.0722, num_kv_heads=1, kv_cache_dtype="int8_per_token",
                       kv_lora_rank=R, qk_rope_head_dim=P)
    nb = 16
    cache = L.allocate_mla_cache(nb, bs, R + P, device=dev)
    cpu_cache = L.allocate_mla_cache(nb, bs, R + P, device="cpu")
    codes, scales = L.mla_cache_views(cpu_cache)
    lay = oracle.MlaLayout.from_views(cpu_cache, codes, scales, R)
    bt = torch.tensor([[3, 1, 0, 0, 0, 0, 0, 0, 0], [2, 4, 5, 6, 7, 8, 9, 10, 11]], dtype=torch.int32)
    for i, c in enumerate(ctx):
        kv_c = torch.randn((c, R), generator=g).to(torch.bfloat16)
        k_pe = torch.randn((c, 1, P), generator=g).to(torch.bfloat16)
        pos = torch.arange(c)
        slots = bt[i, pos // bs].long() * bs + pos % bs
        impl.do_kv_cache_update(kv_c.to(dev), k_pe.to(dev), cache, slots.to(dev))
        oracle.mla_cache_write(kv_c, k_pe.reshape(c, P), cpu_cache, lay, slots)
    torch.cuda.synchronize()
    assert torch.equal(cache.cpu(), cpu_cache)
    ql = torch.randn((2, H, R), generator=g).to(torch.bfloat16)
    qp = torch.randn((2, H, P), generator=g).to(torch.bfloat16)
    md = SimpleNamespace(decode=SimpleNamespace(block_table=bt.to(dev), seq_lens=torch.tensor(ctx, dtype=torch.int32, device=dev)))
    o, lse = impl.forward_mqa((ql.to(dev), qp.to(dev)), cache, md)
    torch.cuda.synchronize()
    want, want_lse = oracle.mla_decode(torch.cat([ql, qp], -1), cpu_cache, lay, bt, torch.tensor(ctx, dtype=torch.int32), 0.0722)
    T.assert_close_attn(o, want, what="forward_mqa")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)
    # the next step as one call: cache update and decode in one launch
    ctx2 = [c + 1 for c in ctx]
    new_c = torch.randn((2, R), generator=g).to(torch.bfloat16)
    new_pe = torch.randn((2, 1, P), generator=g).to(torch.bfloat16)
    slots = torch.tensor([int(bt[i, (c - 1) // bs]) * bs + (c - 1) % bs for i, c in enumerate(ctx2)])
    oracle.mla_cache_write(new_c, new_pe.reshape(2, P), cpu_cache, lay, slots)
    md.decode.seq_lens = torch.tensor(ctx2, dtype=torch.int32, device=dev)
    o, lse = impl.forward_mqa_with_cache_update((ql.to(dev), qp.to(dev)), new_c.to(dev), new_pe.to(dev), cache, md)
    torch.cuda.synchronize()
    assert torch.equal(cache.cpu(), cpu_cache)
    want, want_lse = oracle.mla_decode(torch.cat([ql, qp], -1), cpu_cache, lay, bt, torch.tensor(ctx2, dtype=torch.int32), 0.0722)
    T.assert_close_attn(o, want, what="forward_mqa_with_cache_update")
    torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


def test_mla_decode_caller_absorb_decode_up_proj(gpu_device):
    """The steps either side of forward_mqa (vllm_metax/model_executor/layers/attention/mla_attention.py:
    833-848, 874, 902, 1087-1110): q_nope x W_UK_T -> decode -> x W_UV, the query handed over as the
    strided views the GEMM leaves.  Checked against the same chain in fp32 on the CPU with the
    reference's bf16 roundings of ql_nope and of the decode output."""
    from types import SimpleNamespace

    from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLADecodeCaller, Int8MLAImpl

    dev = gpu_device
    N, Pn, V = 16, 128, 128
    ctx = [300, 1000, 64]
    cache, lay, bt, sl = _build(ctx, 64, seed=41)
    g = torch.Generator().manual_seed(42)
    W_UK_T = (torch.randn((N, Pn, R), generator=g) / Pn ** 0.5).to(torch.bfloat16)
    W_UV = (torch.randn((N, R, V), generator=g) / R ** 0.5).to(torch.bfloat16)
    q_nope = torch.randn((3, N, Pn), generator=g).to(torch.bfloat16)
    q_pe = torch.randn((3, N, P), generator=g).to(torch.bfloat16)
    scale = (Pn + P) ** -0.5
    impl = Int8MLAImpl(num_heads=N, head_size=R + P, scale=scale, num_kv_heads=1, kv_cache_dtype="int8_per_token",
                       kv_lora_rank=R, qk_rope_head_dim=P)
    caller = Int8MLADecodeCaller(impl, W_UK_T.to(dev), W_UV.to(dev))
    md = SimpleNamespace(decode=SimpleNamespace(block_table=bt.to(dev), seq_lens=sl.to(dev)))
    out = torch.full((3, N * V), float("nan"), dtype=torch.bfloat16, device=dev)
    ql_view = caller.absorb_q(q_nope.to(dev))
    assert ql_view.shape == (3, N, R) and not ql_view.is_contiguous()      # handed over as a view
    lse = caller.forward_decode(q_nope.to(dev), q_pe.to(dev), cache.to(dev), md, out)
    torch.cuda.synchronize()
    ql = torch.einsum("bnp,npl->bnl", q_nope.float(), W_UK_T.float()).to(torch.bfloat16)
    o_ref, lse_ref = oracle.mla_decode(torch.cat([ql, q_pe], -1), cache, lay, bt, sl, scale)
    want = torch.einsum("bnl,nlv->bnv", o_ref.to(torch.bfloat16).float(), W_UV.float()).reshape(3, N * V)
    torch.testing.assert_close(out.float().cpu(), want, atol=3e-2, rtol=2e-2)
    torch.testing.assert_close(lse.cpu(), lse_ref, atol=2e-2, rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,Pn,ctx", [
    (16, 128, [300, 1000, 64]),
    (128, 128, [700] * 5 + [33]),
    (20, 64, [5, 0, 95, 1000, 31, 32] * 7),      # 42 sequences: a second block of 32, a last tile of 10; 20 heads: a group of 4
    (128, 128, [70, 0, 130, 33] * 65),           # 260 sequences: one split each, the decode kernel stores the result itself
    (16, 128, [50, 120, 1, 0, 64] * 60),         # the same through the one-head-tile kernel
    (32, 128, [40, 7, 90] * 30),                 # 90 sequences: two tiles of 16 per absorption workgroup
    (256, 128, [100, 33, 70]),                   # 16 head groups: two of them per XCD in the absorption's numbering
])
def test_mla_decode_with_fused_absorption(gpu_device, dtype, N, Pn, ctx):
    """kvq_mla_decode_absorb_int8: q_nope x W_UK_T on the MFMA inside the launch, written as the decode's int8
    operands (vllm_metax/model_executor/layers/attention/mla_attention.py:835-848 + the decode).  Checked
    against the oracle's decode of the fp32 product -- the fused path never rounds it to the activation type."""
    dev = gpu_device
    B = len(ctx)
    cache, lay, bt, sl = _build(ctx, 64, seed=51, dtype=dtype)
    g = torch.Generator().manual_seed(52)
    W_UK_T = (torch.randn((N, Pn, R), generator=g) / Pn ** 0.5).to(dtype)
    q_nope = torch.randn((B, N, Pn), generator=g).to(dtype)
    q_pe = torch.randn((B, N, P), generator=g).to(dtype)
    scale = (Pn + P) ** -0.5
    o = torch.full((B, N, R), float("nan"), dtype=dtype, device=dev)
    lse = torch.full((B, N), float("nan"), dtype=torch.float32, device=dev)
    # q_nope as the strided view a fused q projection leaves: the nope slice of [B, N, Pn + P]
    q_full = torch.cat([q_nope, q_pe], dim=-1).to(dev)
    ops.mla_decode_absorb_int8(q_full[..., :Pn], W_UK_T.to(dev), q_full[..., Pn:], cache.to(dev), o, lse, bt.to(dev),
                               sl.to(dev), scale, R)
    torch.cuda.synchronize()
    ql = torch.einsum("bnp,npl->bnl", q_nope.float(), W_UK_T.float())
    want, want_lse = oracle.mla_decode(torch.cat([ql, q_pe.float()], -1), cache, lay, bt, sl, scale)
    live = sl > 0
    T.assert_close_attn(o[live.to(dev)], want[live], what="fused absorption")
    assert torch.all(o[(~live).to(dev)] == 0)
    torch.testing.assert_close(lse.cpu()[live], want_lse[live], atol=5e-3, rtol=1e-3)


def test_decode_caller_makes_no_library_gemm(gpu_device, monkeypatch):
    """Int8MLADecodeCaller.forward_decode in a serving dtype: the Q absorption runs in the decode launch and the V
    up-projection (mla_attention.py:902, 1087-1110) is kvq_mla_v_up_proj -- no torch.bmm is left."""
    from types import SimpleNamespace

    from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLADecodeCaller, Int8MLAImpl

    dev = gpu_device
    N, Pn, V = 16, 128, 128
    cache, lay, bt, sl = _build([100, 40], 64, seed=61)
    g = torch.Generator().manual_seed(62)
    W_UK_T = (torch.randn((N, Pn, R), generator=g) / Pn ** 0.5).to(torch.bfloat16).to(dev)
    W_UV = (torch.randn((N, R, V), generator=g) / R ** 0.5).to(torch.bfloat16).to(dev)
    impl = Int8MLAImpl(num_heads=N, head_size=R + P, scale=0.07, kv_lora_rank=R, qk_rope_head_dim=P)
    caller = Int8MLADecodeCaller(impl, W_UK_T, W_UV)
    md = SimpleNamespace(decode=SimpleNamespace(block_table=bt.to(dev), seq_lens=sl.to(dev)))
    calls = []
    real_bmm = torch.bmm
    monkeypatch.setattr(torch, "bmm", lambda *a, **k: (calls.append(a[0].shape), real_bmm(*a, **k))[1])
    out = torch.empty((2, N * V), dtype=torch.bfloat16, device=dev)
    caller.forward_decode(torch.randn((2, N, Pn), generator=g).to(torch.bfloat16).to(dev),
                          torch.randn((2, N, P), generator=g).to(torch.bfloat16).to(dev), cache.to(dev), md, out)
    torch.cuda.synchronize()
    assert calls == []


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,N,L,V", [
    (32, 128, 512, 128),     # the decode batch of the 128-head configuration
    (3, 16, 512, 128),       # a tensor-parallel shard, a tile of 3 live rows
    (17, 20, 512, 128),      # a second sequence tile of one row; heads that do not fill the last XCD round
    (1, 5, 256, 256),        # another latent width (run-time step count), two blocks of output dims
    (70, 9, 384, 128),       # 5 tiles of 16 sequences: two per workgroup
    (130, 16, 512, 128),
    (300, 8, 512, 128),      # 19 tiles: the last workgroup with one, partial
    (40, 256, 512, 128),
])
def test_v_up_proj_matches_the_fp32_product(gpu_device, dtype, B, N, L, V):
    """kvq_mla_v_up_proj against the product in fp32 (the reference's _v_up_proj is a bmm over [N, B, L] x
    [N, L, V], vllm_metax/model_executor/layers/attention/mla_attention.py:1087-1109): fp32 accumulation and one
    rounding to the activation type, so the result is within one rounding step of the exact product."""
    dev = gpu_device
    g = torch.Generator().manual_seed(B * 131 + N)
    x_full = torch.randn((B, N, L + 64), generator=g).to(dtype)          # x as a strided view: rows L + 64 apart
    W = (torch.randn((N, L, V), generator=g) / L ** 0.5).to(dtype)
    out = torch.full((B, N * V), float("nan"), dtype=dtype, device=dev)
    ops.mla_v_up_proj(x_full.to(dev)[..., :L], W.to(dev), out)
    torch.cuda.synchronize()
    want = torch.einsum("bnl,nlv->bnv", x_full[..., :L].float(), W.float()).reshape(B, N * V)
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    torch.testing.assert_close(out.float().cpu(), want, atol=5e-5, rtol=eps)
    # a few exactly representable cases: x = one-hot rows pick rows of W
    x1 = torch.zeros((B, N, L), dtype=dtype)
    pick = torch.randint(0, L, (B, N), generator=g)
    x1.scatter_(2, pick.unsqueeze(-1), 1.0)
    out3 = torch.empty((B, N, V), dtype=dtype, device=dev)
    ops.mla_v_up_proj(x1.to(dev), W.to(dev), out3)
    torch.cuda.synchronize()
    want1 = W[torch.arange(N).unsqueeze(0).expand(B, N), pick]            # [B, N, V]
    assert torch.equal(out3.cpu(), want1)


def test_v_up_proj_errors(gpu_device):
    dev = gpu_device
    x = torch.zeros((2, 4, 512), dtype=torch.bfloat16, device=dev)
    W = torch.zeros((4, 512, 128), dtype=torch.bfloat16, device=dev)
    out = torch.zeros((2, 4 * 128), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        ops.mla_v_up_proj(x, W.half(), out)                      # mixed dtypes
    with pytest.raises(RuntimeError):
        ops.mla_v_up_proj(x[..., :500], W[:, :500], out)         # latent width not a multiple of 128
    with pytest.raises(RuntimeError):
        ops.mla_v_up_proj(x, W[..., :64], out[:, :4 * 64])       # 64 output dims
    with pytest.raises(RuntimeError):
        ops.mla_v_up_proj(x.float(), W.float(), out.float())     # fp32 goes to the library GEMM in the caller
    with pytest.raises(RuntimeError):
        ops.mla_v_up_proj(x, W, out[:, :-1])


def test_mla_decode_errors(gpu_device):
    dev = gpu_device
    cache = L.allocate_mla_cache(4, 64, R + P, device=dev)
    q = torch.zeros((1, 8, R + P), dtype=torch.bfloat16, device=dev)
    o = torch.empty((1, 8, R), dtype=torch.bfloat16, device=dev)
    bt = torch.zeros((1, 4), dtype=torch.int32, device=dev)
    sl = torch.tensor([10], dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        ops.mla_decode_int8(q[:, :, :500], cache, o, None, bt, sl, 0.1, R)
    with pytest.raises(RuntimeError):
        ops.mla_decode_int8(q, cache, o, None, bt.long(), sl, 0.1, R)
    with pytest.raises(RuntimeError):
        ops.mla_decode_int8(q, cache, o, None, bt, sl, 0.1, R, workspace=torch.empty(16, dtype=torch.uint8, device=dev))

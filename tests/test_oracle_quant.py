"""Pins the oracle's quantiser (oracle/kvq_oracle.c: kvq_oracle_quant_rows) against things it did
not come from: torch's CPU round/div (a library routine), closed forms, tie cases and an exact
rational-arithmetic brute force."""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref


def _rand(shape, dtype, seed, kind):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32)
    if kind == "outlier":
        x[..., ::37] *= 20.0
    elif kind == "tiny":
        x *= 1e-12
    elif kind == "huge":
        x *= 1e20
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["normal", "outlier", "tiny", "huge"])
@pytest.mark.parametrize("d", [64, 128, 576])
def test_matches_torch_cpu_op_bit_exact(dtype, kind, d):
    if dtype == torch.float16 and kind == "huge":
        pytest.skip("overflows fp16")
    x = _rand((257, 3, d), dtype, 1234 + d, kind)
    codes, scales = oracle.quant_rows(x)
    ref_codes, ref_scales = torch_ref.per_token_head_quant_int8(x, d)
    assert torch.equal(scales, ref_scales.reshape(scales.shape))
    assert torch.equal(codes, ref_codes)


def test_zero_rows_use_floor_in_source_dtype():
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = torch.zeros((4, 128), dtype=dtype)
        codes, scales = oracle.quant_rows(x)
        ref_codes, ref_scales = torch_ref.per_token_head_quant_int8(x, 128)
        assert torch.equal(codes, torch.zeros_like(codes)) and torch.equal(codes, ref_codes)
        assert torch.equal(scales, ref_scales.reshape(-1))
        # eps = 1e-10 underflows to 0 in fp16: scale 0, codes defined as 0 (the as-written op divides 0/0)
        assert (scales > 0).all() or dtype == torch.float16


def test_closed_forms():
    x = _rand((1000, 128), torch.float32, 7, "outlier")
    codes, scales = oracle.quant_rows(x)
    c = codes.to(torch.int32)
    assert c.abs().max() <= 127                      # absmax maps to +-127, nothing beyond
    idx = x.abs().argmax(dim=-1)
    top = c[torch.arange(x.shape[0]), idx]
    assert torch.equal(top.abs(), torch.full_like(top, 127))
    assert torch.equal(torch.sign(top).float(), torch.sign(x[torch.arange(x.shape[0]), idx]))
    err = (c.double() * scales.double()[:, None] - x.double()).abs()
    assert (err <= 0.5 * scales.double()[:, None] * (1 + 1e-4)).all()   # half a step (+ fp32 rounding of x/scale)
    assert torch.equal(scales, x.abs().amax(dim=-1) / 127.0)


def test_ties_round_half_to_even():
    # absmax 127 -> scale exactly 1.0, so x / scale = x and k + 0.5 is a true tie
    row = torch.tensor([127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 126.5, -126.5, 125.5] + [0.0] * 117)
    codes, scales = oracle.quant_rows(row[None])
    assert scales.item() == 1.0
    assert codes[0, :11].tolist() == [127, 0, 2, 2, 4, 0, -2, -2, 126, -126, 126]
    # bf16 source with an exactly representable tie
    rowb = torch.tensor([254.0, 1.0, 3.0, 5.0, -7.0] + [0.0] * 123, dtype=torch.bfloat16)  # scale 2.0
    codes, scales = oracle.quant_rows(rowb[None])
    assert scales.item() == 2.0 and codes[0, :5].tolist() == [127, 0, 2, 2, -4]


def test_negative_extreme_is_minus_127_not_minus_128():
    row = torch.zeros(128)
    row[5] = -3.0
    row[9] = 1.0
    codes, _ = oracle.quant_rows(row[None])
    assert codes[0, 5].item() == -127 and codes.min().item() == -127


def _f32(fr: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) float32 of an exact rational, via Python's float:
    double rounding cannot bite here because inputs are float32 and one double division
    of two float32-exact values is itself exact to 53 bits, well past float32's 24."""
    return np.float32(float(fr))


def test_bruteforce_exact_rational():
    g = torch.Generator().manual_seed(99)
    x = torch.randn((64, 16), generator=g)
    codes, scales = oracle.quant_rows(x)
    for r in range(x.shape[0]):
        vals = [Fraction(float(v)) for v in x[r]]
        amax = max(abs(v) for v in vals)
        scale32 = _f32(amax / 127)
        # float32(amax/127): numerator and denominator are float32-exact, so the double quotient
        # rounds correctly to float32 unless it sits on a float32 rounding boundary of the double
        assert np.float32(scales[r].item()) == scale32
        sfr = Fraction(float(scale32))
        for j, v in enumerate(vals):
            q32 = Fraction(float(_f32(v / sfr)))           # fp32 quotient, then round half even
            fl = q32.__floor__()
            frac = q32 - fl
            if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and fl % 2 == 1):
                fl += 1
            assert codes[r, j].item() == max(-128, min(127, fl))


def test_within_one_code_of_reciprocal_formulation():
    x = _rand((512, 128), torch.bfloat16, 5, "normal")
    codes, _ = oracle.quant_rows(x)
    alt, _ = torch_ref.dynamic_per_token_quant_int8_reciprocal(x)
    assert (codes.int() - alt.int()).abs().max() <= 1


def test_mla_gather_dequant_is_the_python_gather_loop():
    """The oracle's gather + dequantise against a gather written with the typed cache views
    (the reference's test pattern for gather ops, tests/kernels/attention/test_cache.py:706-863:
    per-sequence block lookup, then row copy), with and without seq_starts."""
    import oracle
    from vllm_metax_amd import layout as L

    R, P, bs, nb = 512, 64, 16, 20
    g = torch.Generator().manual_seed(2)
    cache = L.allocate_mla_cache(nb, bs, R + P, device="cpu")
    codes, scales = L.mla_cache_views(cache)
    codes.copy_(torch.randint(-128, 128, codes.shape, generator=g, dtype=torch.int8))
    scales.copy_(torch.rand(scales.shape, generator=g) * 0.05 + 1e-3)
    lay = oracle.MlaLayout.from_views(cache, codes, scales, R)
    bt = torch.randperm(nb, generator=g)[:18].to(torch.int32).reshape(3, 6)
    for starts, chunk in (([0, 0, 0], [50, 96, 7]), ([30, 5, 90], [40, 16, 6])):
        cu = torch.tensor([0] + torch.tensor(chunk).cumsum(0).tolist(), dtype=torch.int32)
        n = int(cu[-1])
        t2s = torch.repeat_interleave(torch.arange(3, dtype=torch.int32), torch.tensor(chunk))
        got = oracle.mla_gather_dequant(cache, lay, bt, cu, t2s, n, torch.tensor(starts, dtype=torch.int32))
        want = torch.empty((n, R + P))
        for t in range(n):
            b = int(t2s[t])
            pos = t - int(cu[b]) + starts[b]
            blk, off = int(bt[b, pos // bs]), pos % bs
            want[t] = codes[blk, off].to(torch.float32) * scales[blk, off]
        assert torch.equal(got, want)


# ---- rotary embedding of the fused MLA write (oracle.rope_rotate) -------------------------------

def _cos_sin(max_pos, rot, dtype=torch.float32, base=10000.0):
    inv = 1.0 / (base ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.cat([ang.cos(), ang.sin()], -1).to(dtype)


def test_rope_quarter_turns_and_pair_layouts():
    """Exact cases: cos = 0, sin = 1 sends (x, y) to (-y, x); the NeoX layout pairs (i, rot/2 + i), the
    GPT-J layout pairs (2i, 2i + 1); position 0 (cos = 1, sin = 0) is the identity."""
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    cs = torch.tensor([[1.0, 1.0, 0.0, 0.0], [0.0, 0.0, 1.0, 1.0]])        # pos 0: identity, pos 1: quarter turn
    pos = torch.tensor([1])
    assert oracle.rope_rotate(x, pos, cs, True).tolist() == [[-3.0, -4.0, 1.0, 2.0]]
    assert oracle.rope_rotate(x, pos, cs, False).tolist() == [[-2.0, 1.0, -4.0, 3.0]]
    assert torch.equal(oracle.rope_rotate(x, torch.tensor([0]), cs, True), x)
    assert torch.equal(oracle.rope_rotate(x, torch.tensor([0]), cs, False), x)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 2e-2), (torch.float16, 3e-3)])
@pytest.mark.parametrize("is_neox", [True, False])
def test_rope_matches_complex_rotation(dtype, tol, is_neox):
    """Against exact complex arithmetic in float64: each pair is multiplied by e^{i theta}; the norm of
    every pair is preserved to rounding; heads of a token share the token's angles."""
    g = torch.Generator().manual_seed(3)
    T_, H, rot = 9, 5, 64
    cs = _cos_sin(50, rot)
    pos = torch.randint(0, 50, (T_,), generator=g)
    x = torch.randn((T_, H, rot), generator=g).to(dtype)
    got = oracle.rope_rotate(x, pos, cs, is_neox).double()
    xd = x.double()
    xs, ys = (xd[..., :rot // 2], xd[..., rot // 2:]) if is_neox else (xd[..., 0::2], xd[..., 1::2])
    z = torch.complex(xs, ys) * torch.polar(torch.ones(T_, rot // 2, dtype=torch.float64),
                                            torch.arange(0, rot, 2, dtype=torch.float64)[None, :].mul(0)
                                            + pos[:, None].double() / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot)))[:, None, :]
    gs, gy = (got[..., :rot // 2], got[..., rot // 2:]) if is_neox else (got[..., 0::2], got[..., 1::2])
    assert float((gs - z.real).abs().max()) <= tol * 4 and float((gy - z.imag).abs().max()) <= tol * 4
    assert float(((gs ** 2 + gy ** 2).sqrt() - (xs ** 2 + ys ** 2).sqrt()).abs().max()) <= tol * 4


def test_rope_cache_write_is_rotate_then_write_and_skips_padding():
    """The fused op equals rotation followed by the latent write; tokens with slot < 0 keep their
    q_pe / k_pe and leave the cache alone."""
    from vllm_metax_amd import layout as L
    g = torch.Generator().manual_seed(5)
    R, P, bs, nb, T_, H = 512, 64, 16, 4, 6, 3
    cs = _cos_sin(64, P)
    pos = torch.randint(0, 64, (T_,), generator=g)
    q_pe = torch.randn((T_, H, P), generator=g).to(torch.bfloat16)
    k_pe = torch.randn((T_, P), generator=g).to(torch.bfloat16)
    kv_c = torch.randn((T_, R), generator=g).to(torch.bfloat16)
    slots = torch.tensor([5, -1, 17, 0, 33, -1], dtype=torch.int64)
    a = L.allocate_mla_cache(nb, bs, R + P, device="cpu", fill=0x11)
    b = a.clone()
    la = oracle.MlaLayout.from_views(a, *L.mla_cache_views(a), R)
    lb = oracle.MlaLayout.from_views(b, *L.mla_cache_views(b), R)
    q1, k1 = q_pe.clone(), k_pe.clone()
    oracle.mla_rope_cache_write(pos, q1, k1, kv_c, cs, True, a, la, slots)
    k2 = oracle.rope_rotate(k_pe, pos, cs, True)
    oracle.mla_cache_write(kv_c, k2, b, lb, slots)
    assert torch.equal(a, b)
    live = slots >= 0
    assert torch.equal(k1[live], k2[live]) and torch.equal(k1[~live], k_pe[~live]) and torch.equal(q1[~live], q_pe[~live])
    assert torch.equal(q1[live], oracle.rope_rotate(q_pe, pos, cs, True)[live])


# ---------------------------------------------------------------------------------------------
# fp8 (e4m3fn) per-token-head mode of the same record layout
# ---------------------------------------------------------------------------------------------

def test_e4m3fn_table_matches_torch_for_every_code():
    tab = oracle.e4m3fn_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32)
    finite = ~torch.isnan(ref)
    assert finite.sum() == 254 and torch.equal(tab[finite], ref[finite])
    assert tab[0x7e] == 448 and tab[0x08] == 2.0 ** -6 and tab[0x01] == 2.0 ** -9 and tab[0x80] == 0


def test_fp8_conversion_matches_torch_on_a_dense_sweep_and_on_ties():
    """Every fp32 whose low 12 mantissa bits are zero between 2^-12 and 448, both signs, plus all exact
    midpoints between neighbouring codes (ties go to the even code): the oracle's conversion equals
    torch's float8_e4m3fn cast (an independent implementation of round-to-nearest-even)."""
    bits = torch.arange(0x39800000, 0x43e00001, 1 << 12, dtype=torch.int64).to(torch.int32)
    y = bits.view(torch.float32)
    y = torch.cat([y, -y])
    codes, scales = oracle.quant_rows_fp8(torch.cat([y, torch.tensor([448.0])]).view(1, -1))   # absmax 448 -> scale 1
    assert scales.item() == 1.0
    want = y.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(codes.view(-1)[:-1], want)
    tab = oracle.e4m3fn_table()[:0x7f]                       # positive codes in increasing order
    mid = (tab[:-1] + tab[1:]) / 2                            # exact in fp32
    codes, _ = oracle.quant_rows_fp8(torch.cat([mid, torch.tensor([448.0])]).view(1, -1))
    got = codes.view(-1)[:-1].to(torch.int64)
    lower = torch.arange(0x7e)
    assert torch.equal(got, torch.where(lower % 2 == 0, lower, lower + 1)), "ties must go to the even code"
    assert torch.equal(got.to(torch.uint8), mid.to(torch.float8_e4m3fn).view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fp8_quant_rows_rule_and_closed_forms(dtype):
    g = torch.Generator().manual_seed(11)
    x = (torch.randn((300, 128), generator=g) * 3).to(dtype)
    x[7] = 0                                                   # a zero row
    codes, scales = oracle.quant_rows_fp8(x)
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=-1).clamp(min=oracle.eps_for(dtype))
    assert torch.equal(scales, amax / 448.0)                   # fp32 true division
    safe = torch.where(scales > 0, scales, torch.ones_like(scales))
    want = (xf / safe[:, None]).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(codes, want)
    assert bool((codes[7] == 0).all())
    deq = oracle.e4m3fn_table()[codes.to(torch.int64)] * scales[:, None]
    # the absmax element maps to +-448 exactly, and every element is within half a code step
    idx = xf.abs().argmax(dim=-1)
    rows = torch.arange(300)
    live = amax > 1e-9
    assert torch.equal(deq[rows, idx][live].abs(), (scales * 448.0)[live])
    step = torch.maximum(deq.abs() / 16.0, scales[:, None] * 2.0 ** -10)   # half of 2^-3 relative / half the subnormal step
    assert bool(((deq - xf).abs() <= step * 1.0001 + 1e-30).all())


# ---- int4 per-token-head codes (kvq_oracle_quant_rows_int4): the rule is this build's decision (the reference
# states the record width only), so these pin the oracle against what the stated rule fixes, not against upstream

def test_int4_closed_forms_and_nibble_order():
    # a row whose absmax is 7 has scale 1: every integer in [-7, 7] is its own code; +-0.5 ties go to the even
    # neighbour; values beyond the range clamp; dim 2 i sits in the low nibble of byte i
    x = torch.tensor([[7.0, -7.0, 3.0, -3.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 6.49, 6.51, 0.0, -6.5, 5.5, 1.0]])
    codes, scales = oracle.quant_rows_int4(x)
    assert scales.item() == 1.0
    want = torch.tensor([7, -7, 3, -3, 0, 2, 2, 0, -2, -2, 6, 7, 0, -6, 6, 1], dtype=torch.int8)
    assert torch.equal(oracle.unpack_int4(codes)[0], want)
    assert codes[0, 0].item() == (7 | ((-7 & 15) << 4)) and codes[0, 7].item() == (6 | (1 << 4))
    # -8 is reachable only through rounding past the symmetric range: the scale is absmax / 7, so it is not
    x = torch.tensor([[-10.0, 10.0, 9.99, -9.99]])
    codes, scales = oracle.quant_rows_int4(x)
    assert torch.equal(oracle.unpack_int4(codes)[0], torch.tensor([-7, 7, 7, -7], dtype=torch.int8))
    assert scales.item() == np.float32(10.0) / np.float32(7.0)


def test_int4_zero_rows_and_floor():
    z = torch.zeros((3, 64), dtype=torch.bfloat16)
    codes, scales = oracle.quant_rows_int4(z)
    assert torch.equal(codes, torch.zeros_like(codes))
    assert torch.all(scales == np.float32(oracle.eps_for(torch.bfloat16)) / np.float32(7.0))
    codes, scales = oracle.quant_rows_int4(torch.zeros((2, 64), dtype=torch.float16))   # 1e-10 underflows in fp16
    assert torch.equal(codes, torch.zeros_like(codes)) and torch.all(scales == 0)


def test_int4_bruteforce_exact_rational():
    g = torch.Generator().manual_seed(4)
    x = torch.randn((40, 32), generator=g, dtype=torch.float32)
    x[:, 5] *= 9
    codes, scales = oracle.quant_rows_int4(x)
    vals = oracle.unpack_int4(codes)
    for r in range(x.shape[0]):
        amax = max(abs(float(v)) for v in x[r])
        s32 = np.float32(amax) / np.float32(7.0)
        assert scales[r].item() == s32
        for d in range(x.shape[1]):
            y = np.float32(np.float32(x[r, d].item()) / s32)          # the fp32 quotient the rule rounds
            f = Fraction(float(y))
            lo = f.numerator // f.denominator
            frac = f - lo
            k = lo + (1 if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and lo % 2) else 0)
            assert vals[r, d].item() == max(-8, min(7, k)), (r, d)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_int4_matches_torch_round_div(dtype):
    """The same rule in torch's CPU ops (a library routine's division and rounding)."""
    x = _rand((64, 128), dtype, 11, "outlier")
    codes, scales = oracle.quant_rows_int4(x)
    xf = x.to(torch.float32)
    amax = xf.abs().amax(-1).clamp(min=oracle.eps_for(dtype))
    s = amax / 7.0
    q = torch.clamp(torch.round(xf / s[:, None]), -8, 7).to(torch.int8)
    assert torch.equal(scales, s) and torch.equal(oracle.unpack_int4(codes), q)


def test_int4_cache_write_and_attention_read_the_same_nibbles():
    """Write through the oracle, then attend: the result equals attention over code * scale computed in torch
    from the unpacked bytes of the cache (pins the write's packing against the read's unpacking)."""
    import kvq_testlib as T
    hq, hkv, d, bs = 4, 2, 64, 16
    ctx = [37, 5]
    g = torch.Generator().manual_seed(3)
    nb = 8
    kv, (k, v, ks, vs), lay = T.cpu_cache(nb, bs, hkv, d, "NHD", code_type=oracle.CODE_INT4)
    assert k.shape[-1] == d // 2 + 4 and lay.head_size == d
    bt = T.make_block_tables(ctx, bs, nb, g)
    srcs = [(torch.randn((c, hkv, d), generator=g), torch.randn((c, hkv, d), generator=g)) for c in ctx]
    T.fill_cache_from_sources(kv, lay, bt, ctx, bs, [a for a, _ in srcs], [b for _, b in srcs], code_type=oracle.CODE_INT4)
    q = torch.randn((2, hq, d), generator=g)
    sl = torch.tensor(ctx, dtype=torch.int32)
    cu = torch.arange(3, dtype=torch.int32)
    got = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, 0.125, code_type=oracle.CODE_INT4)
    for i, c in enumerate(ctx):
        slots = T.slots_for(bt, ctx, bs)[i]
        kc = oracle.unpack_int4(k.reshape(-1, hkv, d // 2 + 4)[slots][..., : d // 2].contiguous().view(torch.uint8))
        vc = oracle.unpack_int4(v.reshape(-1, hkv, d // 2 + 4)[slots][..., : d // 2].contiguous().view(torch.uint8))
        kd = kc.float() * ks.reshape(-1, hkv)[slots][..., None]
        vd = vc.float() * vs.reshape(-1, hkv)[slots][..., None]
        # the written codes are the quantiser's
        wc, wscale = oracle.quant_rows_int4(srcs[i][0])
        assert torch.equal(oracle.unpack_int4(wc), kc) and torch.equal(wscale, ks.reshape(-1, hkv)[slots])
        want = torch_ref.sdpa_gathered(q[i:i + 1], kd, vd, 0.125)
        torch.testing.assert_close(got[i:i + 1], want, atol=1e-5, rtol=1e-5)

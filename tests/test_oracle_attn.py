"""Pins the attention side of the oracle (paged GQA attention, split-K partition + reduce, LSE
merge, MLA decode) against torch library routines (SDPA, softmax, logsumexp) on gathered
contiguous K/V, against the as-written restatement of the reference's test ops, and against
invariants (block permutation, partition-size independence, NaN poisoning of unused slots)."""
import math

import pytest
import torch
from hypothesis import given, settings, strategies as st

import kvq_testlib as T
import oracle
from oracle import torch_ref
from vllm_metax_amd import layout as L


def _build(ctx_lens, q_lens, hq, hkv, d, bs, layout, seed, num_blocks=None, poison=False):
    g = torch.Generator().manual_seed(seed)
    nb = num_blocks or (sum((c + bs - 1) // bs for c in ctx_lens) + 3)
    kv, views, lay = T.cpu_cache(nb, bs, hkv, d, layout)
    if poison:  # unreferenced slots hold NaN scales and extreme codes
        T.storage_bytes(kv).fill_(0xFF)
    bt = T.make_block_tables(ctx_lens, bs, nb, g)
    ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx_lens]
    vs = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx_lens]
    T.fill_cache_from_sources(kv, lay, bt, ctx_lens, bs, ks, vs)
    q = torch.randn((sum(q_lens), hq, d), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    sl = torch.tensor(ctx_lens, dtype=torch.int32)
    return kv, views, lay, bt, q, cu, sl


def _gather_dequant(views, bt_row, ctx, d):
    k, v, ks, vs = views
    bs = k.shape[1]
    pos = torch.arange(ctx)
    blk = bt_row[pos // bs].long()
    off = pos % bs
    kd = k[blk, off][..., :d].float() * ks[blk, off][..., None]
    vd = v[blk, off][..., :d].float() * vs[blk, off][..., None]
    return kd, vd


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("hq,hkv,d,bs", [(8, 2, 128, 16), (7, 1, 64, 32), (4, 4, 128, 16)])
def test_paged_attn_equals_sdpa_on_gathered_kv(layout, hq, hkv, d, bs):
    ctx = [37, 1, 130, 64]
    ql = [1, 1, 5, 64]
    kv, views, lay, bt, q, cu, sl = _build(ctx, ql, hq, hkv, d, bs, layout, 11, poison=True)
    scale = 1.0 / math.sqrt(d)
    out, lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, causal=True, return_lse=True)
    assert torch.isfinite(out).all()
    row = 0
    for i, (c, n) in enumerate(zip(ctx, ql)):
        kd, vd = _gather_dequant(views, bt[i], c, d)
        want = torch_ref.sdpa_gathered(q[row:row + n].float(), kd, vd, scale)
        torch.testing.assert_close(out[row:row + n], want, atol=2e-5, rtol=1e-5)
        # lse against torch.logsumexp with the same bottom-right causal mask
        rep = hq // hkv
        s = torch.einsum("qhd,khd->hqk", q[row:row + n].float(), kd.repeat_interleave(rep, 1)) * scale
        mask = torch.ones(n, c, dtype=torch.bool).tril(diagonal=c - n)
        s = s.masked_fill(~mask, float("-inf"))
        torch.testing.assert_close(lse[row:row + n], torch.logsumexp(s, -1).T, atol=2e-5, rtol=1e-5)
        row += n


def test_paged_attn_vs_as_written_reference_op():
    hq, hkv, d, bs = 8, 2, 128, 16
    ctx, ql = [100, 463, 18], [1, 129, 5]
    kv, views, lay, bt, q, cu, sl = _build(ctx, ql, hq, hkv, d, bs, "NHD", 3)
    scale = d ** -0.5
    out = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    k, v, ks, vs = views
    # fp32 instance of the as-written op: tight
    kd, vd = torch_ref.dequant_cache(k, v, ks, vs, d, torch.float32)
    want32 = torch_ref.paged_attn(q.float(), kd, vd, ql, ctx, bt, scale)
    torch.testing.assert_close(out, want32, atol=3e-5, rtol=1e-5)
    # bf16 instance (what the CPU baseline times): inside the north-star tolerance
    kd, vd = torch_ref.dequant_cache(k, v, ks, vs, d, torch.bfloat16)
    want16 = torch_ref.paged_attn(q, kd, vd, ql, ctx, bt, scale)
    T.assert_close_attn(want16, out, what="as-written bf16 op vs oracle")


@pytest.mark.parametrize("window,cap", [(16, 0.0), (64, 0.0), (1000, 0.0), (0, 30.0), (40, 5.0)])
def test_sliding_window_and_soft_cap_vs_as_written_reference_op(window, cap):
    """The same op with its sliding_window / soft_cap arguments
    (tests/kernels/attention/test_triton_unified_attention.py:38-39,60-68), fp32 instance; and two
    closed forms: a window at least as long as the sequence changes nothing, a huge cap changes nothing."""
    hq, hkv, d, bs = 8, 2, 64, 16
    ctx, ql = [100, 463, 18, 1], [1, 129, 5, 1]
    kv, views, lay, bt, q, cu, sl = _build(ctx, ql, hq, hkv, d, bs, "NHD", 11)
    q = q * 3.0                                    # logits large enough for the cap to bite
    scale = d ** -0.5
    out = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, sliding_window=window, soft_cap=cap)
    k, v, ks, vs = views
    kd, vd = torch_ref.dequant_cache(k, v, ks, vs, d, torch.float32)
    want = torch_ref.paged_attn(q.float(), kd, vd, ql, ctx, bt, scale, sliding_window=window or None, soft_cap=cap or None)
    torch.testing.assert_close(out, want, atol=3e-5, rtol=1e-5)
    plain = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale)
    if window >= max(ctx) and cap == 0.0:
        assert torch.equal(out, plain)
    else:
        assert not torch.equal(out, plain)
    big = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, soft_cap=1e6)
    torch.testing.assert_close(big, plain, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("window,cap", [(0, 0.0), (40, 0.0), (0, 20.0)])
def test_attention_sinks_vs_softmax_over_one_more_column(window, cap):
    """Attention sinks (the `sinks` argument the reference passes to unified_attention,
    vllm_metax/v1/attention/backends/triton_attn.py:712): the oracle against torch's softmax over the logits and
    one more column that is dropped afterwards; closed forms: a sink of -inf changes nothing, a sink equal to a
    single key's logit halves that row, a huge sink empties the output; lse = logsumexp over logits and sink."""
    hq, hkv, d, bs = 8, 2, 64, 16
    ctx, ql = [100, 463, 18, 1], [1, 129, 5, 1]
    kv, views, lay, bt, q, cu, sl = _build(ctx, ql, hq, hkv, d, bs, "NHD", 23)
    scale = d ** -0.5
    sinks = torch.linspace(-3.0, 4.0, hq)
    out, lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, sliding_window=window, soft_cap=cap,
                                 sinks=sinks, return_lse=True)
    k, v, ks, vs = views
    kd, vd = torch_ref.dequant_cache(k, v, ks, vs, d, torch.float32)
    want = torch_ref.paged_attn(q.float(), kd, vd, ql, ctx, bt, scale, sliding_window=window or None,
                                soft_cap=cap or None, sinks=sinks)
    torch.testing.assert_close(out, want, atol=3e-5, rtol=1e-5)
    plain, plain_lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, sliding_window=window,
                                         soft_cap=cap, return_lse=True)
    # out = plain * exp(plain_lse - lse), lse = logaddexp(plain_lse, sink): the sink only enlarges the denominator
    torch.testing.assert_close(lse, torch.logaddexp(plain_lse, sinks[None, :].expand_as(plain_lse)), atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(out, plain * torch.exp(plain_lse - lse)[..., None], atol=3e-5, rtol=1e-5)
    none = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, sliding_window=window, soft_cap=cap,
                             sinks=torch.full((hq,), float("-inf")))
    assert torch.equal(none, plain)
    huge = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, sliding_window=window, soft_cap=cap,
                             sinks=torch.full((hq,), 80.0))
    assert huge.abs().max() < 1e-20
    # the last sequence has ONE key: with the sink equal to that key's logit the row is half the value row
    one = oracle.paged_attn(q[-1:], T.storage_bytes(kv), lay, bt[-1:], sl[-1:], torch.tensor([0, 1], dtype=torch.int32),
                            scale, sliding_window=window, soft_cap=cap, sinks=plain_lse[-1])
    torch.testing.assert_close(one, plain[-1:] * 0.5, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("window,cap", [(0, 0.0), (40, 0.0), (0, 20.0)])
def test_alibi_vs_explicit_bias_matrix_sdpa_and_closed_forms(window, cap):
    """ALiBi (alibi_slopes of the reference's attention op, vllm_metax/v1/attention/backends/triton_attn.py:699; the
    bias of tests/kernels/attention/test_attention.py:109-117): the oracle against the restated reference op with
    the explicit bias matrix, against torch's scaled_dot_product_attention fed the same matrix as attn_mask, and
    closed forms: zero slopes change nothing; with equal keys the weights are a geometric series in the slope;
    a one-token run equals a decode row; a huge slope leaves the query's own key."""
    hq, hkv, d, bs = 8, 2, 64, 16
    ctx, ql = [100, 463, 18, 1], [1, 129, 5, 1]
    kv, views, lay, bt, q, cu, sl = _build(ctx, ql, hq, hkv, d, bs, "NHD", 29)
    scale = d ** -0.5
    slopes = torch.tensor([2.0 ** -(i + 1) for i in range(hq)])     # the usual ALiBi slopes of 8 heads
    base = T.storage_bytes(kv)
    kw = dict(sliding_window=window, soft_cap=cap)
    out, lse = oracle.paged_attn(q, base, lay, bt, sl, cu, scale, alibi_slopes=slopes, return_lse=True, **kw)
    k, v, ks, vs = views
    kd, vd = torch_ref.dequant_cache(k, v, ks, vs, d, torch.float32)
    want = torch_ref.paged_attn(q.float(), kd, vd, ql, ctx, bt, scale, sliding_window=window or None,
                                soft_cap=cap or None, alibi_slopes=slopes)
    torch.testing.assert_close(out, want, atol=3e-5, rtol=1e-5)
    plain, plain_lse = oracle.paged_attn(q, base, lay, bt, sl, cu, scale, return_lse=True, **kw)
    zero = oracle.paged_attn(q, base, lay, bt, sl, cu, scale, alibi_slopes=torch.zeros(hq), **kw)
    assert torch.equal(zero, plain)
    assert not torch.allclose(out, plain, atol=1e-3)
    if not cap and not window:
        # a library routine with the bias as an additive mask: sequence 1 (129 rows on 463 keys)
        kl, n = ctx[1], ql[1]
        blocks = bt[1, : (kl + bs - 1) // bs].long()
        kk = kd[blocks].reshape(-1, hkv, d)[:kl].repeat_interleave(hq // hkv, dim=1).permute(1, 0, 2)
        vv = vd[blocks].reshape(-1, hkv, d)[:kl].repeat_interleave(hq // hkv, dim=1).permute(1, 0, 2)
        qq = q[int(cu[1]):int(cu[2])].float().permute(1, 0, 2)
        rel = (torch.arange(kl).view(1, kl) - (kl - n + torch.arange(n)).view(n, 1)).float()
        mask = slopes.view(-1, 1, 1) * rel
        mask = mask.masked_fill(rel > 0, float("-inf"))
        ref = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, attn_mask=mask, scale=scale)
        torch.testing.assert_close(out[int(cu[1]):int(cu[2])], ref.permute(1, 0, 2), atol=3e-5, rtol=1e-5)
        # the bias of the query's own key is zero and every other is negative: lse <= the plain lse
        assert bool((lse <= plain_lse + 1e-6).all())
    # a huge slope leaves the query's own key: the row is that key's value row (sequence 0, a decode row of 100 keys)
    big = oracle.paged_attn(q[:1], base, lay, bt[:1], sl[:1], torch.tensor([0, 1], dtype=torch.int32), scale,
                            alibi_slopes=torch.full((hq,), 1000.0), **kw)
    last = vd[bt[0, (ctx[0] - 1) // bs].long(), (ctx[0] - 1) % bs].repeat_interleave(hq // hkv, dim=0)
    torch.testing.assert_close(big[0], last, atol=1e-6, rtol=1e-6)


def test_alibi_with_equal_keys_is_a_geometric_series():
    """Every key and value record of the sequence is the same except the value's first element, which is the
    position: the logits are then equal, the weights are exp(slope * (j - p)) / sum, and out[0] is the
    slope-weighted mean position -- a closed form that a wrong sign or a wrong origin of the positions fails."""
    hq, hkv, d, bs = 4, 1, 64, 16
    n = 77
    kvc, views, lay = T.cpu_cache(8, bs, hkv, d, "NHD")
    g = torch.Generator().manual_seed(3)
    krow = torch.randn((1, hkv, d), generator=g).expand(n, hkv, d).contiguous()
    vrow = torch.zeros((n, hkv, d))
    vrow[:, 0, 0] = torch.arange(n, dtype=torch.float32)
    vrow[:, 0, 1] = 127.0                         # keeps every row's scale at 1: codes are the positions
    bt = torch.arange(5, dtype=torch.int32).view(1, 5)
    slots = torch.arange(n, dtype=torch.int64)
    oracle.cache_write(krow, vrow, T.storage_bytes(kvc), lay, slots)
    q = torch.randn((3, hq, d), generator=g)
    slopes = torch.tensor([0.5, 0.1, 0.01, 0.0])
    out = oracle.paged_attn(q, T.storage_bytes(kvc), lay, bt, torch.tensor([n], dtype=torch.int32),
                            torch.tensor([0, 3], dtype=torch.int32), 0.3, alibi_slopes=slopes)
    for r in range(3):
        p = n - 3 + r                             # the row's position; it sees keys 0..p
        j = torch.arange(p + 1, dtype=torch.float64)
        for h in range(hq):
            w = torch.exp(slopes[h].double() * (j - p))
            want = float((w * j).sum() / w.sum())
            assert abs(float(out[r, h, 0]) - want) < 1e-4 * max(1.0, want), (r, h, float(out[r, h, 0]), want)


def test_block_permutation_invariance_and_noncausal():
    hq, hkv, d, bs = 4, 2, 64, 16
    ctx, ql = [50, 33], [1, 3]
    kv, views, lay, bt, q, cu, sl = _build(ctx, ql, hq, hkv, d, bs, "NHD", 5, num_blocks=12)
    base = T.storage_bytes(kv)
    out = oracle.paged_attn(q, base, lay, bt, sl, cu, 0.2)
    nb = kv.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1))
    kv2, _, lay2 = T.cpu_cache(nb, bs, hkv, d, "NHD")
    b1 = base.view(nb, -1)
    T.storage_bytes(kv2).view(nb, -1)[perm] = b1          # physical block i moves to perm[i]
    bt2 = perm[bt.long()].to(torch.int32)
    out2 = oracle.paged_attn(q, T.storage_bytes(kv2), lay2, bt2, sl, cu, 0.2)
    assert torch.equal(out, out2)
    nc = oracle.paged_attn(q, base, lay, bt, sl, cu, 0.2, causal=False)
    assert torch.equal(nc[0], out[0]) and not torch.equal(nc[1], out[1])


@settings(max_examples=25, deadline=None)
@given(lens=st.lists(st.integers(1, 700), min_size=1, max_size=4), part=st.sampled_from([32, 64, 96, 512]))
def test_partition_then_reduce_equals_unsplit(lens, part):
    hq, hkv, d, bs = 4, 2, 64, 16
    kv, views, lay, bt, q, cu, sl = _build(lens, [1] * len(lens), hq, hkv, d, bs, "NHD", sum(lens))
    base = T.storage_bytes(kv)
    want, want_lse = oracle.paged_attn(q, base, lay, bt, sl, cu, 0.125, return_lse=True)
    maxp = (max(lens) + part - 1) // part
    tmp, ml, es = oracle.paged_attn_partition(q, base, lay, bt, sl, 0.125, part, maxp)
    got, lse = oracle.splitk_reduce(tmp, ml, es, sl, part, return_lse=True)
    torch.testing.assert_close(got, want, atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(lse, want_lse, atol=2e-6, rtol=1e-5)
    for i, n in enumerate(lens):       # single partition is a passthrough of the normalised partial
        if n <= part:
            torch.testing.assert_close(got[i], tmp[i, :, 0], atol=1e-7, rtol=1e-6)


def test_reduce_matches_reference_formula_in_torch():
    g = torch.Generator().manual_seed(2)
    B, H, P, D = 3, 4, 5, 32
    tmp = torch.randn((B, H, P, D), generator=g)
    ml = torch.randn((B, H, P), generator=g) * 3
    es = torch.rand((B, H, P), generator=g) * 100 + 1
    sl = torch.tensor([P * 512, 512 * 2 + 1, 7], dtype=torch.int32)
    got = oracle.splitk_reduce(tmp, ml, es, sl, 512)
    for b in range(B):
        n = min(P, (int(sl[b]) + 511) // 512)
        m = ml[b, :, :n].max(-1, keepdim=True).values
        w = es[b, :, :n] * torch.exp(ml[b, :, :n] - m)
        want = (tmp[b, :, :n] * w[..., None]).sum(1) / w.sum(-1, keepdim=True)
        torch.testing.assert_close(got[b], want, atol=1e-5, rtol=1e-5)


def test_merge_attn_states_against_torch_and_inf_cases():
    g = torch.Generator().manual_seed(4)
    Tn, H, D = 37, 6, 64
    po, so = torch.randn((Tn, H, D), generator=g), torch.randn((Tn, H, D), generator=g)
    pl, sl = torch.randn((H, Tn), generator=g) * 4, torch.randn((H, Tn), generator=g) * 4
    pl[0, 3] = float("inf")
    sl[1, 5] = float("inf")
    pl[2, 7] = float("-inf")
    out, lse = oracle.merge_attn_states(po, pl, so, sl)
    want, want_lse = torch_ref.merge_attn_states(po, pl, so, sl)
    torch.testing.assert_close(out, want, atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(lse, want_lse, atol=1e-6, rtol=1e-5)
    assert torch.equal(out[3, 0], so[3, 0]) and torch.equal(out[5, 1], po[5, 1])   # +inf side drops out
    # both -inf: prefix output and -inf lse are emitted, no NaN
    pl[4, 9] = sl[4, 9] = float("-inf")
    out, lse = oracle.merge_attn_states(po, pl, so, sl)
    assert torch.equal(out[9, 4], po[9, 4]) and lse[4, 9] == float("-inf")
    # rows at or beyond prefix_num_tokens copy the suffix
    out, lse = oracle.merge_attn_states(po, pl, so, sl, prefix_num_tokens=10)
    assert torch.equal(out[10:], so[10:]) and torch.equal(lse[:, 10:], sl[:, 10:])
    # associativity of the merge (split-K algebra): merge(merge(a,b),c) == merge(a,merge(b,c))
    co, cl = torch.randn((Tn, H, D), generator=g), torch.randn((H, Tn), generator=g)
    ab, abl = oracle.merge_attn_states(po, torch.randn((H, Tn), generator=g), so, sl)
    l1 = oracle.merge_attn_states(*oracle.merge_attn_states(po, abl, so, sl), co, cl)
    l2 = oracle.merge_attn_states(po, abl, *oracle.merge_attn_states(so, sl, co, cl))
    torch.testing.assert_close(l1[0], l2[0], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("bs", [16, 64])
def test_mla_decode_against_torch(bs):
    g = torch.Generator().manual_seed(8)
    B, H, R, P = 3, 16, 512, 64
    lens = [70, 1, 200]
    nb = sum((c + bs - 1) // bs for c in lens) + 2
    cache = L.allocate_mla_cache(nb, bs, R + P, device="cpu")
    cache.fill_(-1)                                   # poison: NaN scales in unused slots
    codes, scales = L.mla_cache_views(cache)
    lay = oracle.MlaLayout.from_views(cache, codes, scales, R)
    bt = T.make_block_tables(lens, bs, nb, g)
    for i, slots in enumerate(T.slots_for(bt, lens, bs)):
        kv_c = torch.randn((lens[i], R), generator=g).to(torch.bfloat16)
        k_pe = torch.randn((lens[i], P), generator=g).to(torch.bfloat16)
        oracle.mla_cache_write(kv_c, k_pe, cache, lay, slots)
        # the write is the per-row quantiser over the concatenated row
        c, s = oracle.quant_rows(torch.cat([kv_c, k_pe], -1))
        assert torch.equal(codes.reshape(-1, R + P)[slots], c) and torch.equal(scales.reshape(-1)[slots], s)
    q = (torch.randn((B, H, R + P), generator=g) * 0.5).to(torch.bfloat16)
    sl = torch.tensor(lens, dtype=torch.int32)
    scale = (128 + 64) ** -0.5
    out, lse = oracle.mla_decode(q, cache, lay, bt, sl, scale)
    assert torch.isfinite(out).all()
    latent = torch.nan_to_num(codes.float() * scales[..., None], nan=0.0, posinf=0.0, neginf=0.0)
    bt_l = [bt[i, : (lens[i] + bs - 1) // bs].long() for i in range(B)]
    want, want_lse = torch_ref.mla_decode_lse(q.float(), latent, scale, bt_l, lens, R)
    torch.testing.assert_close(out, want, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(lse, want_lse, atol=2e-5, rtol=1e-5)
    want2 = torch_ref.mla_decode(q.float(), latent, scale, bt_l, lens, R)   # SDPA(enable_gqa) form
    torch.testing.assert_close(out, want2, atol=2e-5, rtol=1e-5)


def test_cache_write_matches_python_scatter_and_skips_padding():
    hkv, d, bs, nb = 2, 128, 16, 6
    g = torch.Generator().manual_seed(21)
    for layout in ("NHD", "HND"):
        kv, (k, v, ks, vs), lay = T.cpu_cache(nb, bs, hkv, d, layout, fill=0x5A)
        before = T.storage_bytes(kv).clone()
        key = torch.randn((9, hkv, d), generator=g).to(torch.bfloat16)
        val = torch.randn((9, hkv, d), generator=g).to(torch.bfloat16)
        slots = torch.tensor([5, 17, -1, 95, 0, 33, -1], dtype=torch.int64)   # 7 < 9: key is padded
        oracle.cache_write(key, val, T.storage_bytes(kv), lay, slots)
        exp = L.allocate_kv_cache(nb, bs, hkv, d, device="cpu", layout=layout, fill=0x5A)
        ek, ev = L.key_value_views(exp)
        eks, evs = L.scale_views(exp)
        for t, s in enumerate(slots.tolist()):        # the python scatter loop of the reference's test
            if s < 0:
                continue
            kc, ksc = torch_ref.per_token_head_quant_int8(key[t], d)
            vc, vsc = torch_ref.per_token_head_quant_int8(val[t], d)
            ek[s // bs, s % bs, :, :d] = kc
            ev[s // bs, s % bs, :, :d] = vc
            eks[s // bs, s % bs] = ksc[:, 0]
            evs[s // bs, s % bs] = vsc[:, 0]
        assert torch.equal(T.storage_bytes(kv), T.storage_bytes(exp))
        assert not torch.equal(T.storage_bytes(kv), before)

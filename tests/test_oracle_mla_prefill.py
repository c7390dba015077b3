"""Pins of the fp32 statements behind the MLA prefill tests (CPU only).

``torch_ref.varlen_attn_lse`` is checked against the library attention on the special cases that reduce to
it, its LSE against the defining sum on tiny inputs, and the chunk-and-merge identity the chunked-context
loop rests on (mla_attention.py:2017-2140) against the one-pass result; the chunk planner against the
worked example in the reference's comments (mla_attention.py:1407-1409) and against the invariants the
loop needs."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import torch_ref as TR
from vllm_metax_amd.v1.attention.backends.mla import prefill as PF


def _rand(shape, g):
    return torch.randn(shape, generator=g)


@pytest.mark.parametrize("causal,ql,kl", [(False, 7, 19), (True, 9, 9), (True, 4, 11)])
def test_varlen_attn_reduces_to_the_library_routine(causal, ql, kl):
    g = torch.Generator().manual_seed(3)
    H, nope, rope, dv = 3, 16, 8, 12
    q, kn, kpe, v = _rand((ql, H, nope + rope), g), _rand((kl, H, nope), g), _rand((kl, rope), g), _rand((kl, H, dv), g)
    out, lse = TR.varlen_attn_lse(q, kn, kpe, v, [0, ql], [0, kl], 0.3, causal)
    k_full = torch.cat([kn, kpe[:, None].expand(-1, H, -1)], -1)
    mask = torch.ones(ql, kl, dtype=torch.bool).tril(diagonal=kl - ql) if causal else None
    want = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None], k_full.permute(1, 0, 2)[None],
                                          v.permute(1, 0, 2)[None], attn_mask=mask, scale=0.3)[0].permute(1, 0, 2)
    torch.testing.assert_close(out, want, atol=1e-5, rtol=1e-5)
    # the LSE from its definition, element by element
    for h in range(H):
        for i in range(ql):
            vis = [j for j in range(kl) if not causal or j <= i + kl - ql]
            tot = sum(math.exp(0.3 * float(q[i, h] @ k_full[j, h])) for j in vis)
            assert abs(float(lse[h, i]) - math.log(tot)) < 1e-4


def test_varlen_attn_ragged_batch_and_rows_without_keys():
    g = torch.Generator().manual_seed(4)
    H, nope, rope, dv = 2, 8, 8, 8
    qlens, klens = [3, 2, 4], [5, 0, 2]
    T, S = sum(qlens), sum(klens)
    q, kn, kpe, v = _rand((T, H, nope + rope), g), _rand((S, H, nope), g), _rand((S, rope), g), _rand((S, H, dv), g)
    cu_q, cu_k = [0, 3, 5, 9], [0, 5, 5, 7]
    out, lse = TR.varlen_attn_lse(q, kn, kpe, v, cu_q, cu_k, 1.0, True)
    # sequence 1 has no keys; in sequence 2 (4 rows, 2 keys, diagonal at the end) rows 0 and 1 see nothing
    assert torch.all(out[3:5] == 0) and torch.all(lse[:, 3:5] == -torch.inf)
    assert torch.all(out[5:7] == 0) and torch.all(lse[:, 5:7] == -torch.inf)
    assert torch.isfinite(lse[:, 7:9]).all() and torch.isfinite(lse[:, 0:3]).all()
    # each sequence alone gives the same rows
    o0, _ = TR.varlen_attn_lse(q[:3], kn[:5], kpe[:5], v[:5], [0, 3], [0, 5], 1.0, True)
    torch.testing.assert_close(out[:3], o0)


def test_chunk_and_merge_equals_one_pass():
    g = torch.Generator().manual_seed(5)
    H, nope, rope, dv, ql, ctx = 2, 16, 8, 16, 6, 23
    q = _rand((ql, H, nope + rope), g)
    kn, kpe, v = _rand((ctx + ql, H, nope), g), _rand((ctx + ql, rope), g), _rand((ctx + ql, H, dv), g)
    want, want_lse = TR.varlen_attn_lse(q, kn, kpe, v, [0, ql], [0, ctx + ql], 0.25, True)
    state = None
    for lo in range(0, ctx, 10):
        hi = min(ctx, lo + 10)
        o, l = TR.varlen_attn_lse(q, kn[lo:hi], kpe[lo:hi], v[lo:hi], [0, ql], [0, hi - lo], 0.25, False)
        state = (o, l) if state is None else TR.merge_attn_states(state[0], state[1], o, l)
    o, l = TR.varlen_attn_lse(q, kn[ctx:], kpe[ctx:], v[ctx:], [0, ql], [0, ql], 0.25, True)
    got, got_lse = TR.merge_attn_states(state[0], state[1], o, l)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(got_lse, want_lse, atol=1e-5, rtol=1e-5)


def test_chunk_planner_worked_example_and_invariants():
    # mla_attention.py:1407-1409: max_context_chunk=256, num_chunks=3, num_prefills=4 -> starts rows 0 / 256 / 512
    ws = torch.empty(1024, 8)
    md = PF.build_mla_chunked_context_metadata(
        context_lens_cpu=torch.tensor([700, 10, 300, 768]), prefill_query_start_loc_cpu=torch.tensor([0, 4, 9, 11, 30]),
        num_prefills=4, chunked_prefill_workspace=ws, chunked_prefill_workspace_size=1024, block_size=64)
    assert md.starts.tolist() == [[0] * 4, [256] * 4, [512] * 4]
    assert md.seq_lens.tolist() == [[256, 10, 256, 256], [256, 0, 44, 256], [188, 0, 0, 256]]
    assert md.cu_seq_lens.tolist() == [[0, 256, 266, 522, 778], [0, 256, 256, 300, 556], [0, 188, 188, 188, 444]]
    assert md.seq_tot == md.chunk_total_token == [778, 556, 444] and md.max_seq_lens == [256, 256, 256]
    assert md.has_empty_context == [False, True, True] and md.prefill_tokens_with_context == 30
    assert md.token_to_seq[1, :556].tolist() == [0] * 256 + [2] * 44 + [3] * 256
    # invariants for ragged inputs: chunks tile every context exactly, each chunk fits the workspace, starts are
    # block-aligned, rows map to the sequence whose range holds them
    g = torch.Generator().manual_seed(7)
    for _ in range(20):
        n = int(torch.randint(1, 9, (1,), generator=g))
        ctx = torch.randint(0, 2000, (n,), generator=g)
        ctx[torch.rand(n, generator=g) < 0.3] = 0
        qsl = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(torch.randint(2, 50, (n,), generator=g), 0)])
        bs = int([16, 64][int(torch.randint(0, 2, (1,), generator=g))])
        size = int(torch.randint(n * bs, 3000, (1,), generator=g))
        md = PF.build_mla_chunked_context_metadata(
            context_lens_cpu=ctx, prefill_query_start_loc_cpu=qsl, num_prefills=n,
            chunked_prefill_workspace=torch.empty(size, 8), chunked_prefill_workspace_size=size, block_size=bs)
        if int(ctx.max()) == 0:
            assert md is None
            continue
        assert md.seq_lens.sum(0).tolist() == ctx.tolist()
        assert max(md.seq_tot) <= size and (md.starts % bs == 0).all()
        for i in range(len(md.seq_tot)):
            cu = md.cu_seq_lens[i].tolist()
            for b in range(n):
                assert (md.token_to_seq[i, cu[b]:cu[b + 1]] == b).all()
                lo = int(md.starts[i, b])
                assert md.seq_lens[i, b] == max(0, min(int(ctx[b]), lo + int(md.starts[1, 0] if len(md.seq_tot) > 1 else size)) - lo) \
                    or len(md.seq_tot) == 1
        last = max(b for b in range(n) if ctx[b] > 0)
        assert md.prefill_tokens_with_context == int(qsl[last + 1])

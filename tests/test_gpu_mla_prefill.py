"""MLA prefill over the int8 latent cache on the GPU: the varlen attention with LSE against its fp32
statement, and the chunked-context chain (gather + dequantise -> kv_b_proj -> attention with LSE -> merge)
through ``Int8MLAImpl.forward_mha`` against one causal pass over context + new tokens
(vllm_metax/model_executor/layers/attention/mla_attention.py:2017-2140, 2298-2378).
Tolerance for attention outputs: atol 2e-2, rtol 1e-2 (bf16 / fp16 activations); LSE atol 5e-3."""
import math
from types import SimpleNamespace

import pytest
import torch

import kvq_testlib as T
import oracle
from oracle import torch_ref as TR
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLAImpl, Int8MLAMetadataBuilder
from vllm_metax_amd.v1.attention.backends.mla.prefill import Int8MLAPrefillBackend, Int8MLAPrefillMetadata

pytestmark = pytest.mark.gpu

R, P = 512, 64


def _cu(lens):
    out = [0]
    for n in lens:
        out.append(out[-1] + n)
    return out


def _inputs(qlens, klens, H, nope, rope, dv, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    Tq, S = sum(qlens), sum(klens)
    q = torch.randn((Tq, H, nope + rope), generator=g).to(dtype)
    kv = torch.randn((S, H, nope + dv), generator=g).to(dtype)     # k_nope and v as views of one GEMM output
    kpe = torch.randn((S, rope), generator=g).to(dtype) if rope else None
    return q, kv, kpe


def _check(got, lse, want, want_lse, what):
    T.assert_close_attn(got, want, what=what)
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin), what + ": rows without keys"
    assert torch.all(lse.cpu()[~fin] == -torch.inf)
    torch.testing.assert_close(lse.cpu()[fin], want_lse[fin], atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,nope,rope,dv", [(16, 128, 64, 128), (4, 64, 32, 64), (8, 128, 0, 128)])
@pytest.mark.parametrize("causal,qlens,klens", [
    (True, [70, 1, 33, 128], None),                 # the new-tokens pass: keys = queries
    (False, [70, 1, 33, 128], [100, 0, 31, 257]),   # a context chunk, one sequence without rows in it
    (True, [5, 40, 3], [37, 40, 1]),                # diagonal aligned to the end of the keys; rows that see nothing
    (False, [300], [1]),
])
def test_varlen_attention_matches_fp32_statement(gpu_device, dtype, H, nope, rope, dv, causal, qlens, klens):
    dev = gpu_device
    klens = klens or qlens
    q, kv, kpe = _inputs(qlens, klens, H, nope, rope, dv, dtype, seed=11)
    scale = 1.0 / math.sqrt(nope + rope)
    cu_q, cu_k = _cu(qlens), _cu(klens)
    kvd = kv.to(dev)
    out, lse = ops.mla_prefill_attention(
        q.to(dev), kvd[..., :nope], kpe.to(dev) if rope else None, kvd[..., nope:],
        torch.tensor(cu_q, dtype=torch.int32, device=dev), torch.tensor(cu_k, dtype=torch.int32, device=dev),
        max(qlens), scale, causal, return_softmax_lse=True)
    torch.cuda.synchronize()
    want, want_lse = TR.varlen_attn_lse(q, kv[..., :nope], kpe, kv[..., nope:], cu_q, cu_k, scale, causal)
    _check(out, lse, want, want_lse, "varlen attention")


def test_prefill_backend_calls_and_given_buffers(gpu_device):
    """run_prefill_new_tokens / run_prefill_context_chunk (prefill/base.py:154-176) with the key as a pair and
    as the concatenated tensor; ``out`` given; many heads and long rows of keys."""
    dev = gpu_device
    H, nope, rope, dv = 128, 128, 64, 128
    qlens, klens = [130, 64], [700, 1500]
    q, kv, kpe = _inputs(qlens, qlens, H, nope, rope, dv, torch.bfloat16, seed=12)
    _, kvc, kpec = _inputs(qlens, klens, H, nope, rope, dv, torch.bfloat16, seed=13)
    scale = 1.0 / math.sqrt(nope + rope)
    be = Int8MLAPrefillBackend(H, scale, R, nope, rope, dv)
    cu_q = torch.tensor(_cu(qlens), dtype=torch.int32, device=dev)
    cc = SimpleNamespace(cu_seq_lens=torch.tensor([_cu(klens)], dtype=torch.int32, device=dev))
    be.prepare_metadata(Int8MLAPrefillMetadata(block_table=None, query_start_loc=cu_q, max_query_len=max(qlens),
                                               chunked_context=cc))
    qd, kvd = q.to(dev), kv.to(dev)
    out = torch.full((sum(qlens), H, dv), float("nan"), dtype=torch.bfloat16, device=dev)
    got = be.run_prefill_new_tokens(q=qd, k=(kvd[..., :nope], kpe.to(dev)[:, None]), v=kvd[..., nope:],
                                    return_softmax_lse=False, out=out)
    assert got is out
    k_cat = torch.cat([kvd[..., :nope], kpe.to(dev)[:, None].expand(-1, H, -1)], dim=-1)
    got2, lse2 = be.run_prefill_new_tokens(q=qd, k=k_cat, v=kvd[..., nope:], return_softmax_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got2, out)
    want, want_lse = TR.varlen_attn_lse(q, kv[..., :nope], kpe, kv[..., nope:], _cu(qlens), _cu(qlens), scale, True)
    _check(out, lse2, want, want_lse, "new tokens")
    kvcd = kvc.to(dev)
    o3, l3 = be.run_prefill_context_chunk(chunk_idx=0, q=qd, k=(kvcd[..., :nope], kpec.to(dev)), v=kvcd[..., nope:])
    torch.cuda.synchronize()
    want, want_lse = TR.varlen_attn_lse(q, kvc[..., :nope], kpec, kvc[..., nope:], _cu(qlens), _cu(klens), scale, False)
    _check(o3, l3, want, want_lse, "context chunk")


def test_varlen_attention_refuses_what_is_not_built(gpu_device):
    dev = gpu_device
    cu = torch.tensor([0, 4], dtype=torch.int32, device=dev)
    q = torch.zeros((4, 2, 192), device=dev)
    with pytest.raises(RuntimeError, match="bf16 or fp16"):
        ops.mla_prefill_attention(q, q[..., :128], q[:, 0, 128:], q[..., :128], cu, cu, 4, 1.0, True)
    qb = torch.zeros((4, 2, 96), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="not built"):
        ops.mla_prefill_attention(qb, qb[..., :32], qb[:, 0, 32:], qb[..., :32], cu, cu, 4, 1.0, True)
    qh = torch.zeros((4, 2, 192), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="k_pe"):
        ops.mla_prefill_attention(qh, qh[..., :128], None, qh[..., :128], cu, cu, 4, 1.0, True)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        odd = torch.zeros((4, 2, 129), dtype=torch.bfloat16, device=dev)
        ops.mla_prefill_attention(qh, odd[..., :128], qh[:, 0, 128:], qh[..., :128], cu, cu, 4, 1.0, True)


@pytest.mark.parametrize("dtype,workspace_rows", [(torch.bfloat16, 640), (torch.float16, 4096)])
def test_forward_mha_chunked_context_equals_one_causal_pass(gpu_device, dtype, workspace_rows):
    """Two decode requests first, then four prefills (context 300 / none / 700 / 64); the context workspace is
    small enough for several chunks (640 rows over three prefills = 192-row shares -> four chunks, the later
    ones with sequences that have nothing left) or large enough for one."""
    dev = gpu_device
    H, nope, dv, bs = 16, 128, 128, 64
    dec_ctx = [50, 200]
    pre_ctx, pre_q = [300, 0, 700, 64], [17, 40, 5, 64]
    ctx_all = dec_ctx + pre_ctx
    cache, lay, bt, _ = T.build_mla_cache([c + q for c, q in zip(ctx_all, [1, 1] + pre_q)], bs, seed=21, dtype=dtype)
    g = torch.Generator().manual_seed(22)
    w_kv_b = (torch.randn((R, H * (nope + dv)), generator=g) / math.sqrt(R)).to(dtype)
    Tp = sum(pre_q)
    q = torch.randn((Tp, H, nope + P), generator=g).to(dtype)
    kv_c_new = torch.randn((Tp, R), generator=g).to(dtype)
    k_pe_new = torch.randn((Tp, 1, P), generator=g).to(dtype)
    scale = 1.0 / math.sqrt(nope + P)

    qlens_all = [1, 1] + pre_q
    qsl = torch.tensor(_cu(qlens_all), dtype=torch.int32)
    seq_lens = torch.tensor([c + n for c, n in zip(ctx_all, qlens_all)], dtype=torch.int32)
    common = SimpleNamespace(
        num_reqs=6, num_actual_tokens=int(qsl[-1]), max_query_len=max(qlens_all), max_seq_len=int(seq_lens.max()),
        query_start_loc=qsl.to(dev), query_start_loc_cpu=qsl, seq_lens=seq_lens.to(dev), seq_lens_cpu=seq_lens,
        block_table_tensor=bt.to(dev), slot_mapping=torch.zeros(int(qsl[-1]), dtype=torch.int64, device=dev))
    cfg = SimpleNamespace(
        model_config=SimpleNamespace(dtype=dtype, max_model_len=2048,
                                     hf_text_config=SimpleNamespace(kv_lora_rank=R, qk_nope_head_dim=nope,
                                                                    qk_rope_head_dim=P, v_head_dim=dv),
                                     get_num_attention_heads=lambda pc: H),
        parallel_config=None, scheduler_config=SimpleNamespace(max_num_seqs=8),
        mla_chunked_prefill_workspace_size=workspace_rows)
    builder = Int8MLAMetadataBuilder(SimpleNamespace(block_size=bs), ["layer.0"], cfg, dev)
    md = builder.build(0, common)
    assert md.num_decodes == 2 and md.num_prefills == 4 and md.prefill is not None
    cc = md.prefill.chunked_context
    assert cc is not None and len(cc.seq_tot) == (4 if workspace_rows == 640 else 1)
    assert md.prefill.query_start_loc.tolist() == _cu(pre_q) and cc.prefill_tokens_with_context == sum(pre_q)

    wd = w_kv_b.to(dev)
    impl = Int8MLAImpl(num_heads=H, head_size=R + P, scale=scale, num_kv_heads=1, kv_cache_dtype="int8_per_token",
                       kv_lora_rank=R, qk_rope_head_dim=P, qk_nope_head_dim=nope, v_head_dim=dv,
                       kv_b_proj=lambda x: (x @ wd, None))
    output = torch.full((Tp, H * dv), float("nan"), dtype=dtype, device=dev)
    impl.forward_mha(q.to(dev), kv_c_new.to(dev), k_pe_new.to(dev), cache.to(dev), md, None, output)
    torch.cuda.synchronize()

    # the same through the fp32 statement: the context rows as the oracle dequantises them
    rows = []
    for b, c in enumerate(pre_ctx):
        t2s = torch.zeros(max(c, 1), dtype=torch.int32)
        rows.append(oracle.mla_gather_dequant(cache, lay, bt[2 + b:3 + b], torch.tensor([0, c], dtype=torch.int32),
                                              t2s, c) if c else torch.zeros((0, R + P)))
    want = TR.mla_prefill_unchunked(q, kv_c_new, k_pe_new[:, 0], rows, w_kv_b, pre_q, pre_ctx, R, nope, scale, dtype)
    T.assert_close_attn(output.view(Tp, H, dv), want, what="forward_mha")


def test_forward_mha_without_context_is_the_causal_pass(gpu_device):
    dev = gpu_device
    H, nope, dv = 16, 128, 128
    g = torch.Generator().manual_seed(31)
    qlens = [33, 128]
    Tp = sum(qlens)
    w_kv_b = (torch.randn((R, H * (nope + dv)), generator=g) / math.sqrt(R)).to(torch.bfloat16)
    q = torch.randn((Tp, H, nope + P), generator=g).to(torch.bfloat16)
    kv_c = torch.randn((Tp, R), generator=g).to(torch.bfloat16)
    k_pe = torch.randn((Tp, 1, P), generator=g).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(nope + P)
    be = Int8MLAPrefillBackend(H, scale, R, nope, P, dv)
    pm = Int8MLAPrefillMetadata(block_table=None, query_start_loc=torch.tensor(_cu(qlens), dtype=torch.int32, device=dev),
                                max_query_len=max(qlens), chunked_context=None, prefill_backend=be)
    be.prepare_metadata(pm)
    wd = w_kv_b.to(dev)
    impl = Int8MLAImpl(num_heads=H, head_size=R + P, scale=scale, kv_lora_rank=R, qk_rope_head_dim=P,
                       qk_nope_head_dim=nope, v_head_dim=dv, kv_b_proj=lambda x: x @ wd)
    out = impl.forward_mha(q.to(dev), kv_c.to(dev), k_pe.to(dev), torch.empty(0, device=dev),
                           SimpleNamespace(prefill=pm), None, None)
    torch.cuda.synchronize()
    want = TR.mla_prefill_unchunked(q, kv_c, k_pe[:, 0], [torch.zeros((0, R + P))] * 2, w_kv_b, qlens, [0, 0], R, nope,
                                    scale, torch.bfloat16)
    T.assert_close_attn(out.view(Tp, H, dv), want, what="forward_mha, no context")

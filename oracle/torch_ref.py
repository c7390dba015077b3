"""As-written torch restatement of the reference's tests/kernels reference ops.

TEST INFRASTRUCTURE ONLY (same rule as the rest of ``oracle/``).  These keep the
numeric form the reference's own test ops use (bf16 Q.K, fp32 softmax, P cast to
the value dtype before P.V), so they serve two purposes: the CPU baseline that
``bench.py`` times, and an independent cross-check of ``kvq_oracle.c``.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def per_token_head_quant_int8(x: torch.Tensor, group_size: int, eps: float = 1e-10):
    """tests/kernels/quant_utils.py:192-220 (native_per_token_group_quant_int8).

    absmax over each group of ``group_size`` trailing elements, floored at eps in
    the input dtype, cast to fp32; scale = absmax / 127; code = clamp(round(x / scale)).
    """
    if x.shape[-1] % group_size:
        raise ValueError("last dim must be a multiple of group_size")
    lo, hi = torch.iinfo(torch.int8).min, torch.iinfo(torch.int8).max
    g = x.contiguous().reshape(-1, group_size)
    absmax = g.abs().amax(dim=-1, keepdim=True).clamp(min=eps).to(torch.float32)
    scale = absmax / hi
    q = (g.to(torch.float32) / scale).round().clamp(lo, hi).to(torch.int8)
    return q.reshape(x.shape), scale.reshape(*x.shape[:-1], x.shape[-1] // group_size)


def dynamic_per_token_quant_int8_reciprocal(x: torch.Tensor):
    """tests/kernels/quant_utils.py:23-70 (ref_dynamic_per_token_quant, int8 branch):
    the reciprocal formulation, x * (1 / scale).  Differs from the division form on
    ties by at most one code (the reference accepts +-1,
    tests/kernels/quantization/test_int8_quant.py:60-62)."""
    amax = x.abs().amax(dim=-1).to(torch.float32)
    scale = (amax / 127.0)[..., None]
    q = (x.to(torch.float32) * (1.0 / scale)).round().clamp(-128, 127).to(torch.int8)
    return q, scale


def dequant_cache(key_cache, value_cache, k_scale_cache, v_scale_cache, head_size, dtype):
    """Dequantise the whole cache the way the backend's views expose it
    (vllm_metax/v1/attention/backends/triton_attn.py:418-479, 729-739):
    key_cache/value_cache (nb, bs, Hkv, D+4) int8, scales (nb, bs, Hkv) fp32.
    ``dtype`` is the query dtype (the reference dequantises K/V to it before the dot,
    vllm_metax/v1/attention/ops/triton_decode_attention.py:154-155)."""
    k = key_cache[..., :head_size].to(torch.float32) * k_scale_cache[..., None]
    v = value_cache[..., :head_size].to(torch.float32) * v_scale_cache[..., None]
    return k.to(dtype), v.to(dtype)


def paged_attn(query, key_cache, value_cache, query_lens, kv_lens, block_tables, scale,
               sliding_window=None, soft_cap=None, sinks=None, alibi_slopes=None):
    """tests/kernels/attention/test_triton_unified_attention.py:26-78 (ref_paged_attn).
    ``alibi_slopes`` ``[Hq]`` (not in that test either): the bias matrix ``slope * (key position - query position)``
    is added to the scaled, capped logits -- ``alibi_slopes.view(-1, 1, 1) * (position_ids - seq_len + 1)`` of
    tests/kernels/attention/test_attention.py:109-117 for the last position, the same for every row of a run.
    ``sinks`` ``[Hq]`` (not in the reference's copy of that test; the definition of upstream's argument): the
    softmax runs over the masked logits and one more column holding ``sinks[h]``, which is dropped afterwards.

    key_cache/value_cache: dequantised (nb, bs, Hkv, D) in the query dtype.
    The reference op scales ``query`` in place; a scaled copy is used instead so the
    caller's tensor survives."""
    nb, bs, hkv, d = key_cache.shape
    tables = block_tables.cpu().tolist()
    outs, row = [], 0
    for i, (ql, kl) in enumerate(zip(query_lens, kv_lens)):
        q = query[row:row + ql] * scale
        row += ql
        blocks = tables[i][: (kl + bs - 1) // bs]
        k = key_cache[blocks].reshape(-1, hkv, d)[:kl]
        v = value_cache[blocks].reshape(-1, hkv, d)[:kl]
        rep = q.shape[1] // hkv
        if rep != 1:
            k = k.repeat_interleave(rep, dim=1)
            v = v.repeat_interleave(rep, dim=1)
        logits = torch.einsum("qhd,khd->hqk", q, k).float()
        ones = torch.ones(ql, kl)
        hide = torch.triu(ones, diagonal=kl - ql + 1).bool()
        if sliding_window is not None:
            hide |= torch.triu(ones, diagonal=kl - (ql + sliding_window) + 1).bool().logical_not()
        if soft_cap:
            logits = soft_cap * torch.tanh(logits / soft_cap)
        if alibi_slopes is not None:
            rel = torch.arange(kl).view(1, kl) - (kl - ql + torch.arange(ql)).view(ql, 1)
            logits = logits + alibi_slopes.float().view(-1, 1, 1) * rel.float()
        logits.masked_fill_(hide, float("-inf"))
        if sinks is not None:
            col = sinks.float().reshape(-1, 1, 1).expand(-1, ql, 1)
            probs = torch.softmax(torch.cat([logits, col], dim=-1), dim=-1)[..., :-1].to(v.dtype)
        else:
            probs = torch.softmax(logits, dim=-1).to(v.dtype)
        outs.append(torch.einsum("hqk,khd->qhd", probs, v))
    return torch.cat(outs, dim=0)


def sdpa_gathered(query_f32, k_f32, v_f32, scale):
    """Textbook attention on one sequence's gathered, contiguous K/V (fp32):
    query [ql, Hq, D], k/v [kl, Hkv, D].  Bottom-right causal.  Used only to pin the
    oracle against a library routine."""
    ql, hq, d = query_f32.shape
    kl, hkv, _ = k_f32.shape
    qh = query_f32.permute(1, 0, 2)[None]
    kh = k_f32.permute(1, 0, 2)[None]
    vh = v_f32.permute(1, 0, 2)[None]
    mask = torch.ones(ql, kl, dtype=torch.bool).tril(diagonal=kl - ql)
    o = F.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask, scale=scale, enable_gqa=True)
    return o[0].permute(1, 0, 2)


def mla_decode(query, latent_cache, scale, block_tables, seq_lens, v_head_dim):
    """tests/kernels/attention/test_mla_decode_cpu.py:14-41 (ref_mla).

    latent_cache: dequantised (nb, bs, W) in the query dtype; returns out [B, H, v_head_dim]."""
    b, h, w = query.shape
    out = query.new_zeros(b, h, v_head_dim)
    for i in range(b):
        kv = latent_cache[block_tables[i]].reshape(1, -1, w)[:, : int(seq_lens[i])]
        o = F.scaled_dot_product_attention(query[i].reshape(h, 1, w), kv, kv[..., :v_head_dim],
                                           scale=scale, enable_gqa=True)
        out[i] = o.reshape(h, v_head_dim)
    return out


def mla_decode_lse(query_f32, latent_f32, scale, block_tables, seq_lens, v_head_dim):
    """fp32 MLA reference that also returns the log-sum-exp
    (tests/kernels/attention/test_flashmla.py:114-153)."""
    b, h, w = query_f32.shape
    out = torch.zeros(b, h, v_head_dim)
    lse = torch.zeros(b, h)
    for i in range(b):
        kv = latent_f32[block_tables[i]].reshape(-1, w)[: int(seq_lens[i])]
        s = (query_f32[i] @ kv.T) * scale
        lse[i] = torch.logsumexp(s, dim=-1)
        out[i] = torch.softmax(s, dim=-1) @ kv[:, :v_head_dim]
    return out, lse


def merge_attn_states(prefix_output, prefix_lse, suffix_output, suffix_lse):
    """tests/kernels/attention/test_merge_attn_states.py:17-46 (merge_attn_states_torch).
    outputs [T, H, D], lse [H, T].  +inf is read as -inf."""
    pl = prefix_lse.clone()
    sl = suffix_lse.clone()
    pl[pl == torch.inf] = -torch.inf
    sl[sl == torch.inf] = -torch.inf
    mx = torch.maximum(pl, sl)
    pe, se = torch.exp(pl - mx), torch.exp(sl - mx)
    tot = pe + se
    out_lse = torch.log(tot) + mx
    pw = (pe / tot).T.unsqueeze(2)
    sw = (se / tot).T.unsqueeze(2)
    return prefix_output * pw + suffix_output * sw, out_lse


def varlen_attn_lse(q, k_nope, k_pe, v, cu_q, cu_k, scale, causal):
    """fp32 statement of the varlen attention the MLA prefill calls
    (vllm_metax/v1/attention/backends/mla/prefill/flash_attn.py:176-221 ->
    flash_attn_varlen_func with return_softmax_lse): q [T, H, nope + rope], k_nope [S, H, nope],
    k_pe [S, rope] shared by the heads (the broadcast of mla_attention.py:1995-2015), v [S, H, dv].
    With ``causal``, key j is visible to query row i iff j <= i + (k_len - q_len).  Returns
    out [T, H, dv] fp32 and lse [H, T] fp32 (natural log); a row without visible keys gets 0 / -inf."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=torch.float32)
    lse = torch.full((H, T), -torch.inf, dtype=torch.float32)
    for b in range(len(cu_q) - 1):
        qs, qe, ks, ke = int(cu_q[b]), int(cu_q[b + 1]), int(cu_k[b]), int(cu_k[b + 1])
        if qe == qs or ke == ks:
            continue
        kk = k_nope[ks:ke].float()
        if k_pe is not None:
            kk = torch.cat([kk, k_pe[ks:ke].float()[:, None].expand(-1, H, -1)], dim=-1)
        s = torch.einsum("qhd,khd->hqk", q[qs:qe].float(), kk) * scale
        if causal:
            i = torch.arange(qe - qs)[:, None]
            j = torch.arange(ke - ks)[None]
            s = s.masked_fill(j > i + (ke - ks) - (qe - qs), -torch.inf)
        l = torch.logsumexp(s, dim=-1)
        p = torch.nan_to_num(torch.exp(s - l[..., None]), nan=0.0)
        out[qs:qe] = torch.einsum("hqk,khd->qhd", p, v[ks:ke].float())
        lse[:, qs:qe] = l
    return out, lse


def mla_prefill_unchunked(q, kv_c_new, k_pe_new, context_rows, w_kv_b, query_lens, context_lens, kv_lora_rank,
                          nope, scale, act_dtype):
    """What the chunked-context prefill of the MLA layer must equal
    (vllm_metax/model_executor/layers/attention/mla_attention.py:2017-2140, 2298-2378), stated without
    chunks: every prefill attends, causally and in one pass, to its cached context followed by its new
    tokens.  ``context_rows[b]`` are the dequantised latent rows [context_len, R + P] of prefill b, the
    new tokens come as (kv_c_new [T, R], k_pe_new [T, P]); both are up-projected with ``w_kv_b``
    [R, H * (nope + dv)] and the products rounded to ``act_dtype`` as the layer's GEMM output is.
    Returns out [T, H, dv] fp32."""
    T, H, _ = q.shape
    hd = w_kv_b.shape[1] // H
    outs = []
    t0 = 0
    for b, (ql, cl) in enumerate(zip(query_lens, context_lens)):
        lat = torch.cat([context_rows[b][:, :kv_lora_rank].to(act_dtype).float(), kv_c_new[t0:t0 + ql].float()])
        pe = torch.cat([context_rows[b][:, kv_lora_rank:].to(act_dtype).float(), k_pe_new[t0:t0 + ql].float()])
        kv = (lat @ w_kv_b.float()).to(act_dtype).float().view(cl + ql, H, hd)
        o, _ = varlen_attn_lse(q[t0:t0 + ql], kv[..., :nope], pe, kv[..., nope:], [0, ql], [0, cl + ql], scale, True)
        outs.append(o)
        t0 += ql
    return torch.cat(outs)

#!/usr/bin/env python3
"""Writes tests/golden/kvq_golden_small.pt: seeded inputs and the outputs the pinned oracle gives
for them (quantised cache bytes, decode and chunked-prefill attention, split-K partials, MLA latent
cache and decode).  The reference tree holds no golden vectors for the int8 KV path (none of its
tests passes kv_quant_mode / int8_per_token_head), so these are this build's own, generated once
from the oracle after it was pinned against torch, closed forms and brute force.

Run from the repo root:  python tests/golden/make_golden.py
"""
import math
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path[:0] = [ROOT, os.path.join(ROOT, "vllm-metax_amd"), os.path.join(ROOT, "tests")]

import torch  # noqa: E402

import kvq_testlib as T  # noqa: E402
import oracle  # noqa: E402
from vllm_metax_amd import layout as L  # noqa: E402


def main():
    g = torch.Generator().manual_seed(20240607)
    hq, hkv, d, bs, nb = 8, 2, 128, 16, 14
    ctx = [40, 17, 100]
    qlens = [1, 5, 1]                       # a mixed batch: decode, a 5-token prefill chunk, decode
    bt = T.make_block_tables(ctx, bs, nb, g)
    kv, views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    key = [T.outlier_sources((c, hkv, d), g, torch.bfloat16) for c in ctx]
    val = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    slots = T.slots_for(bt, ctx, bs)
    for i in range(len(ctx)):
        oracle.cache_write(key[i], val[i], T.storage_bytes(kv), lay, slots[i])
    q = torch.randn((sum(qlens), hq, d), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    sl = torch.tensor(ctx, dtype=torch.int32)
    scale = 1 / math.sqrt(d)
    out, lse = oracle.paged_attn(q, T.storage_bytes(kv), lay, bt, sl, cu, scale, return_lse=True)
    # decode-only view of the same cache for the split-K contract (32-token partitions)
    qd = q[[0, 1, 6]].contiguous()
    tmp, ml, es = oracle.paged_attn_partition(qd, T.storage_bytes(kv), lay, bt, sl, scale, 32, 4)
    red = oracle.splitk_reduce(tmp, ml, es, sl, 32)
    # MLA
    R, P, mbs, mnb = 512, 64, 16, 10
    mctx = [33, 70]
    mbt = T.make_block_tables(mctx, mbs, mnb, g)
    mcache = L.allocate_mla_cache(mnb, mbs, R + P, device="cpu")
    codes, scales = L.mla_cache_views(mcache)
    mlay = oracle.MlaLayout.from_views(mcache, codes, scales, R)
    kv_c = [torch.randn((c, R), generator=g).to(torch.bfloat16) for c in mctx]
    k_pe = [torch.randn((c, P), generator=g).to(torch.bfloat16) for c in mctx]
    mslots = T.slots_for(mbt, mctx, mbs)
    for i in range(len(mctx)):
        oracle.mla_cache_write(kv_c[i], k_pe[i], mcache, mlay, mslots[i])
    mq = (torch.randn((len(mctx), 16, R + P), generator=g) * 0.5).to(torch.bfloat16)
    mout, mlse = oracle.mla_decode(mq, mcache, mlay, mbt, torch.tensor(mctx, dtype=torch.int32), 192 ** -0.5)
    blob = dict(
        hq=torch.tensor(hq), hkv=torch.tensor(hkv), d=torch.tensor(d), bs=torch.tensor(bs), nb=torch.tensor(nb),
        ctx=sl, qlens=torch.tensor(qlens, dtype=torch.int32), block_table=bt, cu=cu,
        key=torch.cat(key), value=torch.cat(val), slots=torch.cat(slots), q=q, scale=torch.tensor(scale),
        cache_bytes=T.storage_bytes(kv).clone(), out=out, lse=lse,
        part_tmp=tmp, part_max=ml, part_sum=es, part_reduced=red,
        mla_ctx=torch.tensor(mctx, dtype=torch.int32), mla_bs=torch.tensor(mbs), mla_nb=torch.tensor(mnb),
        mla_block_table=mbt, mla_kv_c=torch.cat(kv_c), mla_k_pe=torch.cat(k_pe), mla_slots=torch.cat(mslots),
        mla_q=mq, mla_cache=mcache.clone(), mla_out=mout, mla_lse=mlse,
    )
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kvq_golden_small.pt")
    torch.save(blob, path)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

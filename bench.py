#!/usr/bin/env python3
"""Benchmark of the int8 KV-cache decode path on one MI355X.

A "step" is one layer's worth of the hot path on one decode batch: quantise-on-write of the
batch's new tokens into the paged int8 cache, then paged decode attention over the whole
context.  Steps rotate over several layer caches (same block table, different cache tensor, as
in a real model) so that a step's KV bytes come from HBM and not from what the previous step
left in the last-level cache.  All inputs are resident in HBM before the timed region.

Prints ONE JSON line (see the keys below).  `value` is the algorithmic HBM bytes of a step
divided by the step time; `roofline` is the same for the decode attention launch alone, timed
with events on the launch stream; `cpu_baseline` times the as-written torch restatement of the
reference's tests/kernels ops on a bounded sample of the same batch on the host cores.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "vllm-metax_amd"))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

HBM_PEAK_GBPS = 8000.0
METRIC = "int8-KV paged decode: achieved HBM GB/s (% peak), µs/layer @B=64 ctx=8k"
# Untimed steps run for this long before the counted warm-up, so that a short run (the driver's 20 steps) is
# timed at the clocks a long one reaches; printed in the line as "prewarm_s".
PREWARM_S = 0.5
# rocprofv3 summaries that carry the measured HBM traffic of a workload's attention launch
# (a line "traffic_bytes_per_launch: N" and a line "measured_at_commit: HASH")
TRAFFIC_PROFILE = {"llama3_8b_decode_b64_ctx1k-8k": "paged_decode_streamk_llama3_8b_b64_ctx1k-8k.md",
                   "longctx_splitk_b8_32k-128k": "paged_decode_streamk_longctx_b8_32k-128k.md",
                   "qwen2_7b_mixed_4x2048_prefill_60_decode": "paged_prefill_flash_qwen2_7b_mixed_4x2048_prefill_60_decode.md",
                   "mla_decode_b32_h128_ctx4096": "mla_decode_b32_h128_ctx4096.md",
                   "mla_decode_b32_h16_ctx4096": "mla_decode_b32_h16_ctx4096.md"}


def measured_traffic(workload):
    """(bytes per launch, source) from the workload's rocprofv3 summary under profiles/, or (None, None): the
    figure is what a profiler run measured at the named commit, never a constant of this file."""
    name = TRAFFIC_PROFILE.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return None, None
    nbytes = commit = None
    for line in open(path, encoding="utf-8"):
        if line.startswith("traffic_bytes_per_launch:"):
            nbytes = float(line.split(":", 1)[1].split()[0])
        elif line.startswith("measured_at_commit:"):
            commit = line.split(":", 1)[1].strip()
    if nbytes is None:
        return None, None
    return nbytes, f"profiles/{name} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, measured at commit {commit})"


def prewarm(step, seconds=PREWARM_S):
    """Run `step(i)` untimed for a fixed wall time."""
    t0, i = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            step(i)
            i += 1
        torch.cuda.synchronize()


def time_back_to_back(fn, n):
    """Average duration of `fn(i)` over n launches issued back to back between two events on the launch
    stream (torch's current stream, which the ops launch on)."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(n):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n * 1e-3


def time_graph_replay(fn, n, replays=5):
    """GPU time of one `fn(i)`: n of them captured into one HIP graph, the graph replayed and timed between two
    events.  Inside a graph the launches follow each other without the host in between, so a kernel far shorter
    than a host-side call (the decode write) is timed as what the GPU spends on it."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n):
            fn(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(n):
            fn(i)
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (n * replays) * 1e-3


def make_batch(workload: str, seed: int = 0):
    """Context lengths and pool size of the named workload (BASELINE.json configs)."""
    g = torch.Generator().manual_seed(seed)
    if workload == "llama3_8b_decode_b64_ctx1k-8k":      # configs[1]
        ctx = torch.randint(1024, 8193, (64,), generator=g).tolist()
        return dict(hq=32, hkv=8, d=128, bs=16, ctx=ctx, pool=40000)
    if workload == "llama3_8b_decode_b64_ctx8k_fixed":   # the headline's fixed-context variant
        return dict(hq=32, hkv=8, d=128, bs=16, ctx=[8192] * 64, pool=40000)
    if workload == "longctx_splitk_b8_32k-128k":         # configs[2]
        ctx = torch.randint(32768, 131073, (8,), generator=g).tolist()
        return dict(hq=32, hkv=8, d=128, bs=16, ctx=ctx, pool=66000)
    if workload == "config1_b4_ctx512":                  # configs[0]
        return dict(hq=32, hkv=8, d=128, bs=16, ctx=[512] * 4, pool=129)
    if workload == "qwen2_7b_mixed_4x2048_prefill_60_decode":   # configs[4]
        dctx = torch.randint(512, 4097, (60,), generator=g).tolist()
        return dict(mixed=True, hq=28, hkv=4, d=128, bs=16, ctx=[2048, 4096, 6144, 8192] + dctx,
                    qlens=[2048] * 4 + [1] * 60, pool=12000)
    if workload == "llama3_8b_chunk512_ctx32k":          # one request's 512-token prefill chunk on 32k cached tokens
        return dict(mixed=True, chunk=True, hq=32, hkv=8, d=128, bs=16, ctx=[32768 + 512], qlens=[512], pool=2200)
    if workload == "llama3_8b_spec_decode_b64_q4_ctx1k-8k":   # configs[1]'s batch in a speculative-decoding step: 1 + 3 query tokens per sequence
        ctx = torch.randint(1024, 8193, (64,), generator=g).tolist()
        return dict(mixed=True, spec=True, hq=32, hkv=8, d=128, bs=16, ctx=ctx, qlens=[4] * 64, pool=40000)
    if workload == "mla_decode_b32_h128_ctx4096":        # configs[3]: DeepSeek-V2 MLA decode
        return dict(mla=True, heads=128, r=512, p=64, bs=64, ctx=[4096] * 32, pool=32 * 64 + 8)
    if workload == "mla_prefill_h128":                   # the MLA layer's prefill attention calls, DeepSeek-V2 shapes
        return dict(mla_prefill=True, heads=128, nope=128, rope=64, dv=128)
    if workload == "mla_decode_b32_h16_ctx4096":         # the same step on one of eight tensor-parallel shards
        return dict(mla=True, heads=16, r=512, p=64, bs=64, ctx=[4096] * 32, pool=32 * 64 + 8)
    raise SystemExit(f"unknown workload {workload}")


def algorithmic_bytes(cfg, include_write=True):
    """Bytes the decode step must move once: every context token's K+V codes and both scales for
    all kv heads, Q and output rows, the block-table entries and seq_lens; plus, for the write,
    the new tokens' bf16 K/V rows in and their int8 records out."""
    hq, hkv, d, bs = cfg["hq"], cfg["hkv"], cfg["d"], cfg["bs"]
    ctx = cfg["ctx"]
    B = len(ctx)
    cb = d // 2 if cfg.get("kv_dtype") == "int4" else d   # code bytes of a half record (int4: two codes per byte)
    attn = sum(ctx) * hkv * 2 * (cb + 4) + 2 * B * hq * d * 2 + sum((c + bs - 1) // bs for c in ctx) * 4 + 4 * B
    write = B * hkv * (2 * d * 2 + 2 * (cb + 4)) if include_write else 0
    return attn, write


def _quant_mode(cfg):
    from vllm_metax_amd.kv_cache_interface import KVQuantMode

    return {"fp8": KVQuantMode.FP8_PER_TOKEN_HEAD, "int4": KVQuantMode.INT4_PER_TOKEN_HEAD}.get(
        cfg.get("kv_dtype"), KVQuantMode.INT8_PER_TOKEN_HEAD)


def _cache_dtype_str(cfg):
    return {"fp8": "fp8_per_token_head", "int4": "int4_per_token_head"}.get(cfg.get("kv_dtype"), "int8_per_token_head")


def build_device_state(cfg, dev, layers, seed=0, layout="NHD", permute=True):
    from vllm_metax_amd import _custom_ops as ops
    from vllm_metax_amd import layout as L

    hq, hkv, d, bs, ctx, pool = cfg["hq"], cfg["hkv"], cfg["d"], cfg["bs"], cfg["ctx"], cfg["pool"]
    B = len(ctx)
    g = torch.Generator().manual_seed(seed)
    need = [(c + bs - 1) // bs for c in ctx]
    perm = torch.randperm(pool - 1, generator=g)[: sum(need)] + 1          # block 0 stays the null block
    if not permute:
        perm = torch.arange(sum(need)) + 1
    bt = torch.zeros((B, max(need)), dtype=torch.int32)
    o = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[o:o + n].to(torch.int32)
        o += n
    bt_d = bt.to(dev)
    sl_d = torch.tensor(ctx, dtype=torch.int32, device=dev)
    cu_d = torch.arange(B + 1, dtype=torch.int32, device=dev)
    # slot of the newest token of every sequence (the one this step writes) and of all the others
    last = torch.tensor([int(bt[i, (c - 1) // bs]) * bs + (c - 1) % bs for i, c in enumerate(ctx)], dtype=torch.int64)
    caches = []
    torch.manual_seed(seed)
    for _ in range(layers):
        kv = L.allocate_kv_cache(pool, bs, hkv, d, device=dev, layout=layout, fill=0, cache_dtype_str=_cache_dtype_str(cfg))
        k, v = L.key_value_views(kv)
        ks, vs = L.scale_views(kv)
        ks.fill_(1.0)
        vs.fill_(1.0)
        geom = L.geometry_from_views(k, v, ks, vs, L.code_type_of(_quant_mode(cfg)))
        # fill the context with N(0,1) bf16 sources through the quantise-on-write kernel itself
        for i, c in enumerate(ctx):
            pos = torch.arange(c, device=dev)
            slots = bt_d[i, pos // bs].to(torch.int64) * bs + pos % bs
            for s0 in range(0, c, 32768):
                n = min(32768, c - s0)
                ksrc = torch.randn((n, hkv, d), device=dev, dtype=torch.float32).to(torch.bfloat16)
                vsrc = torch.randn((n, hkv, d), device=dev, dtype=torch.float32).to(torch.bfloat16)
                ops.reshape_and_cache_flash_per_token_head_quant(ksrc, vsrc, k, v, ks, vs, slots[s0:s0 + n],
                                                                 kv_quant_mode=_quant_mode(cfg), geometry=geom)
        caches.append(dict(kv=kv, k=k, v=v, ks=ks, vs=vs, geom=geom))
    q = torch.randn((B, hq, d), device=dev, dtype=torch.float32).to(torch.bfloat16)
    new_k = torch.randn((B, hkv, d), device=dev, dtype=torch.float32).to(torch.bfloat16)
    new_v = torch.randn((B, hkv, d), device=dev, dtype=torch.float32).to(torch.bfloat16)
    out = torch.empty_like(q)
    ws = torch.empty(ops.paged_attn_workspace_bytes(B, hq, d), dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    return dict(bt=bt, bt_d=bt_d, sl_d=sl_d, cu_d=cu_d, slots_new=last.to(dev), caches=caches, q=q, new_k=new_k,
                new_v=new_v, out=out, ws=ws, scale=1.0 / math.sqrt(d), max_ctx=max(ctx), mode=_quant_mode(cfg))


def _window_kwargs(st):
    """window_size / softcap keywords of the attention call (the plain causal call when neither is set)."""
    w, cap = st.get("window", 0), st.get("softcap", 0.0)
    return dict(window_size=(w - 1, 0) if w else (-1, -1), softcap=cap)


def run_step(st, layer, ops, write=True, attn=True, fused=False):
    c = st["caches"][layer]
    if fused:   # the same step in one launch: the attention kernel writes the new tokens itself
        ops.decode_attention_with_cache_update(st["q"], st["new_k"], st["new_v"], c["k"], c["v"], st["out"], st["sl_d"],
                                               st["max_ctx"], st["scale"], st["bt_d"], c["ks"], c["vs"],
                                               workspace=st["ws"], geometry=c["geom"], kv_quant_mode=st["mode"],
                                               **_window_kwargs(st))
        return
    if write:
        ops.reshape_and_cache_flash_per_token_head_quant(st["new_k"], st["new_v"], c["k"], c["v"], c["ks"], c["vs"],
                                                         st["slots_new"], kv_quant_mode=st["mode"], geometry=c["geom"])
    if attn:
        ops.unified_attention(st["q"], c["k"], c["v"], st["out"], st["cu_d"], 1, st["sl_d"], st["max_ctx"], st["scale"],
                              True, block_table=st["bt_d"], k_scale_cache=c["ks"], v_scale_cache=c["vs"],
                              workspace=st["ws"], geometry=c["geom"], kv_quant_mode=st["mode"], **_window_kwargs(st))


MFMA_F16_PEAK_TFLOPS = 2500.0


def mla_algorithmic(cfg):
    """(bytes, flops) of one MLA decode launch: every context row's 576 codes + fp32 scale, Q in, O and
    lse out, block table; 2 flops per multiply-add of q.k over 576 dims and p.v over 512 dims."""
    H, R, P, bs, ctx = cfg["heads"], cfg["r"], cfg["p"], cfg["bs"], cfg["ctx"]
    B = len(ctx)
    nbytes = sum(ctx) * (R + P + 4) + B * H * ((R + P) * 2 + R * 2 + 4) + sum((c + bs - 1) // bs for c in ctx) * 4 + 4 * B
    flops = 2 * sum(ctx) * H * ((R + P) + R)
    return nbytes, flops


def build_mla_state(cfg, dev, layers, seed=0):
    from vllm_metax_amd import _custom_ops as ops
    from vllm_metax_amd import layout as L

    H, R, P, bs, ctx, pool = cfg["heads"], cfg["r"], cfg["p"], cfg["bs"], cfg["ctx"], cfg["pool"]
    B = len(ctx)
    g = torch.Generator().manual_seed(seed)
    need = [(c + bs - 1) // bs for c in ctx]
    perm = torch.randperm(pool - 1, generator=g)[: sum(need)] + 1
    bt = torch.zeros((B, max(need)), dtype=torch.int32)
    o = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[o:o + n].to(torch.int32)
        o += n
    bt_d = bt.to(dev)
    sl_d = torch.tensor(ctx, dtype=torch.int32, device=dev)
    last = torch.tensor([int(bt[i, (c - 1) // bs]) * bs + (c - 1) % bs for i, c in enumerate(ctx)], dtype=torch.int64)
    torch.manual_seed(seed)
    caches = []
    for _ in range(layers):
        cache = L.allocate_mla_cache(pool, bs, R + P, device=dev)
        for i, c in enumerate(ctx):
            pos = torch.arange(c, device=dev)
            slots = bt_d[i, pos // bs].to(torch.int64) * bs + pos % bs
            ops.concat_and_cache_mla(torch.randn((c, R), device=dev).to(torch.bfloat16),
                                     torch.randn((c, P), device=dev).to(torch.bfloat16), cache, slots)
        caches.append(cache)
    q = (torch.randn((B, H, R + P), device=dev) * 0.5).to(torch.bfloat16)
    st = dict(bt=bt, bt_d=bt_d, sl_d=sl_d, caches=caches, q=q, out=torch.empty((B, H, R), dtype=torch.bfloat16, device=dev),
              lse=torch.empty((B, H), dtype=torch.float32, device=dev), slots_new=last.to(dev),
              new_c=torch.randn((B, R), device=dev).to(torch.bfloat16), new_pe=torch.randn((B, P), device=dev).to(torch.bfloat16),
              ws=torch.empty(ops.mla_decode_workspace_bytes(B, H, R), dtype=torch.uint8, device=dev),
              scale=(128 + P) ** -0.5)
    torch.cuda.synchronize()
    return st


def run_mla_step(st, layer, ops, cfg, write=True, attn=True, fused=False):
    cache = st["caches"][layer]
    if fused:   # the same step in one launch: the decode kernel writes the new rows itself
        ops.mla_decode_with_cache_update(st["q"], st["new_c"], st["new_pe"], cache, st["out"], st["lse"], st["bt_d"],
                                         st["sl_d"], st["scale"], cfg["r"], workspace=st["ws"])
        return
    if write:
        ops.concat_and_cache_mla(st["new_c"], st["new_pe"], cache, st["slots_new"])
    if attn:
        ops.mla_decode_int8(st["q"], cache, st["out"], st["lse"], st["bt_d"], st["sl_d"], st["scale"], cfg["r"],
                            workspace=st["ws"])


def mla_cpu_baseline(cfg, st, seconds_target=15.0):
    """The reference's CPU-runnable MLA decode contract (tests/kernels/attention/test_mla_decode_cpu.py:14-41,
    as-written torch ops) on dequantised rows of a bounded sample of the batch."""
    from oracle import torch_ref
    from vllm_metax_amd import layout as L

    H, R, P, bs, ctx = cfg["heads"], cfg["r"], cfg["p"], cfg["bs"], cfg["ctx"]
    cache = st["caches"][0]
    t_total, done, reps = 0.0, 0, 0
    q_cpu = st["q"].cpu()
    for i in range(len(ctx)):
        if t_total >= seconds_target:
            break
        n = (ctx[i] + bs - 1) // bs
        sub = cache[st["bt_d"][i, :n].long()].cpu().contiguous()
        codes, scales = L.mla_cache_views(sub)
        t0 = time.perf_counter()
        latent = (codes.to(torch.float32) * scales[..., None]).to(torch.bfloat16)     # dequantised (n, bs, 576)
        torch_ref.mla_decode(q_cpu[i:i + 1], latent, st["scale"], torch.arange(n)[None], [ctx[i]], R)
        t_total += time.perf_counter() - t0
        done += ctx[i]
        reps += 1
    flops = 2 * done * H * (2 * R + P)
    return dict(value=flops / t_total / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{reps} sequence(s) of the batch ({done} context rows), oracle/torch_ref.py mla_decode "
                       f"(as-written torch), {t_total:.1f} s, torch threads={torch.get_num_threads()}")


def mla_main(args, cfg, dev, ops):
    st = build_mla_state(cfg, dev, args.layers)
    nbytes, flops = mla_algorithmic(cfg)
    L = args.layers
    prewarm(lambda i: run_mla_step(st, i % L, ops, cfg))
    for i in range(args.warmup):
        run_mla_step(st, i % L, ops, cfg)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        run_mla_step(st, i % L, ops, cfg)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    n_ev = max(args.steps, 100)
    attn_s = time_back_to_back(lambda i: run_mla_step(st, i % L, ops, cfg, write=False, attn=True), n_ev)
    fused_s = None
    if not args.no_one_launch:
        for i in range(args.warmup):
            run_mla_step(st, i % L, ops, cfg, fused=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            run_mla_step(st, i % L, ops, cfg, fused=True)
        torch.cuda.synchronize()
        fused_s = (time.perf_counter() - t0) / args.steps
    traffic, traffic_source = measured_traffic(args.workload)
    small = cfg["heads"] <= 16   # one head tile: a kernel of its own, which also prepares the query
    # at 16 heads the launch moves few flops per byte: the HBM roof is the one that binds
    roof = ({"bound": "hbm", "achieved": round(nbytes / attn_s / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": round(nbytes / attn_s / 1e9 / HBM_PEAK_GBPS, 4)} if small else
            {"bound": "mfma", "achieved": round(flops / attn_s / 1e12, 1), "peak": MFMA_F16_PEAK_TFLOPS,
             "unit": "TFLOP/s", "frac": round(flops / attn_s / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)})
    res = {
        "metric": f"int8 MLA latent-cache decode: achieved HBM GB/s, µs/layer @B=32 H={cfg['heads']} ctx=4096",
        "value": round(nbytes / dt / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 latent codes, fp16 MFMA operands, fp32 softmax/accumulate, bf16 Q/out", "data": "synthetic",
        "config": {"workload": args.workload, "batch": len(cfg["ctx"]), "sum_ctx": sum(cfg["ctx"]), "heads": cfg["heads"],
                   "kv_lora_rank": cfg["r"], "rope_dim": cfg["p"], "block_size": cfg["bs"], "layer_caches_rotated": L,
                   **({"batch_invariant": True} if ops.batch_invariant() else {})},
        "prewarm_s": PREWARM_S, "us_per_layer": round(dt * 1e6, 2), "attn_launch_us": round(attn_s * 1e6, 2),
        "roofline": {**roof, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": ("MLA decode launch on an absorbed query = mla_decode_small_kernel + mla_reduce_kernel" if small else
                                "MLA decode launch on an absorbed query = mla_decode_kernel (quantises the query itself) + mla_reduce_kernel"),
                     "timing": f"{n_ev} decode launches back to back between two events on the launch stream",
                     "algorithmic_flops_per_launch": flops, "algorithmic_bytes_per_launch": nbytes,
                     "hbm_frac_of_peak": round(nbytes / attn_s / 1e9 / HBM_PEAK_GBPS, 4)},
    }
    if fused_s is not None:
        res["one_launch_step"] = {"what": "the same layer step with the latent write inside the decode launch "
                                          "(kvq_mla_decode_int8_fused_write)",
                                  "us_per_layer": round(fused_s * 1e6, 2), "value": round(nbytes / fused_s / 1e9, 1),
                                  "unit": "GB/s"}
        res["decode_caller"] = mla_caller_chain(cfg, st, dev, ops, n_ev)
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = mla_cpu_baseline(cfg, st, args.cpu_seconds)
    print(json.dumps(res))


def mla_caller_chain(cfg, st, dev, ops, n):
    """The layer-level decode step around the launch above, from the un-absorbed query (q_nope x W_UK_T ->
    decode -> x W_UV, mla_attention.py:835-848, 902): with the absorption inside the decode launch, and as
    the reference's three steps (library GEMM, decode of the bf16 product, library GEMM)."""
    from types import SimpleNamespace

    from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLADecodeCaller, Int8MLAImpl

    H, R, P, B, Pn, V = cfg["heads"], cfg["r"], cfg["p"], len(cfg["ctx"]), 128, 128
    impl = Int8MLAImpl(num_heads=H, head_size=R + P, scale=st["scale"], kv_lora_rank=R, qk_rope_head_dim=P)
    w_uk_t = (torch.randn((H, Pn, R), device=dev) / Pn ** 0.5).to(torch.bfloat16)
    w_uv = (torch.randn((H, R, V), device=dev) / R ** 0.5).to(torch.bfloat16)
    caller = Int8MLADecodeCaller(impl, w_uk_t, w_uv)
    q_nope = (torch.randn((B, H, Pn), device=dev) * 0.5).to(torch.bfloat16)
    q_pe = (torch.randn((B, H, P), device=dev) * 0.5).to(torch.bfloat16)
    out = torch.empty((B, H * V), dtype=torch.bfloat16, device=dev)
    md = SimpleNamespace(decode=SimpleNamespace(block_table=st["bt_d"], seq_lens=st["sl_d"]), workspace=st["ws"],
                         decode_out=st["out"], decode_lse=st["lse"])
    L = len(st["caches"])

    def fused(i):
        caller.forward_decode(q_nope, q_pe, st["caches"][i % L], md, out)

    def three_steps(i):
        attn_out, _ = impl.forward_mqa((caller.absorb_q(q_nope), q_pe), st["caches"][i % L], md)
        caller.v_up_proj_library(attn_out, out)

    res = {}
    for name, fn in (("absorb_in_launch_us", fused), ("library_gemm_then_decode_us", three_steps)):
        prewarm(fn, 0.2)
        res[name] = round(time_back_to_back(fn, n) * 1e6, 2)
    res["steps"] = "q_nope [B,H,128] x W_UK_T -> decode -> x W_UV [H,512,128] -> out [B, H*128], bf16"
    return res


MLA_PREFILL_SHAPES = (("context chunk: 4 x 2048 queries, 8192 keys each, unmasked", 4, 2048, 8192, False),
                      ("new tokens: 4 x 2048 causal", 4, 2048, 2048, True),
                      ("new tokens: 1 x 8192 causal", 1, 8192, 8192, True))


def mla_prefill_main(args, cfg, dev, ops):
    """The attention call of the MLA layer's prefill (kvq_mla_prefill_attn: dense bf16 K / V behind the gather
    and the up-projection) at DeepSeek-V2 shapes.  A step is one call of the first shape; the other two are
    timed the same way and reported beside it.  --steps 1 --warmup 0 makes one call per shape (counter runs)."""
    H, nope, rope, dv = cfg["heads"], cfg["nope"], cfg["rope"], cfg["dv"]
    rows = []
    for name, B, ql, kl, causal in MLA_PREFILL_SHAPES:
        T, S = B * ql, B * kl
        q = torch.randn(T, H, nope + rope, device=dev, dtype=torch.bfloat16)
        kv = torch.randn(S, H, nope + dv, device=dev, dtype=torch.bfloat16)
        kpe = torch.randn(S, rope, device=dev, dtype=torch.bfloat16)
        cuq = torch.arange(0, T + 1, ql, dtype=torch.int32, device=dev)
        cuk = torch.arange(0, S + 1, kl, dtype=torch.int32, device=dev)
        out = torch.empty(T, H, dv, device=dev, dtype=torch.bfloat16)
        lse = torch.empty(H, T, device=dev)

        def call(_i=0):
            ops.mla_prefill_attention(q, kv[..., :nope], kpe, kv[..., nope:], cuq, cuk, ql, (nope + rope) ** -0.5,
                                      causal, out=out, lse=lse)

        n = min(args.steps, 10)
        for _ in range(min(args.warmup, 3)):
            call()
        s = time_back_to_back(call, n)
        flops = B * ql * kl * (0.5 if causal else 1.0) * H * (nope + rope + dv) * 2
        nbytes = (q.numel() + kv.numel() + kpe.numel() + out.numel()) * 2 + lse.numel() * 4
        rows.append(dict(shape=name, ms_per_call=round(s * 1e3, 4), tflops=round(flops / s / 1e12, 1),
                         frac=round(flops / s / 1e12 / MFMA_F16_PEAK_TFLOPS, 4), calls_timed=n,
                         algorithmic_flops=int(flops), algorithmic_bytes=nbytes))
        if name == MLA_PREFILL_SHAPES[0][0] and not args.no_cpu_baseline:
            cpu = mla_prefill_cpu_baseline(q, kv, kpe, nope, ql, kl, args.cpu_seconds)
        del q, kv, kpe, out, lse
    r0 = rows[0]
    res = {
        "metric": "MLA prefill attention (bf16 K/V behind the latent gather): TFLOP/s over visible (query, key) pairs, 128 heads",
        "value": r0["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": r0["calls_timed"], "warmup": min(args.warmup, 3),
        "ms_per_step": r0["ms_per_call"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 Q/K/V, fp16-range MFMA operands, fp32 softmax/accumulate", "data": "synthetic",
        "config": {"workload": args.workload, "heads": H, "qk_nope_head_dim": nope, "qk_rope_head_dim": rope,
                   "v_head_dim": dv, "shape": r0["shape"]},
        "roofline": {"bound": "mfma", "achieved": r0["tflops"], "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": r0["frac"], "traffic": None, "kernel": "varlen_attn_kernel<1, 128, 64, 128>",
                     "timing": f"{r0['calls_timed']} calls back to back between two events on the launch stream",
                     "algorithmic_flops_per_launch": r0["algorithmic_flops"],
                     "algorithmic_bytes_per_launch": r0["algorithmic_bytes"]},
        "shapes": rows,
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu
    print(json.dumps(res))


def mla_prefill_cpu_baseline(q, kv, kpe, nope, ql, kl, seconds_target):
    """fp32 torch statement of the same varlen attention on the host, on a slice of the first shape: the first
    sequence, its last 128 query rows, a few heads at a time until the time is spent."""
    from oracle import torch_ref

    rows, hb = 128, 8
    kn = kv[:kl, :, :nope].float().cpu()
    vv = kv[:kl, :, nope:].float().cpu()
    pe = kpe[:kl].float().cpu()
    cu_q, cu_k = torch.tensor([0, rows], dtype=torch.int32), torch.tensor([0, kl], dtype=torch.int32)
    t_total, blocks, r1 = 0.0, 0, ql
    while t_total < seconds_target and r1 >= rows:       # row blocks from the end of the sequence backwards
        qs = q[r1 - rows:r1].float().cpu()
        for h in range(0, q.shape[1], hb):
            t0 = time.perf_counter()
            torch_ref.varlen_attn_lse(qs[:, h:h + hb], kn[:, h:h + hb], pe, vv[:, h:h + hb], cu_q, cu_k,
                                      q.shape[-1] ** -0.5, False)
            t_total += time.perf_counter() - t0
            blocks += 1
            if t_total >= seconds_target:
                break
        r1 -= rows
    flops = blocks * rows * kl * hb * (q.shape[-1] + vv.shape[-1]) * 2
    return dict(value=flops / t_total / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{blocks} blocks of {rows} query rows x {kl} keys x {hb} heads of the first shape's first sequence, "
                       f"oracle/torch_ref.py varlen_attn_lse (fp32), {t_total:.1f} s, torch threads={torch.get_num_threads()}")


def mixed_cpu_baseline(cfg, caches, bt, q, cu, scale, seconds_target):
    """The reference's CPU path (as-written torch ops of its unified-attention test) on a bounded sample of the
    mixed batch: the decode rows one after the other, then the last 64 query rows of each prefill chunk, in whole
    passes until the time is spent.  Reported in the line's unit over the sample's algorithmic bytes, with its flops."""
    from oracle import torch_ref

    hq, hkv, d, bs, ctx, qls = (cfg[k] for k in ("hq", "hkv", "d", "bs", "ctx", "qlens"))
    c0 = caches[0]
    threads = torch.get_num_threads()
    done_bytes = done_flops = 0
    t_total, reps = 0.0, 0
    order = [i for i, ql in enumerate(qls) if ql == 1] + [i for i, ql in enumerate(qls) if ql > 1]
    host, idx = {}, 0
    while t_total < seconds_target:                        # whole passes over the sample until the time is spent
        i = order[idx % len(order)]
        idx += 1
        n = (ctx[i] + bs - 1) // bs
        rows = min(qls[i], 64)
        if i not in host:                                  # gathered to the host untimed: the reference's cache lives there
            blocks = bt[i, :n].long().to(c0["k"].device)
            host[i] = tuple(c0[name][blocks].cpu() for name in ("k", "v", "ks", "vs")) + (
                q[int(cu[i + 1]) - rows:int(cu[i + 1])].cpu(),)
        kb, vb, ksb, vsb, qi = host[i]
        t0 = time.perf_counter()
        kd, vd = torch_ref.dequant_cache(kb, vb, ksb, vsb, d, torch.bfloat16)
        torch_ref.paged_attn(qi, kd, vd, [rows], [ctx[i]], torch.arange(n, dtype=torch.int32)[None], scale)
        t_total += time.perf_counter() - t0
        done_bytes += ctx[i] * hkv * 2 * (d + 4) + 2 * rows * hq * d * 2
        done_flops += 4 * d * hq * (rows * (ctx[i] - rows) + rows * (rows + 1) // 2)
        reps += 1
        if idx % len(order) == 0 and t_total > 0.6 * seconds_target:
            break
    return dict(value=done_bytes / t_total / 1e9, unit="GB/s", cores=threads, kind="port",
                tflops=done_flops / t_total / 1e12,
                sample=f"{reps} sequence runs = {reps / len(order):.2f} passes over the 60 decode rows and the last 64 query rows of each of the four chunks ("
                       f"{done_bytes / 1e6:.1f} MB of algorithmic bytes, {done_flops / 1e9:.1f} GFLOP), oracle/torch_ref.py "
                       f"dequant_cache + paged_attn (bf16, as-written), {t_total:.1f} s, torch threads={threads}")


def mixed_main(args, cfg, dev, ops):
    """configs[4]: write all new tokens (quantise-on-write), then ONE varlen attention call over the
    mixed batch.  ctx here is the sequence length INCLUDING the run's own tokens."""
    from vllm_metax_amd import layout as L

    hq, hkv, d, bs, ctx, qls, pool = (cfg[k] for k in ("hq", "hkv", "d", "bs", "ctx", "qlens", "pool"))
    mode = _quant_mode(cfg)
    B = len(ctx)
    g = torch.Generator().manual_seed(0)
    need = [(c + bs - 1) // bs for c in ctx]
    perm = torch.randperm(pool - 1, generator=g)[: sum(need)] + 1
    bt = torch.zeros((B, max(need)), dtype=torch.int32)
    o = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[o:o + n].to(torch.int32)
        o += n
    bt_d = bt.to(dev)
    sl_d = torch.tensor(ctx, dtype=torch.int32, device=dev)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    cu_d = cu.to(dev)
    n_tok = int(cu[-1])
    torch.manual_seed(0)
    caches = []
    new_slots = []
    for i, c in enumerate(ctx):
        pos = torch.arange(c - qls[i], c)
        new_slots.append(bt[i, pos // bs].long() * bs + pos % bs)
    new_slots = torch.cat(new_slots).to(dev)
    for _ in range(args.layers):
        kv = L.allocate_kv_cache(pool, bs, hkv, d, device=dev, layout=args.kv_layout, fill=0,
                                 cache_dtype_str=_cache_dtype_str(cfg))
        k, v = L.key_value_views(kv)
        ks, vs = L.scale_views(kv)
        ks.fill_(1.0)
        vs.fill_(1.0)
        geom = L.geometry_from_views(k, v, ks, vs, L.code_type_of(mode))
        for i, c in enumerate(ctx):
            pos = torch.arange(c, device=dev)
            slots = bt_d[i, pos // bs].to(torch.int64) * bs + pos % bs
            ops.reshape_and_cache_flash_per_token_head_quant(
                torch.randn((c, hkv, d), device=dev).to(torch.bfloat16), torch.randn((c, hkv, d), device=dev).to(torch.bfloat16),
                k, v, ks, vs, slots, geometry=geom, kv_quant_mode=mode)
        caches.append(dict(k=k, v=v, ks=ks, vs=vs, geom=geom, kv=kv))
    q = torch.randn((n_tok, hq, d), device=dev).to(torch.bfloat16)
    new_k = torch.randn((n_tok, hkv, d), device=dev).to(torch.bfloat16)
    new_v = torch.randn((n_tok, hkv, d), device=dev).to(torch.bfloat16)
    out = torch.empty_like(q)
    ws = torch.empty(ops.paged_attn_workspace_bytes(B, hq, d), dtype=torch.uint8, device=dev)
    scale = 1.0 / math.sqrt(d)

    # context splits of the long runs, as the metadata builder proposes them from the run lengths
    splits = ops.prefill_context_splits(qls, max(ctx), hq, hkv) if cfg.get("chunk") else 1
    if splits > 1:
        ws = torch.empty(ops.split_prefill_workspace_bytes(B, hq, d, n_tok, splits), dtype=torch.uint8, device=dev)

    def step(layer, write=True, attn=True, splits=splits):
        c = caches[layer]
        if write:
            ops.reshape_and_cache_flash_per_token_head_quant(new_k, new_v, c["k"], c["v"], c["ks"], c["vs"], new_slots,
                                                             geometry=c["geom"], kv_quant_mode=mode)
        if attn:
            ops.unified_attention(q, c["k"], c["v"], out, cu_d, max(qls), sl_d, max(ctx), scale, True, block_table=bt_d,
                                  k_scale_cache=c["ks"], v_scale_cache=c["vs"], workspace=ws, geometry=c["geom"],
                                  kv_quant_mode=mode, prefill_splits=splits,
                                  **_window_kwargs(dict(window=args.sliding_window, softcap=args.soft_cap)))

    Lr = args.layers
    prewarm(lambda i: step(i % Lr))
    for i in range(args.warmup):
        step(i % Lr)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i % Lr)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    n_ev = min(max(args.steps, 20), 100)
    attn_s = time_back_to_back(lambda i: step(i % Lr, write=False, attn=True), n_ev)
    # causal prefill flops: 4 D Hq (q_len * cached + q_len (q_len + 1) / 2); decode rows: 4 D Hq ctx
    flops = sum(4 * d * hq * (ql * (c - ql) + ql * (ql + 1) // 2) for c, ql in zip(ctx, qls))
    cb = d // 2 if cfg.get("kv_dtype") == "int4" else d
    dec_bytes = sum(c for c, ql in zip(ctx, qls) if ql == 1) * hkv * 2 * (cb + 4)
    pre_bytes = sum(c for c, ql in zip(ctx, qls) if ql > 1) * hkv * 2 * (cb + 4) + 2 * n_tok * hq * d * 2
    write_bytes = n_tok * hkv * (2 * d * 2 + 2 * (cb + 4))
    traffic, traffic_source = measured_traffic(args.workload)
    if args.sliding_window or args.soft_cap or cfg.get("kv_dtype") != "int8" or args.kv_layout != "HND":
        traffic, traffic_source = None, None
    if cfg.get("chunk"):
        unsplit_s = time_back_to_back(lambda i: step(i % Lr, write=False, attn=True, splits=1), min(n_ev, 20))
        res = {
            "metric": f"{cfg.get('kv_dtype', 'int8')}-KV prefill chunk of one request ({qls[0]} tokens on {ctx[0] - qls[0]} cached): TFLOP/s of the attention launch",
            "value": round(flops / attn_s / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None,
            "dtype": f"{cfg.get('kv_dtype', 'int8')} KV codes, fp16 MFMA operands, fp32 softmax/accumulate, bf16 Q/out",
            "data": "synthetic",
            "config": {"workload": args.workload, "batch": B, "new_tokens": n_tok, "sum_ctx": sum(ctx), "q_heads": hq,
                       "kv_heads": hkv, "head_dim": d, "block_size": bs, "layer_caches_rotated": Lr,
                       "kv_layout": args.kv_layout, "context_splits": splits},
            "prewarm_s": PREWARM_S, "attn_launch_us": round(attn_s * 1e6, 1),
            "attn_launch_us_without_context_splits": round(unsplit_s * 1e6, 1),
            "roofline": {"bound": "mfma", "achieved": round(flops / attn_s / 1e12, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(flops / attn_s / 1e12 / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                         "timing": f"{n_ev} attention launches back to back between two events on the launch stream",
                         "kernel": "varlen attention launch = prefill_plan_kernel + paged_prefill_flash32_kernel (context splits) + prefill_split_merge_kernel",
                         "algorithmic_flops_per_launch": flops},
        }
        print(json.dumps(res))
        return
    if cfg.get("spec"):
        # a memory-bound step: every record of every context is read once, as in a decode step
        res = {
            "metric": f"{cfg.get('kv_dtype', 'int8')}-KV speculative-decoding step ({B} sequences x {qls[0]} query tokens): achieved HBM GB/s",
            "value": round(pre_bytes / attn_s / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None,
            "dtype": f"{cfg.get('kv_dtype', 'int8')} KV codes, fp16 MFMA operands, fp32 softmax/accumulate, bf16 Q/out",
            "data": "synthetic",
            "config": {"workload": args.workload, "batch": B, "new_tokens": n_tok, "sum_ctx": sum(ctx), "q_heads": hq,
                       "kv_heads": hkv, "head_dim": d, "block_size": bs, "layer_caches_rotated": Lr,
                       "kv_layout": args.kv_layout},
            "prewarm_s": PREWARM_S, "attn_launch_us": round(attn_s * 1e6, 1),
            "roofline": {"bound": "hbm", "achieved": round(pre_bytes / attn_s / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(pre_bytes / attn_s / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None,
                         "timing": f"{n_ev} attention launches back to back between two events on the launch stream",
                         "kernel": "varlen attention launch = prefill_plan_kernel + paged_prefill_kernel (an item's tiles spread over a workgroup's waves)",
                         "algorithmic_bytes_per_launch": pre_bytes},
        }
        print(json.dumps(res))
        return
    res = {
        "metric": f"{cfg.get('kv_dtype', 'int8')}-KV mixed batch (4 x 2048-token prefill chunks + 60 decode rows): ms per layer",
        "value": round((dec_bytes + pre_bytes + write_bytes) / dt / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": f"{cfg.get('kv_dtype', 'int8')} KV codes, fp16 MFMA operands, fp32 softmax/accumulate, bf16 Q/out", "data": "synthetic",
        "config": {"workload": args.workload,
                   **({"kv_dtype": cfg["kv_dtype"] + "_per_token_head"} if cfg.get("kv_dtype") != "int8" else {}),
                   **({"sliding_window": args.sliding_window} if args.sliding_window else {}),
                   **({"soft_cap": args.soft_cap} if args.soft_cap else {}),
                   "batch": B, "new_tokens": n_tok, "sum_ctx": sum(ctx), "q_heads": hq,
                   "kv_heads": hkv, "head_dim": d, "block_size": bs, "layer_caches_rotated": Lr,
                   "kv_layout": args.kv_layout},
        "prewarm_s": PREWARM_S, "attn_launch_us": round(attn_s * 1e6, 1),
        "roofline": {"bound": "mfma", "achieved": round(flops / attn_s / 1e12, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(flops / attn_s / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "timing": f"{n_ev} attention launches back to back between two events on the launch stream",
                     "kernel": "varlen attention launch = paged_decode_streamk_kernel + reduce + prefill_plan_kernel + paged_prefill_flash32_kernel",
                     "algorithmic_flops_per_launch": flops, "algorithmic_bytes_per_launch": dec_bytes + pre_bytes},
    }
    if not args.no_cpu_baseline and cfg.get("kv_dtype") == "int8":
        res["cpu_baseline"] = mixed_cpu_baseline(cfg, caches, bt, q, cu, scale, args.cpu_seconds)
    print(json.dumps(res))


def cpu_baseline(cfg, st, seconds_target=15.0):
    """The reference's CPU path (as-written torch ops, bf16 Q.K / fp32 softmax / bf16 P.V) on a
    bounded sample of the batch: dequantise the sampled sequences' blocks, then ref_paged_attn."""
    from oracle import torch_ref

    hq, hkv, d, bs, ctx = cfg["hq"], cfg["hkv"], cfg["d"], cfg["bs"], cfg["ctx"]
    c0 = st["caches"][0]
    order = sorted(range(len(ctx)), key=lambda i: ctx[i])
    q_cpu = st["q"].cpu()
    threads = torch.get_num_threads()
    done_bytes, t_total, reps = 0, 0.0, 0
    idx = 0
    cand = [order[len(order) // 2]] + [i for i in order if i != order[len(order) // 2]]
    host = {}                                              # sequence -> its blocks on the host
    while t_total < seconds_target:                        # whole passes over the batch until the time is spent
        i = cand[idx % len(cand)]
        idx += 1
        n = (ctx[i] + bs - 1) // bs
        if i not in host:
            blocks = st["bt"][i, :n].long().to(c0["k"].device)
            # gather this sequence's blocks to the host (not timed: the reference's cache would already live there)
            host[i] = tuple(c0[name][blocks].cpu() for name in ("k", "v", "ks", "vs"))
        kb, vb, ksb, vsb = host[i]
        local_bt = torch.arange(n, dtype=torch.int32)[None]
        t0 = time.perf_counter()
        kd, vd = torch_ref.dequant_cache(kb, vb, ksb, vsb, d, torch.bfloat16)
        torch_ref.paged_attn(q_cpu[i:i + 1], kd, vd, [1], [ctx[i]], local_bt, st["scale"])
        t_total += time.perf_counter() - t0
        done_bytes += ctx[i] * hkv * 2 * (d + 4) + 2 * hq * d * 2 + n * 4 + 4
        reps += 1
        if idx % len(cand) == 0 and t_total > 0.6 * seconds_target:
            break                                          # stop on a pass boundary once most of the time is spent
    return dict(value=done_bytes / t_total / 1e9, unit="GB/s", cores=threads, kind="port",
                sample=f"{reps} sequence runs = {reps / len(cand):.2f} passes over the batch ({done_bytes / 1e6:.1f} MB of algorithmic bytes), "
                       f"oracle/torch_ref.py dequant_cache + paged_attn (bf16, as-written), {t_total:.1f} s, "
                       f"torch threads={threads}, os.cpu_count()={os.cpu_count()}",
                us_per_layer_extrapolated=t_total / done_bytes * algorithmic_bytes(cfg, False)[0] * 1e6)


def time_decode(cfg, st, args, ops):
    """Pre-warm, W untimed and K timed steps (write + attention) on the host clock around a device
    synchronisation; then the attention launch and the write launch on their own, back to back."""
    attn_bytes, write_bytes = algorithmic_bytes(cfg)
    if args.sliding_window:  # a windowed decode row reads only its last `window` tokens
        attn_bytes, _ = algorithmic_bytes(dict(cfg, ctx=[min(c, args.sliding_window) for c in cfg["ctx"]]))
    L = args.layers
    prewarm(lambda i: run_step(st, i % L, ops))
    for i in range(args.warmup):
        run_step(st, i % L, ops)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        run_step(st, i % L, ops)
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / args.steps
    n = max(args.steps, 100)
    attn_s = time_back_to_back(lambda i: run_step(st, i % L, ops, write=False, attn=True), n)
    write_host_s = time_back_to_back(lambda i: run_step(st, i % L, ops, write=True, attn=False), n)
    write_s = time_graph_replay(lambda i: run_step(st, i % L, ops, write=True, attn=False), 100)
    # the attention launch as GPU time only (50 launches in one HIP graph): differs from attn_s where the launch is
    # shorter than the host's call (small batches)
    attn_graph_s = time_graph_replay(lambda i: run_step(st, i % L, ops, write=False, attn=True), 50)
    fused_s = None
    if not args.no_one_launch:
        # the same step as ONE launch (the decode kernel writes the new tokens), timed like the two-launch step
        for i in range(args.warmup):
            run_step(st, i % L, ops, fused=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            run_step(st, i % L, ops, fused=True)
        torch.cuda.synchronize()
        fused_s = (time.perf_counter() - t0) / args.steps
    return dict(step_s=step_s, attn_s=attn_s, write_s=write_s, write_host_s=write_host_s, attn_bytes=attn_bytes, n_attn=n,
                value=(attn_bytes + write_bytes) / step_s / 1e9, fused_s=fused_s, attn_graph_s=attn_graph_s,
                fused_value=(attn_bytes + write_bytes) / fused_s / 1e9 if fused_s else None)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--workload", default="llama3_8b_decode_b64_ctx1k-8k")
    ap.add_argument("--layers", type=int, default=4, help="distinct layer caches the steps rotate over")
    ap.add_argument("--sliding-window", type=int, default=0,
                    help="GQA workloads: attend to the last N keys only (0 = full causal, the configured workloads)")
    ap.add_argument("--soft-cap", type=float, default=0.0, help="GQA workloads: logits soft cap (0 = none)")
    ap.add_argument("--kv-dtype", choices=["int8", "fp8", "int4"], default="int8",
                    help="GQA workloads: code format of the cache (fp8 = e4m3fn per-token-head mode of the same layout; "
                         "int4 = two 4-bit codes per byte, half the code bytes)")
    ap.add_argument("--kv-layout", choices=["HND", "NHD"], default=None,
                    help="GQA workloads: memory order of the cache tensor, both of which the reference defines "
                         "(triton_attn.py:350-372, VLLM_KV_CACHE_LAYOUT).  Default: what the backend itself asks for "
                         "(vllm_metax_amd.layout.get_kv_cache_layout(): HND unless the environment says otherwise), "
                         "so that the headline is the order a deployment gets; the default workload reports the other "
                         "order too")
    ap.add_argument("--seed", type=int, default=0,
                    help="draw of the workload's random context lengths (0 = the draw every published figure uses)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-one-launch", action="store_true",
                    help="skip the one-launch variant of the step (write inside the decode launch): for profiler runs, "
                         "where its dispatches would be averaged into the decode kernel's row")
    ap.add_argument("--no-fixed-8k", action="store_true",
                    help="default workload only: skip the extra fixed-context (64 x 8192) measurement")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU (no collectives, no sharding); use --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible; the HIP kernels have no CPU fallback")
    from vllm_metax_amd import _custom_ops as ops
    from vllm_metax_amd.layout import get_kv_cache_layout

    if args.kv_layout is None:
        args.kv_layout = get_kv_cache_layout()
    dev = torch.device("cuda:0")
    cfg = make_batch(args.workload, args.seed)
    cfg["kv_dtype"] = args.kv_dtype
    if cfg.get("mla_prefill"):
        return mla_prefill_main(args, cfg, dev, ops)
    if cfg.get("mla"):
        return mla_main(args, cfg, dev, ops)
    if cfg.get("mixed"):
        return mixed_main(args, cfg, dev, ops)
    st = build_device_state(cfg, dev, args.layers, layout=args.kv_layout)
    st["window"], st["softcap"] = args.sliding_window, args.soft_cap
    L = args.layers
    t = time_decode(cfg, st, args, ops)
    traffic, traffic_source = measured_traffic(args.workload)
    if args.sliding_window or args.soft_cap or args.kv_dtype != "int8" or args.kv_layout != "HND" or ops.batch_invariant():
        traffic, traffic_source = None, None   # the profiles were taken on the plain int8 workload in HND order

    res = {
        "metric": METRIC,
        "value": round(t["value"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(t["step_s"] * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": f"{args.kv_dtype} KV codes, fp16 MFMA operands, fp32 softmax/accumulate, bf16 Q/out",
        "data": "synthetic",
        "config": {"workload": args.workload, "batch": len(cfg["ctx"]), "sum_ctx": sum(cfg["ctx"]),
                   "q_heads": cfg["hq"], "kv_heads": cfg["hkv"], "head_dim": cfg["d"], "block_size": cfg["bs"],
                   "pool_blocks": cfg["pool"], "layer_caches_rotated": L, "kv_layout": args.kv_layout,
                   **({"batch_invariant": True} if ops.batch_invariant() else {}),
                   **({"lengths_seed": args.seed} if args.seed else {}),
                   **({"kv_dtype": args.kv_dtype + "_per_token_head"} if args.kv_dtype != "int8" else {}),
                   **({"sliding_window": args.sliding_window} if args.sliding_window else {}),
                   **({"soft_cap": args.soft_cap} if args.soft_cap else {})},
        "prewarm_s": PREWARM_S,
        "pct_hbm_peak": round(100 * t["value"] / HBM_PEAK_GBPS, 2),
        "us_per_layer": round(t["step_s"] * 1e6, 2),
        "decode_tokens_per_s": round(len(cfg["ctx"]) / t["step_s"], 1),
        "attn_launch_us": round(t["attn_s"] * 1e6, 2),
        # GPU time of the write kernel (100 launches in one HIP graph, replayed between two events), and what one
        # call costs when the host issues them one by one (bound by the host, not by the kernel)
        "write_launch_us": round(t["write_s"] * 1e6, 2),
        "write_call_host_us": round(t["write_host_s"] * 1e6, 2),
        "attn_launch_in_graph_us": round(t["attn_graph_s"] * 1e6, 2),
        "one_launch_step": None if t["fused_s"] is None else {
            "what": "the same step with the cache update inside the attention launch "
                    "(kvq_paged_attn_int8_fused_write; a backend with forward_includes_kv_cache_update)",
            "us_per_layer": round(t["fused_s"] * 1e6, 2), "value": round(t["fused_value"], 1), "unit": "GB/s",
            "pct_hbm_peak": round(100 * t["fused_value"] / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(t["attn_bytes"] / t["attn_s"] / 1e9, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(t["attn_bytes"] / t["attn_s"] / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "paged decode attention launch = paged_decode_streamk_kernel + a reduce kernel (paged_decode_streamk_reduce_split4_kernel up to 16 sequences, _reduce_by_seq_kernel up to 96, _reduce_kernel beyond)",
                     "timing": f"{t['n_attn']} attention launches back to back between two events on the launch stream",
                     "algorithmic_bytes_per_launch": t["attn_bytes"]},
    }
    if args.workload == "llama3_8b_decode_b64_ctx1k-8k" and not (args.sliding_window or args.soft_cap or args.no_fixed_8k
                                                                  or args.kv_dtype != "int8"):
        # the shape the metric's wording names (every context 8192), same steps, in the same line
        cfg8 = make_batch("llama3_8b_decode_b64_ctx8k_fixed")
        cfg8["kv_dtype"] = "int8"
        st8 = build_device_state(cfg8, dev, args.layers, layout=args.kv_layout)
        st8["window"], st8["softcap"] = 0, 0.0
        t8 = time_decode(cfg8, st8, args, ops)
        res["fixed_ctx_8192"] = {
            "workload": "llama3_8b_decode_b64_ctx8k_fixed", "sum_ctx": sum(cfg8["ctx"]),
            "value": round(t8["value"], 1), "unit": "GB/s", "pct_hbm_peak": round(100 * t8["value"] / HBM_PEAK_GBPS, 2),
            "us_per_layer": round(t8["step_s"] * 1e6, 2), "decode_tokens_per_s": round(len(cfg8["ctx"]) / t8["step_s"], 1),
            "attn_launch_us": round(t8["attn_s"] * 1e6, 2),
            "roofline_frac": round(t8["attn_bytes"] / t8["attn_s"] / 1e9 / HBM_PEAK_GBPS, 4),
            "algorithmic_bytes_per_launch": t8["attn_bytes"]}
        del st8
        # the same workload in the other memory order of the cache, same steps
        other = "NHD" if args.kv_layout == "HND" else "HND"
        sto = build_device_state(cfg, dev, args.layers, layout=other)
        sto["window"], sto["softcap"] = 0, 0.0
        to = time_decode(cfg, sto, args, ops)
        res["other_kv_layout"] = {
            "kv_layout": other, "value": round(to["value"], 1), "unit": "GB/s",
            "pct_hbm_peak": round(100 * to["value"] / HBM_PEAK_GBPS, 2), "us_per_layer": round(to["step_s"] * 1e6, 2),
            "attn_launch_us": round(to["attn_s"] * 1e6, 2),
            "roofline_frac": round(to["attn_bytes"] / to["attn_s"] / 1e9 / HBM_PEAK_GBPS, 4)}
        del sto
    if not args.no_cpu_baseline and args.kv_dtype == "int8":
        res["cpu_baseline"] = cpu_baseline(cfg, st, args.cpu_seconds)
    print(json.dumps(res))


if __name__ == "__main__":
    main()

"""Shared helpers of the test-suite: seeded synthetic inputs and CPU-side cache building.

The cache is always built on the CPU with the oracle's quantiser, as raw int8 storage in
the product's layout; GPU tests copy those bytes to the device.  Nothing here reads the
reference tree."""
from __future__ import annotations

import math

import torch

import oracle
from vllm_metax_amd import layout as L


def make_block_tables(ctx_lens, block_size, num_blocks, gen, reserve_null_block=True):
    """Random-permutation block tables over a pool (block 0 kept as the null block, as the
    reference's backend tests do, tests/v1/attention/test_attention_backends.py:74-171)."""
    need = [(c + block_size - 1) // block_size for c in ctx_lens]
    total = sum(need)
    first = 1 if reserve_null_block else 0
    assert total + first <= num_blocks, (total, num_blocks)
    perm = torch.randperm(num_blocks - first, generator=gen)[:total] + first
    width = max(max(need), 1)
    bt = torch.zeros((len(ctx_lens), width), dtype=torch.int32)
    o = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[o:o + n].to(torch.int32)
        o += n
    return bt


def slots_for(bt, ctx_lens, block_size):
    """slot ids of every context token, per sequence: list of int64 tensors."""
    out = []
    for i, c in enumerate(ctx_lens):
        pos = torch.arange(c)
        out.append(bt[i, pos // block_size].to(torch.int64) * block_size + pos % block_size)
    return out


def _dtype_str(code_type):
    return {oracle.CODE_INT8: "int8_per_token_head", oracle.CODE_FP8: "fp8_per_token_head",
            oracle.CODE_INT4: "int4_per_token_head"}[code_type]


def cpu_cache(num_blocks, block_size, hkv, d, layout="NHD", fill=0, code_type=oracle.CODE_INT8):
    kv = L.allocate_kv_cache(num_blocks, block_size, hkv, d, device="cpu", layout=layout, fill=fill,
                             cache_dtype_str=_dtype_str(code_type))
    k, v = L.key_value_views(kv)
    ks, vs = L.scale_views(kv)
    lay = oracle.RecordLayout.from_views(_storage_base(kv), k, v, ks, vs, code_type)
    return kv, (k, v, ks, vs), lay


class _Base:
    def __init__(self, ptr):
        self._p = ptr

    def data_ptr(self):
        return self._p


def _storage_base(t):
    return _Base(t.untyped_storage().data_ptr())


def storage_bytes(t):
    """The whole underlying storage of a cache tensor as a flat uint8 tensor (shares memory)."""
    return torch.tensor([], dtype=torch.uint8, device=t.device).set_(t.untyped_storage())


def fill_cache_from_sources(kv, lay, bt, ctx_lens, block_size, k_src, v_src, code_type=oracle.CODE_INT8):
    """Quantise per-sequence K/V sources ([ctx, Hkv, D] each) into the CPU cache with the oracle."""
    base = storage_bytes(kv)
    for i, slots in enumerate(slots_for(bt, ctx_lens, block_size)):
        if slots.numel() > 0:  # an empty sequence writes nothing
            oracle.cache_write(k_src[i], v_src[i], base, lay, slots, code_type=code_type)


def to_device_cache(kv_cpu, device, layout, code_type=oracle.CODE_INT8):
    """Same bytes, same layout, on the GPU; returns the logical-shape tensor."""
    nb, hkv, bs, content = kv_cpu.shape
    d = (content // 2 - 4) * (2 if code_type == oracle.CODE_INT4 else 1)
    kv = L.allocate_kv_cache(nb, bs, hkv, d, device=device, layout=layout, fill=None,
                             cache_dtype_str=_dtype_str(code_type))
    storage_bytes(kv).copy_(storage_bytes(kv_cpu).to(device))
    return kv


def outlier_sources(shape, gen, dtype=torch.float32, frac=0.01, mult=20.0):
    """N(0,1) with a fixed 1 % of the (head, dim) channels scaled x20 (the long-context config)."""
    t, h, d = shape
    x = torch.randn(shape, generator=gen, dtype=torch.float32)
    n = max(1, int(round(frac * h * d)))
    ch = torch.randperm(h * d, generator=gen)[:n]
    x.view(t, h * d)[:, ch] *= mult
    return x.to(dtype)


def assert_close_attn(got, want, atol=2e-2, rtol=1e-2, what=""):
    """north-star tolerance for bf16 attention outputs against the fp32-accumulated oracle."""
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max |err| {err.max().item():.4g}, worst excess over atol+rtol*|ref| {worst:.4g}"


def build_mla_cache(ctx, bs, seed, dtype=torch.bfloat16, poison=True, amp=1.0, rows_fn=None, R=512, P=64):
    """A latent cache written by the oracle for sequences of the given lengths, blocks shuffled.
    ``rows_fn(kv_c, k_pe)`` may reshape the random rows of a sequence before they are quantised."""
    g = torch.Generator().manual_seed(seed)
    B = len(ctx)
    per = [(c + bs - 1) // bs for c in ctx]
    nb = sum(per) + 3
    order = torch.randperm(nb, generator=g).tolist()
    cache = L.allocate_mla_cache(nb, bs, R + P, device="cpu", fill=-1 if poison else 0)  # all-ones bytes: unwritten scales read as NaN
    codes, scales = L.mla_cache_views(cache)
    lay = oracle.MlaLayout.from_views(cache, codes, scales, R)
    bt = torch.zeros((B, max(max(per), 1)), dtype=torch.int32)
    it = iter(order)
    for i, c in enumerate(ctx):
        blocks = [next(it) for _ in range(per[i])]
        bt[i, : per[i]] = torch.tensor(blocks, dtype=torch.int32)
        if c == 0:
            continue
        kv_c = (torch.randn((c, R), generator=g) * amp).to(dtype)
        k_pe = (torch.randn((c, P), generator=g) * amp).to(dtype)
        if rows_fn is not None:
            kv_c, k_pe = rows_fn(kv_c.float(), k_pe.float())
            kv_c, k_pe = kv_c.to(dtype), k_pe.to(dtype)
        pos = torch.arange(c)
        slots = (bt[i, pos // bs].long() * bs + pos % bs)
        oracle.mla_cache_write(kv_c, k_pe, cache, lay, slots)
    return cache, lay, bt, torch.tensor(ctx, dtype=torch.int32)

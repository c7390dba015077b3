"""Block moves over the int8 cache format (swap_blocks / swap_blocks_batch), through the C ABI.

Pattern of the reference's tests/kernels/attention/test_cache.py:352-432 (test_swap_blocks: random
non-overlapping pairs, every direction, compare moved blocks with a clone of the source) and
:640-700 (test_swap_blocks_mla), applied to the layouts of this path: a block carries codes and
fp32 scales, so a moved block must dequantise -- and attend -- exactly as before.  Byte moves:
the bar is bit-exact."""
import math
import random

import pytest
import torch

import kvq_testlib as T
import oracle
from test_gpu_prefill import build
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def block_bytes(kv):
    return kv.stride(0) * kv.element_size()


def as_blocks(kv):
    """(nb, block_bytes) uint8 view of a cache tensor's storage."""
    return T.storage_bytes(kv)[: kv.shape[0] * block_bytes(kv)].view(kv.shape[0], block_bytes(kv))


@pytest.mark.parametrize("direction", [("cuda", "cuda"), ("cuda", "cpu"), ("cpu", "cuda")])
@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("num_mappings", [1, 37, 300])
def test_swap_blocks_gqa_cache(gpu_device, direction, layout, num_mappings):
    nb, bs, hkv, d = 700, 16, 8, 128
    random.seed(num_mappings)
    g = torch.Generator().manual_seed(num_mappings)
    devs = [gpu_device if x == "cuda" else torch.device("cpu") for x in direction]
    src = L.allocate_kv_cache(nb, bs, hkv, d, device=devs[0], layout=layout, fill=None)
    dst = L.allocate_kv_cache(nb, bs, hkv, d, device=devs[1], layout=layout, fill=None)
    as_blocks(src).copy_(torch.randint(0, 256, as_blocks(src).shape, generator=g, dtype=torch.uint8))
    as_blocks(dst).copy_(torch.randint(0, 256, as_blocks(dst).shape, generator=g, dtype=torch.uint8))
    src_blocks = random.sample(range(nb), num_mappings)
    dst_blocks = random.sample(range(nb), num_mappings)
    mapping = torch.tensor(list(zip(src_blocks, dst_blocks)), dtype=torch.int64, device="cpu").view(-1, 2)
    src_clone = as_blocks(src).cpu().clone()
    dst_before = as_blocks(dst).cpu().clone()
    ops.swap_blocks(src, dst, block_bytes(src), mapping)
    torch.cuda.synchronize()
    got = as_blocks(dst).cpu()
    want = dst_before.clone()
    want[dst_blocks] = src_clone[src_blocks]
    assert torch.equal(got, want)                         # moved blocks arrived, every other block untouched
    assert torch.equal(as_blocks(src).cpu(), src_clone)   # the source is only read


def test_swap_blocks_same_tensor_and_strided_mapping(gpu_device):
    """Copy inside one allocation (non-overlapping pairs), mapping given as a strided view."""
    nb = 64
    kv = L.allocate_kv_cache(nb, 16, 4, 64, device=gpu_device, fill=None)
    as_blocks(kv).copy_(torch.randint(0, 256, as_blocks(kv).shape, dtype=torch.uint8).to(gpu_device))
    before = as_blocks(kv).cpu().clone()
    wide = torch.zeros((20, 4), dtype=torch.int64)
    wide[:, 0] = torch.arange(0, 20)
    wide[:, 2] = torch.arange(40, 60)
    mapping = wide[:, ::2]                                 # strides (4, 2)
    ops.swap_blocks(kv, kv, block_bytes(kv), mapping)
    torch.cuda.synchronize()
    want = before.clone()
    want[40:60] = before[0:20]
    assert torch.equal(as_blocks(kv).cpu(), want)


def test_swap_blocks_mla_cache(gpu_device):
    nb, bs = 40, 64
    src = L.allocate_mla_cache(nb, bs, 576, device=gpu_device)
    dst = L.allocate_mla_cache(nb, bs, 576, device=gpu_device)
    src.view(torch.uint8).random_(0, 256)
    dst.view(torch.uint8).random_(0, 256)
    src_clone, dst_before = src.cpu().clone(), dst.cpu().clone()
    mapping = torch.tensor([[3, 7], [0, 39], [12, 1]], dtype=torch.int64)
    ops.swap_blocks(src, dst, src.stride(0) * src.element_size(), mapping)
    torch.cuda.synchronize()
    want = dst_before.clone()
    want[[7, 39, 1]] = src_clone[[3, 0, 12]]
    assert torch.equal(dst.cpu(), want)


def test_swapped_out_and_back_in_cache_attends_identically(gpu_device):
    """Swap every block of a filled cache out to pinned host memory, scramble the device cache, swap
    the blocks back in at NEW block numbers and attend through the remapped block table: the output
    is bit-identical to the one before the round trip (codes and scales travel together)."""
    ctx, qls = [300, 77, 129], [1, 1, 1]
    hq, hkv, d, bs = 8, 2, 128, 16
    kv_cpu, lay, bt, q, sl, cu = build(ctx, qls, hq, hkv, d, bs, seed=3)
    dev = gpu_device
    kv = T.to_device_cache(kv_cpu, dev, "NHD")
    nb = kv.shape[0]

    def attend(cache, table):
        k, v = L.key_value_views(cache)
        ks, vs = L.scale_views(cache)
        out = torch.empty(q.shape, dtype=torch.float32, device=dev)
        ops.unified_attention(q.to(dev), k, v, out, cu.to(dev), 1, sl.to(dev), int(sl.max()), 1 / math.sqrt(d), True,
                              block_table=table.to(dev), k_scale_cache=ks, v_scale_cache=vs)
        torch.cuda.synchronize()
        return out.cpu()

    before = attend(kv, bt)
    want = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, 1 / math.sqrt(d))
    T.assert_close_attn(before, want, what="before the swap")

    host = torch.empty((nb, block_bytes(kv)), dtype=torch.uint8, pin_memory=True)
    ident = torch.arange(nb, dtype=torch.int64)
    ops.swap_blocks(kv, host, block_bytes(kv), torch.stack([ident, ident], dim=1))
    torch.cuda.synchronize()
    as_blocks(kv).fill_(0xA5)
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(0))
    ops.swap_blocks(host, kv, block_bytes(kv), torch.stack([ident, perm], dim=1))   # block i -> perm[i]
    torch.cuda.synchronize()
    after = attend(kv, perm[bt.long()].to(torch.int32))
    assert torch.equal(before, after)


@pytest.mark.parametrize("all_on_device", [False, True])
def test_swap_blocks_batch(gpu_device, all_on_device):
    """Arbitrary (pointer, pointer, size) triples, including sizes that are no multiple of 16, a
    zero-length entry and (in the general mode) host memory."""
    g = torch.Generator().manual_seed(5)
    src = torch.randint(0, 256, (1 << 20,), generator=g, dtype=torch.uint8).to(gpu_device)
    dst = torch.zeros(1 << 20, dtype=torch.uint8, device=gpu_device)
    host = torch.zeros(1 << 16, dtype=torch.uint8, pin_memory=True)
    entries = [(0, 0, 33792), (40000, 50000, 4096), (100001, 200003, 777), (300000, 300000, 0), (500000, 600000, 70000)]
    sp = [src.data_ptr() + a for a, _, _ in entries]
    dp = [dst.data_ptr() + b for _, b, _ in entries]
    sz = [n for _, _, n in entries]
    if not all_on_device:
        sp.append(src.data_ptr() + 1234)
        dp.append(host.data_ptr())
        sz.append(5000)
    ops.swap_blocks_batch(torch.tensor(sp, dtype=torch.int64), torch.tensor(dp, dtype=torch.int64),
                          torch.tensor(sz, dtype=torch.int64), all_on_device=all_on_device)
    torch.cuda.synchronize()
    want = torch.zeros(1 << 20, dtype=torch.uint8)
    s_cpu = src.cpu()
    for a, b, n in entries:
        want[b:b + n] = s_cpu[a:a + n]
    assert torch.equal(dst.cpu(), want)
    if not all_on_device:
        assert torch.equal(host[:5000], s_cpu[1234:6234]) and int(host[5000:].sum()) == 0


@pytest.mark.parametrize("kind", ["gqa_nhd", "gqa_hnd", "mla"])
@pytest.mark.parametrize("num_mappings,num_layers", [(1, 1), (7, 3), (60, 5)])
def test_copy_blocks(gpu_device, kind, num_mappings, num_layers):
    """The reference's test_copy_blocks / test_copy_blocks_mla (tests/kernels/attention/test_cache.py:
    55-110, 592-650): every source block goes to TWO destinations, in every layer; compared with the
    same copies done on clones.  Bytes must match, codes and scales alike."""
    nb = 256
    random.seed(num_mappings + num_layers)
    src_blocks = random.sample(range(nb), num_mappings)
    rest = list(set(range(nb)) - set(src_blocks))
    dst_blocks = random.sample(rest, 2 * num_mappings)
    mapping = []
    for i, s_ in enumerate(src_blocks):
        mapping += [(s_, dst_blocks[2 * i]), (s_, dst_blocks[2 * i + 1])]
    caches = []
    for _ in range(num_layers):
        if kind == "mla":
            kv = L.allocate_mla_cache(nb, 64, 576, device=gpu_device)
            kv.view(torch.uint8).random_(0, 256)
        else:
            kv = L.allocate_kv_cache(nb, 16, 4, 128, device=gpu_device, layout="NHD" if kind == "gqa_nhd" else "HND", fill=None)
            as_blocks(kv).random_(0, 256)
        caches.append(kv)
    raw = (lambda kv: kv.view(torch.uint8).reshape(nb, -1)) if kind == "mla" else as_blocks
    want = [raw(kv).cpu().clone() for kv in caches]
    for s_, d_ in mapping:
        for w in want:
            w[d_] = w[s_]
    mapping_t = torch.tensor(mapping, dtype=torch.int64, device=gpu_device).view(-1, 2)
    (ops.copy_blocks_mla if kind == "mla" else ops.copy_blocks)(caches, mapping_t)
    torch.cuda.synchronize()
    for kv, w in zip(caches, want):
        assert torch.equal(raw(kv).cpu(), w)


def test_copy_blocks_skips_bad_pairs_and_checks_arguments(gpu_device):
    nb = 16
    kv = L.allocate_kv_cache(nb, 16, 2, 64, device=gpu_device, fill=None)
    as_blocks(kv).random_(0, 256)
    before = as_blocks(kv).cpu().clone()
    mapping = torch.tensor([[3, 5], [2, 99], [-1, 4], [7, 7]], dtype=torch.int64, device=gpu_device)
    ops.copy_blocks([kv], mapping)                          # one valid pair; the others name no block
    torch.cuda.synchronize()
    want = before.clone()
    want[5] = before[3]
    assert torch.equal(as_blocks(kv).cpu(), want)
    ops.copy_blocks([], mapping)
    ops.copy_blocks([kv], torch.zeros((0, 2), dtype=torch.int64, device=gpu_device))
    with pytest.raises(RuntimeError):                       # mapping on the CPU
        ops.copy_blocks([kv], mapping.cpu())
    with pytest.raises(RuntimeError):
        ops.copy_blocks([kv], mapping.to(torch.int32))
    other = L.allocate_kv_cache(nb + 1, 16, 2, 64, device=gpu_device, fill=None)
    with pytest.raises(RuntimeError):                       # layers of different shapes
        ops.copy_blocks([kv, other], mapping)


def test_argument_errors(gpu_device):
    kv = L.allocate_kv_cache(8, 16, 2, 64, device=gpu_device)
    cpu = L.allocate_kv_cache(8, 16, 2, 64, device="cpu")
    bb = block_bytes(kv)
    with pytest.raises(RuntimeError):                     # mapping on the GPU (the reference refuses it too)
        ops.swap_blocks(kv, kv, bb, torch.zeros((1, 2), dtype=torch.int64, device=gpu_device))
    with pytest.raises(RuntimeError):                     # cpu -> cpu
        ops.swap_blocks(cpu, cpu, bb, torch.zeros((1, 2), dtype=torch.int64))
    with pytest.raises(RuntimeError):                     # block number past the end
        ops.swap_blocks(kv, kv, bb, torch.tensor([[0, 8]], dtype=torch.int64))
    with pytest.raises(RuntimeError):
        ops.swap_blocks(kv, kv, bb, torch.tensor([[-1, 2]], dtype=torch.int64))
    with pytest.raises(RuntimeError):
        ops.swap_blocks_batch(torch.zeros(2, dtype=torch.int64), torch.zeros(3, dtype=torch.int64),
                              torch.zeros(2, dtype=torch.int64))
    ops.swap_blocks(kv, kv, bb, torch.zeros((0, 2), dtype=torch.int64))   # empty mapping: nothing to do

"""GPU test of kvq_paged_attn_int8_static_scratch, the entry point that allocates nothing: called
through the C ABI, its output must equal kvq_paged_attn_int8's bit for bit (same kernels, the
split-K states in the library's own fixed array instead of a caller workspace) and lie within
atol 2e-2 / rtol 1e-2 of the oracle -- on two calls in a row, the second on a smaller batch, so
that what the first call left in the shared array is seen not to leak into the second."""
import ctypes
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _C
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


def _case(ctx, qls, hq, hkv, d, bs, seed):
    g = torch.Generator().manual_seed(seed)
    nb = sum((c + bs - 1) // bs for c in ctx) + 5
    kv, _, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    T.storage_bytes(kv).fill_(0xFF)
    bt = T.make_block_tables(ctx, bs, nb, g)
    ks = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    vs = [torch.randn((c, hkv, d), generator=g).to(torch.bfloat16) for c in ctx]
    T.fill_cache_from_sources(kv, lay, bt, ctx, bs, ks, vs)
    q = torch.randn((sum(qls), hq, d), generator=g).to(torch.bfloat16)
    sl = torch.tensor(ctx, dtype=torch.int32)
    cu = torch.tensor([0] + torch.tensor(qls).cumsum(0).tolist(), dtype=torch.int32)
    return kv, lay, bt, q, sl, cu


def _geometry(kv):
    k, v = L.key_value_views(kv)
    ksc, vsc = L.scale_views(kv)
    return L.geometry_from_views(k, v, ksc, vsc)


def _enqueue(dev, static, kv, bt, q, sl, cu, max_q, scale, out, lse, ws=None, geom=None):
    """One call through the C ABI on torch's current stream, without waiting for it."""
    lib = _C.load()
    geom = geom or _geometry(kv)
    g = geom.as_struct()
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    head = (ctypes.c_void_p(out.data_ptr()), _C.KVQ_BF16, out.stride(0), out.stride(1),
            ctypes.c_void_p(q.data_ptr()), _C.KVQ_BF16, q.stride(0), q.stride(1),
            ctypes.c_void_p(geom.base_ptr), ctypes.byref(g), ctypes.c_void_p(bt.data_ptr()), bt.stride(0),
            ctypes.c_void_p(sl.data_ptr()), ctypes.c_void_p(cu.data_ptr()), sl.shape[0], q.shape[1], max_q,
            scale, 1, 0, 0.0, ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_void_p(lse.data_ptr()))   # no window, cap, sinks or ALiBi
    if static:
        rc = lib.kvq_paged_attn_int8_static_scratch(*head, stream)
        _C.check(rc, "kvq_paged_attn_int8_static_scratch")
    else:
        rc = lib.kvq_paged_attn_int8(*head, ctypes.c_void_p(ws.data_ptr()), ws.numel(), stream)
        _C.check(rc, "kvq_paged_attn_int8")


def _call(dev, static, kv, bt, q, sl, cu, max_q, scale, ws=None):
    """One call through the C ABI; returns (out, lse)."""
    out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full(q.shape[:2], float("nan"), dtype=torch.float32, device=dev)
    _enqueue(dev, static, kv, bt, q, sl, cu, max_q, scale, out, lse, ws=ws)
    torch.cuda.synchronize()
    return out, lse


def test_static_scratch_matches_workspace_entry_twice(gpu_device):
    dev = gpu_device
    hq, hkv, d, bs = 32, 8, 128, 16
    scale = 1 / math.sqrt(d)
    # first call: 24 sequences cut into many split-K states, a prefill row and an empty sequence among them;
    # second call: 3 short sequences, far fewer states, in the same array
    first = ([1500, 33, 0, 2047, 640] + [300 + 37 * i for i in range(19)], [1, 1, 1, 1, 50] + [1] * 19)
    second = ([700, 16, 129], [1, 1, 1])
    for seed, (ctx, qls) in enumerate((first, second)):
        kv_cpu, lay, bt, q, sl, cu = _case(ctx, qls, hq, hkv, d, bs, 100 + seed)
        kv = T.to_device_cache(kv_cpu, dev, "NHD")
        args = (kv, bt.to(dev), q.to(dev), sl.to(dev), cu.to(dev), max(qls), scale)
        ws = torch.empty(ops.paged_attn_workspace_bytes(len(ctx), hq, d), dtype=torch.uint8, device=dev)
        want_out, want_lse = _call(dev, False, *args, ws=ws)
        got_out, got_lse = _call(dev, True, *args)
        assert torch.equal(got_out.view(torch.int16), want_out.view(torch.int16)), f"call {seed}: outputs differ"
        assert torch.equal(got_lse.view(torch.int32), want_lse.view(torch.int32)), f"call {seed}: lse differs"
        ref = oracle.paged_attn(q, T.storage_bytes(kv_cpu), lay, bt, sl, cu, scale)
        T.assert_close_attn(got_out, ref, what=f"static scratch call {seed}")


def test_static_scratch_rejects_oversized_batches(gpu_device):
    """A batch whose split-K states outgrow the array must be refused (and nothing launched)."""
    dev = gpu_device
    hq, hkv, d, bs, n = 64, 8, 256, 16, 1200
    limit = _C.load().kvq_paged_attn_static_scratch_bytes()
    assert ops.paged_attn_workspace_bytes(n, hq, d) > limit
    kv = L.allocate_kv_cache(4, bs, hkv, d, device=dev, layout="NHD", fill=0)
    bt = torch.zeros((n, 1), dtype=torch.int32, device=dev)
    q = torch.zeros((n, hq, d), dtype=torch.bfloat16, device=dev)
    sl = torch.ones(n, dtype=torch.int32, device=dev)
    cu = torch.arange(n + 1, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="too large for the built-in scratch"):
        _call(dev, True, kv, bt, q, sl, cu, 1, 1.0)


def test_static_scratch_captured_and_replayed(gpu_device):
    """The caller the entry point is for: the call recorded into a HIP graph (after the set-up hook,
    kvq_paged_attn_static_scratch_bytes, has resolved the array on this device) and replayed on
    changing lengths and queries, with eager work between the replays; every replay must give the
    workspace entry point's bits."""
    dev = gpu_device
    hq, hkv, d, bs = 32, 8, 128, 16
    scale = 1 / math.sqrt(d)
    assert _C.load().kvq_paged_attn_static_scratch_bytes() == 24 << 20          # the set-up hook, outside the capture
    full = [900, 70, 2100, 333, 16, 1289]
    kv_cpu, lay, bt, q_cpu, _, cu = _case(full, [1] * len(full), hq, hkv, d, bs, 7)
    kv = T.to_device_cache(kv_cpu, dev, "NHD")
    bt_d, cu_d = bt.to(dev), cu.to(dev)
    q = q_cpu.to(dev)
    sl = torch.ones(len(full), dtype=torch.int32, device=dev)
    out = torch.zeros(q.shape, dtype=torch.bfloat16, device=dev)
    lse = torch.zeros(q.shape[:2], dtype=torch.float32, device=dev)
    ws = torch.empty(ops.paged_attn_workspace_bytes(len(full), hq, d), dtype=torch.uint8, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pass
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    geom = _geometry(kv)                                   # torch views are made outside the capture
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):                          # run alone, this is the entry point's first call
        _enqueue(dev, True, kv, bt_d, q, sl, cu_d, 1, scale, out, lse, geom=geom)
    g = torch.Generator().manual_seed(11)
    for it, lens in enumerate((full, [1, 1, 1, 1, 1, 1], [c // 2 for c in full], full)):
        sl_cpu = torch.tensor(lens, dtype=torch.int32)
        sl.copy_(sl_cpu.to(dev))
        qh = torch.randn(q_cpu.shape, generator=g).to(torch.bfloat16)
        q.copy_(qh.to(dev))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want_out, want_lse = _call(dev, False, kv, bt_d, q, sl, cu_d, 1, scale, ws=ws)    # eager, between replays
        assert torch.equal(out.view(torch.int16), want_out.view(torch.int16)), f"replay {it}: outputs differ"
        assert torch.equal(lse.view(torch.int32), want_lse.view(torch.int32)), f"replay {it}: lse differs"
        ref = oracle.paged_attn(qh, T.storage_bytes(kv_cpu), lay, bt, sl_cpu, cu, scale)
        T.assert_close_attn(out, ref, what=f"static scratch graph replay {it}")

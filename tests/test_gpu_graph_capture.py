"""The write + attention step of the path inside a captured HIP graph (the reference's builder
declares full graph support, vllm_metax/v1/attention/backends/triton_attn.py:103): no allocation, no
host synchronisation, no dependence on host-side values that change between steps.  The graph is
replayed several times with new token data, sequence lengths and slots written into the same
buffers, with eager work between the replays, and every replay is checked against the oracle."""
import math

import pytest
import torch

import kvq_testlib as T
import oracle
from vllm_metax_amd import _custom_ops as ops
from vllm_metax_amd import layout as L

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("one_launch", [False, True], ids=["write_then_attention", "one_launch_step"])
def test_decode_step_replays_correctly(gpu_device, one_launch):
    dev = gpu_device
    hq, hkv, d, bs, nb, B = 32, 8, 128, 16, 120, 4
    max_len = 400
    g = torch.Generator().manual_seed(5)
    bt = T.make_block_tables([max_len] * B, bs, nb, g)            # every sequence owns blocks for 400 tokens
    kv_cpu, _views, lay = T.cpu_cache(nb, bs, hkv, d, "NHD")
    ctx = [37, 200, 1, 333]                                       # tokens cached before the first step
    ks = [torch.randn((max_len, hkv, d), generator=g).to(torch.bfloat16) for _ in range(B)]
    vs = [torch.randn((max_len, hkv, d), generator=g).to(torch.bfloat16) for _ in range(B)]
    all_slots = T.slots_for(bt, [max_len] * B, bs)
    for i in range(B):
        oracle.cache_write(ks[i][:ctx[i]], vs[i][:ctx[i]], T.storage_bytes(kv_cpu), lay, all_slots[i][:ctx[i]])
    kv = T.to_device_cache(kv_cpu, dev, "NHD")
    k, v = L.key_value_views(kv)
    ksc, vsc = L.scale_views(kv)
    geom = L.geometry_from_views(k, v, ksc, vsc)
    # static buffers of the captured step
    q = torch.zeros((B, hq, d), dtype=torch.bfloat16, device=dev)
    new_k = torch.zeros((B, hkv, d), dtype=torch.bfloat16, device=dev)
    new_v = torch.zeros((B, hkv, d), dtype=torch.bfloat16, device=dev)
    slots = torch.zeros((B,), dtype=torch.int64, device=dev)
    seq_lens = torch.ones((B,), dtype=torch.int32, device=dev)
    cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
    bt_d = bt.to(dev)
    out = torch.zeros((B, hq, d), dtype=torch.bfloat16, device=dev)
    ws = torch.empty(ops.paged_attn_workspace_bytes(B, hq, d), dtype=torch.uint8, device=dev)
    scale = 1 / math.sqrt(d)

    def step():
        if one_launch:   # the attention launch writes the new tokens itself
            ops.decode_attention_with_cache_update(q, new_k, new_v, k, v, out, seq_lens, max_len, scale, bt_d, ksc, vsc,
                                                   workspace=ws, geometry=geom)
            return
        ops.reshape_and_cache_flash_per_token_head_quant(new_k, new_v, k, v, ksc, vsc, slots, geometry=geom)
        ops.unified_attention(q, k, v, out, cu, 1, seq_lens, max_len, scale, True, block_table=bt_d,
                              k_scale_cache=ksc, v_scale_cache=vsc, workspace=ws, geometry=geom)

    def load_inputs(lens, gen):
        """Next token of every sequence: lens[i] is the length INCLUDING it."""
        qh = torch.randn((B, hq, d), generator=gen).to(torch.bfloat16)
        nk = torch.stack([ks[i][lens[i] - 1] for i in range(B)])
        nv = torch.stack([vs[i][lens[i] - 1] for i in range(B)])
        sl = torch.tensor([int(all_slots[i][lens[i] - 1]) for i in range(B)], dtype=torch.int64)
        q.copy_(qh.to(dev))
        new_k.copy_(nk.to(dev))
        new_v.copy_(nv.to(dev))
        slots.copy_(sl.to(dev))
        seq_lens.copy_(torch.tensor(lens, dtype=torch.int32).to(dev))
        oracle.cache_write(nk, nv, T.storage_bytes(kv_cpu), lay, sl)
        return qh

    lens = [c + 1 for c in ctx]
    load_inputs(lens, g)                       # warm-up on a side stream, as graph capture requires
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it in range(4):
        lens = [n + 1 for n in lens]           # every sequence grows by one token per step
        qh = load_inputs(lens, g)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(T.storage_bytes(kv).cpu(), T.storage_bytes(kv_cpu)), f"replay {it}: cache bytes differ"
        want = oracle.paged_attn(qh, T.storage_bytes(kv_cpu), lay, bt, torch.tensor(lens, dtype=torch.int32),
                                 torch.arange(B + 1, dtype=torch.int32), scale)
        T.assert_close_attn(out, want, what=f"graph replay {it}")
        # eager work between replays: the same step outside the graph gives the same bytes
        eager = torch.empty_like(out)
        ops.unified_attention(q, k, v, eager, cu, 1, seq_lens, max_len, scale, True, block_table=bt_d,
                              k_scale_cache=ksc, v_scale_cache=vsc, workspace=ws, geometry=geom)
        torch.cuda.synchronize()
        assert torch.equal(eager, out), f"replay {it}: graph and eager outputs differ"


@pytest.mark.parametrize("one_launch", [False, True], ids=["write_then_decode", "one_launch_step"])
def test_mla_decode_replays_correctly(gpu_device, one_launch):
    dev = gpu_device
    R, P, H, bs, nb, B = 512, 64, 16, 64, 12, 2
    g = torch.Generator().manual_seed(8)
    max_len = 300
    bt = T.make_block_tables([max_len] * B, bs, nb, g)
    cpu = L.allocate_mla_cache(nb, bs, R + P, device="cpu")
    codes, scales = L.mla_cache_views(cpu)
    lay = oracle.MlaLayout.from_views(cpu, codes, scales, R)
    rows_c = [torch.randn((max_len, R), generator=g).to(torch.bfloat16) for _ in range(B)]
    rows_p = [torch.randn((max_len, P), generator=g).to(torch.bfloat16) for _ in range(B)]
    all_slots = T.slots_for(bt, [max_len] * B, bs)
    ctx = [70, 255]
    for i in range(B):
        oracle.mla_cache_write(rows_c[i][:ctx[i]], rows_p[i][:ctx[i]], cpu, lay, all_slots[i][:ctx[i]])
    cache = cpu.to(dev)
    q = torch.zeros((B, H, R + P), dtype=torch.bfloat16, device=dev)
    kv_c = torch.zeros((B, R), dtype=torch.bfloat16, device=dev)
    k_pe = torch.zeros((B, P), dtype=torch.bfloat16, device=dev)
    slots = torch.zeros((B,), dtype=torch.int64, device=dev)
    seq_lens = torch.ones((B,), dtype=torch.int32, device=dev)
    o = torch.zeros((B, H, R), dtype=torch.bfloat16, device=dev)
    lse = torch.zeros((B, H), dtype=torch.float32, device=dev)
    bt_d = bt.to(dev)
    ws = torch.empty(ops.mla_decode_workspace_bytes(B, H, R), dtype=torch.uint8, device=dev)
    geom = L.mla_geometry(cache, R)

    def step():
        if one_launch:
            ops.mla_decode_with_cache_update(q, kv_c, k_pe, cache, o, lse, bt_d, seq_lens, 0.0722, R, workspace=ws,
                                             geometry=geom)
            return
        ops.concat_and_cache_mla(kv_c, k_pe, cache, slots, geometry=geom)
        ops.mla_decode_int8(q, cache, o, lse, bt_d, seq_lens, 0.0722, R, workspace=ws, geometry=geom)

    def load_inputs(lens):
        qh = (torch.randn((B, H, R + P), generator=g) * 0.5).to(torch.bfloat16)
        c = torch.stack([rows_c[i][lens[i] - 1] for i in range(B)])
        p = torch.stack([rows_p[i][lens[i] - 1] for i in range(B)])
        sl = torch.tensor([int(all_slots[i][lens[i] - 1]) for i in range(B)], dtype=torch.int64)
        q.copy_(qh.to(dev)); kv_c.copy_(c.to(dev)); k_pe.copy_(p.to(dev)); slots.copy_(sl.to(dev))
        seq_lens.copy_(torch.tensor(lens, dtype=torch.int32).to(dev))
        oracle.mla_cache_write(c, p, cpu, lay, sl)
        return qh

    lens = [c + 1 for c in ctx]
    load_inputs(lens)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it in range(3):
        lens = [n + 1 for n in lens]
        qh = load_inputs(lens)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(cache.cpu(), cpu), f"replay {it}: latent cache differs"
        want, want_lse = oracle.mla_decode(qh, cpu, lay, bt, torch.tensor(lens, dtype=torch.int32), 0.0722)
        T.assert_close_attn(o, want, what=f"MLA graph replay {it}")
        torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)


def test_mla_forward_mqa_through_the_builder_replays_correctly(gpu_device):
    """The decode step as the MLA layer runs it -- metadata from ``Int8MLAMetadataBuilder`` (which owns the
    launch's scratch and the output buffers), ``Int8MLAImpl.do_kv_cache_update`` then ``forward_mqa`` -- captured
    in a graph: the call allocates nothing (checked on the allocator's counters too), and every replay
    matches the oracle and the eager call."""
    import types

    from vllm_metax_amd.v1.attention.backends.mla.int8_mla import Int8MLABackend

    dev = gpu_device
    R, P, H, bs, nb, B = 512, 64, 16, 64, 12, 2
    g = torch.Generator().manual_seed(18)
    max_len = 300
    bt = T.make_block_tables([max_len] * B, bs, nb, g)
    cpu = L.allocate_mla_cache(nb, bs, R + P, device="cpu")
    codes, scales = L.mla_cache_views(cpu)
    lay = oracle.MlaLayout.from_views(cpu, codes, scales, R)
    rows_c = [torch.randn((max_len, R), generator=g).to(torch.bfloat16) for _ in range(B)]
    rows_p = [torch.randn((max_len, P), generator=g).to(torch.bfloat16) for _ in range(B)]
    all_slots = T.slots_for(bt, [max_len] * B, bs)
    ctx = [64, 129]
    for i in range(B):
        oracle.mla_cache_write(rows_c[i][:ctx[i]], rows_p[i][:ctx[i]], cpu, lay, all_slots[i][:ctx[i]])
    cache = cpu.to(dev)
    spec = types.SimpleNamespace(block_size=bs, num_kv_heads=1, head_size=R + P, num_heads=H, kv_lora_rank=R)
    cfg = types.SimpleNamespace(scheduler_config=types.SimpleNamespace(max_num_seqs=8))
    assert Int8MLABackend.get_builder_cls()._cudagraph_support.name == "UNIFORM_SINGLE_TOKEN_DECODE"
    builder = Int8MLABackend.get_builder_cls()(spec, ["layer.0"], cfg, dev)
    impl = Int8MLABackend.get_impl_cls()(H, R + P, 0.0722, kv_cache_dtype="int8_per_token")
    ql = torch.zeros((B, H, R), dtype=torch.bfloat16, device=dev)
    qp = torch.zeros((B, H, P), dtype=torch.bfloat16, device=dev)
    kv_c = torch.zeros((B, R), dtype=torch.bfloat16, device=dev)
    k_pe = torch.zeros((B, P), dtype=torch.bfloat16, device=dev)
    slots = torch.zeros((B,), dtype=torch.int64, device=dev)
    seq_lens = torch.ones((B,), dtype=torch.int32, device=dev)
    common = types.SimpleNamespace(
        num_reqs=B, num_actual_tokens=B, max_query_len=1, max_seq_len=max_len,
        query_start_loc=torch.arange(B + 1, dtype=torch.int32, device=dev),
        query_start_loc_cpu=torch.arange(B + 1, dtype=torch.int32),
        seq_lens=seq_lens, block_table_tensor=bt.to(dev), slot_mapping=slots)
    md = builder.build(0, common)
    assert md.num_decodes == B and md.num_prefills == 0 and md.workspace is not None
    held = {}

    def step():
        impl.do_kv_cache_update(kv_c, k_pe, cache, md.slot_mapping)
        held["o"], held["lse"] = impl.forward_mqa((ql, qp), cache, md)

    def load_inputs(lens):
        qh = (torch.randn((B, H, R + P), generator=g) * 0.5).to(torch.bfloat16)
        c = torch.stack([rows_c[i][lens[i] - 1] for i in range(B)])
        p = torch.stack([rows_p[i][lens[i] - 1] for i in range(B)])
        sl = torch.tensor([int(all_slots[i][lens[i] - 1]) for i in range(B)], dtype=torch.int64)
        ql.copy_(qh[..., :R].to(dev)); qp.copy_(qh[..., R:].to(dev))
        kv_c.copy_(c.to(dev)); k_pe.copy_(p.to(dev)); slots.copy_(sl.to(dev))
        seq_lens.copy_(torch.tensor(lens, dtype=torch.int32).to(dev))
        oracle.mla_cache_write(c, p, cpu, lay, sl)
        return qh

    lens = [c + 1 for c in ctx]
    load_inputs(lens)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    step()                                                     # eager: the builder's buffers, no allocation
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before, "forward_mqa allocated"
    assert held["o"].data_ptr() == md.decode_out.data_ptr() and held["lse"].data_ptr() == md.decode_lse.data_ptr()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    o, lse = held["o"], held["lse"]
    for it in range(3):
        lens = [n + 1 for n in lens]
        qh = load_inputs(lens)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(cache.cpu(), cpu), f"replay {it}: latent cache differs"
        want, want_lse = oracle.mla_decode(qh, cpu, lay, bt, torch.tensor(lens, dtype=torch.int32), 0.0722)
        T.assert_close_attn(o, want, what=f"MLA forward_mqa graph replay {it}")
        torch.testing.assert_close(lse.cpu(), want_lse, atol=5e-3, rtol=1e-3)
        got = o.clone()
        eo, _ = impl.forward_mqa((ql, qp), cache, md)          # eager work between the replays, same buffers
        torch.cuda.synchronize()
        assert torch.equal(eo, got), f"replay {it}: graph and eager outputs differ"

"""pa_decode_noalloc, the entry point that allocates nothing: its output must equal pa_decode's bit for bit (the
same kernels run on the same inputs; only where the partition buffers live differs) and the CPU oracle's within
the parity bar, on two calls in a row that share the library's scratch array, the second with a smaller input;
the device's free memory must not move across a call; a call captured into a HIP graph must replay to the same
bits; and a call too large for the array must be refused before anything is launched."""
import ctypes as C

import pytest
import torch

import triton_op_amd as T
from oracle import pa_oracle as O
from triton_op_amd import _cabi
from triton_op_amd import workloads as W

pytestmark = pytest.mark.gpu


def _plan(wl, out, partition_size):
    return T.plan_decode(out, wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                         wl.softmax_scale, wl.q_len, wl.max_context_len, torch.bfloat16, None, wl.key_scale,
                         wl.value_scale, partition_size=partition_size, query_lens=wl.q_lens)


def _workloads(dev):
    # first a ragged MTP batch over per-token scales (shared-stream kernel, sorted dispatch, listed reduce, the
    # queue counters), then a smaller one on the other partition kernel with several partitions per sequence
    g = torch.Generator().manual_seed(11)
    ctx_a = torch.randint(16, 2560, (200,), generator=g, dtype=torch.int32)
    ql_a = torch.randint(1, 4, (200,), generator=g, dtype=torch.int32)
    a = W.make_decode_workload(name="noalloc_a", seed=21, batch=200, num_q_heads=32, num_kv_heads=2, block_size=16,
                               context_lens=ctx_a, q_len=3, q_lens=ql_a, scale_mode="token").to(dev)
    ctx_b = torch.tensor([1500, 17, 700], dtype=torch.int32)
    b = W.make_decode_workload(name="noalloc_b", seed=22, batch=3, num_q_heads=16, num_kv_heads=2, block_size=16,
                               context_lens=ctx_b, q_len=1).to(dev)
    # ... and one whose (sequence, kv head) units run as teams that merge in the partition kernel (no reduce kernel)
    ctx_c = torch.randint(1, 2049, (52,), generator=g, dtype=torch.int32)
    c = W.make_decode_workload(name="noalloc_c", seed=24, batch=52, num_q_heads=64, num_kv_heads=8, block_size=16,
                               context_lens=ctx_c, q_len=1).to(dev)
    return [(a, 256), (b, 256), (c, 256)]


def test_noalloc_matches_pa_decode_on_two_calls_in_a_row():
    dev = torch.device("cuda:0")
    lib = _cabi.load_library()
    stream = torch.cuda.current_stream(dev)
    for wl, ps in _workloads(dev):
        print(f"[noalloc] {wl.name} batch={wl.batch} partition_size={ps}", flush=True)
        if wl.name == "noalloc_c":
            info = _plan(wl, torch.empty_like(wl.query), ps).launch_info()
            assert "teams of 4 waves" in info, info
        ref = torch.full_like(wl.query, float("nan"))
        _plan(wl, ref, ps).run()
        out = torch.full_like(wl.query, float("nan"))
        plan = _plan(wl, out, ps)
        # poison this plan's own buffers: the entry point must not touch them
        plan.tmp_output.fill_(float("nan"))
        plan.exp_sums.fill_(float("nan"))
        plan.run_noalloc(stream.cuda_stream)  # the first call on a device looks the scratch array's address up
        torch.cuda.synchronize()
        out.fill_(float("nan"))
        # free device memory as the driver reports it (torch's own counters only see torch's allocator): a
        # hipMalloc inside the library would move it
        free_before, _ = torch.cuda.mem_get_info(dev)
        torch_before = torch.cuda.memory_allocated(dev)
        plan.run_noalloc(stream.cuda_stream)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(dev)
        assert free_after == free_before, (free_before, free_after)
        assert torch.cuda.memory_allocated(dev) == torch_before
        assert not torch.isnan(out.float()).any()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), wl.name
        assert torch.isnan(plan.tmp_output.float()).all() and torch.isnan(plan.exp_sums).all()
        # ... and against the CPU oracle, like every other entry point
        c = wl.to("cpu")
        oracle = O.paged_attention_decode_oracle(c.query, c.key_cache, c.value_cache, c.context_lens, c.block_tables,
                                                 c.softmax_scale, c.q_len if c.q_lens is None else c.q_lens, c.key_scale,
                                                 c.value_scale, q_max=c.q_len)
        torch.testing.assert_close(out.float().cpu(), oracle.float(), atol=2e-2, rtol=2e-2)


def test_noalloc_call_captured_in_a_graph_replays_to_the_same_bits():
    """The entry point is for callers under graph capture.  One call is made outside capture first (the first call
    on a device asks the runtime for the scratch array's address); then a call is captured and replayed three
    times with eager work and host synchronisations in between, each replay held against pa_decode's result."""
    dev = torch.device("cuda:0")
    wl, ps = _workloads(dev)[0]
    ref = torch.full_like(wl.query, float("nan"))
    _plan(wl, ref, ps).run()
    out = torch.full_like(wl.query, float("nan"))
    plan = _plan(wl, out, ps)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        plan.run_noalloc(side.cuda_stream)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plan.run_noalloc(side.cuda_stream)
    torch.cuda.synchronize()
    for i in range(3):
        out.fill_(float("nan"))
        (wl.key_cache.float()[:1] * 1.0).sum().item()  # unrelated eager work and a host sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"replay {i}"


def test_noalloc_refuses_what_does_not_fit():
    dev = torch.device("cuda:0")
    lib = _cabi.load_library()
    wl = W.make_decode_workload(name="noalloc_big", seed=23, batch=2, num_q_heads=8, num_kv_heads=1, block_size=16,
                                context_lens=torch.tensor([64, 33], dtype=torch.int32), q_len=1).to(dev)
    out = torch.full_like(wl.query, 7.0)
    plan = _plan(wl, out, 256)
    a = _cabi.PaDecodeArgs.from_buffer_copy(plan.args)
    a.exp_sums = a.max_logits = a.tmp_output = a.workspace = None
    a.workspace_bytes = 0
    # claim a partition axis whose buffers would take more than the scratch array: 2 * 1 * P * 8 rows * 264 B
    a.max_num_partitions = _cabi.PA_DECODE_NOALLOC_SCRATCH_BYTES // (2 * 8 * 264) + 1
    rc = lib.pa_decode_noalloc(C.byref(a), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == _cabi.PA_ERR_SCRATCH_TOO_SMALL
    torch.cuda.synchronize()
    assert torch.equal(out, torch.full_like(out, 7.0))  # nothing ran


def test_noalloc_with_the_output_only_flag():
    """PA_DECODE_FLAG_OUTPUT_ONLY through the entry point that allocates nothing: the real query rows equal, bit for
    bit, those of pa_decode with the same flag (under the flag the library cuts the partition axis its own way, the
    same way in both entry points), and agree with the flagless call to the parity tolerance."""
    dev = torch.device("cuda:0")
    wl, ps = _workloads(dev)[0]
    flagless = torch.full_like(wl.query, float("nan"))
    _plan(wl, flagless, ps).run()
    ref = torch.full_like(wl.query, 7.0)
    T.plan_decode(ref, wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                  wl.softmax_scale, wl.q_len, wl.max_context_len, torch.bfloat16, None, wl.key_scale,
                  wl.value_scale, partition_size=ps, query_lens=wl.q_lens, output_only=True).run()
    out = torch.full_like(wl.query, 7.0)
    plan = T.plan_decode(out, wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                         wl.softmax_scale, wl.q_len, wl.max_context_len, torch.bfloat16, None, wl.key_scale,
                         wl.value_scale, partition_size=ps, query_lens=wl.q_lens, output_only=True)
    plan.run_noalloc(torch.cuda.current_stream(dev).cuda_stream)
    torch.cuda.synchronize()
    hkv = wl.key_cache.shape[1]
    view = lambda t: t.view(t.shape[0], hkv, wl.q_len, -1, t.shape[-1])
    for b, ql in enumerate(wl.q_lens.cpu().tolist()):
        assert torch.equal(view(out)[b, :, :ql], view(ref)[b, :, :ql]), f"sequence {b}"
        torch.testing.assert_close(view(out)[b, :, :ql].float(), view(flagless)[b, :, :ql].float(), atol=2e-2, rtol=2e-2)

"""GPU tests of the framework-side adaptor library (lib/libinfinicore_ops.so): every operator through the
immediate and the plan / run / cleanup forms, checked against the CPU oracle, and the behaviour of the
thread-local descriptor cache and workspaces around them."""
import threading

import numpy as np
import pytest
import torch

from infinicore_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture()
def core(lib):
    from infinicore_amd import libinfinicore_ops

    lib.set_device(lib.InfiniDevice.AMD, 0)
    libinfinicore_ops.cache_clear()
    libinfinicore_ops.cache_set_capacity(100)
    yield libinfinicore_ops
    lib.set_device(lib.InfiniDevice.AMD, 0)
    libinfinicore_ops.cache_clear()
    libinfinicore_ops.cache_set_capacity(100)


def bits(t):
    t = t.contiguous().cpu()
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def close(got, want):
    want = want.float()
    return bool(torch.all((got.float().cpu() - want).abs() <= 1e-2 + 2e-3 * want.abs()))


def decode_case(oracle, name, dtype, B, H, Hkv, D, lo, hi, seed):
    cfg = workloads.DecodeConfig(name, dtype, B, H, Hkv, D, 16, lo, hi, seed=seed)
    inp = workloads.make_decode_inputs(cfg)
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens)]
    want = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale)
    return inp, dev, want


def test_immediate_paged_attention_and_the_descriptor_cache(core, oracle):
    print("case immediate paged_attention", flush=True)
    inp, (q, k, v, bt, sl), want = decode_case(oracle, "adaptor", torch.bfloat16, 4, 32, 8, 128, 10, 1500, 71)
    out = torch.zeros_like(q)
    core.paged_attention_(out, q, k, v, bt, sl, None, inp.scale)
    torch.cuda.synchronize()
    assert close(out, want)
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION) == (1, 0, 1)
    out2 = torch.zeros_like(q)
    core.paged_attention_(out2, q, k, v, bt, sl, None, inp.scale)  # same metadata, other output tensor: a hit
    torch.cuda.synchronize()
    assert torch.equal(bits(out), bits(out2))
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION) == (1, 1, 1)
    # another scale is another descriptor (the descriptor stores the scale)
    want_half = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale * 0.5)
    core.paged_attention_(out2, q, k, v, bt, sl, None, inp.scale * 0.5)
    torch.cuda.synchronize()
    assert close(out2, want_half) and not torch.equal(bits(out), bits(out2))
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION) == (2, 1, 2)
    # the other operators' caches are separate
    assert core.cache_stats(core.OpKind.PAGED_CACHING) == (0, 0, 0)


def test_immediate_workspace_grows_with_the_larger_call(core, oracle):
    print("case workspace growth", flush=True)
    small_inp, small, small_want = decode_case(oracle, "small", torch.float16, 2, 8, 8, 128, 1, 100, 72)
    big_inp, big, big_want = decode_case(oracle, "big", torch.float16, 16, 32, 8, 128, 200, 3000, 73)
    for inp, dev, want in ((small_inp, small, small_want), (big_inp, big, big_want), (small_inp, small, small_want)):
        out = torch.zeros_like(dev[0])
        core.paged_attention_(out, *dev, None, inp.scale)
        torch.cuda.synchronize()
        assert close(out, want), inp.config.name


def test_plan_run_cleanup_and_graph_replay(core, oracle, lib):
    print("case plan / run / cleanup", flush=True)
    inp, (q, k, v, bt, sl), want = decode_case(oracle, "plan", torch.bfloat16, 8, 32, 8, 128, 100, 2500, 74)
    out = torch.zeros_like(q)
    plan = core.PlannedOp("paged_attention", out, q, k, v, bt, sl, None, scale=inp.scale)
    assert plan.workspace_bytes > 0
    plan.run()
    torch.cuda.synchronize()
    assert close(out, want)
    eager = out.clone()
    # a second plan on the same metadata shares the cached descriptor and has a workspace of its own
    out_b = torch.zeros_like(q)
    plan_b = core.PlannedOp("paged_attention", out_b, q, k, v, bt, sl, None, scale=inp.scale)
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION) == (1, 1, 1)
    # run allocates nothing: record it into a graph and replay with eager work in between
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan.run(side)  # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plan.run(side)
    for replay in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(out), bits(eager)), f"replay {replay}"
        plan_b.run()
        torch.cuda.synchronize()
        assert torch.equal(bits(out_b), bits(eager)), f"second plan after replay {replay}"
    # a plan runs on the device it was made on only
    import ctypes
    lib.set_device(lib.InfiniDevice.CPU, 0)
    status = core.LIBINFINICORE_OPS.infinicoreOpRun(plan._handle, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    lib.set_device(lib.InfiniDevice.AMD, 0)
    assert status == lib.InfiniStatus.BAD_PARAM
    # the cache forgets the descriptor; the plans keep it alive
    core.cache_clear()
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION)[0] == 0
    out.zero_()
    plan.run()
    torch.cuda.synchronize()
    assert torch.equal(bits(out), bits(eager))
    del graph
    plan.cleanup()
    plan_b.cleanup()
    plan.cleanup()  # idempotent on the Python side


def test_capacity_and_eviction(core, oracle):
    print("case capacity", flush=True)
    a_inp, a, a_want = decode_case(oracle, "a", torch.float16, 2, 8, 8, 128, 1, 100, 75)
    b_inp, b, b_want = decode_case(oracle, "b", torch.float16, 3, 8, 2, 128, 1, 100, 76)
    core.cache_set_capacity(1)
    out_a, out_b = torch.zeros_like(a[0]), torch.zeros_like(b[0])
    with core.PlannedOp("paged_attention", out_a, *a, None, scale=a_inp.scale) as plan_a:
        core.paged_attention_(out_b, *b, None, b_inp.scale)  # evicts a's descriptor, which plan_a still owns
        assert core.cache_stats(core.OpKind.PAGED_ATTENTION)[0] == 1
        plan_a.run()
        torch.cuda.synchronize()
        assert close(out_a, a_want) and close(out_b, b_want)
    core.paged_attention_(out_a, *a, None, a_inp.scale)  # a miss again: created anew
    torch.cuda.synchronize()
    assert close(out_a, a_want)
    entries, hits, misses = core.cache_stats(core.OpKind.PAGED_ATTENTION)
    assert (entries, hits, misses) == (1, 0, 3)


def test_refused_tensors_return_the_operator_status_and_cache_nothing(core, lib):
    q = torch.zeros(2, 8, 128, dtype=torch.float16, device=DEV)
    kc = torch.zeros(4, 8, 16, 128, dtype=torch.float16, device=DEV)
    bt = torch.zeros(2, 2, dtype=torch.int64, device=DEV)
    sl = torch.zeros(2, dtype=torch.int64, device=DEV)
    with pytest.raises(Exception) as err:
        core.paged_attention_(q, q, kc, kc.to(torch.bfloat16), bt, sl, None, 1.0)  # mixed dtypes
    assert "BAD_TENSOR_DTYPE" in str(err.value) or "10" in str(err.value)
    with pytest.raises(Exception):
        core.PlannedOp("paged_attention", q, q, kc, kc, bt, sl.to(torch.int32), None, scale=1.0)  # index dtypes differ
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION)[0] == 0
    with pytest.raises(ValueError):
        core.paged_attention_(q.cpu(), q, kc, kc, bt, sl, None, 1.0)  # host tensor: no fallback


def test_paged_caching_immediate_and_planned(core, oracle):
    print("case paged_caching", flush=True)
    cfg = workloads.CachingConfig("adaptor", torch.bfloat16, 300, 8, 128, 16, 4096, 0.05, seed=77)
    inp = workloads.make_caching_inputs(cfg)
    k_want, v_want = oracle.paged_caching(inp.k_cache.clone(), inp.v_cache.clone(), inp.k, inp.v, inp.slot_mapping)
    kc, vc, k, v, slots = [t.to(DEV) for t in (inp.k_cache, inp.v_cache, inp.k, inp.v, inp.slot_mapping)]
    core.paged_caching_(kc, vc, k, v, slots)
    torch.cuda.synchronize()
    assert torch.equal(bits(kc), bits(k_want)) and torch.equal(bits(vc), bits(v_want))
    kc2, vc2 = inp.k_cache.to(DEV), inp.v_cache.to(DEV)
    with core.PlannedOp("paged_caching", kc2, vc2, k, v, slots) as plan:
        assert plan.workspace_bytes == 0  # the scatter needs none: run gets a null workspace
        plan.run()
        torch.cuda.synchronize()
    assert torch.equal(bits(kc2), bits(k_want)) and torch.equal(bits(vc2), bits(v_want))
    assert core.cache_stats(core.OpKind.PAGED_CACHING) == (1, 1, 1)


def test_kv_caching_immediate_and_planned(core, oracle):
    print("case kv_caching", flush=True)
    cfg = workloads.KVCachingConfig("adaptor", torch.float16, 3, 4, 64, 5, 128, seed=78)
    inp = workloads.make_kv_caching_inputs(cfg)
    k_want, v_want = oracle.kv_caching(inp.k_cache.clone(), inp.v_cache.clone(), inp.k, inp.v, inp.past_kv_lengths)
    kc, vc, k, v, past = [t.to(DEV) for t in (inp.k_cache, inp.v_cache, inp.k, inp.v, inp.past_kv_lengths)]
    core.kv_caching_(kc, vc, k, v, past)
    torch.cuda.synchronize()
    assert torch.equal(bits(kc), bits(k_want)) and torch.equal(bits(vc), bits(v_want))
    kc2, vc2 = inp.k_cache.to(DEV), inp.v_cache.to(DEV)
    with core.PlannedOp("kv_caching", kc2, vc2, k, v, past) as plan:
        plan.run()
        torch.cuda.synchronize()
    assert torch.equal(bits(kc2), bits(k_want)) and torch.equal(bits(vc2), bits(v_want))


def test_paged_attention_prefill_immediate_and_planned(core, oracle):
    print("case prefill", flush=True)
    cfg = workloads.PrefillConfig("adaptor", torch.bfloat16, 3, 32, 8, 128, 16, 1, 200, 0, 300, seed=79)
    inp = workloads.make_prefill_inputs(cfg)
    want = oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                          inp.cum_seq_lens_q, inp.scale)
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    out = torch.zeros_like(dev[0])
    core.paged_attention_prefill_(out, *dev, None, inp.scale)
    torch.cuda.synchronize()
    assert close(out, want)
    out2 = torch.zeros_like(dev[0])
    with core.PlannedOp("paged_attention_prefill", out2, *dev, None, scale=inp.scale) as plan:
        plan.run()
        torch.cuda.synchronize()
    assert torch.equal(bits(out), bits(out2))
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION_PREFILL) == (1, 1, 1)


def test_strided_views_are_part_of_the_key(core, oracle):
    """A padded query (row stride larger than heads x head size) is another descriptor than the packed one."""
    inp, (q, k, v, bt, sl), want = decode_case(oracle, "strided", torch.float16, 3, 8, 8, 128, 1, 200, 80)
    padded = torch.zeros(3, 16, 128, dtype=q.dtype, device=DEV)
    padded[:, :8] = q
    out = torch.zeros_like(q)
    core.paged_attention_(out, q, k, v, bt, sl, None, inp.scale)
    out_p = torch.zeros_like(q)
    core.paged_attention_(out_p, padded[:, :8], k, v, bt, sl, None, inp.scale)
    torch.cuda.synchronize()
    assert close(out, want) and torch.equal(bits(out), bits(out_p))
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION) == (2, 0, 2)


def test_each_thread_has_its_own_cache(core, oracle, lib):
    inp, (q, k, v, bt, sl), want = decode_case(oracle, "threads", torch.float16, 2, 8, 8, 128, 1, 100, 81)
    out = torch.zeros_like(q)
    core.paged_attention_(out, q, k, v, bt, sl, None, inp.scale)
    torch.cuda.synchronize()
    seen = {}

    def worker():
        try:
            lib.set_device(lib.InfiniDevice.AMD, 0)
            seen["before"] = core.cache_stats(core.OpKind.PAGED_ATTENTION)
            out_t = torch.zeros_like(q)
            core.paged_attention_(out_t, q, k, v, bt, sl, None, inp.scale)
            torch.cuda.synchronize()
            seen["equal"] = torch.equal(bits(out_t), bits(out))
            seen["after"] = core.cache_stats(core.OpKind.PAGED_ATTENTION)
            core.cache_clear()  # frees this thread's workspace while the runtime is alive
        except Exception as exc:  # pragma: no cover - reported below
            seen["error"] = exc

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert "error" not in seen, seen.get("error")
    assert seen["before"] == (0, 0, 0) and seen["after"] == (1, 0, 1) and seen["equal"]
    assert core.cache_stats(core.OpKind.PAGED_ATTENTION) == (1, 0, 1)  # this thread's cache is untouched
    assert close(out, want)

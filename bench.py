#!/usr/bin/env python3
"""Paged-attention benchmark on one MI355X: decode (default, the headline) or prefill.

A step is one decode step's worth of attention for a 32-layer model: 32 ``infiniopPagedAttention`` calls
(decode kernel + segment merge each) through the C ABI, one per layer, on the Llama-3-8B GQA batch-32
decode shape (bf16, 32 query / 8 KV heads, head 128, pages of 16 tokens, ragged lengths 512..4096 through a
shuffled block table). Every layer has a KV pool of its own (same content, different addresses, 11 GB
together), so every call streams its K/V from HBM as a real model does when it moves from layer to layer.
Inputs are resident in HBM before the timed region. ``us_per_call`` = step time / 32; ``value`` is the
algorithmic bytes of the step over its time.

With ``--workload p2_llama3_8b_prompt``, ``p3_llama3_8b_chunked`` or ``p4_mla_16_heads_chunked`` (latent
attention: keys 576, values 512) a step is one ``infiniopPagedAttentionPrefill`` call instead, bounded by the
bf16 matrix-core peak; the line then reports TFLOP/s (2 x multiply-adds of Q.K^T and P.V over the visible
query/key pairs).

Prints one JSON line: throughput in algorithmic GB/s (K and V once per KV head + Q + O + the
needed table entries + lengths), the time per call, the HBM roofline of the step measured with
device events on the stream the kernels run on, and a CPU baseline (the CPU oracle, a C restatement
of the reference kernel's arithmetic, timed on this machine's host cores).
"""
from __future__ import annotations

import argparse
import ctypes
import dataclasses
import json
import os
import sys
import time
from ctypes import c_float, c_size_t, c_void_p
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 matrix peak

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# file, each scaled by what the same counter reads for a 256 MiB copy. Counters cannot be read from inside
# this process, so the figures are recorded here per workload, each with the summary under profiles/ that
# holds the command and the raw counter values, and the commit whose kernel sources were measured (a later
# change to that kernel makes the figure stale until it is collected again).
MEASURED_TRAFFIC = {
    # workload: (bytes, summary under profiles/, commit of the measured kernel)
    "c2_llama3_8b_b32": (322_400_000, "decode_balanced_c2_llama3_8b_b32_hbm_traffic.md", "afe7af1"),
    "m1_mla_16_heads_b32": (153_400_000, "decode_mla_m1_m2_kernel_stats_and_traffic.md", "4349d98"),
    "m2_mla_128_heads_b32": (205_500_000, "decode_mla_m1_m2_kernel_stats_and_traffic.md", "3b94ee4"),
    "c5_prefill_scatter": (33_000_000, "paged_caching_c5_prefill_scatter_kernel_stats_and_traffic.md", "3fbf320"),
    "k2_append_prefill_chunk": (33_600_000, "kv_caching_k2_append_prefill_chunk_kernel_stats_and_traffic.md", "3fbf320"),
    "r2_rope_scatter_prefill_chunk": (35_300_000, "rope_paged_caching_r1_r2_kernel_stats_and_traffic.md", "3fbf320"),
    "r4_rope_qk_scatter_prefill_chunk": (103_250_000, "rope_paged_caching_r1_r2_kernel_stats_and_traffic.md", "3fbf320"),
    "p3_llama3_8b_chunked": (552_500_000, "prefill_tiled_p3_llama3_8b_chunked_counters.md", "60c46ff"),  # fetched 508.1 MB + written 44.35 MB
}


def traffic_fields(workload):
    """``roofline.traffic`` and where the figure comes from (both None for a workload without a counter run)."""
    if workload not in MEASURED_TRAFFIC:
        return {"traffic": None, "traffic_profile": None, "traffic_commit": None}
    nbytes, summary, commit = MEASURED_TRAFFIC[workload]
    # flat string fields (not a nested object): they survive tools that keep only scalars of this line
    return {"traffic": nbytes, "traffic_profile": "profiles/" + summary, "traffic_commit": commit}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="default 20 (decode: 32 calls each) / 50 (prefill) / 400 (scatter)")
    ap.add_argument("--warmup", type=int, default=None, help="default 3 (decode) / 5 (prefill) / 40 (scatter)")
    ap.add_argument("--layers", type=int, default=32, help="decode: calls per step, each on a KV pool of its own")
    ap.add_argument("--workload", default="c2_llama3_8b_b32")
    ap.add_argument("--head-size", type=int, default=0,
                    help="run the workload's shape with this head size (64 / 192 / 256 / 576) instead of its own; the "
                         "workload name in the output gets a _d<head> suffix")
    ap.add_argument("--pools", type=int, default=4, help="scatter workloads: distinct cache sets the steps rotate over")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true", help="skip the oracle check of the output")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies, so that a rocprofv3 --pmc run of this "
                         "command records FETCH_SIZE / WRITE_SIZE of a kernel whose traffic is known")
    return ap.parse_args()


def pmc_calibration_copies(torch, dev):
    """Three plain 256 MiB device-to-device copies: a kernel of known traffic that gives hardware byte
    counters their scale when the same run is collected with rocprofv3 --pmc."""
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(3)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def run_prefill(args, torch, L, workloads, dev):
    """One step = one infiniopPagedAttentionPrefill call; inputs resident in HBM."""
    import numpy as np

    cfg = workloads.PREFILL_CONFIGS[args.workload]
    if args.head_size:
        cfg = dataclasses.replace(cfg, head_size=args.head_size, name=f"{cfg.name}_d{args.head_size}")
    inp = workloads.make_prefill_inputs(cfg)
    new, history = workloads.draw_prefill_lens(cfg)
    flops = workloads.prefill_flops(cfg, new, history)
    algo_bytes = workloads.prefill_algorithmic_bytes(cfg, new, history)

    L.set_device(L.InfiniDevice.AMD, 0)
    handle = L.create_handle()
    tensors = [t.to(dev) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    q, k_cache, v_cache, bt, sl, cu = tensors
    out = torch.zeros((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype, device=dev)
    DTYPES = {torch.float16: L.InfiniDtype.F16, torch.bfloat16: L.InfiniDtype.BF16, torch.int64: L.InfiniDtype.I64}
    descs = [L.create_tensor_descriptor(tuple(t.shape), tuple(t.stride()), DTYPES[t.dtype]) for t in (out, *tensors)]
    op = L.infiniopOperatorDescriptor_t()
    L.check_error(L.LIBINFINIOP.infiniopCreatePagedAttentionPrefillDescriptor(
        handle, ctypes.byref(op), *descs, L.infiniopTensorDescriptor_t(), inp.scale))
    for d in descs:
        L.destroy_tensor_descriptor(d)
    ws_size = c_size_t(0)
    L.check_error(L.LIBINFINIOP.infiniopGetPagedAttentionPrefillWorkspaceSize(op, ctypes.byref(ws_size)))
    workspace = torch.empty(max(ws_size.value, 1), dtype=torch.uint8, device=dev)

    stream = c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtStreamCreate(ctypes.byref(stream)))
    ev0, ev1 = c_void_p(), c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtEventCreate(ctypes.byref(ev0)))
    L.check_error(L.LIBINFINIRT.infinirtEventCreate(ctypes.byref(ev1)))

    def step():
        L.check_error(L.LIBINFINIOP.infiniopPagedAttentionPrefill(
            op, c_void_p(workspace.data_ptr()), ws_size.value, c_void_p(out.data_ptr()), c_void_p(q.data_ptr()),
            c_void_p(k_cache.data_ptr()), c_void_p(v_cache.data_ptr()), c_void_p(bt.data_ptr()), c_void_p(sl.data_ptr()),
            c_void_p(cu.data_ptr()), c_void_p(0), stream))

    if args.pmc_calibration:
        pmc_calibration_copies(torch, dev)
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    L.check_error(L.LIBINFINIRT.infinirtEventRecord(ev0, stream))
    for _ in range(args.steps):
        step()
    L.check_error(L.LIBINFINIRT.infinirtEventRecord(ev1, stream))
    L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms = c_float(0)
    L.check_error(L.LIBINFINIRT.infinirtEventElapsedTime(ctypes.byref(ms), ev0, ev1))
    us_wall = wall_s / args.steps * 1e6
    us_dev = ms.value / args.steps * 1e3
    tflops_wall = flops / (us_wall * 1e-6) / 1e12
    tflops_dev = flops / (us_dev * 1e-6) / 1e12

    result = {
        "metric": "PagedAttn prefill achieved TFLOP/s (2 * (head_size + value_size) * heads * visible query-key pairs / "
                  "time per call), 1 GPU",
        "value": round(tflops_wall, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_wall / 1e3, 6),
        "us_per_call": round(us_wall, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg.dtype == torch.bfloat16 else "f16",
        "data": "synthetic",
        "config": {
            "workload": cfg.name,
            "num_seqs": cfg.num_seqs, "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_kv_heads,
            "head_size": cfg.head_size, "value_size": cfg.v_size, "block_size": cfg.block_size,
            "new_tokens": f"uniform[{cfg.min_new},{cfg.max_new}] sum={int(new.sum())}",
            "history_tokens": f"uniform[{cfg.min_history},{cfg.max_history}] sum={int(history.sum())}",
            "flops_per_call": flops,
            "algorithmic_bytes_per_call": algo_bytes,
        },
        "roofline": {
            "bound": "mfma",
            "achieved": round(tflops_dev, 1),
            "peak": MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(tflops_dev / MFMA_PEAK_TFLOPS, 4),
            **traffic_fields(cfg.name),
            "us_per_call_device": round(us_dev, 2),
            "note": "achieved = flops per call / device time per call (events on the kernel's stream); one kernel per call",
        },
    }

    from oracle import paged_oracle

    threads = min(16, os.cpu_count() or 1)
    # a bounded sample of query rows: first, middle and last row of every sequence plus random ones
    rng = np.random.default_rng(1)
    cum = inp.cum_seq_lens_q.tolist()
    rows = []
    for s in range(cfg.num_seqs):
        n = cum[s + 1] - cum[s]
        if n > 0:
            rows += [cum[s] + j for j in sorted({0, n // 2, n - 1} | set(rng.integers(0, n, 5).tolist()))]
    if not args.no_check:
        step()
        L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
        sel = torch.as_tensor(rows)
        _, want32 = paged_oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                                         inp.cum_seq_lens_q, inp.scale, rows=rows, num_threads=threads,
                                                         return_fp32=True)
        err = (out.float().cpu()[sel] - want32[sel]).abs()
        ok = bool((err <= 1e-2 + 2e-3 * want32[sel].abs()).all())
        result["parity"] = {"rows_checked": len(rows), "max_abs_err": float(err.max()), "within_atol1e-2_rtol2e-3": ok}
        if not ok:
            print(json.dumps(result))
            print("bench.py: output does not match the oracle", file=sys.stderr)
            sys.exit(4)
    if not args.no_cpu_baseline:
        # the C oracle on the sampled rows, scaled by the flops those rows stand for
        sample_pairs = 0
        for r in rows:
            s = int(np.searchsorted(np.asarray(cum), r, side="right") - 1)
            sample_pairs += int(history[s]) + (r - cum[s]) + 1
        sample_flops = sample_pairs * cfg.num_heads * 2 * (cfg.head_size + cfg.v_size)
        reps, t0 = 0, time.perf_counter()
        while reps < 50 and time.perf_counter() - t0 < 12.0:
            paged_oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                                 inp.cum_seq_lens_q, inp.scale, rows=rows, num_threads=threads)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        result["cpu_baseline"] = {
            "value": round(sample_flops / cpu_s / 1e12, 5),
            "unit": "TFLOP/s",
            "cores": threads,
            "host_cores": os.cpu_count(),
            "kind": "port",
            "sample": f"{reps} passes of the C oracle over {len(rows)} of the {cum[-1]} query rows "
                      f"({sample_flops / flops * 100:.2f} % of the call's flops), {cpu_s * 1e3:.1f} ms per pass",
        }
    print(json.dumps(result))
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor(op))
    L.check_error(L.LIBINFINIRT.infinirtEventDestroy(ev0))
    L.check_error(L.LIBINFINIRT.infinirtEventDestroy(ev1))
    L.check_error(L.LIBINFINIRT.infinirtStreamDestroy(stream))
    L.destroy_handle(handle)


def run_caching(args, torch, L, workloads, dev):
    """One step = one infiniopPagedCaching call (scatter of a chunk of new K/V rows into the paged pools) or one
    infiniopKVCaching call (append to contiguous caches); inputs resident in HBM, several source / cache sets
    rotated so that the rows are not served from cache."""
    def oracle_fn(*operands):  # the checker and the CPU baseline; never on the timed path
        from oracle import paged_oracle

        if rope:
            if query is not None:
                paged_oracle.rope(query, pos, sin, cos, True)
            return paged_oracle.rope_paged_caching(*operands, pos, sin, cos, True)
        return (paged_oracle.paged_caching if paged else paged_oracle.kv_caching)(*operands)

    paged = args.workload in workloads.CACHING_CONFIGS
    rope = args.workload in workloads.ROPE_CACHING_CONFIGS
    query = None  # workloads that rotate the query in the same launch
    if rope:
        cfg = workloads.ROPE_CACHING_CONFIGS[args.workload]
        inp, pos, sin, cos = workloads.make_rope_caching_inputs(cfg)
        index = inp.slot_mapping
        algo_bytes = workloads.rope_caching_algorithmic_bytes(cfg, index.numpy())
        create = lambda handle, op, *descs: L.LIBINFINIOP.infiniopCreateRoPEPagedCachingDescriptor(handle, op, *descs, L.RoPEAlgo.GPT_NEOX)
        size_of = L.LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize
        call, destroy = L.LIBINFINIOP.infiniopRoPEPagedCaching, L.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor
        if cfg.name in workloads.ROPE_QUERY_HEADS:
            query = workloads.make_rope_query(cfg)
            create = lambda handle, op, *descs: L.LIBINFINIOP.infiniopCreateRoPEQKPagedCachingDescriptor(handle, op, *descs, L.RoPEAlgo.GPT_NEOX)
            call = L.LIBINFINIOP.infiniopRoPEQKPagedCaching
        metric = ("rotary embedding + paged_caching scatter achieved HBM GB/s (rows read + rows written + slot ids + "
                  "positions + table rows / time per call), 1 GPU")
        config = {"workload": cfg.name, "num_tokens": cfg.num_tokens, "valid_tokens": int((index >= 0).sum()),
                  "num_kv_heads": cfg.num_kv_heads, "head_size": cfg.head_size, "block_size": cfg.block_size,
                  "num_slots": cfg.num_slots, "table_len": workloads.ROPE_CACHING_TABLE_LEN, "algo": "gpt_neox",
                  "query_heads_rotated": workloads.ROPE_QUERY_HEADS.get(cfg.name, 0)}
    elif paged:
        cfg = workloads.CACHING_CONFIGS[args.workload]
        inp = workloads.make_caching_inputs(cfg)
        index = inp.slot_mapping
        algo_bytes = workloads.caching_algorithmic_bytes(cfg, index.numpy())
        create, size_of = L.LIBINFINIOP.infiniopCreatePagedCachingDescriptor, L.LIBINFINIOP.infiniopGetPagedCachingWorkspaceSize
        call, destroy = L.LIBINFINIOP.infiniopPagedCaching, L.LIBINFINIOP.infiniopDestroyPagedCachingDescriptor
        metric = "paged_caching scatter achieved HBM GB/s (rows read + rows written + slot ids / time per call), 1 GPU"
        config = {"workload": cfg.name, "num_tokens": cfg.num_tokens, "valid_tokens": int((index >= 0).sum()),
                  "num_kv_heads": cfg.num_kv_heads, "head_size": cfg.head_size, "block_size": cfg.block_size,
                  "num_slots": cfg.num_slots}
    else:
        cfg = workloads.KV_CACHING_CONFIGS[args.workload]
        inp = workloads.make_kv_caching_inputs(cfg)
        index = inp.past_kv_lengths
        algo_bytes = workloads.kv_caching_algorithmic_bytes(cfg)
        create, size_of = L.LIBINFINIOP.infiniopCreateKVCachingDescriptor, L.LIBINFINIOP.infiniopGetKVCachingWorkspaceSize
        call, destroy = L.LIBINFINIOP.infiniopKVCaching, L.LIBINFINIOP.infiniopDestroyKVCachingDescriptor
        metric = "kv_caching append achieved HBM GB/s (rows read + rows written + lengths / time per call), 1 GPU"
        config = {"workload": cfg.name, "batch": cfg.batch, "num_kv_heads": cfg.num_kv_heads, "max_seq_len": cfg.max_seq_len,
                  "new_tokens_per_sequence": cfg.new_tokens, "head_size": cfg.head_size}

    L.set_device(L.InfiniDevice.AMD, 0)
    handle = L.create_handle()
    index_dev = index.to(dev)
    # bound the rotation by memory: a set of the append workload's caches is 2 GiB
    set_bytes = 2 * inp.k_cache.numel() * inp.k_cache.element_size()
    n_sets = max(1, min(args.pools, (8 << 30) // max(set_bytes, 1)))
    sets = [(inp.k_cache.to(dev), inp.v_cache.to(dev), inp.k.to(dev), inp.v.to(dev)) for _ in range(n_sets)]
    DTYPES = {torch.float16: L.InfiniDtype.F16, torch.bfloat16: L.InfiniDtype.BF16, torch.int64: L.InfiniDtype.I64}
    extra = [t.to(dev) for t in (pos, sin, cos)] if rope else []
    # (q_out, q) in front of the other operands; one pair per rotated set
    q_sets = [(torch.empty_like(query, device=dev), query.to(dev)) for _ in sets] if query is not None else [()] * len(sets)
    descs = [L.create_tensor_descriptor(tuple(t.shape), tuple(t.stride()), DTYPES[t.dtype])
             for t in (*q_sets[0], *sets[0], index_dev, *extra)]
    op = L.infiniopOperatorDescriptor_t()
    L.check_error(create(handle, ctypes.byref(op), *descs))
    for d in descs:
        L.destroy_tensor_descriptor(d)
    ws_size = c_size_t(0)
    L.check_error(size_of(op, ctypes.byref(ws_size)))

    stream = c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtStreamCreate(ctypes.byref(stream)))
    ev0, ev1 = c_void_p(), c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtEventCreate(ctypes.byref(ev0)))
    L.check_error(L.LIBINFINIRT.infinirtEventCreate(ctypes.byref(ev1)))

    # The argument lists once, outside the timed loop: a call of 5 - 9 us of device time is short enough for the
    # host side of a step (building a dozen ctypes pointers) to show in the device-event time otherwise.
    call_args = [(op, c_void_p(0), 0, *[c_void_p(t.data_ptr()) for t in (*q_sets[j], *sets[j], index_dev, *extra)], stream)
                 for j in range(len(sets))]

    def step(i):
        status = call(*call_args[i % len(call_args)])
        if status != 0:
            L.check_error(status)

    if args.pmc_calibration:
        pmc_calibration_copies(torch, dev)
    torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    L.check_error(L.LIBINFINIRT.infinirtEventRecord(ev0, stream))
    for i in range(args.steps):
        step(i)
    L.check_error(L.LIBINFINIRT.infinirtEventRecord(ev1, stream))
    L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms = c_float(0)
    L.check_error(L.LIBINFINIRT.infinirtEventElapsedTime(ctypes.byref(ms), ev0, ev1))
    us_wall = wall_s / args.steps * 1e6
    us_dev = ms.value / args.steps * 1e3
    config.update({"sets_rotated": len(sets), "algorithmic_bytes_per_call": algo_bytes})

    result = {
        "metric": metric,
        "value": round(algo_bytes / (us_wall * 1e-6) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_wall / 1e3, 6),
        "us_per_call": round(us_wall, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": config,
        "roofline": {
            "bound": "hbm",
            "achieved": round(algo_bytes / (us_dev * 1e-6) / 1e9, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(algo_bytes / (us_dev * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            **traffic_fields(cfg.name),
            "us_per_call_device": round(us_dev, 2),
            "note": "achieved = algorithmic bytes / device time per call (events on the kernel's stream, back-to-back "
                    "launches); 32 MB per call is 4 us of traffic at 8 TB/s, the size of a kernel launch",
        },
    }

    if not args.no_check:
        kc, vc, k, v = sets[0]
        want_k, want_v = oracle_fn(inp.k_cache.clone(), inp.v_cache.clone(), inp.k, inp.v, index)
        ok = bool(torch.equal(kc.cpu().view(torch.int16), want_k.view(torch.int16))
                  and torch.equal(vc.cpu().view(torch.int16), want_v.view(torch.int16)))
        if query is not None:
            from oracle import paged_oracle

            ok = ok and torch.equal(q_sets[0][0].cpu().view(torch.int16), paged_oracle.rope(query, pos, sin, cos, True).view(torch.int16))
        result["parity"] = {"bit_exact": ok}
        if not ok:
            print(json.dumps(result))
            print("bench.py: caches differ from the oracle's", file=sys.stderr)
            sys.exit(4)
    if not args.no_cpu_baseline:
        kc, vc = inp.k_cache.clone(), inp.v_cache.clone()
        reps, t0 = 0, time.perf_counter()
        while reps < 2000 and time.perf_counter() - t0 < 10.0:
            oracle_fn(kc, vc, inp.k, inp.v, index)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        result["cpu_baseline"] = {
            "value": round(algo_bytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "host_cores": os.cpu_count(), "kind": "port",
            "sample": f"{reps} full calls of the same workload through the C oracle (one thread), {cpu_s * 1e6:.0f} us per call",
        }
    print(json.dumps(result))
    L.check_error(destroy(op))
    L.check_error(L.LIBINFINIRT.infinirtEventDestroy(ev0))
    L.check_error(L.LIBINFINIRT.infinirtEventDestroy(ev1))
    L.check_error(L.LIBINFINIRT.infinirtStreamDestroy(stream))
    L.destroy_handle(handle)


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU (no collective on it); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from infinicore_amd import libinfiniop as L
    from infinicore_amd import workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    if (args.workload in workloads.CACHING_CONFIGS or args.workload in workloads.KV_CACHING_CONFIGS
            or args.workload in workloads.ROPE_CACHING_CONFIGS):
        args.steps = 400 if args.steps is None else args.steps
        args.warmup = 40 if args.warmup is None else args.warmup
        return run_caching(args, torch, L, workloads, dev)
    if args.workload in workloads.PREFILL_CONFIGS:
        args.steps = 50 if args.steps is None else args.steps
        args.warmup = 5 if args.warmup is None else args.warmup
        return run_prefill(args, torch, L, workloads, dev)
    args.steps = 20 if args.steps is None else args.steps
    args.warmup = 3 if args.warmup is None else args.warmup
    layers = max(1, args.layers)
    cfg = workloads.DECODE_CONFIGS[args.workload]
    if args.head_size:
        cfg = dataclasses.replace(cfg, head_size=args.head_size, name=f"{cfg.name}_d{args.head_size}")
    inp = workloads.make_decode_inputs(cfg)
    algo_bytes = workloads.decode_algorithmic_bytes(cfg, inp.seq_lens.numpy())

    L.set_device(L.InfiniDevice.AMD, 0)
    handle = L.create_handle()

    q = inp.q.to(dev)
    bt = inp.block_tables.to(dev)
    sl = inp.seq_lens.to(dev)
    k_pools = [inp.k_cache.to(dev)]
    v_pools = [inp.v_cache.to(dev)]
    for _ in range(1, layers):
        k_pools.append(k_pools[0].clone())
        v_pools.append(v_pools[0].clone())
    out = torch.zeros((*q.shape[:-1], v_pools[0].shape[-1]), dtype=q.dtype, device=dev)

    # descriptor + workspace, exactly as a caller of the C API does it
    def describe(t):
        return L.create_tensor_descriptor(tuple(t.shape), tuple(t.stride()), DTYPES[t.dtype])

    DTYPES = {torch.float16: L.InfiniDtype.F16, torch.bfloat16: L.InfiniDtype.BF16, torch.int64: L.InfiniDtype.I64}
    descs = [describe(t) for t in (out, q, k_pools[0], v_pools[0], bt, sl)]
    op = L.infiniopOperatorDescriptor_t()
    L.check_error(L.LIBINFINIOP.infiniopCreatePagedAttentionDescriptor(
        handle, ctypes.byref(op), *descs, L.infiniopTensorDescriptor_t(), inp.scale))
    for d in descs:
        L.destroy_tensor_descriptor(d)
    ws_size = c_size_t(0)
    L.check_error(L.LIBINFINIOP.infiniopGetPagedAttentionWorkspaceSize(op, ctypes.byref(ws_size)))
    workspace = torch.empty(max(ws_size.value, 1), dtype=torch.uint8, device=dev)

    stream = c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtStreamCreate(ctypes.byref(stream)))
    ev0, ev1 = c_void_p(), c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtEventCreate(ctypes.byref(ev0)))
    L.check_error(L.LIBINFINIRT.infinirtEventCreate(ctypes.byref(ev1)))

    # argument lists built once: the host side of a call must not show in the time of the small workloads
    call_args = [(op, c_void_p(workspace.data_ptr()), ws_size.value, c_void_p(out.data_ptr()), c_void_p(q.data_ptr()),
                  c_void_p(k_pools[p].data_ptr()), c_void_p(v_pools[p].data_ptr()), c_void_p(bt.data_ptr()),
                  c_void_p(sl.data_ptr()), c_void_p(0), stream) for p in range(layers)]
    paged_attention = L.LIBINFINIOP.infiniopPagedAttention

    def call(p):
        status = paged_attention(*call_args[p])
        if status != 0:
            L.check_error(status, "infiniopPagedAttention")

    def step(i):
        for p in range(layers):
            call(p)

    if args.pmc_calibration:
        pmc_calibration_copies(torch, dev)

    torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
    torch.cuda.synchronize()

    t0 = time.perf_counter()
    L.check_error(L.LIBINFINIRT.infinirtEventRecord(ev0, stream))
    for i in range(args.steps):
        step(i)
    L.check_error(L.LIBINFINIRT.infinirtEventRecord(ev1, stream))
    L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms = c_float(0)
    L.check_error(L.LIBINFINIRT.infinirtEventElapsedTime(ctypes.byref(ms), ev0, ev1))

    calls = args.steps * layers
    us_wall = wall_s / calls * 1e6
    us_dev = ms.value / calls * 1e3                # device time per call on the kernels' stream
    gbps_wall = algo_bytes / (us_wall * 1e-6) / 1e9
    gbps_dev = algo_bytes / (us_dev * 1e-6) / 1e9

    result = {
        "metric": "PagedAttn decode achieved HBM GB/s (algorithmic bytes / time per call), 8B-GQA b=32, 1 GPU"
                  if cfg.name == "c2_llama3_8b_b32" else f"PagedAttn decode achieved HBM GB/s, {cfg.name}, 1 GPU",
        "value": round(gbps_wall, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_wall * layers / 1e3, 6),
        "us_per_call": round(us_wall, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if cfg.dtype == torch.bfloat16 else "f16",
        "data": "synthetic",
        "config": {
            "workload": cfg.name,
            "num_seqs": cfg.num_seqs, "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_kv_heads,
            "head_size": cfg.head_size, "value_size": cfg.v_size, "block_size": cfg.block_size,
            "seq_lens": f"uniform[{cfg.min_len},{cfg.max_len}] sum={int(inp.seq_lens.sum())}",
            "calls_per_step": layers,
            "kv_pools": len(k_pools),
            "algorithmic_bytes_per_call": algo_bytes,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbps_dev, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(gbps_dev / HBM_PEAK_GBPS, 4),
            **traffic_fields(cfg.name),
            "us_per_call_device": round(us_dev, 2),
            "note": "achieved = algorithmic bytes / device time per CALL (events on the kernels' stream bracket the "
                    "decode kernel and the small segment-merge kernel that follows it); traffic = HBM bytes of the "
                    "decode kernel per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE",
        },
    }

    if not args.no_check:
        # not timed: one more call on pool 0, compared with the CPU oracle
        from oracle import paged_oracle

        call(0)
        L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
        # against the oracle's value before its final rounding to the storage dtype: two correctly rounded
        # results can sit one bf16 step apart, which above |x| = 2.44 is already more than the tolerance
        _, want = paged_oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                               inp.scale, num_threads=min(16, os.cpu_count() or 1), return_fp32=True)
        err = (out.float().cpu() - want).abs()
        ok = bool((err <= 1e-2 + 2e-3 * want.abs()).all())
        result["parity"] = {"max_abs_err": float(err.max()), "within_atol1e-2_rtol2e-3": ok}
        if not ok:
            print(json.dumps(result))
            print("bench.py: output does not match the oracle", file=sys.stderr)
            sys.exit(4)

    if not args.no_cpu_baseline:
        from oracle import paged_oracle

        threads = min(16, os.cpu_count() or 1)
        paged_oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                     num_threads=threads)
        reps, t0 = 0, time.perf_counter()
        while reps < 50 and time.perf_counter() - t0 < 12.0:
            paged_oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                         num_threads=threads)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        result["cpu_baseline"] = {
            "value": round(algo_bytes / cpu_s / 1e9, 3),
            "unit": "GB/s",
            "cores": threads,
            "host_cores": os.cpu_count(),
            "kind": "port",
            "sample": f"{reps} full calls of the same workload through the C oracle (OpenMP over sequence x head, "
                      f"{threads} threads of the host's {os.cpu_count()} cores), {cpu_s * 1e3:.1f} ms per call",
            "us_per_call": round(cpu_s * 1e6, 1),
        }
        # the torch statement the reference's own test uses as expected value (vectorised gather), one call
        torch.set_num_threads(threads)
        t0 = time.perf_counter()
        paged_oracle.torch_reference_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale)
        torch_s = time.perf_counter() - t0
        result["cpu_baseline_torch"] = {
            "value": round(algo_bytes / torch_s / 1e9, 3), "unit": "GB/s", "cores": threads, "host_cores": os.cpu_count(),
            "kind": "port",
            "sample": f"1 full call of the reference test's torch formulation (vectorised gather) on CPU, "
                      f"torch.get_num_threads() = {torch.get_num_threads()}",
            "us_per_call": round(torch_s * 1e6, 1),
        }
        if cfg.name == "c1_plumbing_mha":
            # the literal form of the reference's test: a Python loop over every token of every sequence
            # (test/infiniop/paged_attention.py:60-73); only on the smallest workload, where it ends in seconds
            t0 = time.perf_counter()
            paged_oracle.torch_reference_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                                   inp.scale, vectorised=False)
            loop_s = time.perf_counter() - t0
            result["cpu_baseline_torch_token_loop"] = {
                "value": round(algo_bytes / loop_s / 1e9, 4), "unit": "GB/s", "cores": threads,
                "host_cores": os.cpu_count(), "kind": "port",
                "sample": "1 full call of the reference test's torch formulation with its per-token Python loop",
                "us_per_call": round(loop_s * 1e6, 1),
            }

    print(json.dumps(result))
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
    L.check_error(L.LIBINFINIRT.infinirtEventDestroy(ev0))
    L.check_error(L.LIBINFINIRT.infinirtEventDestroy(ev1))
    L.check_error(L.LIBINFINIRT.infinirtStreamDestroy(stream))
    L.destroy_handle(handle)


if __name__ == "__main__":
    main()

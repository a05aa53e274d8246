#!/usr/bin/env python3
"""Benchmark of the paged KV-cache data-movement path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops write,prefill,copy,swap]

Headline (`value`): benchmark configuration 2, the Llama-3-8B decode-step KV write
(256 sequences x 1 new token, 32 layers, 8 KV heads x 128, block_size 16, bf16,
pool of 65536 blocks = 128 GiB). One step = the K/V write of one decode step
over all 32 layers through `kvc_reshape_and_cache_layers` (one launch). Inputs
are resident in HBM before the timed region. K/V sources and slot sets rotate
over 16 sets (512 MiB of sources) so no step finds its lines in the 256 MiB
last-level cache. The K timed steps are K eager launches on torch's current
stream; `ops` repeats the measurement with the launches replayed from a hipGraph.

The same JSON line carries `roofline` (algorithmic bytes of one launch over the
launch's mean duration measured with events on the launch stream, against
8 TB/s), `cpu_baseline` (the torch-CPU statement of the same step on the host
cores, bounded sample) and `ops`: every other configuration and entry point
(per-layer launches, page-table addressing, chunked prefill, copy_blocks, swap)
with its own us/call and GB/s.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

REPO_ROOT = os.path.dirname(os.path.abspath(__file__))
if REPO_ROOT not in sys.path:
    sys.path.insert(0, REPO_ROOT)

HBM_PEAK_GBPS = 8000.0
ROTATE_DECODE = 16   # 16 x 32 MiB of K/V sources
PREWARM_S = 0.15     # seconds of untimed launches ahead of every timed region
ROTATE_PREFILL = 8   # 8 x 112 MiB of K/V sources

# HBM bytes per launch of the headline kernel (config 2, all layers in one launch)
# from two rocprofv3 --pmc runs: FETCH_SIZE 16410.8 KiB x 2.0000 + WRITE_SIZE
# 32813.8 KiB x 1.0000, the factors being what the same counters read for a
# plain elementwise kernel of known size (1 GiB read, 1 GiB written); summary in
# profiles/hbm_traffic_fetch_size_write_size.txt. Only valid for the default workload.
MEASURED_TRAFFIC_CFG2_ONE_LAUNCH = 67221046


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=320)
    p.add_argument("--warmup", type=int, default=32)
    p.add_argument("--ops", default="write,prefill,copy,swap,overlap,twoproc,rope,shard,disk,index",
                   help="comma list of extra measurements: write (per-layer / page-table variants "
                        "of config 2), prefill (config 3), copy (config 4), swap (config 5), "
                        "rope (rotation fused with the write vs two launches), "
                        "overlap (write-through behind a stand-in forward pass), "
                        "twoproc (a swap carried out by a KV-worker process on the IPC-mapped pool), "
                        "shard (one rank's head slice of Llama-3.1-70B at tp=8), "
                        "disk (host <-> disk tier), "
                        "index (index preparation of a step: host construction vs one launch), "
                        "sweep (write / copy_blocks / plain kernel over launch sizes; not in the default), "
                        "calib (a plain elementwise kernel of known size, for counter calibration); "
                        "queues (KV workers made one after the other beside a forward pass, to be run with "
                        "--hw-queues 4 and 8; not in the default); "
                        "translation (the config 3 launch with dense, block-run and random slots, for "
                        "address-translation counter runs; not in the default); "
                        "'none' for the headline only")
    p.add_argument("--settle-seconds", type=float, default=8.0,
                   help="quiet time before each section that uses the copy engines, after the bench has freed a pool")
    p.add_argument("--swap-blocks", type=int, default=8192,
                   help="blocks per swap direction; 8192 (40 GiB pinned) is config 5 at its stated size")
    p.add_argument("--pool-blocks", type=int, default=65536)
    p.add_argument("--disk-blocks", type=int, default=256,
                   help="blocks moved by the disk-tier measurement (5 MiB each)")
    p.add_argument("--disk-dir", default=None, help="directory of the disk-tier file (default: tmp)")
    p.add_argument("--hw-queues", type=int, default=8,
                   help="GPU_MAX_HW_QUEUES for this process (0 = leave the environment alone). The write-through "
                        "rows run the model's stream and the KV worker's streams in ONE process; with the "
                        "runtime's default of 4 hardware queues two of those streams can land on one queue "
                        "and wait for each other, which the reference's two processes (a set of queues "
                        "each) never do")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--cpu-seconds", type=float, default=10.0)
    return p.parse_args()


def time_region(fn, steps, warmup, torch, graph_of=0):
    """W untimed + K timed calls of fn(i); returns (wall ms/step, event ms/step).

    graph_of > 0: the launches of `graph_of` consecutive steps are captured once
    into a hipGraph and the timed region replays it (steps // graph_of) times,
    then runs the remaining steps eagerly -- exactly K steps either way, without
    the host's per-launch cost between them.

    Before the W warm-up calls the same fn runs for PREWARM_S of wall time, so
    that the memory and shader clocks have left their idle state (a cold start
    reads about 4 % slower on a 13 us launch); those calls are not counted."""
    t_end = time.perf_counter() + PREWARM_S
    i = 0
    while time.perf_counter() < t_end:
        fn(i)
        i += 1
        if i % 64 == 0:
            torch.cuda.synchronize()
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    graph = None
    if graph_of > 0 and steps >= graph_of:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(graph_of):
                fn(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(graph_of):
                fn(i)
        graph.replay()
        torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    if graph is not None:
        for _ in range(steps // graph_of):
            graph.replay()
        for i in range(steps % graph_of):
            fn(i)
    else:
        for i in range(steps):
            fn(warmup + i)
    end.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, start.elapsed_time(end) / steps


def entry(name, bytes_per_call, ms_wall, ms_event, calls_per_step=1, **extra):
    us = ms_event * 1e3 / calls_per_step
    gbps = bytes_per_call / (us * 1e-6) / 1e9 if us > 0 else 0.0
    d = {"name": name, "us_per_call": round(us, 3), "gbps": round(gbps, 1),
         "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
         "bytes_per_call": int(bytes_per_call),
         "wall_us_per_call": round(ms_wall * 1e3 / calls_per_step, 3)}
    d.update(extra)
    return d


def settle_copy_engines(torch, dev, what, quiet_s=8.0, limit_s=20.0):
    """For some seconds after a large device allocation has been freed (128 GiB:
    under 8 s on MI355X), transfers that hand over between a kernel and a copy
    engine several times per call run at half their rate (the staged swap-in at
    29 instead of 54 GB/s), while kernels and plain back-to-back copies keep
    theirs; waiting is what ends it, wherever the wait sits, so it is taken to be
    the driver working through the freed memory. The bench frees pools of tens of
    GiB between its sections, a serving process does not: let that time pass, then
    check that plain pinned copies run at a steady rate, before timing anything
    that uses the engines."""
    t_start = time.perf_counter()
    torch.cuda.synchronize()
    time.sleep(quiet_s)
    h = torch.empty(128 << 20, dtype=torch.uint8, pin_memory=True)
    d = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    rates = []
    while time.perf_counter() - t_start < quiet_s + limit_s:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        h.copy_(d, non_blocking=True)
        d.copy_(h, non_blocking=True)
        torch.cuda.synchronize()
        rates.append(2 * h.numel() / (time.perf_counter() - t0) / 1e9)
        last = rates[-4:]
        steady = len(last) == 4 and min(last) >= 0.97 * max(rates)
        # a PCIe Gen5 x16 link gives 55-57 GB/s; on a slower link, steady for 10 s is enough
        if steady and (rates[-1] >= 45.0 or time.perf_counter() - t_start >= quiet_s + 10.0):
            break
    waited = time.perf_counter() - t_start
    log(f"waited {waited:.1f} s before {what}; plain pinned copies then: {len(rates)} probes, "
        f"{min(rates):.1f} -> {rates[-1]:.1f} GB/s")
    return waited


class optional_section:
    """A section of rows beyond the headline: if it fails, say so and go on, so
    that the line with the headline is printed whatever happens here."""

    def __init__(self, name, torch):
        self.name, self.torch = name, torch

    def __enter__(self):
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is None or not issubclass(exc_type, Exception):
            return False
        log(f"{self.name} skipped: {exc!r}")
        tb = None
        try:
            self.torch.cuda.synchronize()
            self.torch.cuda.empty_cache()
        except Exception as again:
            log(f"after {self.name}: {again!r}")
        return True


def alloc_pool(torch, shape_cfg, num_blocks, dev):
    """[L, nb, 2, bs, H, D] bf16; drops layers if HBM cannot hold all of them."""
    L = shape_cfg.num_layers
    while L > 0:
        try:
            return torch.empty(L, num_blocks, 2, shape_cfg.block_size, shape_cfg.num_kv_heads,
                               shape_cfg.head_dim, dtype=torch.bfloat16, device=dev), L
        except torch.OutOfMemoryError:
            L //= 2
    raise RuntimeError("cannot allocate the KV pool")


def write_inputs(torch, kvc, workload_fn, shape_cfg, L, num_blocks, dev, rotate, **kw):
    """`rotate` sets of (workload, key, value, device index tensors) for a write config."""
    sets = []
    for r in range(rotate):
        w = workload_fn(shape_cfg, num_blocks=num_blocks, seed=r, **kw)
        key = torch.randn(L, w.num_tokens, shape_cfg.num_kv_heads, shape_cfg.head_dim, device=dev,
                          dtype=torch.float32).to(torch.bfloat16)
        value = torch.randn_like(key)
        sets.append((w, key, value, kvc.to_device(w.index, shape_cfg.block_size, dev)))
    return sets


def bench_write_config(torch, kvc, tag, sets, pool, L, steps, warmup, variants):
    """Measure the write entry points on one configuration.
    Returns (list of entries, {variant: (wall ms, event ms)})."""
    out, results = [], {}
    R = len(sets)
    w0 = sets[0][0]
    bytes_fused = w0.algorithmic_bytes(L)
    bytes_layer = w0.algorithmic_bytes(1)

    # per-layer views made once, as a model holds per-layer tensors (slicing costs
    # the host ~2 us per view and is not part of the operator)
    pool_l = [pool[l] for l in range(L)]
    k_l = [[sets[r][1][l] for l in range(L)] for r in range(R)]
    v_l = [[sets[r][2][l] for l in range(L)] for r in range(R)]

    def fused_slot(i):
        _, k, v, idx = sets[i % R]
        kvc.reshape_and_cache_layers(k, v, pool, idx.slot_mapping)

    def fused_paged(i):
        _, k, v, idx = sets[i % R]
        kvc.append_paged_kv_cache_layers(k, v, idx.batch_indices, idx.positions, pool,
                                         idx.kv_block_indices, idx.kv_block_indptrs,
                                         idx.kv_last_block_lens)

    def per_layer_paged(i):
        r = i % R
        idx = sets[r][3]
        ks, vs = k_l[r], v_l[r]
        for l in range(L):
            kvc.append_paged_kv_cache(ks[l], vs[l], idx.batch_indices, idx.positions, pool_l[l],
                                      idx.kv_block_indices, idx.kv_block_indptrs,
                                      idx.kv_last_block_lens)

    plans = {}

    def planned(i, resolve):
        r = i % R
        _, k, v, idx = sets[r]
        plan = plans.get((r, resolve))
        if plan is None:
            s = sets[r][0].shape
            plan = plans[(r, resolve)] = kvc.PagedKVWritePlan(
                idx.batch_indices, idx.positions, idx.kv_block_indices, idx.kv_block_indptrs,
                idx.kv_last_block_lens, s.num_kv_heads, s.head_dim, s.block_size, k.dtype,
                resolve_slots=resolve)
        ks, vs = k_l[r], v_l[r]
        for l in range(L):
            plan.append(ks[l], vs[l], pool_l[l])

    def per_layer_plan(i):
        planned(i, False)

    def per_layer_plan_resolved(i):
        planned(i, True)

    def per_layer_slot(i):
        r = i % R
        idx = sets[r][3]
        ks, vs = k_l[r], v_l[r]
        for l in range(L):
            kvc.reshape_and_cache(ks[l], vs[l], pool_l[l], idx.slot_mapping)

    table = {
        "fused_slot": (fused_slot, f"reshape_and_cache_layers (1 launch, {L} layers)", bytes_fused, 1),
        "fused_paged": (fused_paged, f"append_paged_kv_cache_layers (1 launch, {L} layers)",
                        bytes_fused, 1),
        "per_layer_paged": (per_layer_paged, f"append_paged_kv_cache (per layer, {L} launches per step)",
                            bytes_layer, L),
        "per_layer_plan": (per_layer_plan, f"PagedKVWritePlan.append (per layer, {L} launches per step)",
                           bytes_layer, L),
        "per_layer_plan_resolved": (per_layer_plan_resolved,
                                    f"PagedKVWritePlan(resolve_slots).append (per layer, {L} launches per step)",
                                    bytes_layer, L),
        "per_layer_slot": (per_layer_slot, f"reshape_and_cache (per layer, {L} launches per step)",
                           bytes_layer, L),
    }
    for variant in variants:
        name, mode = variant.split(":")
        fn, label, nbytes, calls = table[name]
        n = steps if calls == 1 else max(R, steps // 8 // R * R)
        wu = warmup if calls == 1 else max(2, warmup // 8)
        try:
            ms_w, ms_e = time_region(fn, n, wu, torch, graph_of=R if mode == "graph" else 0)
        except Exception as exc:  # a failed graph capture never takes the bench down
            log(f"{tag}/{label} [{mode}] skipped: {exc!r}")
            continue
        results[variant] = (ms_w, ms_e)
        out.append(entry(f"{tag}/{label}", nbytes, ms_w, ms_e, calls_per_step=calls,
                         launch="hipGraph replay" if mode == "graph" else "eager (one Python call per launch)"))
    return out, results


def bench_size_sweep(torch, kvc, wl, pool, L, num_blocks, dev):
    """One-launch write of T tokens x L layers, copy_blocks of P pairs x L layers and
    a plain elementwise kernel of the same byte count, over launch sizes from
    16 MiB to 2 GiB: where the fixed cost of a launch ends and bandwidth begins.
    Sources rotate over at least 512 MiB so no launch finds its lines cached."""
    s8 = wl.LLAMA_3_8B
    out = []
    for T in (64, 128, 256, 512, 1024, 2048, 4096, 8192):
        one_way = T * 2 * s8.row_bytes * L
        R = int(max(2, min(16, (512 << 20) // one_way)))
        sets = []
        for r in range(R):
            slots = torch.from_numpy(wl.random_free_slots(s8, num_blocks, T, seed=r)).to(dev)
            k = torch.randn(L, T, s8.num_kv_heads, s8.head_dim, device=dev, dtype=torch.float32).to(torch.bfloat16)
            sets.append((k, torch.randn_like(k), slots))
        n_el = one_way // 4
        srcs = [torch.zeros(n_el, dtype=torch.int32, device=dev) for _ in range(R)]
        dsts = [torch.empty(n_el, dtype=torch.int32, device=dev) for _ in range(R)]
        steps = max(R, min(64, (8 << 30) // (2 * one_way)) // R * R)
        ms_w, ms_e = time_region(lambda i: kvc.reshape_and_cache_layers(sets[i % R][0], sets[i % R][1], pool,
                                                                          sets[i % R][2]),
                                 steps, 2, torch, graph_of=R)
        ms_w2, ms_e2 = time_region(lambda i: torch.add(srcs[i % R], 1, out=dsts[i % R]), steps, 2, torch,
                                   graph_of=R)
        nbytes = 2 * one_way + 8 * T
        out.append(entry(f"sweep/write, {T} random rows x {L} layers in one launch", nbytes, ms_w, ms_e,
                         launch="hipGraph replay", plain_kernel_same_bytes_us=round(ms_e2 * 1e3, 3),
                         plain_kernel_same_bytes_gbps=round(2 * one_way / (ms_e2 * 1e-3) / 1e9, 1)))
        del sets, srcs, dsts
        torch.cuda.empty_cache()
    for P in (16, 64, 256, 1024, 4096):
        maps = [torch.from_numpy(wl.copy_on_write_pairs(num_blocks, P, seed=r)[0]).to(dev) for r in range(4)]
        nbytes = 2 * P * L * s8.block_bytes + 16 * P
        steps = max(4, min(64, (16 << 30) // nbytes) // 4 * 4)
        ms_w, ms_e = time_region(lambda i: kvc.copy_blocks(pool, maps[i % 4]), steps, 2, torch, graph_of=4)
        out.append(entry(f"sweep/copy_blocks, {P} pairs x {L} layers", nbytes, ms_w, ms_e,
                         launch="hipGraph replay"))
    return out


def bench_disk_tier(kvc, shape_cfg, n, directory):
    """Whole-block save (to the device, fdatasync included) and load through the
    native tier, beside the reference's way of doing it: one task per layer on 4
    threads, one row per entry through a NumPy memory map
    (runtime/worker/llm_worker/kv_worker.py:229-247, :297-322)."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    import numpy as np

    L, E = shape_cfg.num_layers, shape_cfg.block_elems
    directory = directory or tempfile.gettempdir()
    nbytes = n * L * E * 2
    pinned = kvc.PinnedHostPool((n, L, E), np.uint16)   # the pool the KV worker really holds
    host = pinned.array
    host[...] = np.arange(n, dtype=np.uint16)[:, None, None]
    rng = np.random.default_rng(0)
    src, dst = rng.permutation(n), rng.permutation(n)
    out = []
    path = os.path.join(directory, f"kvc-bench-disk-{os.getpid()}.npy")
    try:
        with kvc.DiskTier(path, (n, L, E), np.uint16, direct=True, threads=8) as d:
            t0 = time.perf_counter()
            d.save_blocks(host, src, dst)
            d.sync()
            t1 = time.perf_counter()
            d.load_blocks(host, dst, src)
            t2 = time.perf_counter()
            direct = d.is_direct
            staged = d.last_transfer_staged
        out.append({"name": f"cfg5 rows, Host->Disk ({n} blocks x {L} layers x 64 KiB, native tier, "
                            f"8 threads, O_DIRECT {'on' if direct else 'refused'}"
                            f"{', pinned pool staged through aligned buffers' if staged else ''}"
                            f", fdatasync included)",
                    "ms_per_call": round((t1 - t0) * 1e3, 1), "disk_gbps": round(nbytes / (t1 - t0) / 1e9, 2),
                    "bytes_per_call": int(nbytes)})
        out.append({"name": f"cfg5 rows, Disk->Host ({n} blocks, native tier, "
                            f"{'from the device' if direct else 'page cache warm'})",
                    "ms_per_call": round((t2 - t1) * 1e3, 1), "disk_gbps": round(nbytes / (t2 - t1) / 1e9, 2),
                    "bytes_per_call": int(nbytes)})
    finally:
        if os.path.exists(path):
            os.remove(path)
    try:
        mm = np.lib.format.open_memmap(path, mode="w+", dtype=np.uint16, shape=(n, L, E))

        def save_layer(l):
            for s_, d_ in zip(src, dst):
                mm[d_][l] = host[s_][l]

        def load_layer(l):
            for s_, d_ in zip(dst, src):
                host[d_][l] = mm[s_][l]

        with ThreadPoolExecutor(4) as ex:
            t0 = time.perf_counter()
            list(ex.map(save_layer, range(L)))
            mm.flush()
            t1 = time.perf_counter()
            list(ex.map(load_layer, range(L)))
            t2 = time.perf_counter()
        del mm
        out.append({"name": f"cfg5 rows, Host->Disk, port of the reference's memory-map row copies "
                            f"(4 threads, flush included)",
                    "ms_per_call": round((t1 - t0) * 1e3, 1), "disk_gbps": round(nbytes / (t1 - t0) / 1e9, 2),
                    "bytes_per_call": int(nbytes)})
        out.append({"name": "cfg5 rows, Disk->Host, port of the reference's memory-map row copies "
                            "(4 threads, page cache warm)",
                    "ms_per_call": round((t2 - t1) * 1e3, 1), "disk_gbps": round(nbytes / (t2 - t1) / 1e9, 2),
                    "bytes_per_call": int(nbytes)})
    finally:
        if os.path.exists(path):
            os.remove(path)
        del host
        pinned.close()
    return out


def cpu_baseline_write(torch, shape_cfg, L, seconds):
    """torch-CPU statement of the same step on a pool scaled to fit host RAM
    (same tokens, same rows, same bytes moved)."""
    from lmserve_amd import workloads as wl
    from oracle import torch_cpu
    nb = 2048
    w = wl.decode_step(shape_cfg, num_blocks=nb, batch=256, max_context=8 * shape_cfg.block_size,
                       seed=0)
    slots = torch.from_numpy(w.index.slot_mapping)
    T = w.num_tokens
    pool = torch.zeros(L, nb, 2, shape_cfg.block_size, shape_cfg.num_kv_heads, shape_cfg.head_dim,
                       dtype=torch.bfloat16)
    key = torch.randn(L, T, shape_cfg.num_kv_heads, shape_cfg.head_dim).to(torch.bfloat16)
    value = torch.randn_like(key)
    torch_cpu.reshape_and_cache_layers_cpu(key, value, pool, slots)  # warm-up
    n, t0 = 0, time.perf_counter()
    while True:
        torch_cpu.reshape_and_cache_layers_cpu(key, value, pool, slots)
        n += 1
        el = time.perf_counter() - t0
        if el >= seconds or n >= 20000:
            break
    per_step = el / n
    gbps = w.algorithmic_bytes(L) / per_step / 1e9
    return {"value": round(gbps, 2), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "us_per_step": round(per_step * 1e6, 1),
            "sample": f"{n} steps of the same decode-step write (T={T}, {L} layers) through the "
                      f"torch-CPU statement oracle/torch_cpu.py on a pool scaled to {nb} blocks/layer "
                      f"({pool.numel() * 2 / 2**30:.1f} GiB), {el:.1f} s"}


def cpu_baseline_others(torch, wl, seconds_each):
    """torch-CPU statements of the other operations on bounded samples: the
    prefill-chunk write (config 3 shape), copy_blocks (config 4 shape) and the
    swap in both directions (config 5 rows), pools scaled to fit host RAM."""
    from oracle import torch_cpu

    def timed(fn, nbytes, what):
        fn()  # warm-up
        n, t0 = 0, time.perf_counter()
        while True:
            fn()
            n += 1
            el = time.perf_counter() - t0
            if el >= seconds_each or n >= 5000:
                break
        return {"name": what, "value": round(nbytes * n / el / 1e9, 2), "unit": "GB/s",
                "us_per_call": round(el / n * 1e6, 1), "calls": n, "seconds": round(el, 1)}

    out = []
    # config 3: 2048 tokens x 28 layers, Qwen2.5-7B rows
    sq = wl.QWEN_2_5_7B
    nb = 2048
    w = wl.chunked_prefill(sq, num_blocks=nb, num_seqs=4, chunk_tokens=2048, min_context=16,
                           max_context=4096, seed=0)
    slots = torch.from_numpy(w.index.slot_mapping)
    pool = torch.zeros(sq.num_layers, nb, 2, sq.block_size, sq.num_kv_heads, sq.head_dim, dtype=torch.bfloat16)
    key = torch.randn(sq.num_layers, w.num_tokens, sq.num_kv_heads, sq.head_dim).to(torch.bfloat16)
    value = torch.randn_like(key)
    out.append(timed(lambda: torch_cpu.reshape_and_cache_layers_cpu(key, value, pool, slots),
                     w.algorithmic_bytes(sq.num_layers),
                     f"config 3 write, 2048 tokens x {sq.num_layers} layers, pool scaled to {nb} blocks/layer"))
    del pool, key, value
    # config 4: copy_blocks, 512 pairs x 32 layers x 64 KiB on a 4096-block pool
    s8 = wl.LLAMA_3_8B
    nb, P = 4096, 512
    pool = torch.zeros(s8.num_layers, nb, s8.block_elems, dtype=torch.bfloat16)
    flat, _ = wl.copy_on_write_pairs(nb, P, seed=0)
    src, dst = torch.from_numpy(flat[0::2].copy()), torch.from_numpy(flat[1::2].copy())
    out.append(timed(lambda: torch_cpu.copy_blocks_cpu(pool, src, dst), 2 * P * s8.num_layers * s8.block_bytes,
                     f"config 4 copy_blocks, {P} pairs x {s8.num_layers} layers x 64 KiB, pool scaled to {nb} blocks/layer"))
    del pool
    # config 5: swap rows, 128 blocks x 80 layers x 64 KiB each way
    s70 = wl.LLAMA_3_1_70B
    nb, n = 512, 128
    pool = torch.zeros(s70.num_layers, nb, s70.block_elems, dtype=torch.bfloat16)
    host = torch.zeros(n, s70.num_layers, s70.block_elems, dtype=torch.bfloat16)
    old, host_ids, new = wl.swap_round_trip(nb, n, seed=0)
    old_t, host_t, new_t = (torch.from_numpy(a) for a in (old, host_ids, new))
    nbytes = 2 * n * s70.num_layers * s70.block_bytes     # read + written
    out.append(timed(lambda: torch_cpu.swap_out_cpu(pool, host, old_t, host_t), nbytes,
                     f"config 5 swap-out rows, {n} blocks x {s70.num_layers} layers x 64 KiB (host memory both sides)"))
    out.append(timed(lambda: torch_cpu.swap_in_cpu(pool, host, host_t, new_t), nbytes,
                     f"config 5 swap-in rows, {n} blocks x {s70.num_layers} layers x 64 KiB (host memory both sides)"))
    return out


def bench_write_through_overlap(torch, kvc, wl, dev, scattered=False):
    """What the layer-pipelined protocol is for (kv_worker.py:272-295,
    model_worker.py:254-276): the KV worker saves layer l of the step's blocks to
    the host pool while the model is already computing layer l+1. A stand-in
    forward pass (per layer: four bf16 GEMMs of 0.11 ms, then the layer's K/V
    write through a per-step plan, then the post hook) runs alone, the
    layer-by-layer swap-out runs alone, and then both run together with the
    worker (a thread of this process, as the tests run it) following the hooks:
    once in the default staged mode (DMA engines carry the PCIe leg) and once in
    the direct mode (a kernel writes to the mapped host pool).

    scattered=True: the host blocks are every second block of the host pool (what
    an allocator hands out after churn), so a layer's rows are 64 KiB pieces that
    do not neighbour each other. The worker's default then carries each layer as
    one copy into a dense pinned buffer and lets host threads place the rows;
    beside it, the same worker without that buffer (the direct kernel) and the
    copy engines on the rows as they lie (one copy per block)."""
    import asyncio
    import threading

    import numpy as np

    s8 = wl.LLAMA_3_8B
    L, nb, n = s8.num_layers, 4096, 512            # 8 GiB pool; 512 blocks x 32 layers x 64 KiB = 1 GiB out
    pool = torch.empty(L, nb, 2, s8.block_size, s8.num_kv_heads, s8.head_dim, dtype=torch.bfloat16, device=dev)
    w = wl.decode_step(s8, num_blocks=nb, batch=256, max_context=200, seed=3)
    idx = kvc.to_device(w.index, s8.block_size, dev)
    key = torch.randn(L, 256, s8.num_kv_heads, s8.head_dim, device=dev).to(torch.bfloat16)
    value = torch.randn_like(key)
    a = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
    b = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
    c = torch.empty(4096, 4096, dtype=torch.bfloat16, device=dev)
    plan = kvc.PagedKVWritePlan(idx.batch_indices, idx.positions, idx.kv_block_indices, idx.kv_block_indptrs,
                                idx.kv_last_block_lens, s8.num_kv_heads, s8.head_dim, s8.block_size,
                                torch.bfloat16, resolve_slots=True)
    rng_ids = np.random.default_rng(5).permutation(nb)[:n]
    host_ids = list(range(0, 2 * n, 2)) if scattered else list(range(n))
    nhb = 2 * n if scattered else n
    maps = [kvc.BlockMapping.from_pairs(zip(rng_ids.tolist(), host_ids))]
    model_stream = torch.cuda.Stream()
    nbytes = n * L * s8.block_bytes
    out = []
    variants = [("staged", 0, False, "staged swap"), ("direct", 0, False, "direct swap"),
                ("staged", 1 << 30, True, "consecutive host blocks all the same through the dense pinned buffer: "
                                          "1-D copies + host threads")]
    if scattered:
        variants = [("auto", 1 << 30, False, "scattered host blocks; auto: one copy per layer into a dense pinned "
                                             "buffer, rows placed by host threads"),
                    ("auto", 0, False, "scattered host blocks; auto without the pinned buffer: the direct kernel"),
                    ("staged", 0, False, "scattered host blocks; staged: the copy engines, one copy per block")]
    for mode, bounce_bytes, always, label in variants:
        handle = kvc.KVWorkerHandle.create(L)
        worker = kvc.KVWorker(pool, num_host_blocks=nhb, swap_mode=mode, kv_worker_handle=handle,
                              host_bounce_bytes=bounce_bytes, host_bounce_always=always)
        scattered_timing = scattered or always      # measured through the protocol, not through prepared calls
        hooks = kvc.LayerSyncHooks(handle)

        def protocol_alone(copy_maps, src, dst, saving):
            """The layer-by-layer copy through `copy_kv` with nothing else on the GPU: the
            model side only rings the doorbells (save) or takes them (fetch)."""
            best = None
            for _ in range(4):
                torch.cuda.synchronize()
                th = threading.Thread(target=lambda: asyncio.run(worker.copy_kv(copy_maps, src, dst)))
                hooks.enable_record_after_execute = saving
                hooks.enable_wait_before_execute = not saving
                hooks.timeout = 60
                t0 = time.perf_counter()
                th.start()
                with torch.cuda.stream(model_stream):
                    for l in range(L):
                        hooks.pre(l)
                        hooks.post(l)
                th.join(timeout=120)
                torch.cuda.synchronize()
                t = (time.perf_counter() - t0) * 1e3
                best = t if best is None else min(best, t)
            hooks.enable_record_after_execute = False
            hooks.enable_wait_before_execute = False
            return best

        def forward():
            with torch.cuda.stream(model_stream):
                for l in range(L):
                    hooks.pre(l)
                    for _ in range(4):
                        torch.mm(a, b, out=c)
                    plan.append(key[l], value[l], pool[l])
                    hooks.post(l)

        def timed_forward():
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(model_stream)
            forward()
            e1.record(model_stream)
            return e0, e1

        try:
            forward()                                            # warm up (hooks off: nothing posted)
            torch.cuda.synchronize()
            e0, e1 = timed_forward()
            torch.cuda.synchronize()
            fwd_alone = e0.elapsed_time(e1)
            prepared = None if scattered_timing else worker.prepare_swap("out", maps)
            swap_alone = protocol_alone(maps, kvc.Device.GPU, kvc.Device.Host, True) if scattered_timing else None
            for _ in range(0 if scattered_timing else 4):               # the first pass touches the pinned pool
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for l in range(L):
                    worker.swap_prepared_layers(prepared, l, l + 1)
                worker.dtoh_stream.synchronize()
                t = (time.perf_counter() - t0) * 1e3
                swap_alone = t if swap_alone is None else min(swap_alone, t)

            def kv_thread():
                asyncio.run(worker.copy_kv(maps, kvc.Device.GPU, kvc.Device.Host))

            # three passes, the median by completion time reported (with all of them listed): the
            # first pass of a new worker beside a busy GPU can hold one of its enqueues for the
            # length of the forward pass, a one-time cost a server does not meet again
            hooks.enable_record_after_execute = True
            passes = []
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                th = threading.Thread(target=kv_thread)
                th.start()
                e0, e1 = timed_forward()
                th.join(timeout=120)
                torch.cuda.synchronize()
                passes.append(((time.perf_counter() - t0) * 1e3, e0.elapsed_time(e1)))
            hooks.enable_record_after_execute = False
            total, fwd_with = sorted(passes)[1]
            save_passes = [(round(f, 2), round(t, 2)) for t, f in passes]
            del prepared
            out.append({"name": f"write-through during a stand-in forward pass ({label}; {L} layers; {n} blocks x "
                                f"{L} layers x 64 KiB saved layer by layer behind the model's post hooks)",
                        "forward_alone_ms": round(fwd_alone, 2), "swap_alone_ms": round(swap_alone, 2),
                        "forward_with_write_through_ms": round(fwd_with, 2),
                        "forward_slowdown_pct": round(100.0 * (fwd_with / fwd_alone - 1.0), 1),
                        "both_done_after_ms": round(total, 2),
                        "passes_forward_ms_and_done_after_ms": save_passes,
                        "one_after_the_other_ms": round(fwd_alone + swap_alone, 2),
                        "pcie_gbps_alone": round(nbytes / swap_alone / 1e6, 2),
                        "bytes_per_call": int(nbytes)})
            # the other half of the protocol (kv_worker.py:249-270, model_worker.py:254-263): the
            # blocks of a request come back from the host layer by layer, and the model's layer l
            # waits for "layer l landed" before it runs
            in_maps = [kvc.BlockMapping.from_pairs(zip(host_ids, rng_ids.tolist()))]
            prepared_in = None if scattered_timing else worker.prepare_swap("in", in_maps)
            fetch_alone = protocol_alone(in_maps, kvc.Device.Host, kvc.Device.GPU, False) if scattered_timing else None
            for _ in range(0 if scattered_timing else 4):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for l in range(L):
                    worker.swap_prepared_layers(prepared_in, l, l + 1)
                worker.htod_stream.synchronize()
                t = (time.perf_counter() - t0) * 1e3
                fetch_alone = t if fetch_alone is None else min(fetch_alone, t)

            del prepared_in

            def kv_fetch_thread():
                asyncio.run(worker.copy_kv(in_maps, kvc.Device.Host, kvc.Device.GPU))

            hooks.enable_wait_before_execute = True
            hooks.timeout = 60
            passes = []
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                th = threading.Thread(target=kv_fetch_thread)
                th.start()
                e0, e1 = timed_forward()
                th.join(timeout=120)
                torch.cuda.synchronize()
                passes.append(((time.perf_counter() - t0) * 1e3, e0.elapsed_time(e1)))
            hooks.enable_wait_before_execute = False
            total, fwd_behind = sorted(passes)[1]
            out.append({"name": f"fetch during a stand-in forward pass ({label}; {L} layers; {n} blocks x {L} "
                                f"layers x 64 KiB loaded layer by layer, each layer of the model waits for its own)",
                        "forward_alone_ms": round(fwd_alone, 2), "fetch_alone_ms": round(fetch_alone, 2),
                        "forward_behind_the_fetch_ms": round(fwd_behind, 2),
                        "both_done_after_ms": round(total, 2),
                        "passes_forward_ms_and_done_after_ms": [(round(f, 2), round(t, 2)) for t, f in passes],
                        "one_after_the_other_ms": round(fwd_alone + fetch_alone, 2),
                        "pcie_gbps_alone": round(nbytes / fetch_alone / 1e6, 2),
                        "bytes_per_call": int(nbytes)})
        finally:
            worker.close()
            handle.close()
    del pool
    torch.cuda.empty_cache()
    return out


def bench_small_write_through(torch, kvc, wl, dev):
    """Where the per-call choice between the two swap modes sits: one-layer
    write-throughs of 1, 2, 4 and 8 MiB (16 to 128 blocks of the Llama-3-8B shape,
    consecutive host blocks) behind the same stand-in forward pass, by how much
    they lengthen it in each mode."""
    import asyncio
    import threading

    import numpy as np

    s8 = wl.LLAMA_3_8B
    L, nb = s8.num_layers, 4096
    pool = torch.empty(L, nb, 2, s8.block_size, s8.num_kv_heads, s8.head_dim, dtype=torch.bfloat16, device=dev)
    a = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
    b = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
    c = torch.empty(4096, 4096, dtype=torch.bfloat16, device=dev)
    model_stream = torch.cuda.Stream()
    out = []
    for n in (16, 32, 64, 128):
        ids = np.random.default_rng(5).permutation(nb)[:n]
        maps = [kvc.BlockMapping.from_pairs(zip(ids.tolist(), range(n)))]
        row = {"name": f"write-through of {n * 64 // 1024} MiB per layer ({n} blocks x {L} layers) during a stand-in "
                       f"forward pass: what it adds to the forward pass",
               "bytes_per_call": int(n * L * s8.block_bytes)}
        for mode in ("staged", "direct"):
            handle = kvc.KVWorkerHandle.create(L)
            worker = kvc.KVWorker(pool, num_host_blocks=n, swap_mode=mode, kv_worker_handle=handle)
            hooks = kvc.LayerSyncHooks(handle)
            try:
                def timed_forward():
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(model_stream)
                    with torch.cuda.stream(model_stream):
                        for l in range(L):
                            for _ in range(4):
                                torch.mm(a, b, out=c)
                            hooks.post(l)
                    e1.record(model_stream)
                    return e0, e1

                timed_forward()
                torch.cuda.synchronize()
                alone, beside = [], []
                for _ in range(3):
                    e0, e1 = timed_forward()
                    torch.cuda.synchronize()
                    alone.append(e0.elapsed_time(e1))
                for _ in range(3):
                    hooks.enable_record_after_execute = True
                    th = threading.Thread(
                        target=lambda: asyncio.run(worker.copy_kv(maps, kvc.Device.GPU, kvc.Device.Host)))
                    torch.cuda.synchronize()
                    th.start()
                    e0, e1 = timed_forward()
                    th.join(timeout=60)
                    torch.cuda.synchronize()
                    hooks.enable_record_after_execute = False
                    beside.append(e0.elapsed_time(e1))
                row[f"forward_alone_ms_{mode}"] = round(min(alone), 2)
                row[f"forward_with_write_through_ms_{mode}"] = round(min(beside), 2)
                row[f"forward_slowdown_pct_{mode}"] = round(100.0 * (min(beside) / min(alone) - 1.0), 1)
            finally:
                worker.close()
                handle.close()
        out.append(row)
    del pool
    torch.cuda.empty_cache()
    return out


def bench_worker_states(torch, kvc, wl, dev, workers=9):
    """Not in the default run (`--ops queues`, to be run with `--hw-queues 4` and
    `--hw-queues 8`): KV workers made one after the other in this process, each
    writing 1 GiB through to the host layer by layer beside the stand-in forward
    pass, four passes each. With the runtime's four hardware queues some workers
    spend their whole life in a slow state (their stream shares a queue with the
    model's); the row lists every worker's passes and a plain copy on its stream."""
    import asyncio
    import threading

    import numpy as np

    s8 = wl.LLAMA_3_8B
    L, nb, n = s8.num_layers, 4096, 512
    pool = torch.empty(L, nb, 2, s8.block_size, s8.num_kv_heads, s8.head_dim, dtype=torch.bfloat16, device=dev)
    a = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
    b = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
    c = torch.empty(4096, 4096, dtype=torch.bfloat16, device=dev)
    ids = np.random.default_rng(5).permutation(nb)[:n]
    model_stream = torch.cuda.Stream()
    probe_src = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    probe_dst = torch.empty(64 << 20, dtype=torch.uint8).pin_memory()
    rows = []
    for w in range(workers):
        dense = w % 3 != 2          # two workers on the dense-buffer path, then one on 2-D copies
        host_ids = list(range(0, 2 * n, 2)) if (w % 2 and dense) else list(range(n))
        maps = [kvc.BlockMapping.from_pairs(zip(ids.tolist(), host_ids))]
        handle = kvc.KVWorkerHandle.create(L)
        worker = kvc.KVWorker(pool, num_host_blocks=2 * n, swap_mode="staged", kv_worker_handle=handle,
                              host_bounce_always=dense, host_bounce_bytes=(1 << 30) if dense else 0)
        hooks = kvc.LayerSyncHooks(handle)
        try:
            def both(gemms):
                hooks.enable_record_after_execute = True
                th = threading.Thread(target=lambda: asyncio.run(worker.copy_kv(maps, kvc.Device.GPU, kvc.Device.Host)))
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                th.start()
                e0.record(model_stream)
                with torch.cuda.stream(model_stream):
                    for l in range(L):
                        for _ in range(gemms):
                            torch.mm(a, b, out=c)
                        hooks.post(l)
                e1.record(model_stream)
                th.join(timeout=120)
                torch.cuda.synchronize()
                hooks.enable_record_after_execute = False
                return round(e0.elapsed_time(e1), 1), round((time.perf_counter() - t0) * 1e3, 1)

            both(0)
            both(4)                       # the one-time cost of a new worker's first pass beside a busy GPU
            passes = [both(4) for _ in range(4)]
            rates = []
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                with torch.cuda.stream(worker.dtoh_stream):
                    probe_dst.copy_(probe_src, non_blocking=True)
                worker.dtoh_stream.synchronize()
                rates.append((64 << 20) / (time.perf_counter() - t0) / 1e9)
            rows.append({"worker": w, "path": "dense pinned buffer + host threads" if dense else "2-D copies of the rows as they lie",
                         "host_blocks": "every second" if (w % 2 and dense) else "consecutive",
                         "passes_forward_ms_and_done_after_ms": passes,
                         "plain_64MiB_copy_on_its_stream_gbps": round(max(rates), 1)})
        finally:
            worker.close()
            handle.close()
    del pool
    torch.cuda.empty_cache()
    return [{"name": f"{workers} KV workers one after the other in this process, 1 GiB write-through each beside the "
                     f"stand-in forward pass (GPU_MAX_HW_QUEUES={os.environ.get('GPU_MAX_HW_QUEUES', 'default')})",
             "workers": rows}]


def bench_two_process_swap(torch, kvc, wl, dev):
    """The reference's deployment: the KV worker is a process of its own that maps
    the pool from an IPC handle (kv_worker.py:97-160, cli.py:115-121). A pool in a
    segment of its own below 2 GiB, swapped out and back in by the other process;
    the time is the request's round trip as the model process sees it (queue
    hand-over included)."""
    import gc
    import multiprocessing as mp
    import queue as queue_mod

    s70 = wl.LLAMA_3_1_70B
    L, nb, n = 16, 1536, 768                  # 1.5 GiB pool, 0.75 GiB each way
    gc.collect()
    torch.cuda.empty_cache()
    pool = torch.empty(L, nb, 2, s70.block_size, s70.num_kv_heads, s70.head_dim, dtype=torch.bfloat16,
                       device=dev)
    ctx = mp.get_context("spawn")
    handle = kvc.KVWorkerHandle.create(L, interprocess=True, mp_context=ctx, sync="host")
    params = kvc.make_kv_worker_params(pool, handle, n)
    requests, replies = ctx.Queue(), ctx.Queue()
    mode = "auto"                             # the KV worker's default; consecutive host blocks: staged
    child = ctx.Process(target=kvc.serve_kv_worker, args=(params, dev.index or 0, requests, replies, mode),
                        daemon=True)
    child.start()
    out = []
    try:
        def get(what):
            try:
                msg = replies.get(timeout=60)
            except queue_mod.Empty:
                raise RuntimeError(f"the KV-worker process did not answer ({what})")
            if msg[0] == "error":
                raise RuntimeError(msg[1])
            return msg
        get("start-up")
        hooks = kvc.LayerSyncHooks(handle)
        hooks.timeout = 60
        old, host_ids, new = wl.swap_round_trip(nb, n, seed=1)
        nbytes = n * L * s70.block_bytes
        for direction, pairs, src, dst in (
                ("swap_out", list(zip(old.tolist(), host_ids.tolist())), kvc.Device.GPU, kvc.Device.Host),
                ("swap_in", list(zip(host_ids.tolist(), new.tolist())), kvc.Device.Host, kvc.Device.GPU)):
            best = None
            for _ in range(4):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                requests.put(("copy_kv", [pairs], int(src), int(dst)))
                # the model's half of the layer protocol (model_worker.py:254-276): a save waits
                # for "layer l written" per layer, a load announces "layer l landed" per layer
                if direction == "swap_out":
                    hooks.enable_record_after_execute = True
                    for l in range(L):
                        hooks.post(l)
                    hooks.enable_record_after_execute = False
                else:
                    hooks.enable_wait_before_execute = True
                    for l in range(L):
                        hooks.pre(l)
                    hooks.enable_wait_before_execute = False
                get(direction)
                t = time.perf_counter() - t0
                best = t if best is None else min(best, t)
            out.append({"name": f"two processes: {direction} by a KV-worker process on the IPC-mapped pool "
                                f"({mode}; {n} blocks x {L} layers x 64 KiB, request round trip)",
                        "ms_per_call": round(best * 1e3, 2), "pcie_gbps": round(nbytes / best / 1e9, 2),
                        "bytes_per_call": int(nbytes)})
    finally:
        handle.close()
        requests.put(("stop",))
        child.join(timeout=30)
        if child.is_alive():
            child.kill()
            child.join(timeout=10)
        del pool
        torch.cuda.empty_cache()
    return out


def per_layer_summary(entries):
    """The launches a layer-by-layer forward pass can actually issue (one K/V write
    per attention layer, as runtime/worker/llm_worker/models/layers/attention.py:76-85
    does), pulled out of `ops` for the top level of the line."""
    wanted = (
        ("eager_full_wrapper_us", "cfg2 decode/append_paged_kv_cache (per layer", "eager"),
        ("eager_plan_us", "cfg2 decode/PagedKVWritePlan.append", "eager"),
        ("graph_replay_us", "cfg2 decode/append_paged_kv_cache (per layer", "hipGraph"),
        ("eager_plan_resolved_slots_us", "cfg2 decode/PagedKVWritePlan(resolve_slots).append", "eager"),
        ("graph_replay_plan_resolved_slots_us", "cfg2 decode/PagedKVWritePlan(resolve_slots).append", "hipGraph"),
        ("rotation_then_append_eager_us", "cfg2 decode + rotation/rotary_pos_emb + append_paged_kv_cache", "eager"),
        ("rotation_fused_eager_full_wrapper_us", "cfg2 decode + rotation/rotary_pos_emb_and_append_paged", "eager"),
        ("rotation_fused_eager_plan_us", "cfg2 decode + rotation/PagedRotaryWritePlan.run", "eager"),
        ("rotation_fused_graph_replay_us", "cfg2 decode + rotation/rotary_pos_emb_and_append_paged", "hipGraph"),
        ("rotation_fused_graph_replay_plan_resolved_slots_us",
         "cfg2 decode + rotation/PagedRotaryWritePlan(resolve_slots).run", "hipGraph"),
        ("rotation_then_append_graph_replay_us", "cfg2 decode + rotation/rotary_pos_emb + append_paged_kv_cache", "hipGraph"),
    )
    out = {"workload": "configuration 2, one launch per layer (2 MiB of K/V rows per launch)",
           "note": "us per layer; eager rows are host-bound (wall time = what the serving loop pays)"}
    for key, prefix, launch in wanted:
        for e in entries:
            if e.get("name", "").startswith(prefix) and e.get("launch", "").startswith(launch):
                out[key] = e["wall_us_per_call"] if launch == "eager" else e["us_per_call"]
                if key == "graph_replay_us":
                    out["graph_replay_gbps"] = e["gbps"]
                break
    return out


def main():
    import numpy as np

    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this path has no cross-GPU step "
              f"(--gpus {args.gpus} is not supported)", file=sys.stderr)
        sys.exit(2)
    if args.hw_queues > 0:
        os.environ["GPU_MAX_HW_QUEUES"] = str(min(args.hw_queues, 32))   # read when the runtime starts
    import torch

    import lmserve_amd as kvc
    from lmserve_amd import _lib
    from lmserve_amd import workloads as wl

    from lmserve_amd.build import ensure_built
    ensure_built()  # uses the built library; compiles only if there is none
    _lib.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ops = set() if args.ops == "none" else set(args.ops.split(","))
    extra = []

    # ------------------------------------------------ config 2: decode-step write
    s8 = wl.LLAMA_3_8B
    pool, L = alloc_pool(torch, s8, args.pool_blocks, dev)
    log(f"pool {tuple(pool.shape)} = {pool.numel() * 2 / 2**30:.1f} GiB")
    sets = write_inputs(torch, kvc, wl.decode_step, s8, L, args.pool_blocks, dev, ROTATE_DECODE,
                        batch=256)
    variants = ["fused_slot:eager"]
    if "write" in ops:
        variants += ["fused_slot:graph", "fused_paged:eager", "per_layer_paged:graph",
                     "per_layer_slot:graph", "per_layer_paged:eager", "per_layer_plan:eager",
                     "per_layer_plan_resolved:eager", "per_layer_plan_resolved:graph"]
    entries, res = bench_write_config(torch, kvc, "cfg2 decode", sets, pool, L, args.steps,
                                      args.warmup, variants)
    extra += entries[1:]
    ms_wall, ms_event = res["fused_slot:eager"]
    bytes_step = sets[0][0].algorithmic_bytes(L)
    # One number per kernel: `value` and `roofline.achieved` both come from the event-timed
    # mean of the K timed steps (events recorded on the launch stream, inside the
    # synchronised region). The wall-clock mean of the same region additionally holds one
    # launch latency and one synchronisation (~40 us), which at K = 20 steps of 13 us is a
    # sixth of the region; it is reported as `wall_ms_per_step`.
    achieved = bytes_step / (ms_event * 1e-3) / 1e9
    value_gbps = achieved
    # dispersion of the same measurement: eight more regions of K steps each, event-timed
    # the same way (not part of `value`, which is the first region's mean)
    fused_fn = lambda i: kvc.reshape_and_cache_layers(sets[i % len(sets)][1], sets[i % len(sets)][2], pool,
                                                      sets[i % len(sets)][3].slot_mapping)
    regions = [ms_event]
    for _ in range(8):
        a_ev, b_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a_ev.record()
        for i in range(args.steps):
            fused_fn(i)
        b_ev.record()
        torch.cuda.synchronize()
        regions.append(a_ev.elapsed_time(b_ev) / args.steps)
    ran = _lib.last_launch()   # the launch shape of the headline entry, as the library reports it
    kernel_names = {_lib.KVC_KERNEL_WRITE_PLANES: "write_planes_kernel", _lib.KVC_KERNEL_WRITE_ROWS: "write_rows_kernel"}
    headline_kernel = (f"{kernel_names.get(ran['kernel'], 'kernel ' + str(ran['kernel']))}<{ran['per_lane']} "
                       f"{'planes' if ran['kernel'] == _lib.KVC_KERNEL_WRITE_PLANES else 'vectors'} per lane, slot-mapped, "
                       f"{'non-temporal stores' if ran['non_temporal'] & 1 else 'plain stores'}"
                       f"{', a wait per load' if ran['pipe'] == 1 else ''}>, "
                       f"{ran['grid']} workgroups of {ran['threads']} lanes")
    regions.sort()
    repeats = {"regions_of_k_steps": len(regions), "median_ms_per_step": round(regions[len(regions) // 2], 6),
               "min_ms_per_step": round(regions[0], 6), "max_ms_per_step": round(regions[-1], 6)}

    # a plain elementwise kernel moving the same bytes per launch as the headline
    # (32 MiB read + 32 MiB written), rotated over as many buffers: what a launch
    # of this size can reach on this machine whatever the kernel
    same_size = None
    try:
        n_el = (bytes_step // 2) // 4
        srcs = [torch.zeros(n_el, dtype=torch.int32, device=dev) for _ in range(ROTATE_DECODE)]
        dsts = [torch.empty(n_el, dtype=torch.int32, device=dev) for _ in range(ROTATE_DECODE)]
        ms_w, ms_e = time_region(lambda i: torch.add(srcs[i % ROTATE_DECODE], 1, out=dsts[i % ROTATE_DECODE]),
                                 args.steps, args.warmup, torch)
        same_size = {"kernel": "torch.add(int32, 1, out=...)", "bytes_per_launch": int(n_el * 8),
                     "us_per_launch": round(ms_e * 1e3, 3),
                     "gbps": round(n_el * 8 / (ms_e * 1e-3) / 1e9, 1)}
        del srcs, dsts
    except Exception as exc:
        log(f"same-size plain copy skipped: {exc!r}")

    # ------------------------------------------------ rotation + write, per layer (config 2 shape)
    if "rope" in ops:
        with optional_section("rotation rows", torch):
            Hq, Hkv, D, T = 32, s8.num_kv_heads, s8.head_dim, 256
            cs = kvc.make_cos_sin_cache(D, 8192, 500000.0, dtype=torch.bfloat16).to(dev)
            R = ROTATE_DECODE
            qs = [torch.randn(T, Hq * D, device=dev).to(torch.bfloat16) for _ in range(R)]
            ks = [sets[r][1][0].reshape(T, Hkv * D) for r in range(R)]
            vs = [sets[r][2][0].reshape(T, Hkv * D) for r in range(R)]
            idxs = [sets[r][3] for r in range(R)]
            pool_l = [pool[l] for l in range(L)]
            E = 2
            # q read+write, k read + cache write, v read + cache write, cos/sin row, indices
            rope_bytes = T * (2 * Hq * D * E + 2 * Hkv * D * E + 2 * Hkv * D * E + 2 * D * E + 12)

            def two_launches(i):
                r = i % R
                idx = idxs[r]
                for l in range(L):
                    q_o, k_o = kvc.rotary_pos_emb(qs[r], ks[r], idx.positions, cs, D)
                    kvc.append_paged_kv_cache(k_o, vs[r], idx.batch_indices, idx.positions, pool_l[l],
                                              idx.kv_block_indices, idx.kv_block_indptrs,
                                              idx.kv_last_block_lens)

            def fused(i):
                r = i % R
                idx = idxs[r]
                for l in range(L):
                    kvc.rotary_pos_emb_and_append_paged(qs[r], ks[r], vs[r], idx.batch_indices,
                                                        idx.positions, cs, D, pool_l[l],
                                                        idx.kv_block_indices, idx.kv_block_indptrs,
                                                        idx.kv_last_block_lens, return_key=False)

            plans = [kvc.PagedRotaryWritePlan(ix.batch_indices, ix.positions, ix.kv_block_indices,
                                              ix.kv_block_indptrs, ix.kv_last_block_lens, cs, Hq, Hkv, D,
                                              s8.block_size) for ix in idxs]
            q_buf = torch.empty(T, Hq * D, dtype=torch.bfloat16, device=dev)

            def fused_plan(i):
                r = i % R
                for l in range(L):
                    plans[r].run(qs[r], ks[r], vs[r], pool_l[l], query_out=q_buf)

            plans_r = [kvc.PagedRotaryWritePlan(ix.batch_indices, ix.positions, ix.kv_block_indices,
                                                ix.kv_block_indptrs, ix.kv_last_block_lens, cs, Hq, Hkv, D,
                                                s8.block_size, resolve_slots=True) for ix in idxs]

            def fused_plan_resolved(i):
                r = i % R
                for l in range(L):
                    plans_r[r].run(qs[r], ks[r], vs[r], pool_l[l], query_out=q_buf)

            n = max(R, args.steps // 8 // R * R)
            for fn, label in ((two_launches, "rotary_pos_emb + append_paged_kv_cache (2 launches per layer)"),
                              (fused, "rotary_pos_emb_and_append_paged (1 launch per layer)"),
                              (fused_plan, "PagedRotaryWritePlan.run (1 launch per layer)")):
                ms_w, ms_e = time_region(fn, n, 2, torch)
                extra.append(entry(f"cfg2 decode + rotation/{label}", rope_bytes, ms_w, ms_e,
                                   calls_per_step=L, launch="eager (one Python call per launch)"))
            for fn, label, extra_b in ((two_launches, "rotary_pos_emb + append_paged_kv_cache (2 launches per layer)",
                                        2 * T * Hkv * D * E),   # rotated key written out and read back
                                       (fused, "rotary_pos_emb_and_append_paged (1 launch per layer)", 0),
                                       (fused_plan_resolved,
                                        "PagedRotaryWritePlan(resolve_slots).run (1 launch per layer)", 0)):
                try:
                    ms_w, ms_e = time_region(fn, n, 2, torch, graph_of=R)
                except Exception as exc:
                    log(f"rope variant skipped: {exc!r}")
                    continue
                extra.append(entry(f"cfg2 decode + rotation/{label}", rope_bytes + extra_b, ms_w, ms_e,
                                   calls_per_step=L, launch="hipGraph replay"))
            del qs, ks, vs, idxs

    # ------------------------------------------------ config 4: copy_blocks (same pool)
    if "copy" in ops:
        with optional_section("config 4 copy_blocks row", torch):
            maps = [torch.from_numpy(wl.copy_on_write_pairs(args.pool_blocks, 4096, seed=r)[0]).to(dev)
                    for r in range(2)]
            nbytes = 2 * 4096 * L * s8.block_bytes + 16 * 4096
            ms_w, ms_e = time_region(lambda i: kvc.copy_blocks(pool, maps[i % 2]),
                                     max(5, min(args.steps, 20)), 3, torch)
            extra.append(entry(f"cfg4 copy_blocks (4096 pairs x {L} layers, 64 KiB blocks)", nbytes,
                               ms_w, ms_e, launch="eager"))
    # ------------------------------------------------ index preparation of a step
    if "index" in ops:
        with optional_section("index preparation rows", torch):
            for tag, wk in (("cfg2 decode, 256 requests", sets[0][0]),
                            ("cfg3 prefill chunk, 4 requests",
                             wl.chunked_prefill(wl.QWEN_2_5_7B, num_blocks=16384, seed=0))):
                reqs = wk.inputs
                bs_ = wk.shape.block_size
                n_ids = sum(len(r.block_ids) for r in reqs)

                def host_lists_and_uploads():
                    d = kvc.to_device(kvc.make_kv_index_inputs(reqs, bs_), bs_, dev, with_slot_mapping=False)
                    return d.positions

                def one_launch():
                    return kvc.to_device_one_launch(reqs, bs_, dev, with_slot_mapping=True).positions

                for fn, label in ((host_lists_and_uploads, "host list building + 6 uploads + 2 launches "
                                                          "(the reference's construction)"),
                                  (one_launch, "4 packed uploads + 1 launch (slot_mapping included)")):
                    for _ in range(5):
                        fn()
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    reps = 30
                    for _ in range(reps):
                        fn()
                    torch.cuda.synchronize()
                    us = (time.perf_counter() - t0) / reps * 1e6
                    extra.append({"name": f"index preparation/{tag} ({n_ids} block ids)/{label}",
                                  "wall_us_per_call": round(us, 1)})

    # ------------------------------------------------ launch-size sweep (8B shape, same pool)
    if "sweep" in ops:
        with optional_section("launch size sweep", torch):
            extra += bench_size_sweep(torch, kvc, wl, pool, L, args.pool_blocks, dev)
    del pool, sets
    torch.cuda.empty_cache()

    if "calib" in ops:
        with optional_section("calibration rows", torch):
            # a plain elementwise kernel of known size: reads 1 GiB, writes 1 GiB
            a = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
            b = torch.empty_like(a)
            ms_w, ms_e = time_region(lambda i: torch.add(a, 1, out=b), 10, 2, torch)
            extra.append(entry("calibration: plain elementwise kernel, 1 GiB read + 1 GiB written "
                               "(torch.add(int32, 1))", 2 << 30, ms_w, ms_e, launch="eager"))
            # write-only ceiling of the machine: a plain fill of 1 GiB
            ms_w, ms_e = time_region(lambda i: b.fill_(3), 10, 2, torch)
            extra.append(entry("calibration: plain fill, 1 GiB written (Tensor.fill_)", 1 << 30, ms_w, ms_e,
                               launch="eager"))
            del a, b
            torch.cuda.empty_cache()

    # ------------------------------------------------ config 3: chunked-prefill write
    if "prefill" in ops:
        with optional_section("config 3 rows", torch):
            sq = wl.QWEN_2_5_7B
            pool3, L3 = alloc_pool(torch, sq, 16384, dev)
            sets3 = write_inputs(torch, kvc, wl.chunked_prefill, sq, L3, 16384, dev, ROTATE_PREFILL)
            e3, _ = bench_write_config(torch, kvc, "cfg3 chunked prefill", sets3, pool3, L3,
                                       max(ROTATE_PREFILL, args.steps // 2), max(3, args.warmup // 2),
                                       ["fused_slot:graph", "fused_paged:graph", "per_layer_paged:graph"])
            extra += e3
            if "rope" in ops:
                # rotation + write per layer at the prefill chunk (28 query heads, 4 KV heads x 128)
                Hq3, Hkv3, D3 = 28, sq.num_kv_heads, sq.head_dim
                T3 = sets3[0][0].num_tokens
                R3 = len(sets3)
                cs3 = kvc.make_cos_sin_cache(D3, 65536, 1000000.0, dtype=torch.bfloat16).to(dev)
                q3 = [torch.randn(T3, Hq3 * D3, device=dev).to(torch.bfloat16) for _ in range(R3)]
                k3 = [sets3[r][1][0].reshape(T3, Hkv3 * D3) for r in range(R3)]
                v3 = [sets3[r][2][0].reshape(T3, Hkv3 * D3) for r in range(R3)]
                plans3 = [kvc.PagedRotaryWritePlan(ix.batch_indices, ix.positions, ix.kv_block_indices,
                                                   ix.kv_block_indptrs, ix.kv_last_block_lens, cs3, Hq3,
                                                   Hkv3, D3, sq.block_size) for _, _, _, ix in sets3]
                qo3 = torch.empty(T3, Hq3 * D3, dtype=torch.bfloat16, device=dev)
                pool3_l = [pool3[l] for l in range(L3)]
                bytes3 = T3 * (2 * Hq3 * D3 * 2 + 4 * Hkv3 * D3 * 2 + 2 * D3 * 2 + 12)

                def fused3(i):
                    r = i % R3
                    for l in range(L3):
                        plans3[r].run(q3[r], k3[r], v3[r], pool3_l[l], query_out=qo3)

                def two3(i):
                    r = i % R3
                    ix = sets3[r][3]
                    for l in range(L3):
                        q_o, k_o = kvc.rotary_pos_emb(q3[r], k3[r], ix.positions, cs3, D3)
                        kvc.append_paged_kv_cache(k_o, v3[r], ix.batch_indices, ix.positions, pool3_l[l],
                                                  ix.kv_block_indices, ix.kv_block_indptrs,
                                                  ix.kv_last_block_lens)

                for fn, label, extra_b in ((two3, "rotary_pos_emb + append_paged_kv_cache (2 launches per layer)",
                                            2 * T3 * Hkv3 * D3 * 2),
                                           (fused3, "PagedRotaryWritePlan.run (1 launch per layer)", 0)):
                    try:
                        ms_w, ms_e = time_region(fn, R3, 1, torch, graph_of=R3)
                    except Exception as exc:
                        log(f"prefill rope variant skipped: {exc!r}")
                        continue
                    extra.append(entry(f"cfg3 chunked prefill + rotation/{label}", bytes3 + extra_b, ms_w, ms_e,
                                       calls_per_step=L3, launch="hipGraph replay"))
                del q3, k3, v3, plans3, qo3
            del sets3, pool3
            torch.cuda.empty_cache()

    # ------------------------------------------------ config 3 launch, three slot patterns
    # (for counter runs: the same 2048-token x 28-layer launch writing one dense run per
    # layer, the workload's scattered 16-token block runs, and fully random rows; the
    # write_rows_kernel dispatches appear in that order, `reps` + 2 of each)
    if "translation" in ops:
        with optional_section("slot pattern rows", torch):
            sq = wl.QWEN_2_5_7B
            nbq = 16384
            poolq, Lq = alloc_pool(torch, sq, nbq, dev)
            Tq, Rq, reps = 2048, ROTATE_PREFILL, max(2, min(args.steps, 64))
            srcs = []
            for r in range(Rq):
                kq = torch.randn(Lq, Tq, sq.num_kv_heads, sq.head_dim, device=dev, dtype=torch.float32).to(torch.bfloat16)
                srcs.append((kq, torch.randn_like(kq)))
            patterns = (
                ("one dense run per layer (slots 0..2047)",
                 [torch.arange(Tq, dtype=torch.int64, device=dev) for _ in range(Rq)]),
                ("the workload's block runs (4 sequences x 32 scattered blocks of 16 tokens)",
                 [torch.from_numpy(wl.chunked_prefill(sq, num_blocks=nbq, seed=r).index.slot_mapping).to(dev)
                  for r in range(Rq)]),
                ("random rows (2048 distinct random slots)",
                 [torch.from_numpy(wl.random_free_slots(sq, nbq, Tq, seed=r)).to(dev) for r in range(Rq)]),
            )
            nbytes = 2 * 2 * Tq * sq.row_bytes * Lq + 8 * Tq
            rounds = 3                      # patterns interleaved, so drift hits all of them alike
            per_pattern = {label: [] for label, _ in patterns}
            for rnd in range(rounds):
                for label, slot_sets in patterns:
                    for i in range(2):
                        kvc.reshape_and_cache_layers(srcs[i % Rq][0], srcs[i % Rq][1], poolq, slot_sets[i % Rq])
                    torch.cuda.synchronize()
                    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    start.record()
                    for i in range(reps):
                        kvc.reshape_and_cache_layers(srcs[i % Rq][0], srcs[i % Rq][1], poolq, slot_sets[i % Rq])
                    end.record()
                    torch.cuda.synchronize()
                    per_pattern[label].append(start.elapsed_time(end) / reps)
                    log(f"translation: round {rnd}: {reps + 2} write_rows_kernel dispatches, {label}, "
                        f"{per_pattern[label][-1] * 1e3:.2f} us each")
            for label, _ in patterns:
                ms = sorted(per_pattern[label])[rounds // 2]
                extra.append(entry(f"cfg3 launch, slot pattern: {label}", nbytes, ms, ms, launch="eager",
                                   launches_per_round=reps + 2, rounds=rounds,
                                   us_per_round=[round(x * 1e3, 2) for x in per_pattern[label]]))
            del poolq, srcs
            torch.cuda.empty_cache()

    # ------------------------------------------------ config 5: swap round trip
    if "swap" in ops:
        with optional_section("config 5 swap rows", torch):
            s70 = wl.LLAMA_3_1_70B
            nb5 = 16384
            n = min(args.swap_blocks, nb5 // 2)
            pool5, L5 = alloc_pool(torch, s70, nb5, dev)
            # the pinned host pool first (40 GiB at the stated size): a box that cannot pin
            # that much runs the rows on fewer blocks, and their names say how many
            worker = None
            while worker is None:
                try:
                    worker = kvc.KVWorker(pool5, n)
                except MemoryError as exc:
                    if n <= 256:
                        raise
                    log(f"cannot pin a host pool of {n} blocks ({exc}); trying {n // 2}")
                    n //= 2
            try:
                old, host_ids, new = wl.swap_round_trip(nb5, n, seed=0)
                out_maps = [kvc.BlockMapping.from_pairs(zip(old.tolist(), host_ids.tolist()))]
                in_maps = [kvc.BlockMapping.from_pairs(zip(host_ids.tolist(), new.tolist()))]
                nbytes = n * L5 * s70.block_bytes
                # the on-device half alone: gather to / scatter from a dense HBM buffer (HBM roofline)
                ids_out = torch.from_numpy(old).to(dev)
                ids_in = torch.from_numpy(new).to(dev)
                dense = torch.empty(n, L5, s70.block_elems, dtype=torch.bfloat16, device=dev)
                ms_w, ms_e = time_region(lambda i: kvc.gather_blocks(pool5, ids_out, out=dense), 10, 2, torch)
                extra.append(entry(f"cfg5 gather stage, HBM only ({n} blocks x {L5} layers x 64 KiB -> dense buffer)",
                                   2 * nbytes, ms_w, ms_e, launch="eager"))
                ms_w, ms_e = time_region(lambda i: kvc.scatter_blocks(pool5, ids_in, dense), 10, 2, torch)
                extra.append(entry(f"cfg5 scatter stage, HBM only (dense buffer -> {n} blocks x {L5} layers x 64 KiB)",
                                   2 * nbytes, ms_w, ms_e, launch="eager"))
                del dense
                torch.cuda.empty_cache()
                settle_copy_engines(torch, dev, "the swap rows", args.settle_seconds)
                def timed_sync(fn, reps):
                    fn()   # warm-up (first touch of the pinned pool, staging allocation)
                    times = []
                    for _ in range(reps):
                        torch.cuda.synchronize()
                        t0 = time.perf_counter()
                        fn()
                        times.append(time.perf_counter() - t0)
                    return sorted(times)[len(times) // 2]

                size = f"{n} blocks x {L5} layers x 64 KiB"
                host_in = np.arange(n // 2, n, dtype=np.int64)
                both_out = [kvc.BlockMapping.from_pairs(zip(old[:n // 2].tolist(), range(n // 2)))]
                both_in = [kvc.BlockMapping.from_pairs(zip(host_in.tolist(), new[n // 2:].tolist()))]
                # "staged" (default): gather/scatter kernel + DMA extents on a second stream;
                # "direct": one kernel that addresses the mapped host pool
                for mode in ("staged", "direct"):
                    worker.swap_mode = mode
                    for direction, maps, src, dst in (
                            ("swap_out", out_maps, kvc.Device.GPU, kvc.Device.Host),
                            ("swap_in", in_maps, kvc.Device.Host, kvc.Device.GPU)):
                        t = timed_sync(lambda: worker.copy_kv_sync(maps, src, dst), 3)
                        extra.append({"name": f"cfg5 {direction} ({mode}; {size})", "ms_per_call": round(t * 1e3, 2),
                                      "pcie_gbps": round(nbytes / t / 1e9, 2), "bytes_per_call": int(nbytes)})

                    # one call per layer, as the layer-pipelined protocol issues them: ids checked and
                    # uploaded once (kvc_swap_prepare), then one call per layer
                    enqueue = []

                    def layer_by_layer_prepared():
                        t0 = time.perf_counter()
                        prep = worker.prepare_swap("out", out_maps)
                        t1 = time.perf_counter()
                        for l in range(L5):
                            worker.swap_prepared_layers(prep, l, l + 1)
                        enqueue.append((t1 - t0, time.perf_counter() - t1))
                        worker.dtoh_stream.synchronize()

                    t = timed_sync(layer_by_layer_prepared, 3)
                    prep_s, calls_s = sorted(enqueue[1:])[len(enqueue[1:]) // 2]
                    extra.append({"name": f"cfg5 swap_out layer by layer, ids uploaded once ({mode}; {L5} calls of {n} blocks x 1 layer)",
                                  "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                                  "bytes_per_call": int(nbytes),
                                  "host_ms_flatten_check_upload_once": round(prep_s * 1e3, 3),
                                  "host_ms_to_enqueue_all_layer_calls": round(calls_s * 1e3, 3),
                                  "host_us_per_layer_call": round(calls_s / L5 * 1e6, 2)})

                    # both directions at once on the worker's two streams (PCIe is full duplex):
                    # write-through of one set of blocks while another set is fetched
                    def both():
                        worker.save_kv_blocks_to_host_nowait(both_out)
                        worker.load_kv_blocks_from_host_nowait(both_in)
                        worker.dtoh_stream.synchronize()
                        worker.htod_stream.synchronize()

                    t = timed_sync(both, 3)
                    extra.append({"name": f"cfg5 swap_out and swap_in at once ({mode}; {n // 2} blocks each way)",
                                  "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                                  "pcie_gbps_note": "sum of both directions", "bytes_per_call": int(nbytes)})

                # host blocks that do not neighbour each other (every second block of the host pool:
                # what an allocator hands out after churn): the staged mode's PCIe leg falls apart into
                # one copy per block, the direct kernel does not care, "auto" picks per call
                ns = min(512, n // 2)
                scat_maps = [kvc.BlockMapping.from_pairs(zip(old[:ns].tolist(), range(0, 2 * ns, 2)))]
                sbytes = ns * L5 * s70.block_bytes
                for mode in ("staged", "direct", "auto"):
                    worker.swap_mode = mode
                    picked = {}

                    def scattered_layer_by_layer():
                        prep = worker.prepare_swap("out", scat_maps)
                        for l in range(L5):
                            worker.swap_prepared_layers(prep, l, l + 1)
                        picked["layer"] = _lib.last_swap_mode()
                        worker.dtoh_stream.synchronize()

                    def scattered_one_call():
                        worker.save_kv_blocks_to_host_nowait(scat_maps)
                        picked["all"] = _lib.last_swap_mode()
                        worker.dtoh_stream.synchronize()

                    names = {_lib.KVC_SWAP_STAGED: "staged", _lib.KVC_SWAP_DIRECT: "direct"}
                    t = timed_sync(scattered_layer_by_layer, 3)
                    extra.append({"name": f"cfg5 swap_out to scattered host blocks, layer by layer ({mode}"
                                          f"{' -> ' + names[picked['layer']] if mode == 'auto' else ''}; "
                                          f"{L5} calls of {ns} blocks x 1 layer, 64 KiB extents)",
                                  "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(sbytes / t / 1e9, 2),
                                  "bytes_per_call": int(sbytes)})
                    t = timed_sync(scattered_one_call, 3)
                    extra.append({"name": f"cfg5 swap_out to scattered host blocks, one call ({mode}"
                                          f"{' -> ' + names[picked['all']] if mode == 'auto' else ''}; "
                                          f"{ns} blocks x {L5} layers, 5 MiB extents)",
                                  "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(sbytes / t / 1e9, 2),
                                  "bytes_per_call": int(sbytes)})
                worker.swap_mode = "direct"
                enqueue2 = []

                def layer_by_layer_unprepared():
                    t0 = time.perf_counter()
                    for l in range(L5):
                        worker.save_kv_blocks_to_host_nowait(out_maps, layer_begin=l, layer_end=l + 1)
                    enqueue2.append(time.perf_counter() - t0)
                    worker.dtoh_stream.synchronize()

                t = timed_sync(layer_by_layer_unprepared, 1)
                extra.append({"name": f"cfg5 swap_out layer by layer, ids flattened, checked and uploaded per call (direct; {L5} calls)",
                              "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                              "bytes_per_call": int(nbytes),
                              "host_ms_to_enqueue_all_layer_calls": round(enqueue2[-1] * 1e3, 3)})
            finally:
                worker.close()
            del pool5
            torch.cuda.empty_cache()
    if "overlap" in ops:
        try:
            settle_copy_engines(torch, dev, "the write-through rows", args.settle_seconds)
            extra += bench_write_through_overlap(torch, kvc, wl, dev)
            extra += bench_write_through_overlap(torch, kvc, wl, dev, scattered=True)
            extra += bench_small_write_through(torch, kvc, wl, dev)
        except Exception as exc:
            log(f"write-through overlap skipped: {exc!r}")
    if "queues" in ops:
        with optional_section("worker states", torch):
            extra += bench_worker_states(torch, kvc, wl, dev)
    if "twoproc" in ops:
        try:
            settle_copy_engines(torch, dev, "the two-process rows", args.settle_seconds)
            extra += bench_two_process_swap(torch, kvc, wl, dev)
        except Exception as exc:   # a second process is optional equipment of the bench
            log(f"two-process swap skipped: {exc!r}")

    # ------------------------------------------------ one rank's slice of Llama-3.1-70B at tp=8
    if "shard" in ops:
        with optional_section("tensor-parallel shard rows", torch):
            sh = wl.LLAMA_3_1_70B.shard(8)          # 1 KV head: 256-byte rows, 8 KiB blocks, 80 layers
            nbs = 65536
            pool_s, Ls = alloc_pool(torch, sh, nbs, dev)
            sets_s = write_inputs(torch, kvc, wl.decode_step, sh, Ls, nbs, dev, ROTATE_DECODE, batch=256)
            es, _ = bench_write_config(torch, kvc, "70B/tp8 shard decode", sets_s, pool_s, Ls, args.steps,
                                       args.warmup, ["fused_slot:graph", "per_layer_paged:graph"])
            extra += es
            maps = [torch.from_numpy(wl.copy_on_write_pairs(nbs, 4096, seed=r)[0]).to(dev) for r in range(2)]
            nbytes = 2 * 4096 * Ls * sh.block_bytes + 16 * 4096
            ms_w, ms_e = time_region(lambda i: kvc.copy_blocks(pool_s, maps[i % 2]), 20, 3, torch)
            extra.append(entry(f"70B/tp8 shard copy_blocks (4096 pairs x {Ls} layers, 8 KiB blocks)", nbytes,
                               ms_w, ms_e, launch="eager"))
            n = min(4096, args.swap_blocks * 4, nbs // 2)
            old, host_ids, new = wl.swap_round_trip(nbs, n, seed=0)
            nbytes = n * Ls * sh.block_bytes
            settle_copy_engines(torch, dev, "the shard's swap rows", args.settle_seconds)
            worker = kvc.KVWorker(pool_s, n)
            try:
                for mode in ("staged", "direct"):
                    worker.swap_mode = mode
                    for direction, maps_, src, dst in (
                            ("swap_out", [kvc.BlockMapping.from_pairs(zip(old.tolist(), host_ids.tolist()))],
                             kvc.Device.GPU, kvc.Device.Host),
                            ("swap_in", [kvc.BlockMapping.from_pairs(zip(host_ids.tolist(), new.tolist()))],
                             kvc.Device.Host, kvc.Device.GPU)):
                        worker.copy_kv_sync(maps_, src, dst)
                        times = []
                        for _ in range(3):
                            torch.cuda.synchronize()
                            t0 = time.perf_counter()
                            worker.copy_kv_sync(maps_, src, dst)
                            times.append(time.perf_counter() - t0)
                        t = sorted(times)[1]
                        extra.append({"name": f"70B/tp8 shard {direction} ({mode}; {n} blocks x {Ls} layers x 8 KiB)",
                                      "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                                      "bytes_per_call": int(nbytes)})
            finally:
                worker.close()
            del pool_s, sets_s
            torch.cuda.empty_cache()

    # ------------------------------------------------ host <-> disk tier (config 5 block rows)
    if "disk" in ops:
        try:
            extra += bench_disk_tier(kvc, wl.LLAMA_3_1_70B, args.disk_blocks, args.disk_dir)
        except OSError as exc:
            log(f"disk tier skipped: {exc!r}")

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_write(torch, s8, L, args.cpu_seconds)
        if ops:
            cpu["other_ops"] = cpu_baseline_others(torch, wl, max(1.0, args.cpu_seconds / 4))

    line = {
        "metric": "achieved HBM GB/s, KV write (Llama-3-8B decode step)",
        "value": round(value_gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_event, 6),
        "wall_ms_per_step": round(ms_wall, 6),
        "timing": "mean over the K timed steps between two events on the launch stream; "
                  "wall_ms_per_step is the host clock around the same synchronised region",
        "repeats": repeats,
        "us_per_call": round(ms_event * 1e3, 3),
        "pct_of_hbm_peak": round(100.0 * value_gbps / HBM_PEAK_GBPS, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u16",
        "data": "synthetic",
        "config": {"workload": "configuration 2: Llama-3-8B decode-step KV write, 256 seqs x 1 token, "
                               f"{L} layers, 8 KV heads x 128, block_size 16, bf16 lanes, pool "
                               f"{args.pool_blocks} blocks "
                               f"({L * args.pool_blocks * s8.block_bytes / 2**30:.0f} GiB)",
                   "entry": "kvc_reshape_and_cache_layers (all layers in one launch)",
                   "launch": "one eager launch per step on torch's current stream",
                   "rotation": f"{ROTATE_DECODE} K/V source sets and slot sets cycled",
                   "clock_prewarm_s": PREWARM_S,
                   "hardware_queues_of_the_process": os.environ.get("GPU_MAX_HW_QUEUES", "runtime default")},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_CFG2_ONE_LAUNCH
                     if (L == 32 and args.pool_blocks == 65536) else None,
                     "kernel": headline_kernel,
                     "bytes_per_launch": int(bytes_step),
                     "us_per_launch": round(ms_event * 1e3, 3),
                     "plain_kernel_of_same_size": same_size,
                     "frac_of_plain_kernel_of_same_size":
                         round(achieved / same_size["gbps"], 3) if same_size else None},
        "target": {"wanted_frac_of_hbm_peak": 0.75, "met": bool(achieved / HBM_PEAK_GBPS >= 0.75),
                   "note": "the one-launch form is the upper bound for callers that hold all layers' "
                           "K/V at once; a layer-by-layer forward pass issues one launch per layer "
                           "(per_layer below), which at 2 MiB per launch is bound by launch latency, "
                           "not by HBM"},
        "per_layer": per_layer_summary(extra),
        "cpu_baseline": cpu,
        "ops": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()

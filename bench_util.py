"""Timing helpers shared by bench.py and bench_sections.py (no measurements of
their own): a timed region of K calls between two events on the launch stream,
the row format of the details file, pool and input builders."""
from __future__ import annotations

import sys
import time

HBM_PEAK_GBPS = 8000.0
ROTATE_DECODE = 16   # 16 x 32 MiB of K/V sources
PREWARM_S = 0.15     # seconds of untimed launches ahead of every timed region
ROTATE_PREFILL = 8   # 8 x 112 MiB of K/V sources


def log(*a):
    print(*a, file=sys.stderr, flush=True)



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


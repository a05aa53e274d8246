#!/usr/bin/env python3
"""Benchmark of the paged KV-cache data-movement path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops write,prefill,copy,swap,step]

Headline (`value`): benchmark configuration 2, the Llama-3-8B decode-step KV write
(256 sequences x 1 new token, 32 layers, 8 KV heads x 128, block_size 16, bf16,
pool of 65536 blocks = 128 GiB). One step = the K/V write of one decode step
over all 32 layers through `kvc_reshape_and_cache_layers` (one launch). Inputs
are resident in HBM before the timed region. K/V sources and slot sets rotate
over 16 sets (512 MiB of sources) so no step finds its lines in the 256 MiB
last-level cache. The K timed steps are K eager launches on torch's current
stream, between two events recorded on that stream.

The LAST line of stdout is one compact JSON object (under 4 KiB): the headline,
`roofline` (algorithmic bytes of one launch over the launch's mean duration,
against 8 TB/s), `cpu_baseline` (the torch-CPU statement of the same step on the
host cores, bounded sample) and `configs`: one short object per benchmark
configuration and form (us, GB/s, fraction of 8 TB/s, and counter traffic over
algorithmic bytes where it has been measured). Every other row (variants, passes, names in prose) goes to
the details file (`--details`, default bench_out/bench_details.json) and to
stderr, never to stdout.

Sections beyond the operations the benchmark names are opt-in
(`--ops ...,rope,shard,index,overlap,twoproc,disk,sweep,calib,translation,loads,duplex`) and
live in bench_sections.py.
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

from bench_util import (HBM_PEAK_GBPS, ROTATE_DECODE, ROTATE_PREFILL,  # noqa: E402
                        bench_write_config, entry, log, optional_section, settle_copy_engines, time_region,
                        write_inputs)

MAX_LINE_BYTES = 4096
DEFAULT_OPS = "write,prefill,copy,swap,step"

# HBM bytes per launch over algorithmic bytes, from two rocprofv3 --pmc runs per
# kernel (FETCH_SIZE x 2.0000 + WRITE_SIZE x 1.0000, the factors being what the
# same counters read for a plain elementwise kernel of 1 GiB read + 1 GiB
# written); profiles/hbm_traffic_fetch_size_write_size.txt. Valid for the default
# sizes only.
MEASURED_TRAFFIC_CFG2_ONE_LAUNCH = 67214029
TRAFFIC_RATIO = {
    ("cfg2", "1 launch"): 1.0015,
    ("cfg3", "1 launch"): 1.0014,
    ("cfg3", "1 launch, block runs"): 1.0002,   # profiles/write_runs_kernel_prefill_chunk_kernel_trace_and_translation_counters.txt
    ("cfg3", "per layer, graph"): 1.0208,
    ("cfg4", "1 launch"): 1.0000,
    ("cfg5", "gather"): 1.0000,
    ("cfg5", "scatter"): 1.0000,
}


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=320)
    p.add_argument("--warmup", type=int, default=32)
    p.add_argument("--ops", default=DEFAULT_OPS,
                   help="comma list of sections beside the headline. Default: write (per-layer / page-table "
                        "forms of config 2), prefill (config 3), copy (config 4), swap (config 5), step (a whole "
                        "decode step, index build included, replayed from one hipGraph). Opt-in: rope, shard, "
                        "index, overlap, twoproc, disk, sweep, calib, translation, loads, duplex. 'none' = headline only")
    p.add_argument("--details", default=None,
                   help="file for every row beyond the final line (default bench_out/bench_details.json; "
                        "'-' = stderr only)")
    p.add_argument("--settle-seconds", type=float, default=0.0,
                   help="quiet time before sections that use the copy engines after the bench has freed a "
                        "large pool (the default run frees none: all its pools come from one allocation)")
    p.add_argument("--swap-blocks", type=int, default=8192,
                   help="blocks per swap direction; 8192 (40 GiB pinned) is config 5 at its stated size")
    p.add_argument("--pool-blocks", type=int, default=65536)
    p.add_argument("--disk-blocks", type=int, default=256)
    p.add_argument("--disk-dir", default=None)
    p.add_argument("--hw-queues", type=int, default=0,
                   help="GPU_MAX_HW_QUEUES for this process (0 = leave the environment alone, the default)")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--cpu-seconds", type=float, default=8.0)
    return p.parse_args(argv)


# --------------------------------------------------------------------------- CPU baseline
def cpu_baseline_write(torch, wl, shape_cfg, L, seconds):
    """torch-CPU statement of the same step on a pool scaled to fit host RAM
    (same tokens, same rows, same bytes moved)."""
    from oracle import torch_cpu
    nb = 2048
    w = wl.decode_step(shape_cfg, num_blocks=nb, batch=256, max_context=8 * shape_cfg.block_size, seed=0)
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
            "sample": f"{n} decode-step writes (T={T}, {L} layers) via oracle/torch_cpu.py, "
                      f"pool {nb} blocks/layer, {el:.1f} s"}


def cpu_baseline_others(torch, wl, seconds_each):
    """torch-CPU statements of the other operations on bounded samples: the
    prefill-chunk write (config 3 shape), copy_blocks (config 4 shape) and the
    swap in both directions (config 5 rows), pools scaled to fit host RAM.
    Returns {config id: detail row}."""
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

    rows = {}
    sq = wl.QWEN_2_5_7B
    nb = 2048
    w = wl.chunked_prefill(sq, num_blocks=nb, num_seqs=4, chunk_tokens=2048, min_context=16,
                           max_context=4096, seed=0)
    slots = torch.from_numpy(w.index.slot_mapping)
    pool = torch.zeros(sq.num_layers, nb, 2, sq.block_size, sq.num_kv_heads, sq.head_dim, dtype=torch.bfloat16)
    key = torch.randn(sq.num_layers, w.num_tokens, sq.num_kv_heads, sq.head_dim).to(torch.bfloat16)
    value = torch.randn_like(key)
    rows["cfg3"] = timed(lambda: torch_cpu.reshape_and_cache_layers_cpu(key, value, pool, slots),
                         w.algorithmic_bytes(sq.num_layers),
                         f"config 3 write, 2048 tokens x {sq.num_layers} layers, pool scaled to {nb} blocks/layer")
    del pool, key, value
    s8 = wl.LLAMA_3_8B
    nb, P = 4096, 512
    pool = torch.zeros(s8.num_layers, nb, s8.block_elems, dtype=torch.bfloat16)
    flat, _ = wl.copy_on_write_pairs(nb, P, seed=0)
    src, dst = torch.from_numpy(flat[0::2].copy()), torch.from_numpy(flat[1::2].copy())
    rows["cfg4"] = timed(lambda: torch_cpu.copy_blocks_cpu(pool, src, dst), 2 * P * s8.num_layers * s8.block_bytes,
                         f"config 4 copy_blocks, {P} pairs x {s8.num_layers} layers x 64 KiB, pool scaled to {nb} "
                         f"blocks/layer")
    del pool
    s70 = wl.LLAMA_3_1_70B
    nb, n = 512, 128
    pool = torch.zeros(s70.num_layers, nb, s70.block_elems, dtype=torch.bfloat16)
    host = torch.zeros(n, s70.num_layers, s70.block_elems, dtype=torch.bfloat16)
    old, host_ids, new = wl.swap_round_trip(nb, n, seed=0)
    old_t, host_t, new_t = (torch.from_numpy(a) for a in (old, host_ids, new))
    nbytes = 2 * n * s70.num_layers * s70.block_bytes     # read + written
    rows["cfg5_out"] = timed(lambda: torch_cpu.swap_out_cpu(pool, host, old_t, host_t), nbytes,
                             f"config 5 swap-out rows, {n} blocks x {s70.num_layers} layers x 64 KiB (host memory "
                             f"both sides)")
    rows["cfg5_in"] = timed(lambda: torch_cpu.swap_in_cpu(pool, host, host_t, new_t), nbytes,
                            f"config 5 swap-in rows, {n} blocks x {s70.num_layers} layers x 64 KiB (host memory "
                            f"both sides)")
    return rows


# --------------------------------------------------------------------------- the final line
def config_row(cfg_id, entry_point, form, e, wall=False, **extra):
    """One object of the final line's `configs` array from a detail row."""
    us = e["wall_us_per_call"] if wall else e["us_per_call"]
    gbps = e["bytes_per_call"] / (us * 1e-6) / 1e9 if us > 0 else 0.0
    row = {"id": cfg_id, "entry": entry_point, "form": form, "us": round(us, 2), "gbps": round(gbps),
           "frac": round(gbps / HBM_PEAK_GBPS, 3)}
    if (cfg_id, form) in TRAFFIC_RATIO:      # measured with counters at the default sizes; absent = not measured
        row["traffic_ratio"] = TRAFFIC_RATIO[(cfg_id, form)]
    row.update(extra)
    return row


def find(entries, prefix, launch):
    for e in entries:
        if e.get("name", "").startswith(prefix) and e.get("launch", "").startswith(launch):
            return e
    return None


def build_line(head, configs):
    """The final stdout line: strict JSON under MAX_LINE_BYTES. `head` holds every
    key but `configs`; if the whole does not fit, configs are dropped from the end
    (the details file has them all) and `configs_dropped` says how many."""
    dropped = 0
    configs = [dict(c, entry=c["entry"].replace("kvc_", "")) for c in configs]   # entry points of libkvcache, prefix dropped
    while True:
        line = dict(head)
        line["configs"] = configs[:len(configs) - dropped]
        if dropped:
            line["configs_dropped"] = dropped
        text = json.dumps(line, allow_nan=False, separators=(",", ":"))
        if len(text.encode()) < MAX_LINE_BYTES or dropped >= len(configs):
            break
        dropped += 1
    assert len(text.encode()) < MAX_LINE_BYTES, f"final line is {len(text.encode())} bytes"
    assert json.loads(text)["metric"] == head["metric"]
    assert "\n" not in text
    return text


def write_details(path, details):
    if path == "-":
        return None
    if path is None:
        path = os.path.join(REPO_ROOT, "bench_out", "bench_details.json")
    try:
        os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
        with open(path, "w") as f:
            json.dump(details, f, indent=1)
        return path
    except OSError as exc:
        log(f"details file not written: {exc!r}")
        return None


class Arena:
    """One device allocation that every pool of the run is carved from (the 128 GiB
    of config 2's pool; the other configurations need less). The bench never frees
    a large pool between its sections: for some seconds after such a free,
    transfers that hand over between a kernel and a copy engine run at half their
    rate, and a serving process, which keeps its pool, never meets that."""

    def __init__(self, torch, dev, nbytes):
        self.torch = torch
        while True:
            try:
                self.buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
                break
            except torch.OutOfMemoryError:
                nbytes //= 2
                if nbytes < (1 << 30):
                    raise
        self.nbytes = nbytes
        self.used = 0

    def reset(self):
        self.used = 0

    def take(self, shape, dtype=None):
        torch = self.torch
        dtype = dtype or torch.bfloat16
        n = 1
        for d in shape:
            n *= int(d)
        nbytes = n * torch.empty(0, dtype=dtype).element_size()
        start = (self.used + 4095) // 4096 * 4096
        if start + nbytes > self.nbytes:
            raise MemoryError(f"arena of {self.nbytes} bytes cannot hold {nbytes} more")
        self.used = start + nbytes
        return self.buf[start:start + nbytes].view(dtype).view(*shape)

    def pool(self, shape_cfg, num_blocks):
        """[L, nb, 2, bs, H, D] bf16; drops layers if the arena cannot hold all of them."""
        L = shape_cfg.num_layers
        while L > 0:
            try:
                return self.take((L, num_blocks, 2, shape_cfg.block_size, shape_cfg.num_kv_heads,
                                  shape_cfg.head_dim)), L
            except MemoryError:
                L //= 2
        raise RuntimeError("cannot place the KV pool")


# --------------------------------------------------------------------------- config 5
def bench_swap(torch, kvc, _lib, wl, np, dev, swap_blocks, settle_seconds, arena):
    """Config 5: the on-device gather / scatter stages (HBM roofline) and the
    swap in both directions, staged and direct (PCIe). Returns
    (rows of the final line, detail rows)."""
    compact, detail = [], []
    s70 = wl.LLAMA_3_1_70B
    nb5 = 16384
    n = min(swap_blocks, nb5 // 2)
    pool5, L5 = arena.pool(s70, nb5)
    # the pinned host pool first (40 GiB at the stated size): a box that cannot pin
    # that much runs the rows on fewer blocks, and the rows say how many
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
        ids_out = torch.from_numpy(old).to(dev)
        ids_in = torch.from_numpy(new).to(dev)
        dense = arena.take((n, L5, s70.block_elems))
        for form, fn in (("gather", lambda i: kvc.gather_blocks(pool5, ids_out, out=dense)),
                         ("scatter", lambda i: kvc.scatter_blocks(pool5, ids_in, dense))):
            ms_w, ms_e = time_region(fn, 10, 2, torch)
            e = entry(f"cfg5 {form} stage, HBM only ({n} blocks x {L5} layers x 64 KiB)", 2 * nbytes, ms_w, ms_e,
                      launch="eager")
            detail.append(e)
            compact.append(config_row("cfg5", f"kvc_{form}_blocks", form, e))
        del dense
        if settle_seconds > 0:
            settle_copy_engines(torch, dev, "the swap rows", settle_seconds)

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
        for mode in ("staged", "direct"):
            worker.swap_mode = mode
            for direction, maps, src, dst in (
                    ("swap_out", out_maps, kvc.Device.GPU, kvc.Device.Host),
                    ("swap_in", in_maps, kvc.Device.Host, kvc.Device.GPU)):
                t = timed_sync(lambda: worker.copy_kv_sync(maps, src, dst), 3)
                detail.append({"name": f"cfg5 {direction} ({mode}; {size})", "ms_per_call": round(t * 1e3, 2),
                               "pcie_gbps": round(nbytes / t / 1e9, 2), "bytes_per_call": int(nbytes)})
                compact.append({"id": "cfg5", "entry": f"kvc_{direction}", "form": mode,
                                "ms": round(t * 1e3, 1), "pcie_gbps": round(nbytes / t / 1e9, 1)})
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
            detail.append({"name": f"cfg5 swap_out layer by layer, ids uploaded once ({mode}; {L5} calls of {n} "
                                   f"blocks x 1 layer)",
                           "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                           "bytes_per_call": int(nbytes),
                           "host_ms_flatten_check_upload_once": round(prep_s * 1e3, 3),
                           "host_us_per_layer_call": round(calls_s / L5 * 1e6, 2)})
        # both directions at once on the worker's two streams (PCIe is full duplex)
        worker.swap_mode = "staged"
        host_in = np.arange(n // 2, n, dtype=np.int64)
        both_out = [kvc.BlockMapping.from_pairs(zip(old[:n // 2].tolist(), range(n // 2)))]
        both_in = [kvc.BlockMapping.from_pairs(zip(host_in.tolist(), new[n // 2:].tolist()))]

        def both():
            worker.save_kv_blocks_to_host_nowait(both_out)
            worker.load_kv_blocks_from_host_nowait(both_in)
            worker.dtoh_stream.synchronize()
            worker.htod_stream.synchronize()

        t = timed_sync(both, 3)
        detail.append({"name": f"cfg5 swap_out and swap_in at once (staged; {n // 2} blocks each way)",
                       "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                       "pcie_gbps_note": "sum of both directions", "bytes_per_call": int(nbytes)})
        compact.append({"id": "cfg5", "entry": "kvc_swap_out+kvc_swap_in", "form": "staged, both at once",
                        "ms": round(t * 1e3, 1), "pcie_gbps": round(nbytes / t / 1e9, 1)})
        # host blocks that do not neighbour each other (every second block of the host pool:
        # what an allocator hands out after churn), one layer per call
        ns = min(512, n // 2)
        scat_maps = [kvc.BlockMapping.from_pairs(zip(old[:ns].tolist(), range(0, 2 * ns, 2)))]
        sbytes = ns * L5 * s70.block_bytes
        names = {_lib.KVC_SWAP_STAGED: "staged", _lib.KVC_SWAP_DIRECT: "direct"}
        for mode in ("staged", "direct", "auto"):
            worker.swap_mode = mode
            picked = {}

            def scattered_layer_by_layer():
                prep = worker.prepare_swap("out", scat_maps)
                for l in range(L5):
                    worker.swap_prepared_layers(prep, l, l + 1)
                picked["layer"] = _lib.last_swap_mode()
                worker.dtoh_stream.synchronize()

            t = timed_sync(scattered_layer_by_layer, 3)
            detail.append({"name": f"cfg5 swap_out to scattered host blocks, layer by layer ({mode}"
                                   f"{' -> ' + names[picked['layer']] if mode == 'auto' else ''}; "
                                   f"{L5} calls of {ns} blocks x 1 layer, 64 KiB extents)",
                           "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(sbytes / t / 1e9, 2),
                           "bytes_per_call": int(sbytes)})
    finally:
        worker.close()
    return compact, detail, n


def main(argv=None):
    import numpy as np

    args = parse_args(argv)
    if args.gpus != 1:
        print("bench.py measures one GPU only: this path has no cross-GPU step "
              f"(--gpus {args.gpus} is not supported)", file=sys.stderr)
        sys.exit(2)
    if args.hw_queues > 0:
        os.environ["GPU_MAX_HW_QUEUES"] = str(min(args.hw_queues, 32))   # read when the runtime starts
    import torch

    import lmserve_amd as kvc
    import workloads as wl
    from lmserve_amd import _lib
    from lmserve_amd.build import ensure_built

    t_begin = time.perf_counter()
    ensure_built()  # uses the built library; compiles only if there is none
    _lib.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ops = set() if args.ops == "none" else set(args.ops.split(","))
    details, configs = [], []
    swap_blocks_run = None
    default_sizes = args.pool_blocks == 65536

    # ------------------------------------------------ config 2: decode-step write (headline)
    s8 = wl.LLAMA_3_8B
    arena = Arena(torch, dev, s8.num_layers * args.pool_blocks * s8.block_bytes)
    pool, L = arena.pool(s8, args.pool_blocks)
    log(f"pool {tuple(pool.shape)} = {pool.numel() * 2 / 2**30:.1f} GiB")
    sets = write_inputs(torch, kvc, wl.decode_step, s8, L, args.pool_blocks, dev, ROTATE_DECODE, batch=256)
    variants = ["fused_slot:eager"]
    if "write" in ops:
        variants += ["fused_slot:graph", "fused_paged:eager", "per_layer_paged:graph",
                     "per_layer_slot:graph", "per_layer_paged:eager", "per_layer_plan:eager",
                     "per_layer_plan_resolved:eager", "per_layer_plan_resolved:graph"]
    entries, res = bench_write_config(torch, kvc, "cfg2 decode", sets, pool, L, args.steps, args.warmup, variants)
    details += entries
    ms_wall, ms_event = res["fused_slot:eager"]
    bytes_step = sets[0][0].algorithmic_bytes(L)
    # `value` and `roofline.achieved` both come from the event-timed mean of the K timed
    # steps (events on the launch stream, inside the synchronised region); the wall-clock
    # mean of the same region also holds one launch latency and one synchronisation.
    achieved = bytes_step / (ms_event * 1e-3) / 1e9
    # dispersion: eight more regions of K steps each, event-timed the same way
    n_sets = len(sets)
    regions = [ms_event]
    for _ in range(8):
        a_ev, b_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a_ev.record()
        for i in range(args.steps):
            r = i % n_sets
            kvc.reshape_and_cache_layers(sets[r][1], sets[r][2], pool, sets[r][3].slot_mapping)
        b_ev.record()
        torch.cuda.synchronize()
        regions.append(a_ev.elapsed_time(b_ev) / args.steps)
    ran = _lib.last_launch()   # the launch shape of the headline entry, as the library reports it
    kernel_names = {_lib.KVC_KERNEL_WRITE_PLANES: "write_planes_kernel", _lib.KVC_KERNEL_WRITE_ROWS: "write_rows_kernel"}
    headline_kernel = (f"{kernel_names.get(ran['kernel'], 'kernel ' + str(ran['kernel']))}<{ran['per_lane']} per lane>, "
                       f"{ran['grid']} wgs x {ran['threads']} lanes")
    regions.sort()
    configs.insert(0, config_row("cfg2", "kvc_reshape_and_cache_layers", "1 launch", entries[0],
                                 us_median=round(regions[len(regions) // 2] * 1e3, 2),
                                 us_min=round(regions[0] * 1e3, 2), us_max=round(regions[-1] * 1e3, 2)))

    # a plain elementwise kernel moving the same bytes per launch as the headline
    same_size = None
    with optional_section("same-size plain kernel", torch):
        n_el = (bytes_step // 2) // 4
        srcs = [torch.zeros(n_el, dtype=torch.int32, device=dev) for _ in range(ROTATE_DECODE)]
        dsts = [torch.empty(n_el, dtype=torch.int32, device=dev) for _ in range(ROTATE_DECODE)]
        ms_w, ms_e = time_region(lambda i: torch.add(srcs[i % ROTATE_DECODE], 1, out=dsts[i % ROTATE_DECODE]),
                                 args.steps, args.warmup, torch)
        same_size = {"us": round(ms_e * 1e3, 2), "gbps": round(n_el * 8 / (ms_e * 1e-3) / 1e9)}
        details.append(entry("plain elementwise kernel of the headline's size (torch.add int32)", n_el * 8, ms_w,
                             ms_e, launch="eager"))
        del srcs, dsts

    if "write" in ops:
        # (the page-table one-launch form, the full-argument eager call and the plan under a
        # graph are in the details file)
        for form, prefix, launch, entry_point, wall in (
                ("per layer, graph", "cfg2 decode/append_paged_kv_cache (per layer", "hipGraph",
                 "kvc_append_paged_kv_cache", False),
                ("per layer, plan, eager wall", "cfg2 decode/PagedKVWritePlan(resolve_slots).append", "eager",
                 "kvc_write_plan_append", True)):
            e = find(entries, prefix, launch)
            if e is not None:
                configs.append(config_row("cfg2", entry_point, form, e, wall=wall))
    log(f"[{time.perf_counter() - t_begin:.1f} s] config 2 done")

    if "rope" in ops:
        with optional_section("rotation rows", torch):
            from bench_sections import bench_rope_decode
            details += bench_rope_decode(torch, kvc, s8, sets, pool, L, dev, args.steps)

    # ------------------------------------------------ config 4: copy_blocks (same pool)
    if "copy" in ops:
        with optional_section("config 4 copy_blocks row", torch):
            maps = [torch.from_numpy(wl.copy_on_write_pairs(args.pool_blocks, 4096, seed=r)[0]).to(dev)
                    for r in range(2)]
            nbytes = 2 * 4096 * L * s8.block_bytes + 16 * 4096
            ms_w, ms_e = time_region(lambda i: kvc.copy_blocks(pool, maps[i % 2]),
                                     max(5, min(args.steps, 20)), 3, torch)
            e = entry(f"cfg4 copy_blocks (4096 pairs x {L} layers, 64 KiB blocks)", nbytes, ms_w, ms_e, launch="eager")
            details.append(e)
            configs.append(config_row("cfg4", "kvc_copy_blocks", "1 launch", e))
    if "index" in ops:
        with optional_section("index preparation rows", torch):
            from bench_sections import bench_index_prep
            details += bench_index_prep(torch, kvc, wl, sets[0][0], dev)
    if "sweep" in ops:
        with optional_section("launch size sweep", torch):
            from bench_sections import bench_size_sweep
            details += bench_size_sweep(torch, kvc, wl, pool, L, args.pool_blocks, dev)
    del pool, sets
    arena.reset()
    torch.cuda.empty_cache()   # the rotating K/V sources; the arena stays

    if "calib" in ops:
        with optional_section("calibration rows", torch):
            from bench_sections import bench_calibration
            details += bench_calibration(torch, dev)

    # ------------------------------------------------ config 3: chunked-prefill write
    if "prefill" in ops:
        with optional_section("config 3 rows", torch):
            sq = wl.QWEN_2_5_7B
            pool3, L3 = arena.pool(sq, 16384)
            sets3 = write_inputs(torch, kvc, wl.chunked_prefill, sq, L3, 16384, dev, ROTATE_PREFILL)
            e3, _ = bench_write_config(torch, kvc, "cfg3 chunked prefill", sets3, pool3, L3,
                                       max(ROTATE_PREFILL, args.steps // 2), max(3, args.warmup // 2),
                                       ["fused_slot:graph", "fused_paged:graph", "per_layer_paged:graph"])
            details += e3
            with optional_section("config 3 run write", torch):
                # the same launch as tile copies over the block runs the index build emits
                runs3 = []
                for w3, _, _, _ in sets3:
                    order = sorted(range(len(w3.inputs)), key=lambda i: -w3.inputs[i].input_len)
                    rs = [w3.inputs[i] for i in order]
                    up = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)   # noqa: E731
                    runs3.append(kvc.build_write_index(
                        up([r.input_len for r in rs]), up([r.context_len for r in rs]),
                        up([len(r.block_ids) for r in rs]), up([b for r in rs for b in r.block_ids]),
                        sq.block_size, w3.num_tokens, with_runs=True)[6])
                R3 = len(sets3)
                ms_w, ms_e = time_region(
                    lambda i: kvc.write_block_runs_layers(sets3[i % R3][1], sets3[i % R3][2], pool3, runs3[i % R3]),
                    max(ROTATE_PREFILL, args.steps // 2), max(3, args.warmup // 2), torch, graph_of=R3)
                e = entry(f"cfg3 chunked prefill/write_block_runs_layers (1 launch, {L3} layers, tile copies over "
                          f"{runs3[0].max_runs} run descriptors)", sets3[0][0].algorithmic_bytes(L3), ms_w, ms_e,
                          launch="hipGraph replay")
                details.append(e)
                configs.append(config_row("cfg3", "kvc_write_runs_layers", "1 launch, block runs", e))
            for form, prefix, entry_point in (
                    ("1 launch", "cfg3 chunked prefill/reshape_and_cache_layers", "kvc_reshape_and_cache_layers"),
                    ("per layer, graph", "cfg3 chunked prefill/append_paged_kv_cache (per layer",
                     "kvc_append_paged_kv_cache")):
                e = find(e3, prefix, "hipGraph")
                if e is not None:
                    configs.append(config_row("cfg3", entry_point, form, e))
            if "rope" in ops:
                from bench_sections import bench_rope_prefill
                details += bench_rope_prefill(torch, kvc, sq, sets3, pool3, L3, dev)
            del sets3, pool3
            arena.reset()
            torch.cuda.empty_cache()
        log(f"[{time.perf_counter() - t_begin:.1f} s] config 3 done")

    # ------------------------------------------------ config 5: swap round trip (pool and dense
    # buffer from the same arena: nothing large has been freed before its copies run)
    if "swap" in ops:
        with optional_section("config 5 swap rows", torch):
            c5, d5, swap_blocks_run = bench_swap(torch, kvc, _lib, wl, np, dev, args.swap_blocks,
                                                 args.settle_seconds, arena)
            configs += c5
            details += d5
        arena.reset()
        log(f"[{time.perf_counter() - t_begin:.1f} s] config 5 done")

    # ------------------------------------------------ a whole decode step from one hipGraph
    # (after the swap rows: whether swap-out and swap-in issued together overlap on the link
    # depends on the streams the KV worker is handed, which depends on how many streams the
    # process has made before; this order keeps that row comparable from run to run)
    if "step" in ops:
        with optional_section("decode step graph", torch):
            from bench_sections import bench_decode_step_graph
            pool, L = arena.pool(s8, args.pool_blocks)
            c, d = bench_decode_step_graph(torch, kvc, wl, s8, pool, L, args.pool_blocks, dev)
            configs += c
            details += d
            del pool
        arena.reset()
        log(f"[{time.perf_counter() - t_begin:.1f} s] decode step graph done")

    del arena
    torch.cuda.empty_cache()
    if "translation" in ops:
        with optional_section("slot pattern rows", torch):
            from bench_sections import bench_slot_patterns
            details += bench_slot_patterns(torch, kvc, wl, dev, args.steps)
    if "loads" in ops:
        with optional_section("load policy rows", torch):
            from bench_sections import bench_load_policy
            details += bench_load_policy(torch, kvc, wl, dev)
    if "duplex" in ops:
        with optional_section("both swap directions by stream choice", torch):
            from bench_sections import bench_duplex_streams
            details += bench_duplex_streams(torch, kvc, wl, dev)
    if "overlap" in ops:
        with optional_section("write-through overlap", torch):
            from bench_sections import bench_small_write_through, bench_write_through_overlap
            settle_copy_engines(torch, dev, "the write-through rows", max(args.settle_seconds, 8.0))
            details += bench_write_through_overlap(torch, kvc, wl, dev)
            details += bench_write_through_overlap(torch, kvc, wl, dev, scattered=True)
            details += bench_small_write_through(torch, kvc, wl, dev)
    if "twoproc" in ops:
        with optional_section("two-process swap", torch):
            from bench_sections import bench_two_process_swap
            settle_copy_engines(torch, dev, "the two-process rows", max(args.settle_seconds, 8.0))
            details += bench_two_process_swap(torch, kvc, wl, dev)
    if "shard" in ops:
        with optional_section("tensor-parallel shard rows", torch):
            from bench_sections import bench_tp_shard
            details += bench_tp_shard(torch, kvc, wl, dev, args.steps, args.warmup, args.swap_blocks,
                                      args.settle_seconds)
    if "disk" in ops:
        try:
            from bench_sections import bench_disk_tier
            details += bench_disk_tier(kvc, wl.LLAMA_3_1_70B, args.disk_blocks, args.disk_dir)
        except OSError as exc:
            log(f"disk tier skipped: {exc!r}")

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline_write(torch, wl, s8, L, args.cpu_seconds)
        if ops:
            others = cpu_baseline_others(torch, wl, max(1.0, args.cpu_seconds / 4))
            details += [dict(r, name="cpu baseline: " + r["name"]) for r in others.values()]
            cpu["others_gbps"] = {k: r["value"] for k, r in others.items()}

    head = {
        "metric": "achieved HBM GB/s, KV write (Llama-3-8B decode step)",
        "value": round(achieved, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_event, 6),
        "wall_ms_per_step": round(ms_wall, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u16",
        "data": "synthetic",
        "config": {"workload": f"config 2: Llama-3-8B decode-step KV write, 256 seqs x 1 token, {L} layers, "
                               f"8 KV heads x 128, block_size 16, pool {args.pool_blocks} blocks "
                               f"({L * args.pool_blocks * s8.block_bytes / 2**30:.0f} GiB)",
                   "entry": "kvc_reshape_and_cache_layers",
                   "launch": "one eager launch per step",
                   "rotation": ROTATE_DECODE,
                   "hw_queues": os.environ.get("GPU_MAX_HW_QUEUES", "runtime default"),
                   "cfg5_blocks": swap_blocks_run},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_CFG2_ONE_LAUNCH if (L == 32 and default_sizes) else None,
                     "kernel": headline_kernel,
                     "bytes_per_launch": int(bytes_step),
                     "us_per_launch": round(ms_event * 1e3, 3),
                     "plain_kernel_same_bytes": same_size},
        "target": {"frac": 0.75, "met": bool(achieved / HBM_PEAK_GBPS >= 0.75)},
        "cpu_baseline": cpu,
    }
    details_doc = {"line": head, "configs": configs, "rows": details,
                   "bench_seconds": round(time.perf_counter() - t_begin, 1)}
    path = write_details(args.details, details_doc)
    head["details"] = os.path.relpath(path, REPO_ROOT) if path else None
    for row in details:
        log(json.dumps(row))
    log(f"bench.py took {time.perf_counter() - t_begin:.1f} s")
    text = build_line(head, configs)
    sys.stderr.flush()
    print(text, flush=True)


if __name__ == "__main__":
    main()

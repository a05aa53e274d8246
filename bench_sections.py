"""Opt-in sections of bench.py (`--ops sweep,calib,translation,rope,shard,index,
overlap,twoproc,disk`): measurements beyond the four operations the headline
benchmark names. Each returns rows for the details file; none of them feeds the
final JSON line."""
from __future__ import annotations

import os
import time

from bench_util import (HBM_PEAK_GBPS, ROTATE_DECODE, ROTATE_PREFILL, alloc_pool, bench_write_config, entry, log,
                        optional_section, settle_copy_engines, time_region, write_inputs)


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
                              host_bounce_bytes=bounce_bytes, host_bounce_always=always,
                              model_streams=[model_stream, torch.cuda.current_stream()])
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
            worker = kvc.KVWorker(pool, num_host_blocks=n, swap_mode=mode, kv_worker_handle=handle,
                                  model_streams=[model_stream, torch.cuda.current_stream()])
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
        # take what the child still says until it reports that it has stopped, then
        # close both queues (their feeder threads) and collect the child: nothing of
        # this section is alive when it returns
        try:
            while replies.get(timeout=30)[0] != "stopped":
                pass
        except queue_mod.Empty:
            log("the KV-worker process did not report that it stopped")
        child.join(timeout=30)
        if child.is_alive():
            child.kill()
            child.join(timeout=10)
        for q in (requests, replies):
            q.close()
            q.join_thread()
        exitcode = child.exitcode
        child.close()
        del pool
        torch.cuda.empty_cache()
    if exitcode != 0:
        raise RuntimeError(f"the KV-worker process ended with exit code {exitcode}")
    return out



def bench_rope_decode(torch, kvc, s8, sets, pool, L, dev, steps):
    """Rotation + write per layer at the config 2 shape: the reference's two
    launches, the fused launch, and the fused launch through a per-step plan."""
    out = []
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

    n = max(R, steps // 8 // R * R)
    for fn, label in ((two_launches, "rotary_pos_emb + append_paged_kv_cache (2 launches per layer)"),
                      (fused, "rotary_pos_emb_and_append_paged (1 launch per layer)"),
                      (fused_plan, "PagedRotaryWritePlan.run (1 launch per layer)")):
        ms_w, ms_e = time_region(fn, n, 2, torch)
        out.append(entry(f"cfg2 decode + rotation/{label}", rope_bytes, ms_w, ms_e,
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
        out.append(entry(f"cfg2 decode + rotation/{label}", rope_bytes + extra_b, ms_w, ms_e,
                         calls_per_step=L, launch="hipGraph replay"))
    return out


def bench_rope_prefill(torch, kvc, sq, sets3, pool3, L3, dev):
    """Rotation + write per layer at the prefill chunk (28 query heads, 4 KV heads x 128)."""
    out = []
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
        out.append(entry(f"cfg3 chunked prefill + rotation/{label}", bytes3 + extra_b, ms_w, ms_e,
                         calls_per_step=L3, launch="hipGraph replay"))
    return out


def bench_index_prep(torch, kvc, wl, decode_workload, dev):
    """Index preparation of a step: the reference's host construction with its
    uploads against four packed uploads and one launch."""
    out = []
    for tag, wk in (("cfg2 decode, 256 requests", decode_workload),
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
            out.append({"name": f"index preparation/{tag} ({n_ids} block ids)/{label}",
                        "wall_us_per_call": round(us, 1)})
    return out


def bench_calibration(torch, dev):
    """A plain elementwise kernel of known size (1 GiB read, 1 GiB written) and a
    plain fill of 1 GiB: what the FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    out = []
    a = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
    b = torch.empty_like(a)
    ms_w, ms_e = time_region(lambda i: torch.add(a, 1, out=b), 10, 2, torch)
    out.append(entry("calibration: plain elementwise kernel, 1 GiB read + 1 GiB written "
                     "(torch.add(int32, 1))", 2 << 30, ms_w, ms_e, launch="eager"))
    ms_w, ms_e = time_region(lambda i: b.fill_(3), 10, 2, torch)
    out.append(entry("calibration: plain fill, 1 GiB written (Tensor.fill_)", 1 << 30, ms_w, ms_e,
                     launch="eager"))
    del a, b
    torch.cuda.empty_cache()
    return out


def bench_slot_patterns(torch, kvc, wl, dev, steps):
    """For counter runs: the config 3 launch (2048 tokens x 28 layers) writing one
    dense run per layer, the workload's scattered 16-token block runs, and fully
    random rows; the write kernel's dispatches appear in that order, `reps` + 2 of
    each per round."""
    out = []
    sq = wl.QWEN_2_5_7B
    nbq = 16384
    poolq, Lq = alloc_pool(torch, sq, nbq, dev)
    Tq, Rq, reps = 2048, ROTATE_PREFILL, max(2, min(steps, 64))
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
            log(f"translation: round {rnd}: {reps + 2} write-kernel dispatches, {label}, "
                f"{per_pattern[label][-1] * 1e3:.2f} us each")
    for label, _ in patterns:
        ms = sorted(per_pattern[label])[rounds // 2]
        out.append(entry(f"cfg3 launch, slot pattern: {label}", nbytes, ms, ms, launch="eager",
                         launches_per_round=reps + 2, rounds=rounds,
                         us_per_round=[round(x * 1e3, 2) for x in per_pattern[label]]))
    # the workload's block runs once more, moved as tile copies over run descriptors
    # (write_runs_kernel dispatches, after all write_rows_kernel ones)
    run_sets = []
    for r in range(Rq):
        wq = wl.chunked_prefill(sq, num_blocks=nbq, seed=r)
        order = sorted(range(len(wq.inputs)), key=lambda i: -wq.inputs[i].input_len)
        rs = [wq.inputs[i] for i in order]
        up = lambda a: torch.tensor(a, dtype=torch.int32, device=dev)   # noqa: E731
        run_sets.append(kvc.build_write_index(up([x.input_len for x in rs]), up([x.context_len for x in rs]),
                                              up([len(x.block_ids) for x in rs]),
                                              up([b for x in rs for b in x.block_ids]), sq.block_size, Tq,
                                              with_runs=True)[6])
    torch.cuda.synchronize()
    times = []
    for rnd in range(rounds):
        for i in range(2):
            kvc.write_block_runs_layers(srcs[i % Rq][0], srcs[i % Rq][1], poolq, run_sets[i % Rq])
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(reps):
            kvc.write_block_runs_layers(srcs[i % Rq][0], srcs[i % Rq][1], poolq, run_sets[i % Rq])
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end) / reps)
        log(f"translation: round {rnd}: {reps + 2} write_runs_kernel dispatches, the workload's block runs, "
            f"{times[-1] * 1e3:.2f} us each")
    ms = sorted(times)[rounds // 2]
    out.append(entry("cfg3 launch, the workload's block runs as tile copies over run descriptors (write_runs_kernel)",
                     nbytes, ms, ms, launch="eager", launches_per_round=reps + 2, rounds=rounds,
                     us_per_round=[round(x * 1e3, 2) for x in times]))
    del poolq, srcs
    torch.cuda.empty_cache()
    return out


def bench_tp_shard(torch, kvc, wl, dev, steps, warmup, swap_blocks, settle_seconds):
    """One rank's slice of Llama-3.1-70B at tp=8: 1 KV head, 256-byte rows, 8 KiB
    blocks, 80 layers."""
    out = []
    sh = wl.LLAMA_3_1_70B.shard(8)
    nbs = 65536
    pool_s, Ls = alloc_pool(torch, sh, nbs, dev)
    sets_s = write_inputs(torch, kvc, wl.decode_step, sh, Ls, nbs, dev, ROTATE_DECODE, batch=256)
    es, _ = bench_write_config(torch, kvc, "70B/tp8 shard decode", sets_s, pool_s, Ls, steps,
                               warmup, ["fused_slot:graph", "per_layer_paged:graph"])
    out += es
    maps = [torch.from_numpy(wl.copy_on_write_pairs(nbs, 4096, seed=r)[0]).to(dev) for r in range(2)]
    nbytes = 2 * 4096 * Ls * sh.block_bytes + 16 * 4096
    ms_w, ms_e = time_region(lambda i: kvc.copy_blocks(pool_s, maps[i % 2]), 20, 3, torch)
    out.append(entry(f"70B/tp8 shard copy_blocks (4096 pairs x {Ls} layers, 8 KiB blocks)", nbytes,
                     ms_w, ms_e, launch="eager"))
    n = min(4096, swap_blocks * 4, nbs // 2)
    old, host_ids, new = wl.swap_round_trip(nbs, n, seed=0)
    nbytes = n * Ls * sh.block_bytes
    if settle_seconds > 0:
        settle_copy_engines(torch, dev, "the shard's swap rows", settle_seconds)
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
                out.append({"name": f"70B/tp8 shard {direction} ({mode}; {n} blocks x {Ls} layers x 8 KiB)",
                            "ms_per_call": round(t * 1e3, 2), "pcie_gbps": round(nbytes / t / 1e9, 2),
                            "bytes_per_call": int(nbytes)})
    finally:
        worker.close()
    del pool_s, sets_s
    torch.cuda.empty_cache()
    return out


def bench_decode_step_graph(torch, kvc, wl, s8, pool, L, num_blocks, dev, steps=200):
    """A whole decode step of configuration 2 (index build + one K/V write per
    layer) replayed from ONE hipGraph for consecutive, different steps, beside
    the eager ways of doing the same step. Times are per 32-layer step.
    Returns (rows of the final line, detail rows)."""
    import numpy as np

    from lmserve_amd.step_graph import KVWriteStep

    R, B = 4, 256
    H, D, bs = s8.num_kv_heads, s8.head_dim, s8.block_size
    works = [wl.decode_step(s8, num_blocks=num_blocks, batch=B, seed=100 + r) for r in range(R)]
    packed = []
    for w in works:
        order = sorted(range(len(w.inputs)), key=lambda i: -w.inputs[i].input_len)
        rs = [w.inputs[i] for i in order]
        packed.append((np.asarray([r.input_len for r in rs], dtype=np.int32),
                       np.asarray([r.context_len for r in rs], dtype=np.int32),
                       np.asarray([len(r.block_ids) for r in rs], dtype=np.int32),
                       np.asarray([b for r in rs for b in r.block_ids], dtype=np.int32)))
    cap_ids = max(p[3].shape[0] for p in packed)
    step = KVWriteStep(H, D, bs, torch.bfloat16, dev, max_requests=B, max_tokens=B, max_block_ids=cap_ids)
    key = torch.randn(L, B, H, D, device=dev).to(torch.bfloat16)
    value = torch.randn_like(key)
    keys, values, caches = [key[l] for l in range(L)], [value[l] for l in range(L)], [pool[l] for l in range(L)]
    step.set_arrays(*packed[0])
    graph = step.capture(keys, values, caches)
    bytes_step = works[0].algorithmic_bytes(L)

    def timed(fn, n):
        for i in range(8):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6, e0.elapsed_time(e1) / n * 1e3

    def replay_only(i):
        graph.replay()

    def new_step_then_replay(i):
        step.set_arrays(*packed[i % R])       # host packing + one upload: a NEW step every time
        graph.replay()

    def eager_one_launch_index_and_plan(i):
        w = works[i % R]
        idx = kvc.to_device_one_launch(w.inputs, bs, dev)
        plan = kvc.PagedKVWritePlan(idx.batch_indices, idx.positions, idx.kv_block_indices, idx.kv_block_indptrs,
                                    idx.kv_last_block_lens, H, D, bs, torch.bfloat16, slots=idx.slot_mapping)
        for l in range(L):
            plan.append(keys[l], values[l], caches[l])

    def eager_reference_construction(i):
        w = works[i % R]
        idx = kvc.to_device(kvc.make_kv_index_inputs(w.inputs, bs), bs, dev, with_slot_mapping=False)
        for l in range(L):
            kvc.append_paged_kv_cache(keys[l], values[l], idx.batch_indices, idx.positions, caches[l],
                                      idx.kv_block_indices, idx.kv_block_indptrs, idx.kv_last_block_lens)

    def eager_writes_only(i):
        for l in range(L):
            step.append(keys[l], values[l], caches[l])

    # the same step with the rotation of Q and K fused into each layer's write
    Hq = 32
    cs = kvc.make_cos_sin_cache(D, 8192, 500000.0, dtype=torch.bfloat16).to(dev)
    rstep = KVWriteStep(H, D, bs, torch.bfloat16, dev, max_requests=B, max_tokens=B, max_block_ids=cap_ids,
                        cos_sin_cache=cs, num_heads=Hq)
    query = torch.randn(B, Hq * D, device=dev).to(torch.bfloat16)
    q_out = torch.empty_like(query)
    rstep.set_arrays(*packed[0])
    rgraph = rstep.capture([k.view(B, H * D) for k in keys], [v.view(B, H * D) for v in values], caches,
                           queries=[query] * L, query_outs=[q_out] * L)

    def rotary_replay_only(i):
        rgraph.replay()

    write_bytes_step = bytes_step
    rotary_bytes_step = L * B * (2 * Hq * D * 2 + 4 * H * D * 2 + 2 * D * 2 + 12)

    # the floor of a graph node on this machine: L kernels that touch one element each
    one = torch.zeros(1, device=dev)
    floor_graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(floor_graph):
        for _ in range(L):
            one.add_(1.0)

    def floor_replay(i):
        floor_graph.replay()

    compact, detail = [], []
    floor_wall, floor_dev = timed(floor_replay, steps)
    detail.append({"name": f"cfg2 decode step: {L} one-element kernels replayed from a hipGraph (what a graph node costs "
                           f"at least)", "wall_us_per_step": round(floor_wall, 1), "device_us_per_step": round(floor_dev, 1),
                   "us_per_node": round(floor_dev / L, 2)})
    # `us` of these rows is WALL time per 32-layer step (what the serving loop pays)
    for fn, n, form, short, what in (
            (rotary_replay_only, steps, "step wall, graph, rotation fused", "graph{index+32 rotate+write}",
             "one hipGraph replay = index build + 32 x (rotation of Q and K + K/V write) in one launch per layer"),
            (replay_only, steps, "step wall, graph", "graph{index+32 writes}",
             "one hipGraph replay = index build + 32 per-layer writes (the step's scalars already uploaded)"),
            (new_step_then_replay, steps, "step wall, new step: pack+upload+graph", "set_arrays+graph",
             "a NEW step each time: host packs 3 x 256 scalars + the block tables, one upload, one replay"),
            (eager_writes_only, steps, "step wall, 32 eager plan calls", None,
             "the 32 per-layer writes alone, eager, through the same plan (no index work)"),
            (eager_one_launch_index_and_plan, max(20, steps // 8), "step wall, eager index+plan", None,
             "eager: host packing from request objects, 2 uploads, one-launch index, 32 plan calls"),
            (eager_reference_construction, max(10, steps // 16), "step wall, eager reference way",
             "host lists+32 append calls",
             "eager: the reference's host list building and six uploads, then 32 full-argument calls")):
        wall_us, dev_us = timed(fn, n)
        # the fused rows also read and write Q and read the cos/sin rows
        bytes_step = rotary_bytes_step if fn is rotary_replay_only else write_bytes_step
        detail.append({"name": f"cfg2 decode step ({L} layers, {B} requests): {what}", "wall_us_per_step": round(wall_us, 1),
                       "device_us_per_step": round(dev_us, 1), "bytes_per_step": int(bytes_step),
                       "note": "K/V sources of all steps are one 64 MiB set (per-layer launches of 2 MiB are bound by "
                               "launch latency, not by where their lines come from)"})
        if short is not None:
            compact.append({"id": "cfg2", "entry": short, "form": form, "us": round(wall_us, 1),
                            "gbps": round(bytes_step / wall_us / 1e3),
                            "frac": round(bytes_step / wall_us / 1e3 / HBM_PEAK_GBPS, 3)})
    return compact, detail


def bench_load_policy(torch, kvc, wl, dev):
    """A/B of plain against non-temporal loads of the source rows, per layer, in one
    process: the per-layer write (`write_nt` 1 against 3) and the fused rotation
    (`rope_nt` 0 against 3), with the layers of a replayed step cycling through
    `sets` distinct source sets (1 = rows still in cache, as after the projection
    of a forward pass; one set per layer = rows from HBM or the last-level cache).
    Two rounds, interleaved; microseconds per layer from a hipGraph replay."""
    from lmserve_amd import _lib
    out = []
    nb = 16384
    for label, shape, Hq, T, decode in (("cfg2 decode batch", wl.LLAMA_3_8B, 32, 256, True),
                                        ("cfg3 prefill chunk", wl.QWEN_2_5_7B, 28, 2048, False)):
        L, Hkv, D = shape.num_layers, shape.num_kv_heads, shape.head_dim
        pool, _ = alloc_pool(torch, shape, nb, dev)
        w = wl.decode_step(shape, num_blocks=nb, batch=T, max_context=100, seed=1) if decode \
            else wl.chunked_prefill(shape, num_blocks=nb, seed=1)
        idx = kvc.to_device(w.index, shape.block_size, dev)
        cs = kvc.make_cos_sin_cache(D, 40000, 500000.0, dtype=torch.bfloat16).to(dev)
        q = torch.randn(L, T, Hq * D, device=dev).to(torch.bfloat16)
        k = torch.randn(L, T, Hkv, D, device=dev).to(torch.bfloat16)
        v = torch.randn(L, T, Hkv, D, device=dev).to(torch.bfloat16)
        qo = torch.empty(T, Hq * D, dtype=torch.bfloat16, device=dev)
        wplan = kvc.PagedKVWritePlan(idx.batch_indices, idx.positions, idx.kv_block_indices, idx.kv_block_indptrs,
                                     idx.kv_last_block_lens, Hkv, D, shape.block_size, torch.bfloat16)
        rplan = kvc.PagedRotaryWritePlan(idx.batch_indices, idx.positions, idx.kv_block_indices,
                                         idx.kv_block_indptrs, idx.kv_last_block_lens, cs, Hq, Hkv, D,
                                         shape.block_size, resolve_slots=True)
        for sets in (1, 4, L):
            def write(i):
                for l in range(L):
                    wplan.append(k[l % sets], v[l % sets], pool[l])

            def rotate(i):
                for l in range(L):
                    rplan.run(q[l % sets], k[l % sets].view(T, Hkv * D), v[l % sets].view(T, Hkv * D), pool[l],
                              query_out=qo)

            for fn, knob, values, what in ((write, "write_nt", (1, 3), "PagedKVWritePlan.append"),
                                           (rotate, "rope_nt", (0, 3), "PagedRotaryWritePlan.run")):
                us = {val: [] for val in values}
                for _ in range(2):
                    for val in values:
                        _lib.reset_tuning()
                        _lib.set_tuning(knob, val)
                        _, ms_e = time_region(fn, 32, 4, torch, graph_of=1)
                        us[val].append(round(ms_e * 1e3 / L, 3))
                _lib.reset_tuning()
                out.append({"name": f"load policy/{label}, {what} per layer, {sets} source set(s)", "knob": knob,
                            "us_per_layer": {f"{knob}={val}": us[val] for val in values}})
                log(f"  {out[-1]['name']}: {out[-1]['us_per_layer']}")
        del pool, q, k, v
        torch.cuda.empty_cache()
    return out


def bench_duplex_streams(torch, kvc, wl, dev, workers=6):
    """Swap-out beside swap-in for KV workers made one after another once a
    recorded step graph has run, with the two streams taken as they come and
    with streams chosen apart by hardware queue; for each worker, which of its
    streams share a queue (with each other, with the current stream) and the
    rate of each direction alone and of both together."""
    from lmserve_amd import _lib
    from lmserve_amd.step_graph import KVWriteStep

    s8, s70 = wl.LLAMA_3_8B, wl.LLAMA_3_1_70B
    L8, B, nb8 = 8, 256, 2048
    pool8 = torch.empty(L8, nb8, 2, 16, 8, 128, dtype=torch.bfloat16, device=dev)
    w = wl.decode_step(s8, num_blocks=nb8, batch=B, max_context=200, seed=1)
    step = KVWriteStep(8, 128, 16, torch.bfloat16, dev, max_requests=B, max_tokens=B, max_block_ids=B * 16)
    step.set_requests(w.inputs)
    k = torch.zeros(L8, B, 8, 128, dtype=torch.bfloat16, device=dev)
    graph = step.capture([k[l] for l in range(L8)], [k[l] for l in range(L8)], [pool8[l] for l in range(L8)])
    for _ in range(50):
        graph.replay()
    torch.cuda.synchronize()
    nb, n = 4096, 2048                                   # 5 GiB each way
    pool = torch.empty(s70.num_layers, nb, 2, 16, 8, 128, dtype=torch.bfloat16, device=dev)
    old, _, new = wl.swap_round_trip(nb, n, seed=0)
    out_maps = [kvc.BlockMapping.from_pairs(zip(old[:n // 2].tolist(), range(n // 2)))]
    in_maps = [kvc.BlockMapping.from_pairs(zip(range(n // 2, n), new[n // 2:].tolist()))]
    half = n // 2 * s70.num_layers * s70.block_bytes
    cur = torch.cuda.current_stream()
    rows = []
    for own in (False, True):
        for number in range(1, workers + 1):
            worker = kvc.KVWorker(pool, n, swap_mode="staged", own_queues=own)
            a, b = worker.dtoh_stream, worker.htod_stream
            try:
                shares = {"out/in": _lib.streams_share_hw_queue(a.cuda_stream, b.cuda_stream),
                          "current/out": _lib.streams_share_hw_queue(cur.cuda_stream, a.cuda_stream),
                          "current/in": _lib.streams_share_hw_queue(cur.cuda_stream, b.cuda_stream)}

                def run(do_out, do_in):
                    if do_out:
                        worker.save_kv_blocks_to_host_nowait(out_maps)
                    if do_in:
                        worker.load_kv_blocks_from_host_nowait(in_maps)
                    a.synchronize()
                    b.synchronize()

                rates = {}
                for label, do_out, do_in in (("out", True, False), ("in", False, True), ("both", True, True)):
                    run(do_out, do_in)
                    ts = []
                    for _ in range(3):
                        torch.cuda.synchronize()
                        t0 = time.perf_counter()
                        run(do_out, do_in)
                        ts.append(time.perf_counter() - t0)
                    rates[label] = round(half * (int(do_out) + int(do_in)) / sorted(ts)[1] / 1e9, 1)
            finally:
                worker.close()
            rows.append({"name": f"duplex/worker {number} after a recorded step ran, streams "
                                 f"{'chosen apart by hardware queue' if own else 'as they come'}",
                         "share_a_queue": shares, "pcie_gbps": rates})
            log(f"  {rows[-1]['name']}: share {shares}; GB/s {rates}")
    return rows

"""The layer-pipelined swap protocol (events + doorbell queues between a model
thread and the swap engine) and hipGraph replay of the write/copy operators."""
import asyncio
import threading

import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from oracle import kvc_oracle as orc
from tests.helpers import FifoBlockIds, bf16_bits, bits_of, random_pool, sentinel_pool, to_bf16

pytestmark = pytest.mark.gpu


def _busy(dev, n=3):
    """Some real GPU time on the current stream (stands in for a layer's compute)."""
    a = torch.ones(2048, 2048, device=dev)
    for _ in range(n):
        a = a @ a * 1e-4
    return a


@pytest.mark.parametrize("bounce", [True, False])
@pytest.mark.parametrize("mode", ["direct", "staged", "auto"])
@pytest.mark.parametrize("sync", ["events", "host"])
def test_write_through_waits_for_each_layers_kv_write(gpu, mode, sync, bounce):
    """GPU->Host runs concurrently with the forward pass; layer l may be saved
    only after the model recorded post_events[l] (sync="events": the worker's
    stream waits for the event; sync="host": the doorbell itself is rung only
    once the event has completed), so the host copy must hold the K/V written
    in THIS step for every layer."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, bs, H, D = 6, 32, 8, s.block_size, s.num_kv_heads, s.head_dim
    pool_np = random_pool((L, nb, 2, bs, H, D), 1)
    dpool = to_bf16(pool_np, gpu)
    handle = kvc.KVWorkerHandle.create(L, sync=sync)
    worker = kvc.KVWorker(dpool, nhb, swap_mode=mode, kv_worker_handle=handle,
                          host_bounce_bytes=(1 << 30) if bounce else 0)
    hooks = kvc.LayerSyncHooks(handle)
    hooks.enable_record_after_execute = True
    try:
        worker.host_kv_caches[...] = sentinel_pool(worker.host_kv_caches.shape, 2)
        blocks = np.asarray([3, 17, 9, 30], dtype=np.int64)           # blocks written to this step
        host_ids = np.asarray([5, 0, 2, 7], dtype=np.int64)
        T = len(blocks) * bs
        slots = (blocks[:, None] * bs + np.arange(bs)[None, :]).reshape(-1)
        key, value = bf16_bits((L, T, H, D), 3), bf16_bits((L, T, H, D), 4)
        want_pool = pool_np.copy()
        for l in range(L):
            orc.reshape_and_cache_np(key[l], value[l], want_pool[l], slots)
        want_host = worker.host_kv_caches.copy()
        orc.save_blocks_to_host_np(want_pool.reshape(L, nb, -1), want_host, blocks, host_ids)

        maps = [kvc.BlockMapping.from_pairs(zip(blocks.tolist(), host_ids.tolist()))]
        errors = []

        def kv_thread():
            try:
                asyncio.run(worker.copy_kv(maps, kvc.Device.GPU, kvc.Device.Host))
            except Exception as exc:  # surfaced in the main thread below
                errors.append(exc)

        th = threading.Thread(target=kv_thread, daemon=True)
        th.start()
        dk, dv, dslots = to_bf16(key, gpu), to_bf16(value, gpu), torch.from_numpy(slots).to(gpu)
        model_stream = torch.cuda.Stream()
        with torch.cuda.stream(model_stream):
            for l in range(L):
                hooks.pre(l)
                _busy(gpu)                                   # the save must not overtake this
                kvc.reshape_and_cache(dk[l], dv[l], dpool[l], dslots)
                hooks.post(l)
        th.join(timeout=60)
        assert not th.is_alive() and not errors, errors
        model_stream.synchronize()
        assert np.array_equal(bits_of(dpool), want_pool)
        assert np.array_equal(worker.host_kv_caches, want_host)
        assert handle.kv_queue.empty()
        # four scattered host blocks, one layer per call: rows of 32 KiB, so the copy goes
        # through the dense pinned buffer wherever the copy engines would carry it
        assert worker.last_copy_went_through_host_bounce == (bounce and mode != "direct")
    finally:
        worker.close()
        handle.close()


@pytest.mark.parametrize("budget_regions", [4, 2, 1])
def test_scattered_host_blocks_layer_by_layer_through_the_dense_pinned_buffer(gpu, budget_regions):
    """Forty blocks to scattered host blocks and back onto other pool blocks, one
    layer per call over nine layers: more layers than the buffer has regions, so
    regions are reused while host threads still empty (or the GPU still reads)
    the earlier ones. With room for a single region the copy goes the usual way.
    Host pool and GPU pool must be the oracle's after each direction."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, n = 9, 128, 100, 40
    pool_np = random_pool((L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), 31)
    dpool = to_bf16(pool_np, gpu)
    handle = kvc.KVWorkerHandle.create(L)
    block_bytes = 2 * s.block_size * s.num_kv_heads * s.head_dim * 2
    worker = kvc.KVWorker(dpool, nhb, kv_worker_handle=handle, host_copy_threads=3,
                          host_bounce_bytes=budget_regions * n * block_bytes)
    hooks = kvc.LayerSyncHooks(handle)
    try:
        worker.host_kv_caches[...] = sentinel_pool(worker.host_kv_caches.shape, 32)
        rng = np.random.default_rng(33)
        perm = rng.permutation(nb).astype(np.int64)
        old, new = perm[:n], perm[n:2 * n]
        host_ids = (rng.permutation(nhb // 2)[:n] * 2).astype(np.int64)      # never neighbours
        gpu_np = pool_np.reshape(L, nb, -1).copy()
        host_np = worker.host_kv_caches.copy()
        orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids)

        def run(maps, src, dst):
            errors = []

            def body():
                try:
                    asyncio.run(worker.copy_kv(maps, src, dst))
                except Exception as exc:
                    errors.append(exc)
            th = threading.Thread(target=body, daemon=True)
            th.start()
            return th, errors

        hooks.enable_record_after_execute = True
        th, errors = run(_split(old, host_ids), kvc.Device.GPU, kvc.Device.Host)
        for l in range(L):
            _busy(gpu, 1)
            hooks.post(l)
        th.join(timeout=60)
        assert not th.is_alive() and not errors, errors
        assert worker.last_copy_went_through_host_bounce == (budget_regions >= 2)
        assert np.array_equal(worker.host_kv_caches, host_np)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)

        hooks.enable_record_after_execute = False
        hooks.enable_wait_before_execute = True
        hooks.timeout = 30
        orc.c_load_blocks_from_host(gpu_np, host_np, host_ids, new)
        th, errors = run(_split(host_ids, new), kvc.Device.Host, kvc.Device.GPU)
        for l in range(L):
            hooks.pre(l)
        th.join(timeout=60)
        assert not th.is_alive() and not errors, errors
        torch.cuda.synchronize()
        assert worker.last_copy_went_through_host_bounce == (budget_regions >= 2)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)
        assert np.array_equal(worker.host_kv_caches, host_np)
        assert handle.model_queue.empty() and handle.kv_queue.empty()
    finally:
        worker.close()
        handle.close()


def _split(src, dst, pieces=3):
    cuts = np.linspace(0, len(src), pieces + 1).astype(int)
    return [kvc.BlockMapping.from_pairs(zip(src[a:b].tolist(), dst[a:b].tolist()))
            for a, b in zip(cuts[:-1], cuts[1:])]


@pytest.mark.parametrize("bounce", [True, False])
@pytest.mark.parametrize("mode", ["direct", "staged", "auto"])
@pytest.mark.parametrize("sync", ["events", "host"])
def test_fetch_releases_each_layer_to_the_model_in_order(gpu, mode, sync, bounce):
    """Host->GPU: the model waits per layer on pre_events[l] (after the doorbell;
    with sync="host" the doorbell alone, rung after the layer's load completed)
    and must then see that layer's fetched blocks."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb = 5, 24, 8
    pool_np = random_pool((L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), 5)
    dpool = to_bf16(pool_np, gpu)
    handle = kvc.KVWorkerHandle.create(L, sync=sync)
    worker = kvc.KVWorker(dpool, nhb, swap_mode=mode, kv_worker_handle=handle,
                          host_bounce_bytes=(1 << 30) if bounce else 0)
    hooks = kvc.LayerSyncHooks(handle)
    hooks.enable_wait_before_execute = True
    hooks.timeout = 30
    try:
        host = random_pool(worker.host_kv_caches.shape, 6)
        worker.host_kv_caches[...] = host
        src = np.asarray([1, 6, 4], dtype=np.int64)
        dst = np.asarray([20, 2, 11], dtype=np.int64)
        maps = [kvc.BlockMapping.from_pairs(zip(src.tolist(), dst.tolist()))]
        th = threading.Thread(target=lambda: asyncio.run(
            worker.copy_kv(maps, kvc.Device.Host, kvc.Device.GPU)), daemon=True)
        th.start()
        seen = []
        model_stream = torch.cuda.Stream()
        with torch.cuda.stream(model_stream):
            for l in range(L):
                hooks.pre(l)                                 # blocks until layer l is on its way
                seen.append(dpool[l, torch.from_numpy(dst).to(gpu)].clone())
                hooks.post(l)
        th.join(timeout=60)
        assert not th.is_alive()
        model_stream.synchronize()
        for l in range(L):
            got = bits_of(seen[l]).reshape(len(dst), -1)
            assert np.array_equal(got, host[src, l]), f"layer {l} was read before its fetch landed"
        assert handle.model_queue.empty()
        assert worker.last_copy_went_through_host_bounce == (bounce and mode != "direct")
        assert np.array_equal(worker.host_kv_caches, host)      # the host pool is only read
    finally:
        worker.close()
        handle.close()


def test_allocator_order_drives_a_realistic_decode_step(gpu):
    """Block tables produced by the FIFO allocator under churn, written through
    the page-table path, equal the oracle."""
    s = wl.LLAMA_3_2_1B
    nb, bs, L = 128, s.block_size, 2
    alloc = FifoBlockIds(nb)
    rng = np.random.default_rng(0)
    live = {}
    for step in range(40):                                    # churn: sequences come and go
        sid = step
        live[sid] = alloc.take(int(rng.integers(1, 6)))
        if len(live) > 8:
            victim = list(live)[int(rng.integers(0, len(live)))]
            alloc.give_back(live.pop(victim))
    reqs = []
    for i, (sid, blocks) in enumerate(live.items()):
        ctx = int(rng.integers((len(blocks) - 1) * bs + 1, len(blocks) * bs + 1))
        new = 1 if i % 2 else min(ctx, int(rng.integers(2, 20)))
        reqs.append(kvc.InferInput(sid, [0] * new, new, ctx - new, ctx, blocks))
    idx = kvc.make_kv_index_inputs(reqs, bs)
    assert sorted(set(idx.kv_block_indices.tolist())) != list(range(len(set(idx.kv_block_indices.tolist()))))
    T = len(idx.slot_mapping)
    key, value = bf16_bits((L, T, s.num_kv_heads, s.head_dim), 1), bf16_bits((L, T, s.num_kv_heads, s.head_dim), 2)
    pool = sentinel_pool((L, nb, 2, bs, s.num_kv_heads, s.head_dim), 3)
    want = pool.copy()
    for l in range(L):
        orc.c_append_paged_kv_cache(key[l], value[l], idx.batch_indices, idx.positions, want[l],
                                    idx.kv_block_indices, idx.kv_block_indptrs)
    dev = kvc.to_device(idx, bs, gpu)
    dpool = to_bf16(pool, gpu)
    kvc.append_paged_kv_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dev.batch_indices,
                                     dev.positions, dpool, dev.kv_block_indices, dev.kv_block_indptrs,
                                     dev.kv_last_block_lens)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)


def test_graph_replay_of_write_and_copy_matches_eager_every_time(gpu):
    """A captured decode step (per-layer page-table writes + a block copy) is
    replayed several times with new K/V in the static input buffers and eager
    work in between; every replay must equal the oracle."""
    s = wl.LLAMA_3_8B
    L, nb, bs = 4, 128, s.block_size
    w = wl.decode_step(s, num_blocks=nb, batch=24, max_context=60, seed=3)
    idx = kvc.to_device(w.index, bs, gpu)
    T = w.num_tokens
    pool_np = sentinel_pool((L, nb, 2, bs, s.num_kv_heads, s.head_dim), 1)
    dpool = to_bf16(pool_np, gpu)
    static_k = torch.zeros(L, T, s.num_kv_heads, s.head_dim, dtype=torch.bfloat16, device=gpu)
    static_v = torch.zeros_like(static_k)
    used = set(w.index.kv_block_indices.tolist())
    free = [b for b in range(nb) if b not in used]
    flat = np.asarray([int(w.index.kv_block_indices[0]), free[0],
                       int(w.index.kv_block_indices[1]), free[1]], dtype=np.int64)
    dmaps = torch.from_numpy(flat).to(gpu)

    def step():
        for l in range(L):
            kvc.append_paged_kv_cache(static_k[l], static_v[l], idx.batch_indices, idx.positions,
                                      dpool[l], idx.kv_block_indices, idx.kv_block_indptrs,
                                      idx.kv_last_block_lens)
        kvc.copy_blocks(dpool, dmaps)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()

    want = pool_np.copy()
    for rep in range(4):
        key, value = bf16_bits((L, T, s.num_kv_heads, s.head_dim), 10 + rep), \
            bf16_bits((L, T, s.num_kv_heads, s.head_dim), 20 + rep)
        dpool.copy_(to_bf16(pool_np, gpu))                    # eager work between replays
        static_k.copy_(to_bf16(key, gpu))
        static_v.copy_(to_bf16(value, gpu))
        _busy(gpu, 1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want[...] = pool_np
        for l in range(L):
            orc.c_append_paged_kv_cache(key[l], value[l], w.index.batch_indices, w.index.positions,
                                        want[l], w.index.kv_block_indices, w.index.kv_block_indptrs)
        orc.c_copy_blocks(want, flat)
        assert np.array_equal(bits_of(dpool), want), f"replay {rep} differs from the oracle"


def test_dispatcher_registered_ops_run_the_same_kernels(gpu):
    """torch.ops.kvcache.* (lmserve_amd.torch_ops) mutate their cache argument
    exactly as the plain functions do."""
    import lmserve_amd.torch_ops  # noqa: F401  (registers the ops)
    s = wl.LLAMA_3_2_1B
    nb, bs = 64, s.block_size
    w = wl.decode_step(s, num_blocks=nb, batch=16, max_context=40, seed=8)
    idx = kvc.to_device(w.index, bs, gpu)
    T = w.num_tokens
    key, value = bf16_bits((T, s.num_kv_heads, s.head_dim), 1), bf16_bits((T, s.num_kv_heads, s.head_dim), 2)
    pool = sentinel_pool((2, nb, 2, bs, s.num_kv_heads, s.head_dim), 3)
    want = pool.copy()
    orc.c_append_paged_kv_cache(key, value, w.index.batch_indices, w.index.positions, want[0],
                                w.index.kv_block_indices, w.index.kv_block_indptrs)
    orc.reshape_and_cache_np(key, value, want[1], w.index.slot_mapping)
    used = set(w.index.kv_block_indices.tolist())
    free = [b for b in range(nb) if b not in used]
    flat = np.asarray([int(w.index.kv_block_indices[0]), free[0]], dtype=np.int64)
    orc.c_copy_blocks(want, flat)
    dpool = to_bf16(pool, gpu)
    dk, dv = to_bf16(key, gpu), to_bf16(value, gpu)
    torch.ops.kvcache.append_paged_kv_cache(dk, dv, idx.batch_indices, idx.positions, dpool[0],
                                            idx.kv_block_indices, idx.kv_block_indptrs,
                                            idx.kv_last_block_lens)
    torch.ops.kvcache.reshape_and_cache(dk, dv, dpool[1], idx.slot_mapping)
    torch.ops.kvcache.copy_blocks(dpool, torch.from_numpy(flat).to(gpu))
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)

    # swap through the functional operators: a torch-pinned host pool and one from the library
    old, host_ids, new = wl.swap_round_trip(nb, 10, seed=4)
    block_elems = 2 * bs * s.num_kv_heads * s.head_dim
    lib_pool = kvc.PinnedHostPool((12, 2, block_elems), np.uint16)
    try:
        for host_t in (torch.zeros(12, 2, block_elems, dtype=torch.int16).pin_memory(),
                       torch.from_numpy(lib_pool.array.view(np.int16))):
            host_t.zero_()
            dpool2 = to_bf16(want, gpu)
            want_host = np.zeros((12, 2, block_elems), dtype=np.uint16)
            gpu_np = want.reshape(2, nb, -1).copy()
            orc.c_save_blocks_to_host(gpu_np, want_host, old, host_ids)
            orc.c_load_blocks_from_host(gpu_np, want_host, host_ids, new)
            torch.ops.kvcache.swap_out(dpool2, host_t, torch.from_numpy(old), torch.from_numpy(host_ids))
            torch.ops.kvcache.swap_in(dpool2, host_t, torch.from_numpy(host_ids), torch.from_numpy(new))
            torch.cuda.synchronize()
            assert np.array_equal(host_t.numpy().view(np.uint16), want_host)
            assert np.array_equal(bits_of(dpool2).reshape(2, nb, -1), gpu_np)
        # a layer range, lists as ids, and the guards
        host_t.zero_()
        kvc.swap_out(dpool2, host_t, old.tolist(), host_ids.tolist(), layer_begin=1)
        torch.cuda.synchronize()
        assert not host_t[:, 0].any() and np.array_equal(host_t.numpy().view(np.uint16)[:, 1], want_host[:, 1])
        with pytest.raises(IndexError):
            kvc.swap_out(dpool2, host_t, [0], [12])
        with pytest.raises(ValueError):
            kvc.swap_in(dpool2, torch.zeros(12, 2, block_elems, dtype=torch.int16), [0], [0])   # pageable
        with pytest.raises(ValueError):
            kvc.swap_in(dpool2, host_t, torch.tensor([0], device=gpu), [0])
        del host_t
    finally:
        lib_pool.close()

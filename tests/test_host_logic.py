"""Host-side logic of the operator surface: pair-list flattening, mapping
flattening, index construction, workload generators, and the loud failures of
the operators when they are handed CPU tensors."""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from lmserve_amd.index_prep import InferInput, make_kv_index_inputs
from oracle import kvc_oracle as orc
from tests.helpers import FifoBlockIds


def test_flatten_block_maps_keeps_dict_order_and_fans_out():
    assert kvc.flatten_block_maps({}) == []
    assert kvc.flatten_block_maps({5: [1, 2], 3: [9]}) == [5, 1, 5, 2, 3, 9]


def test_check_block_maps():
    kvc.check_block_maps([0, 1, 2, 3, 4, 4], 8)          # self pair is fine
    with pytest.raises(IndexError):
        kvc.check_block_maps([0, 8], 8)
    with pytest.raises(ValueError):
        kvc.check_block_maps([0, 2, 1, 2], 8)            # duplicate dst
    with pytest.raises(ValueError):
        kvc.check_block_maps([0, 1, 1, 2], 8)            # chain: 1 is dst and src


def test_flatten_block_mappings_concatenates_in_order():
    a = kvc.BlockMapping.from_pairs([(1, 10), (2, 11)])
    b = kvc.BlockMapping.from_pairs([(7, 3)])
    src, dst = kvc.flatten_block_mappings([a, kvc.BlockMapping(), b])
    assert src.tolist() == [1, 2, 7] and dst.tolist() == [10, 11, 3]
    assert src.dtype == np.int64
    src, dst = kvc.flatten_block_mappings([])
    assert src.shape == (0,)


def test_pairs_of_a_swap_call_are_ordered_by_host_block_id():
    from lmserve_amd.kv_worker import order_by_host_id
    gpu = np.asarray([70, 71, 72, 73, 74, 75], dtype=np.int64)
    host = np.asarray([9, 3, 4, 10, 2, 3], dtype=np.int64)
    g, h = order_by_host_id(gpu, host)
    assert h.tolist() == [2, 3, 3, 4, 9, 10]
    assert g.tolist() == [74, 71, 75, 72, 70, 73]            # pairs stay together, ties keep their order
    assert g.flags["C_CONTIGUOUS"] and h.flags["C_CONTIGUOUS"] and g.dtype == np.int64
    # an ascending list is handed back as it is
    asc = np.asarray([1, 2, 5], dtype=np.int64)
    g2, h2 = order_by_host_id(gpu[:3], asc)
    assert g2 is not None and h2 is asc
    e = np.zeros(0, dtype=np.int64)
    assert order_by_host_id(e, e)[1].size == 0


def test_duplicate_destinations_of_a_swap_call_are_found():
    from lmserve_amd.kv_worker import check_distinct_destinations
    check_distinct_destinations(np.asarray([4, 1, 9], dtype=np.int64), "x")
    check_distinct_destinations(np.zeros(0, dtype=np.int64), "x")
    with pytest.raises(ValueError, match=r"Host->GPU: destination block ids \[1, 9\]"):
        check_distinct_destinations(np.asarray([9, 1, 4, 1, 9], dtype=np.int64), "Host->GPU")


def test_device_enum_matches_the_wire_values():
    assert (int(kvc.Device.GPU), int(kvc.Device.Host), int(kvc.Device.Disk)) == (0, 1, 2)


def test_make_kv_index_inputs_orders_prefill_first_and_builds_the_page_table():
    bs = 4
    inputs = [
        InferInput(0, [1], 1, 6, 7, [3, 9]),                 # decode
        InferInput(1, [1] * 5, 5, 0, 5, [4, 2]),             # prefill chunk
        InferInput(2, [1], 1, 3, 4, [7]),                    # decode
        InferInput(3, [1] * 3, 3, 8, 11, [1, 5, 6]),         # chunked prefill continuation
    ]
    idx = make_kv_index_inputs(inputs, bs)
    assert idx.order == [1, 3, 0, 2]                         # stable sort by -input_len
    assert idx.cu_seqlens_q.tolist() == [0, 5, 8, 9, 10]
    assert idx.prefill_input_len == 8
    assert idx.position_ids.tolist() == [0, 1, 2, 3, 4, 8, 9, 10, 6, 3]
    assert idx.kv_block_indices.tolist() == [4, 2, 1, 5, 6, 3, 9, 7]
    assert idx.kv_block_indptrs.tolist() == [0, 2, 5, 7, 8]
    assert idx.kv_last_block_lens.tolist() == [1, 3, 3, 4]
    assert idx.batch_indices.tolist() == [0] * 5 + [1] * 3 + [2, 3]
    # slot(pos) = table[pos // bs] * bs + pos % bs
    assert idx.slot_mapping.tolist() == [16, 17, 18, 19, 8, 24, 25, 26, 9 * 4 + 2, 7 * 4 + 3]
    # and the page-table oracles give the same (batch, position) pairs from these arrays
    seq_lens = orc.get_seq_lens_np(idx.kv_block_indptrs, idx.kv_last_block_lens, bs)
    bi, pos = orc.get_batch_indices_positions_np(idx.cu_seqlens_q, seq_lens, 10)
    assert bi.tolist() == idx.batch_indices.tolist() and pos.tolist() == idx.positions.tolist()


def test_index_oracle_reproduces_the_hand_case_and_its_own_loops():
    """`oracle.build_write_index_*` on the step written out by hand above (requests
    already in batch order), then NumPy against loops on random steps, and against
    the two pinned page-table functions."""
    bs = 4
    #            prefill 5   continuation 3   decode      decode
    input_lens, context_lens, tables = [5, 3, 1, 1], [5, 11, 7, 4], [[4, 2], [1, 5, 6], [3, 9], [7]]
    flat = [b for t in tables for b in t]
    for build in (orc.build_write_index_np, orc.build_write_index_loops):
        cu, indptr, last, bi, pos, slots = build(input_lens, context_lens, [len(t) for t in tables], flat, bs)
        assert cu.tolist() == [0, 5, 8, 9, 10]
        assert indptr.tolist() == [0, 2, 5, 7, 8]
        assert last.tolist() == [1, 3, 3, 4]
        assert bi.tolist() == [0] * 5 + [1] * 3 + [2, 3]
        assert pos.tolist() == [0, 1, 2, 3, 4, 8, 9, 10, 6, 3]
        assert slots.tolist() == [16, 17, 18, 19, 8, 24, 25, 26, 9 * 4 + 2, 7 * 4 + 3]
        assert slots.dtype == np.int64 and pos.dtype == np.int32
    # a request whose table is too short for its context: slot -1, never the next request's block
    _, _, _, _, pos, slots = orc.build_write_index_np([1, 1], [20, 5], [1, 1], [7, 3], 16)
    assert pos.tolist() == [19, 4] and slots.tolist() == [-1, 3 * 16 + 4]
    assert orc.build_write_index_loops([1, 1], [20, 5], [1, 1], [7, 3], 16)[5].tolist() == [-1, 52]
    rng = np.random.default_rng(3)
    for _ in range(20):
        B = int(rng.integers(0, 9))
        q = rng.integers(0, 40, size=B)
        ctx = q + rng.integers(0, 100, size=B)
        extra = rng.integers(0, 3, size=B)             # tables may hold blocks beyond the context
        nblk = (ctx + bs - 1) // bs + extra
        table = rng.permutation(int(nblk.sum()) + 5)[:int(nblk.sum())]
        a = orc.build_write_index_np(q, ctx, nblk, table, bs)
        b = orc.build_write_index_loops(q, ctx, nblk, table, bs)
        for x, y in zip(a, b):
            assert np.array_equal(x, y) and x.dtype == y.dtype
        seq_lens = orc.get_seq_lens_np(a[1], a[2], bs)
        keep = (ctx > 0) & (extra == 0)
        # model_worker.py:399-408 passes exactly the blocks of [0, context_len): seq_len == context_len
        assert np.array_equal(seq_lens[keep], ctx[keep])
        bi, pos = orc.get_batch_indices_positions_np(a[0], ctx.astype(np.int32), int(q.sum()))
        assert np.array_equal(bi, a[3]) and np.array_equal(pos, a[4])
    # and the host-side construction of the package agrees with the oracle on a mixed step
    w = wl._write_workload(wl.LLAMA_3_2_1B, 256, [0, 37, 5, 64], [70, 1, 1, 33], np.random.default_rng(1))
    host = make_kv_index_inputs(w.inputs, 16)
    reqs = [w.inputs[i] for i in host.order]
    got = orc.build_write_index_np([r.input_len for r in reqs], [r.context_len for r in reqs],
                                   [len(r.block_ids) for r in reqs],
                                   [b for r in reqs for b in r.block_ids], 16)
    for x, y in zip(got, (host.cu_seqlens_q, host.kv_block_indptrs, host.kv_last_block_lens,
                          host.batch_indices, host.positions, host.slot_mapping)):
        assert np.array_equal(x, y)


def test_slot_oracle_of_the_page_table_write_is_pinned():
    """`oracle.paged_write_slots_np`: the hand case, every skip rule on its own, and the
    property that defines it: writing through its slots with the slot-mapped oracle
    gives the pool the page-table oracle gives."""
    bs = 4
    indptr, table = [0, 2, 5, 7, 8], [4, 2, 1, 5, 6, 3, 9, 7]
    bi = [0] * 5 + [1] * 3 + [2, 3]
    pos = [0, 1, 2, 3, 4, 8, 9, 10, 6, 3]
    assert orc.paged_write_slots_np(bi, pos, table, indptr, bs).tolist() == \
        [16, 17, 18, 19, 8, 24, 25, 26, 9 * 4 + 2, 7 * 4 + 3]
    #                        no request   beyond batch   negative pos   beyond own table   page id < 0
    skip = orc.paged_write_slots_np([-1, 4, 0, 0, 3], [0, 0, -1, 8, 1], [4, 2, 1, 5, 6, 3, 9, -7], indptr, bs)
    assert skip.tolist() == [-1, -1, -1, -1, -1]
    # an entry that exists in the array but belongs to the next request is not this request's page
    assert orc.paged_write_slots_np([0], [2 * bs], table, indptr, bs).tolist() == [-1]
    # the indptr may promise more entries than the array holds
    assert orc.paged_write_slots_np([3], [bs], table, [0, 2, 5, 7, 10], bs).tolist() == [-1]
    rng = np.random.default_rng(11)
    for seed in range(6):
        w = wl._write_workload(wl.LLAMA_3_2_1B, 64, rng.integers(0, 60, size=4).tolist(),
                               rng.integers(1, 20, size=4).tolist(), np.random.default_rng(seed))
        idx, s = w.index, w.shape
        T = w.num_tokens
        key = rng.integers(0, 1 << 16, size=(T, s.num_kv_heads, s.head_dim), dtype=np.uint16)
        value = rng.integers(0, 1 << 16, size=(T, s.num_kv_heads, s.head_dim), dtype=np.uint16)
        bad_bi, bad_pos = idx.batch_indices.copy(), idx.positions.copy()
        bad_bi[0], bad_pos[-1] = -1, 1 << 20
        pool = rng.integers(0, 1 << 16, size=(64, 2, s.block_size, s.num_kv_heads, s.head_dim), dtype=np.uint16)
        by_table, by_slots = pool.copy(), pool.copy()
        # the page-table oracle states the write for valid tokens only: hand it those
        orc.append_paged_kv_cache_np(key[1:-1], value[1:-1], bad_bi[1:-1], bad_pos[1:-1], by_table,
                                     idx.kv_block_indices, idx.kv_block_indptrs)
        slots = orc.paged_write_slots_np(bad_bi, bad_pos, idx.kv_block_indices, idx.kv_block_indptrs, s.block_size)
        assert slots[0] == -1 and slots[-1] == -1 and (slots[1:-1] >= 0).all()
        keep = slots >= 0
        orc.reshape_and_cache_np(key[keep], value[keep], by_slots, slots[keep])
        assert np.array_equal(by_table, by_slots)
        assert np.array_equal(orc.paged_write_slots_np(idx.batch_indices, idx.positions, idx.kv_block_indices,
                                                       idx.kv_block_indptrs, s.block_size), idx.slot_mapping)


def test_make_kv_index_inputs_rejects_inconsistent_requests():
    with pytest.raises(ValueError):
        make_kv_index_inputs([InferInput(0, [1, 1], 2, 0, 3, [0])], 4)   # len mismatch
    with pytest.raises(ValueError):
        make_kv_index_inputs([InferInput(0, [1] * 5, 5, 0, 5, [0])], 4)  # too few blocks


def test_workloads_have_the_configured_shapes_and_distinct_slots():
    s = wl.random_free_slots()
    assert s.shape == (256,) and len(set(s.tolist())) == 256 and s.max() < 1024 * 16
    assert np.array_equal(s, wl.random_free_slots())         # seeded

    dec = wl.decode_step(num_blocks=65536, batch=256)
    assert dec.num_tokens == 256 and dec.shape.row_bytes == 2048
    slots = dec.index.slot_mapping
    assert len(set(slots.tolist())) == 256 and slots.max() < 65536 * 16
    for req in dec.inputs:
        assert req.input_len == 1 and req.context_len == req.filled_token_len + 1
    assert dec.algorithmic_bytes(1) == 2 * 256 * 2 * 2048 + 8 * 256

    pre = wl.chunked_prefill()
    assert pre.num_tokens == 2048 and pre.shape.row_bytes == 1024
    assert len(set(pre.index.slot_mapping.tolist())) == 2048
    for req in pre.inputs:
        assert 1024 <= req.filled_token_len <= 32768 and req.input_len == 512

    flat, d = wl.copy_on_write_pairs()
    assert flat.shape == (8192,) and len(d) == 4096
    kvc.check_block_maps(flat.tolist(), 65536)
    assert kvc.flatten_block_maps(d) == flat.tolist()

    out_ids, host_ids, in_ids = wl.swap_round_trip()
    assert len(set(out_ids.tolist()) | set(in_ids.tolist())) == 16384
    assert host_ids.tolist() == list(range(8192))


def test_kv_shapes():
    assert wl.LLAMA_3_8B.block_bytes == 64 * 1024 and wl.LLAMA_3_2_1B.block_bytes == 32 * 1024
    assert wl.QWEN_2_5_7B.row_bytes == 1024 and wl.LLAMA_3_1_70B.num_layers == 80


def test_operators_refuse_cpu_tensors_loudly():
    pool = torch.zeros(2, 4, 2, 4, 1, 8, dtype=torch.bfloat16)
    k = torch.zeros(3, 1, 8, dtype=torch.bfloat16)
    slots = torch.zeros(3, dtype=torch.int64)
    i32 = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(ValueError, match="GPU"):
        kvc.copy_blocks(pool, {0: [1]})
    with pytest.raises(ValueError, match="GPU"):
        kvc.fill_key_cache(k, k, pool[0, :, 0], pool[0, :, 1], slots)
    with pytest.raises(ValueError, match="GPU"):
        kvc.reshape_and_cache(k, k, pool[0], slots)
    with pytest.raises(ValueError, match="GPU"):
        kvc.append_paged_kv_cache(k, k, i32, i32, pool[0], i32, i32, i32)
    with pytest.raises(ValueError, match="GPU"):
        kvc.KVWorker(pool, 4)


def test_torch_cpu_statements_agree_with_the_oracle():
    """The multi-threaded torch-CPU baseline is itself checked against the oracle."""
    from oracle import torch_cpu
    from tests.helpers import bf16_bits, random_pool, sentinel_pool, to_bf16, bits_of

    T, H, D, nb, bs, L = 40, 2, 8, 16, 4, 3
    rng = np.random.default_rng(1)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((T, H, D), 2), bf16_bits((T, H, D), 3)
    pool = sentinel_pool((nb, 2, bs, H, D), 4)
    want = pool.copy()
    orc.c_reshape_and_cache(key, value, want, slots)
    got = to_bf16(pool)
    torch_cpu.reshape_and_cache_cpu(to_bf16(key), to_bf16(value), got, torch.from_numpy(slots))
    assert np.array_equal(bits_of(got), want)

    kc, vc = sentinel_pool((nb * bs, H, D), 5), sentinel_pool((nb * bs, H, D), 6)
    wk, wv = kc.copy(), vc.copy()
    orc.c_fill_key_cache(key, value, wk, wv, slots)
    gk, gv = to_bf16(kc), to_bf16(vc)
    torch_cpu.fill_key_cache_cpu(to_bf16(key), to_bf16(value), gk, gv, torch.from_numpy(slots))
    assert np.array_equal(bits_of(gk), wk) and np.array_equal(bits_of(gv), wv)

    big = random_pool((L, nb, 2, bs, H, D), 7)
    perm = rng.permutation(nb)
    src, dst = perm[:4].astype(np.int64), perm[4:8].astype(np.int64)
    want = big.copy()
    orc.c_copy_blocks(want, np.stack([src, dst], 1).reshape(-1))
    got = to_bf16(big)
    torch_cpu.copy_blocks_cpu(got, torch.from_numpy(src), torch.from_numpy(dst))
    assert np.array_equal(bits_of(got), want)

    gpu = random_pool((L, nb, 32), 8)
    host = sentinel_pool((6, L, 32), 9)
    want_host = host.copy()
    hid = np.asarray([4, 0, 5, 2], dtype=np.int64)
    orc.c_save_blocks_to_host(gpu, want_host, src, hid)
    got_host = torch.from_numpy(host.view(np.int16).copy())
    torch_cpu.swap_out_cpu(torch.from_numpy(gpu.view(np.int16)), got_host, torch.from_numpy(src),
                           torch.from_numpy(hid))
    assert np.array_equal(got_host.numpy().view(np.uint16), want_host)
    want_gpu = gpu.copy()
    orc.c_load_blocks_from_host(want_gpu, want_host, hid, dst)
    got_gpu = torch.from_numpy(gpu.view(np.int16).copy())
    torch_cpu.swap_in_cpu(got_gpu, got_host, torch.from_numpy(hid), torch.from_numpy(dst))
    assert np.array_equal(got_gpu.numpy().view(np.uint16), want_gpu)


def test_fifo_id_source_follows_the_allocator_order():
    """The test-input generator reproduces the id order of block_manager.rs:62-140:
    front of the queue on allocation, back of the queue on the last release."""
    a = FifoBlockIds(6)
    assert a.take(4) == [0, 1, 2, 3]
    a.give_back([1])
    a.give_back([0])
    assert a.take(3) == [4, 5, 1]                   # released ids queue up behind the untouched ones
    assert a.take() == [0]
    with pytest.raises(RuntimeError):
        a.take()
    a.share(2)                                      # shared prefix block: two users
    a.give_back([2])
    assert not a.queue
    a.give_back([2])
    assert a.take() == [2]
    b = FifoBlockIds(10)
    b.share(7)
    assert b.take(8) == [0, 1, 2, 3, 4, 5, 6, 8]


def test_plan_cache_matches_the_configured_pools():
    p = kvc.plan_cache(128 << 30, 16 << 30, 0, 32, 8, 128, 16, torch.bfloat16)
    assert (p.kv_block_size, p.num_gpu_blocks, p.num_host_blocks, p.num_disk_blocks) == \
        (32768, 65536, 8192, 0)
    p = kvc.plan_cache(80 << 30, 40 << 30, 1 << 30, 80, 8, 128, 16, torch.float16)
    assert (p.num_gpu_blocks, p.num_host_blocks, p.num_disk_blocks) == (16384, 8192, 204)


# ------------------------------------------------------------------ waits of the layer protocol give up
class _NeverDone:
    """Stand-in for a GPU event whose work never completes (handled on the host only)."""
    def query(self):
        return False


class _Done:
    def query(self):
        return True


def test_notifier_rings_in_order_gives_up_at_its_deadline_and_stops():
    import queue
    import time
    from lmserve_amd.kv_pool import KVWorkerHandle, _Notifier
    bell = queue.Queue()
    n = _Notifier(timeout=0.15)
    n.submit(_Done(), bell)
    n.submit(_Done(), bell)
    assert bell.get(timeout=2) == b"" and bell.get(timeout=2) == b""
    t0 = time.monotonic()
    n.submit(_NeverDone(), bell)
    n.submit(_Done(), bell)              # queued behind the stuck one: dropped with it, never rung
    while n.failed is None and time.monotonic() - t0 < 3:
        time.sleep(0.01)
    assert n.failed is not None and 0.14 <= time.monotonic() - t0 < 2.0
    time.sleep(0.05)
    assert bell.empty()
    with pytest.raises(TimeoutError):
        n.submit(_Done(), bell)
    t0 = time.monotonic()
    n.stop()
    assert not n.thread.is_alive() and time.monotonic() - t0 < 1.0
    # without a deadline, stop() still ends a wait that would never finish
    n = _Notifier(timeout=None)
    n.submit(_NeverDone(), bell)
    time.sleep(0.05)
    t0 = time.monotonic()
    n.stop()
    assert not n.thread.is_alive() and time.monotonic() - t0 < 1.0 and bell.empty()
    # the handle passes its own deadline on
    h = KVWorkerHandle([], [], host_wait_timeout=0.1, sync="host")
    h.ring_when_done(_NeverDone(), bell)
    assert h._notifier.timeout == 0.1
    h.close()


def test_save_loop_gives_up_when_the_model_stops_posting_layers():
    """`KVWorker._doorbell` (the poll of kv_worker.py:279-281 with a deadline) on a
    queue nobody rings: TimeoutError after `host_wait_timeout`, not a hang."""
    import asyncio
    import queue
    import time
    from lmserve_amd.kv_worker import KVWorker

    class Stub:
        host_wait_timeout = 0.1
    bell = queue.Queue()
    t0 = time.monotonic()
    with pytest.raises(TimeoutError):
        asyncio.run(KVWorker._doorbell(Stub(), bell, 3))
    assert 0.09 <= time.monotonic() - t0 < 2.0
    bell.put(b"")
    asyncio.run(KVWorker._doorbell(Stub(), bell, 3))       # a token that is there is taken at once
    assert bell.empty()


def test_few_hardware_queues_are_warned_about_once():
    import warnings
    from lmserve_amd import kv_worker
    kv_worker._warned_about_queues = False
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        assert kv_worker.warn_if_few_hardware_queues({"GPU_MAX_HW_QUEUES": "8"}) is False
        assert kv_worker.warn_if_few_hardware_queues({"GPU_MAX_HW_QUEUES": "4"}) is True
        assert kv_worker.warn_if_few_hardware_queues({}) is False          # once per process
    assert len(caught) == 1 and "GPU_MAX_HW_QUEUES" in str(caught[0].message)
    kv_worker._warned_about_queues = False
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        assert kv_worker.warn_if_few_hardware_queues({}) is True           # unset = the runtime's 4
    kv_worker._warned_about_queues = False


def test_streams_are_picked_apart_by_hardware_queue():
    """Stand-in streams are integers and their queue is the integer modulo the
    number of queues, which is what the picker cannot see and has to find out."""
    import warnings
    from lmserve_amd import kv_worker

    def world(queues, first=0):
        counter = [first]

        def make():
            counter[0] += 1
            return counter[0]
        return make, (lambda a, b: a % queues == b % queues), counter

    # 4 queues, the model on stream 1: 2 shares nothing, 3 shares nothing, done after two draws
    make, share, counter = world(4, first=1)
    got, apart = kv_worker.pick_streams_apart(2, [1], make, share)
    assert (got, apart) == ([2, 3], True) and counter[0] == 3
    # the model's queue and the first pick's queue are skipped
    make, share, counter = world(4, first=4)
    got, apart = kv_worker.pick_streams_apart(2, [5, 2], make, share)      # queues 1 and 2 are taken
    assert apart and [g % 4 for g in got] == [3, 0] and got == [7, 8]
    # two queues, one of them the model's: one stream fits, the second cannot; the picker gives up and says so
    make, share, counter = world(2)
    got, apart = kv_worker.pick_streams_apart(2, [0], make, share, tries=10)
    assert not apart and len(got) == 2 and got[0] % 2 == 1 and counter[0] == 11
    # nothing to avoid, one queue
    make, share, _ = world(1)
    got, apart = kv_worker.pick_streams_apart(2, [], make, share, tries=5)
    assert not apart and len(got) == 2
    kv_worker._warned_about_shared_queue = False
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        assert kv_worker.warn_streams_share_a_queue({"GPU_MAX_HW_QUEUES": "2"}) is True
        assert kv_worker.warn_streams_share_a_queue({}) is False
    assert len(caught) == 1 and "GPU_MAX_HW_QUEUES=2" in str(caught[0].message)
    kv_worker._warned_about_shared_queue = False


def test_pool_in_a_segment_of_two_gib_or_more_is_not_exported():
    """The IPC handle of a tensor covers its whole allocator segment; segments of
    2 GiB or more must never be shared between processes here."""
    import torch
    from lmserve_amd import kv_pool
    t = torch.zeros(16, dtype=torch.bfloat16)
    base = t.untyped_storage().data_ptr()
    small = [{"address": base - 4096, "total_size": 1 << 30}]
    large = [{"address": base - 4096, "total_size": 2 << 30}]
    elsewhere = [{"address": base + (1 << 40), "total_size": 4 << 30}]
    assert kv_pool.allocator_segment_bytes(t, small) == 1 << 30
    assert kv_pool.allocator_segment_bytes(t, elsewhere) is None
    kv_pool.check_ipc_segment(t, small)
    kv_pool.check_ipc_segment(t, elsewhere)          # not listed: judged by the storage's own size
    with pytest.raises(ValueError, match="segment"):
        kv_pool.check_ipc_segment(t, large)

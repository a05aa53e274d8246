"""GPU parity of the HBM <-> pinned-host swap against the CPU oracle (bit-exact
on the whole host pool and the whole GPU pool), both transfer modes."""
import asyncio

import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from lmserve_amd import _lib
from oracle import kvc_oracle as orc
from tests.helpers import bits_of, random_pool, sentinel_pool, to_bf16

pytestmark = pytest.mark.gpu

MODES = ["staged", "direct", "auto"]


def _mappings(src, dst, pieces=3):
    """Split (src, dst) id lists into several BlockMappings, as one arrives per sequence."""
    cuts = np.linspace(0, len(src), pieces + 1).astype(int)
    return [kvc.BlockMapping.from_pairs(zip(src[a:b].tolist(), dst[a:b].tolist()))
            for a, b in zip(cuts[:-1], cuts[1:])]


def _worker(gpu, L, nb, block_shape, nhb, mode, chunk=0, seed=0):
    pool = random_pool((L, nb) + block_shape, seed)
    dpool = to_bf16(pool, gpu)
    w = kvc.KVWorker(dpool, nhb, swap_mode=mode, staging_chunk_blocks=chunk)
    w.host_kv_caches[...] = sentinel_pool(w.host_kv_caches.shape, seed + 1)
    return pool, dpool, w


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("chunk", [0, 1, 3])
def test_swap_out_then_in_matches_oracle(gpu, mode, chunk):
    s = wl.LLAMA_3_8B
    L, nb, nhb, n = 5, 64, 24, 11
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, mode, chunk, seed=chunk)
    try:
        rng = np.random.default_rng(10 + chunk)
        perm = rng.permutation(nb)
        old, new = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
        # host ids: a run of 4, singles, and a run of 3, so extents of every kind occur
        host_ids = np.asarray([5, 6, 7, 8, 20, 2, 11, 12, 13, 0, 17], dtype=np.int64)
        gpu_np = pool.reshape(L, nb, -1).copy()
        host_np = w.host_kv_caches.copy()
        orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids)
        w.copy_kv_sync(_mappings(old, host_ids), kvc.Device.GPU, kvc.Device.Host)
        assert np.array_equal(w.host_kv_caches, host_np)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)   # pool untouched

        orc.c_load_blocks_from_host(gpu_np, host_np, host_ids, new)
        w.copy_kv_sync(_mappings(host_ids, new), kvc.Device.Host, kvc.Device.GPU)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)
        assert np.array_equal(w.host_kv_caches, host_np)                    # host untouched
        # round trip: payload of the old blocks now sits in the new blocks
        assert np.array_equal(gpu_np[:, new], pool.reshape(L, nb, -1)[:, old])
    finally:
        w.close()


@pytest.mark.parametrize("cap_out,cap_in", [(1, 1), (3, 2), (96, 16), (96, 0), (4096, 4096)])
def test_direct_swap_under_every_grid_cap(gpu, cap_out, cap_in):
    """The direct kernel walks its chunks grid-stride under a cap per direction
    (`direct_max_wgs`, `direct_max_wgs_in`; 0 = the other's): one workgroup, a
    few, the defaults and more workgroups than chunks all move the same bytes."""
    s = wl.LLAMA_3_8B
    L, nb, nhb, n = 3, 48, 40, 29
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, "direct", 0, seed=31)
    try:
        _lib.set_tuning("direct_max_wgs", cap_out)
        _lib.set_tuning("direct_max_wgs_in", cap_in)
        rng = np.random.default_rng(32)
        perm = rng.permutation(nb)
        old, new = perm[:n].astype(np.int64), perm[n:n + 19].astype(np.int64)
        host_ids = rng.permutation(nhb)[:n].astype(np.int64)
        gpu_np = pool.reshape(L, nb, -1).copy()
        host_np = w.host_kv_caches.copy()
        orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids)
        w.copy_kv_sync(_mappings(old, host_ids), kvc.Device.GPU, kvc.Device.Host)
        assert _lib.last_swap_mode() == _lib.KVC_SWAP_DIRECT
        assert np.array_equal(w.host_kv_caches, host_np)
        orc.c_load_blocks_from_host(gpu_np, host_np, host_ids[:19], new)
        w.copy_kv_sync(_mappings(host_ids[:19], new), kvc.Device.Host, kvc.Device.GPU)
        ran = _lib.last_launch()
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)
        want_cap = cap_in if cap_in > 0 else cap_out
        assert ran["kernel"] == _lib.KVC_KERNEL_COPY_TILES and 1 <= ran["grid"] <= want_cap
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_swap_layer_ranges_compose_to_the_full_swap(gpu, mode):
    """One call per layer range (the reference's layer-pipelined protocol) equals
    one call for all layers, and each call touches only its own layers."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, n = 6, 32, 16, 7
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, mode, chunk=2, seed=4)
    try:
        rng = np.random.default_rng(5)
        old = rng.permutation(nb)[:n].astype(np.int64)
        host_ids = rng.permutation(nhb)[:n].astype(np.int64)
        maps = _mappings(old, host_ids, pieces=2)
        gpu_np = pool.reshape(L, nb, -1)
        host_np = w.host_kv_caches.copy()
        for lb, le in ((0, 1), (1, 4), (4, 6)):
            orc.save_blocks_to_host_np(gpu_np, host_np, old, host_ids, lb, le)
            w.save_kv_blocks_to_host_nowait(maps, layer_begin=lb, layer_end=le)
            w.dtoh_stream.synchronize()
            assert np.array_equal(w.host_kv_caches, host_np), (lb, le)
        full = sentinel_pool(host_np.shape, 5)
        orc.c_save_blocks_to_host(gpu_np.copy(), full, old, host_ids)
        assert np.array_equal(host_np[host_ids], full[host_ids])

        new = np.setdiff1d(np.arange(nb), old)[:n].astype(np.int64)
        back = _mappings(host_ids, new, pieces=1)
        want = gpu_np.copy()
        for lb, le in ((3, 6), (0, 3)):
            orc.load_blocks_from_host_np(want, host_np, host_ids, new, lb, le)
            w.load_kv_blocks_from_host_nowait(back, layer_begin=lb, layer_end=le)
            w.htod_stream.synchronize()
            assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), want), (lb, le)
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_prepared_swap_per_layer_equals_the_oracle(gpu, mode):
    """Ids checked and uploaded once (`kvc_swap_prepare`), then one call per layer
    range (`kvc_swap_out_prepared` / `kvc_swap_in_prepared`): every intermediate
    state of the host pool and of the GPU pool equals the oracle's, in both
    transfer modes; several swaps prepared back to back keep their own id lists."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, n = 6, 40, 20, 9
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, mode, chunk=2, seed=21)
    try:
        rng = np.random.default_rng(22)
        perm = rng.permutation(nb)
        old, new = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
        host_ids = rng.permutation(nhb)[:n].astype(np.int64)
        gpu_np = pool.reshape(L, nb, -1).copy()
        host_np = w.host_kv_caches.copy()
        out = w.prepare_swap("out", _mappings(old, host_ids))
        assert out.n == n
        for lb, le in ((0, 1), (1, 2), (2, 5), (5, 6)):
            orc.save_blocks_to_host_np(gpu_np, host_np, old, host_ids, lb, le)
            w.swap_prepared_layers(out, lb, le)
            w.dtoh_stream.synchronize()
            assert np.array_equal(w.host_kv_caches, host_np), (lb, le)
        back = w.prepare_swap("in", _mappings(host_ids, new))
        for lb, le in ((4, 6), (0, 4)):
            orc.load_blocks_from_host_np(gpu_np, host_np, host_ids, new, lb, le)
            w.swap_prepared_layers(back, lb, le)
            w.htod_stream.synchronize()
            assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np), (lb, le)
        assert np.array_equal(w.host_kv_caches, host_np)
        # empty mappings prepare to nothing and move nothing
        assert w.prepare_swap("out", []) is None
        w.swap_prepared_layers(None, 0, L)
        with pytest.raises(IndexError):
            w.prepare_swap("out", _mappings(np.asarray([nb]), np.asarray([0]), 1))
        with pytest.raises(IndexError):
            w.prepare_swap("in", _mappings(np.asarray([nhb]), np.asarray([0]), 1))
    finally:
        w.close()


def test_many_swaps_in_flight_keep_their_id_lists(gpu):
    """More swaps enqueued back to back on one thread than the library has id
    bounce slots, with growing id counts (so bounce buffers are outgrown while
    earlier uploads may still be queued): every swap moves its own blocks."""
    L, nb, nhb = 2, 4200, 4200
    block_shape = (2, 16, 1, 8)                # 512-byte blocks
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, "direct", seed=31)
    try:
        rng = np.random.default_rng(32)
        gpu_np = pool.reshape(L, nb, -1)
        host_np = w.host_kv_caches.copy()
        # call k uses bounce slot k % 4; 2n > 4096 entries outgrows a slot's first buffer
        for k, n in enumerate([3, 500, 10, 20, 2100, 30, 3000, 40, 4100, 4200, 7]):
            old = rng.permutation(nb)[:n].astype(np.int64)
            hid = rng.permutation(nhb)[:n].astype(np.int64)
            orc.save_blocks_to_host_np(gpu_np, host_np, old, hid, 0, L)
            w.save_kv_blocks_to_host_nowait(_mappings(old, hid, 2))
        w.dtoh_stream.synchronize()
        assert np.array_equal(w.host_kv_caches, host_np)
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_swap_odd_block_bytes_and_other_dtypes(gpu, mode):
    """Blocks whose byte size is not a multiple of 16, and fp32 / fp16 pools."""
    for dtype, np_dtype, block_shape in ((torch.bfloat16, np.uint16, (2, 3, 1, 5)),
                                         (torch.float16, np.float16, (2, 4, 2, 8)),
                                         (torch.float32, np.float32, (2, 4, 1, 6))):
        L, nb, nhb, n = 3, 20, 9, 6
        rng = np.random.default_rng(11)
        width = np.dtype(np_dtype).itemsize
        raw = rng.integers(0, 1 << (8 * width), size=(L, nb) + block_shape,
                           dtype=np.uint16 if width == 2 else np.uint32)
        t = torch.from_numpy(raw.view(np.int16 if width == 2 else np.int32).copy()).view(dtype).to(gpu)
        w = kvc.KVWorker(t, nhb, swap_mode=mode)
        try:
            assert w.host_kv_caches.dtype == np.dtype(np_dtype)
            w.host_kv_caches.view(raw.dtype)[...] = 0
            old = rng.permutation(nb)[:n].astype(np.int64)
            hid = rng.permutation(nhb)[:n].astype(np.int64)
            want = np.zeros((nhb, L, raw[0, 0].size), dtype=raw.dtype)
            orc.c_save_blocks_to_host(raw.reshape(L, nb, -1), want, old, hid)
            w.copy_kv_sync(_mappings(old, hid), kvc.Device.GPU, kvc.Device.Host)
            assert np.array_equal(w.host_kv_caches.view(raw.dtype), want)
        finally:
            w.close()


def test_copy_kv_async_dispatcher_errors_and_empty_lists(gpu):
    pool, dpool, w = _worker(gpu, 2, 16, (2, 16, 1, 64), 8, "staged", seed=7)
    try:
        host0 = w.host_kv_caches.copy()
        asyncio.run(w.copy_kv([], kvc.Device.GPU, kvc.Device.Host))       # no mappings: no-op
        w.copy_kv_sync([kvc.BlockMapping()], kvc.Device.GPU, kvc.Device.Host)  # empty mapping
        assert np.array_equal(w.host_kv_caches, host0)
        with pytest.raises(ValueError, match="Unsupported copy direction"):
            asyncio.run(w.copy_kv([], kvc.Device.GPU, kvc.Device.Disk))
        with pytest.raises(ValueError, match="Unsupported copy direction"):
            w.copy_kv_sync([], kvc.Device.GPU, kvc.Device.GPU)
        with pytest.raises(IndexError):
            w.copy_kv_sync([kvc.BlockMapping.from_pairs([(16, 0)])], kvc.Device.GPU, kvc.Device.Host)
        with pytest.raises(IndexError):
            w.copy_kv_sync([kvc.BlockMapping.from_pairs([(0, 8)])], kvc.Device.GPU, kvc.Device.Host)
        assert np.array_equal(w.host_kv_caches, host0)
        # the async path moves data too
        maps = [kvc.BlockMapping.from_pairs([(3, 1), (9, 6)])]
        asyncio.run(w.copy_kv(maps, kvc.Device.GPU, kvc.Device.Host))
        want = host0.copy()
        orc.save_blocks_to_host_np(pool.reshape(2, 16, -1), want, [3, 9], [1, 6])
        assert np.array_equal(w.host_kv_caches, want)
    finally:
        w.close()
    with pytest.raises(TypeError, match="Unsupported dtype"):
        kvc.KVWorker(torch.zeros(2, 4, 8, dtype=torch.int8, device=gpu), 2)


def test_disk_tier_round_trip(gpu, tmp_path):
    """GPU -> Host -> Disk -> Host -> GPU carries the payload bit-exactly, and
    the disk file is reopened when shape and dtype match."""
    path = str(tmp_path / "disk-kv-cache-0.npy")
    L, nb, nhb, ndb = 2, 16, 6, 5
    pool, dpool, w = _worker(gpu, L, nb, (2, 16, 1, 64), nhb, "staged", seed=8)
    try:
        w.close()
        w = kvc.KVWorker(dpool, nhb, num_disk_blocks=ndb, disk_kv_cache_file=path)
        w.copy_kv_sync([kvc.BlockMapping.from_pairs([(2, 0), (7, 3)])], kvc.Device.GPU, kvc.Device.Host)
        w.copy_kv_sync([kvc.BlockMapping.from_pairs([(0, 4), (3, 1)])], kvc.Device.Host, kvc.Device.Disk)
        w.disk_tier.sync()
        # the pinned pool is mapped by the GPU driver: O_DIRECT cannot take it in place
        assert w.disk_tier.last_transfer_staged == w.disk_tier.is_direct
        w.close()
        w = kvc.KVWorker(dpool, nhb, num_disk_blocks=ndb, disk_kv_cache_file=path)  # reopen
        w.copy_kv_sync([kvc.BlockMapping.from_pairs([(4, 5), (1, 2)])], kvc.Device.Disk, kvc.Device.Host)
        w.copy_kv_sync([kvc.BlockMapping.from_pairs([(5, 10), (2, 11)])], kvc.Device.Host, kvc.Device.GPU)
        got = bits_of(dpool).reshape(L, nb, -1)
        src = pool.reshape(L, nb, -1)
        assert np.array_equal(got[:, 10], src[:, 2]) and np.array_equal(got[:, 11], src[:, 7])
        with pytest.raises(ValueError):
            kvc.KVWorker(dpool, nhb).copy_kv_sync([kvc.BlockMapping.from_pairs([(0, 0)])],
                                                  kvc.Device.Host, kvc.Device.Disk)
    finally:
        w.close()


@pytest.mark.parametrize("chunk", [0, 4])
def test_staged_swap_of_a_layer_range_with_runs_of_consecutive_host_ids(gpu, chunk):
    """A partial layer range makes each host block a strided row; runs of
    consecutive host ids then go out as one pitched (2-D) extent."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb = 6, 40, 16
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, "staged", chunk, seed=21)
    try:
        rng = np.random.default_rng(22)
        old = rng.permutation(nb)[:7].astype(np.int64)
        host_ids = np.asarray([3, 4, 5, 6, 9, 10, 0], dtype=np.int64)   # runs of 4, 2 and 1
        maps = _mappings(old, host_ids, pieces=1)
        gpu_np = pool.reshape(L, nb, -1)
        host_np = w.host_kv_caches.copy()
        orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids, 1, 4)
        w.save_kv_blocks_to_host_nowait(maps, layer_begin=1, layer_end=4)
        w.dtoh_stream.synchronize()
        assert np.array_equal(w.host_kv_caches, host_np)
        new = np.setdiff1d(np.arange(nb), old)[:7].astype(np.int64)
        want = gpu_np.copy()
        orc.c_load_blocks_from_host(want, host_np, host_ids, new, 2, 5)
        w.load_kv_blocks_from_host_nowait(_mappings(host_ids, new, pieces=1), layer_begin=2, layer_end=5)
        w.htod_stream.synchronize()
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), want)
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_both_directions_at_once_on_disjoint_blocks(gpu, mode):
    """Write-through of one set of blocks while another set is fetched, each on
    the worker's stream of its direction and both in flight together (the
    reference's two dedicated streams, kv_worker.py:159-160): every byte of both
    pools must be what the oracle leaves, whichever transfer runs first."""
    s = wl.LLAMA_3_8B
    L, nb, nhb, n = 6, 96, 64, 20
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, mode, chunk=3, seed=51)
    try:
        rng = np.random.default_rng(52)
        perm = rng.permutation(nb)
        out_gpu, in_gpu = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
        hperm = rng.permutation(nhb)
        out_host = np.sort(hperm[:n]).astype(np.int64)            # the blocks being saved
        in_host = hperm[n:2 * n].astype(np.int64)                 # the blocks being fetched: disjoint from them
        gpu_np = pool.reshape(L, nb, -1).copy()
        host_np = w.host_kv_caches.copy()
        orc.c_save_blocks_to_host(gpu_np, host_np, out_gpu, out_host)
        orc.c_load_blocks_from_host(gpu_np, host_np, in_host, in_gpu)
        for _ in range(3):                                        # again and again onto the same state: idempotent
            w.save_kv_blocks_to_host_nowait(_mappings(out_gpu, out_host))
            w.load_kv_blocks_from_host_nowait(_mappings(in_host, in_gpu))
        w.dtoh_stream.synchronize()
        w.htod_stream.synchronize()
        assert np.array_equal(w.host_kv_caches, host_np)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_copies_prepared_side_by_side_keep_their_own_id_lists(gpu, mode):
    """Two prepared swaps of one direction are alive at once (two CopyKV requests
    whose layers interleave), an unprepared call runs between their layers, and a
    prepared swap on a caller's own stream joins them: every copy moves its own
    blocks, as the oracle does, whatever the order of the layer calls."""
    s = wl.LLAMA_3_2_1B
    L, nb, nhb = 6, 96, 40
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, mode, seed=91)
    try:
        rng = np.random.default_rng(92)
        gperm = rng.permutation(nb).astype(np.int64)
        hperm = rng.permutation(nhb).astype(np.int64)
        parts = [(gperm[0:7], hperm[0:7]), (gperm[7:20], hperm[7:20]), (gperm[20:23], hperm[20:23]),
                 (gperm[23:32], hperm[23:32])]
        gpu_np = pool.reshape(L, nb, -1).copy()
        host_np = w.host_kv_caches.copy()
        for g, h in parts:
            orc.c_save_blocks_to_host(gpu_np, host_np, g, h)
        side = torch.cuda.Stream()
        a = w.prepare_swap("out", _mappings(*parts[0]))
        b = w.prepare_swap("out", _mappings(*parts[1]))
        c = w.prepare_swap("out", _mappings(*parts[3]), stream=side)
        assert a.staging.data_ptr() != b.staging.data_ptr() != c.staging.data_ptr()
        for layer in range(L):
            w.swap_prepared_layers(b, layer, layer + 1)
            if layer == 2:
                w.save_kv_blocks_to_host_nowait(_mappings(*parts[2]))
            w.swap_prepared_layers(c, layer, layer + 1)
            w.swap_prepared_layers(a, layer, layer + 1)
        torch.cuda.synchronize()
        assert np.array_equal(w.host_kv_caches, host_np)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)   # pool untouched

        # the same the other way, onto fresh pool blocks
        fresh = gperm[40:72]
        targets = [fresh[0:7], fresh[7:20], fresh[20:23], fresh[23:32]]
        for (g, h), t in zip(parts, targets):
            orc.c_load_blocks_from_host(gpu_np, host_np, h, t)
        del a, b, c
        a = w.prepare_swap("in", _mappings(parts[0][1], targets[0]))
        b = w.prepare_swap("in", _mappings(parts[1][1], targets[1]))
        c = w.prepare_swap("in", _mappings(parts[3][1], targets[3]), stream=side)
        for layer in range(L):
            w.swap_prepared_layers(a, layer, layer + 1)
            w.swap_prepared_layers(c, layer, layer + 1)
            if layer == 3:
                w.load_kv_blocks_from_host_nowait(_mappings(parts[2][1], targets[2]))
            w.swap_prepared_layers(b, layer, layer + 1)
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)
        assert np.array_equal(w.host_kv_caches, host_np)
        # once the copies are gone, the kept workspace serves the next one again
        kept = a.staging.data_ptr()
        del a, b, c
        d = w.prepare_swap("in", _mappings(parts[0][1], targets[0]))
        assert d.staging.data_ptr() == kept
        torch.cuda.synchronize()
    finally:
        w.close()


def test_c_entry_points_order_the_pairs_of_an_unprepared_call_themselves(gpu):
    """kvc_swap_out / kvc_swap_in called straight through the C ABI with a dense
    range of host blocks in shuffled order: the library orders the pairs on its
    own copy, so the call is one run, the per-call choice takes the staged path,
    the caller's arrays stay as they were and the result is the oracle's."""
    from lmserve_amd import _lib
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, n = 4, 64, 32, 12
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, "auto", seed=81)
    try:
        _lib.set_tuning("auto_min_extent_bytes", 256 << 10)
        rng = np.random.default_rng(82)
        host_ids = rng.permutation(np.arange(10, 10 + n)).astype(np.int64)
        old = rng.permutation(nb)[:n].astype(np.int64)
        new = rng.permutation(nb)[:n].astype(np.int64)
        keep_host, keep_old = host_ids.copy(), old.copy()
        gpu_np = pool.reshape(L, nb, -1).copy()
        host_np = w.host_kv_caches.copy()
        staging = torch.empty(int(_lib.lib().kvc_swap_staging_bytes(n, L, w.block_stride, _lib.KVC_SWAP_AUTO, 0)),
                              dtype=torch.uint8, device=gpu)
        stream = torch.cuda.current_stream().cuda_stream

        def call(fn, src, dst):
            _lib.check(fn(dpool.data_ptr(), w._host_pool.ptr, src.ctypes.data, dst.ctypes.data, n, L,
                          w.layer_stride, w.block_stride, nb, nhb, 0, L, staging.data_ptr(), staging.numel(),
                          _lib.KVC_SWAP_AUTO, stream, stream))
            assert _lib.last_swap_mode() == _lib.KVC_SWAP_STAGED
            torch.cuda.synchronize()

        orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids)
        call(_lib.lib().kvc_swap_out, old, host_ids)
        assert np.array_equal(w.host_kv_caches, host_np)
        assert np.array_equal(host_ids, keep_host) and np.array_equal(old, keep_old)
        orc.c_load_blocks_from_host(gpu_np, host_np, host_ids, new)
        call(_lib.lib().kvc_swap_in, host_ids, new)
        assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)
    finally:
        _lib.reset_tuning()
        w.close()


def test_validating_worker_refuses_two_pairs_with_one_destination(gpu):
    s = wl.LLAMA_3_2_1B
    L, nb, nhb = 2, 16, 8
    pool = random_pool((L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), 71)
    dpool = to_bf16(pool, gpu)
    w = kvc.KVWorker(dpool, nhb, validate=True)
    try:
        w.host_kv_caches[...] = sentinel_pool(w.host_kv_caches.shape, 72)
        before_host = w.host_kv_caches.copy()
        with pytest.raises(ValueError, match="GPU->Host: destination block ids \\[3\\]"):
            w.copy_kv_sync(_mappings(np.asarray([1, 2, 5]), np.asarray([3, 0, 3]), pieces=1),
                           kvc.Device.GPU, kvc.Device.Host)
        with pytest.raises(ValueError, match="Host->GPU: destination block ids \\[7\\]"):
            w.prepare_swap("in", _mappings(np.asarray([0, 1]), np.asarray([7, 7]), pieces=1))
        torch.cuda.synchronize()
        assert np.array_equal(w.host_kv_caches, before_host)                  # nothing ran
        assert np.array_equal(bits_of(dpool), pool)
        # one source fanned out to two destinations is fine
        w.copy_kv_sync(_mappings(np.asarray([4, 4]), np.asarray([9, 10]), pieces=1), kvc.Device.Host, kvc.Device.GPU)
    finally:
        w.close()


def test_seeded_random_swaps_match_the_oracle(gpu):
    """Forty seeded cases over what a call can vary: number of blocks, layer range,
    shape of the host id list (runs, singles, shuffled, reversed), ring size and
    mode, in both directions on the same worker one after the other."""
    from lmserve_amd import _lib
    s = wl.LLAMA_3_2_1B
    L, nb, nhb = 5, 80, 48
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)
    rng = np.random.default_rng(61)
    pool = random_pool((L, nb) + block_shape, 62)
    dpool = to_bf16(pool, gpu)
    gpu_np = pool.reshape(L, nb, -1).copy()
    try:
        for case in range(40):
            mode = MODES[case % 3]
            chunk = int(rng.choice([0, 1, 2, 5]))
            w = kvc.KVWorker(dpool, nhb, swap_mode=mode, staging_chunk_blocks=chunk)
            try:
                _lib.set_tuning("auto_min_extent_bytes", int(rng.choice([1, 64 << 10, 4 << 20])))
                w.host_kv_caches[...] = sentinel_pool(w.host_kv_caches.shape, 100 + case)
                host_np = w.host_kv_caches.copy()
                n = int(rng.integers(1, 24))
                lb = int(rng.integers(0, L))
                le = int(rng.integers(lb + 1, L + 1))
                kind = case % 4
                if kind == 0:                                    # one run, somewhere in the pool
                    start = int(rng.integers(0, nhb - n + 1))
                    host_ids = np.arange(start, start + n)
                elif kind == 1:                                  # scattered singles
                    host_ids = rng.permutation(nhb)[:n]
                elif kind == 2:                                  # a run handed over in reverse
                    start = int(rng.integers(0, nhb - n + 1))
                    host_ids = np.arange(start, start + n)[::-1]
                else:                                            # runs of three with gaps
                    host_ids = np.sort(rng.permutation(nhb // 4)[:(n + 2) // 3])[:, None] * 4 + np.arange(3)[None, :]
                    host_ids = host_ids.reshape(-1)[:n]
                host_ids = np.ascontiguousarray(host_ids, dtype=np.int64)
                n = len(host_ids)
                perm = rng.permutation(nb)
                old, new = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
                tag = f"case {case}: {mode}, chunk {chunk}, n {n}, layers [{lb}, {le}), host ids {host_ids.tolist()}"
                orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids, lb, le)
                w.save_kv_blocks_to_host_nowait(_mappings(old, host_ids, pieces=2), layer_begin=lb, layer_end=le)
                w.dtoh_stream.synchronize()
                assert np.array_equal(w.host_kv_caches, host_np), tag
                orc.c_load_blocks_from_host(gpu_np, host_np, host_ids, new, lb, le)
                prepared = w.prepare_swap("in", _mappings(host_ids, new, pieces=2))
                for l in range(lb, le):                          # layer by layer, as the protocol does
                    w.swap_prepared_layers(prepared, l, l + 1)
                w.htod_stream.synchronize()
                assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np), tag
                assert np.array_equal(w.host_kv_caches, host_np), tag
            finally:
                w.close()
    finally:
        _lib.reset_tuning()


def test_auto_mode_takes_the_copy_engines_for_long_runs_and_the_kernel_for_scattered_blocks(gpu):
    """"auto" decides per call from the host ids: runs of consecutive host blocks
    whose PCIe extents reach the threshold go through the staging ring, scattered
    blocks through the direct kernel; both give the oracle's bytes. The worker
    sorts a call's pairs by host id, so a shuffled dense range still forms one run."""
    from lmserve_amd import _lib
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, n = 4, 64, 32, 12
    block_shape = (2, s.block_size, s.num_kv_heads, s.head_dim)      # 32 KiB per layer and block
    pool, dpool, w = _worker(gpu, L, nb, block_shape, nhb, "auto", seed=41)
    cases = [
        ("one run, all layers", np.arange(4, 4 + n), (0, L), 256 << 10, _lib.KVC_SWAP_STAGED),
        ("one run given in shuffled order", np.random.default_rng(1).permutation(np.arange(4, 4 + n)), (0, L),
         256 << 10, _lib.KVC_SWAP_STAGED),
        ("every second host block", np.arange(0, 2 * n, 2), (0, L), 256 << 10, _lib.KVC_SWAP_DIRECT),
        ("one run, one layer, under the threshold", np.arange(4, 4 + n), (1, 2), 1 << 20, _lib.KVC_SWAP_DIRECT),
        ("one run, one layer, over the threshold", np.arange(4, 4 + n), (1, 2), 256 << 10, _lib.KVC_SWAP_STAGED),
        ("the default threshold, one run of 384 KiB", np.arange(4, 4 + n), (1, 2), None, _lib.KVC_SWAP_DIRECT),
        ("the default threshold, one run of 1.5 MiB", np.arange(4, 4 + n), (0, L), None, _lib.KVC_SWAP_STAGED),
    ]
    try:
        gpu_np = pool.reshape(L, nb, -1).copy()
        rng = np.random.default_rng(42)
        for name, host_ids, (lb, le), threshold, want_mode in cases:
            _lib.reset_tuning()
            if threshold is not None:
                _lib.set_tuning("auto_min_extent_bytes", threshold)
            host_ids = np.asarray(host_ids, dtype=np.int64)
            old = rng.permutation(nb)[:n].astype(np.int64)
            host_np = w.host_kv_caches.copy()
            orc.c_save_blocks_to_host(gpu_np, host_np, old, host_ids, lb, le)
            w.save_kv_blocks_to_host_nowait(_mappings(old, host_ids), layer_begin=lb, layer_end=le)
            assert _lib.last_swap_mode() == want_mode, name
            w.dtoh_stream.synchronize()
            assert np.array_equal(w.host_kv_caches, host_np), name
            new = rng.permutation(nb)[:n].astype(np.int64)
            orc.c_load_blocks_from_host(gpu_np, host_np, host_ids, new, lb, le)
            prepared = w.prepare_swap("in", _mappings(host_ids, new))
            w.swap_prepared_layers(prepared, lb, le)
            assert _lib.last_swap_mode() == want_mode, name
            w.htod_stream.synchronize()
            assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np), name
    finally:
        _lib.reset_tuning()
        w.close()


@pytest.mark.parametrize("layers", [(0, None), (1, 4)])
def test_device_gather_and_scatter_match_the_swap_oracle(gpu, layers):
    """gather_blocks / scatter_blocks are the swap's row semantics with the host
    pool replaced by a dense device buffer and host ids 0..n-1."""
    s = wl.LLAMA_3_8B
    L, nb, n = 5, 48, 13
    lb, le = layers
    le = L if le is None else le
    pool = random_pool((L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), 31)
    dpool = to_bf16(pool, gpu)
    rng = np.random.default_rng(32)
    perm = rng.permutation(nb)
    ids, fresh = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
    gpu_np = pool.reshape(L, nb, -1)
    want_buf = np.zeros((n, L, gpu_np.shape[2]), dtype=np.uint16)
    orc.c_save_blocks_to_host(gpu_np, want_buf, ids, np.arange(n), lb, le)
    buf = kvc.gather_blocks(dpool, torch.from_numpy(ids).to(gpu), layer_begin=lb, layer_end=le)
    assert buf.shape == (n, le - lb, gpu_np.shape[2])
    assert np.array_equal(bits_of(buf), want_buf[:, lb:le])
    assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), gpu_np)          # pool untouched
    want = gpu_np.copy()
    orc.c_load_blocks_from_host(want, want_buf, np.arange(n), fresh, lb, le)
    kvc.scatter_blocks(dpool, torch.from_numpy(fresh).to(gpu), buf, layer_begin=lb, layer_end=le)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool).reshape(L, nb, -1), want)
    # ids outside the pool are skipped, the rest still lands
    bad = torch.tensor([int(fresh[0]), nb, -1], dtype=torch.int64, device=gpu)
    out = kvc.gather_blocks(dpool, bad)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(out[0]), want[:, fresh[0]])
    with pytest.raises(ValueError):
        kvc.scatter_blocks(dpool, torch.from_numpy(fresh).to(gpu), buf[:, :1].contiguous())

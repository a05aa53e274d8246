"""The swap entry point that allocates nothing (`kvc_swap_noalloc`): its id lists
live in a static device array of the library and travel as kernel arguments.
Checked through the C ABI against `kvc_swap_out` / `kvc_swap_in` (the entry
points it is a variant of) and the CPU oracle, bit-exact on the whole host pool
and the whole GPU pool, on calls in a row that share the static array."""
import ctypes

import numpy as np
import pytest
import torch

import lmserve_amd as kvc
from lmserve_amd import _lib
from oracle import kvc_oracle as orc
from tests.helpers import bits_of, random_pool, sentinel_pool, to_bf16

pytestmark = pytest.mark.gpu

L, NB, NHB = 3, 1500, 1400
BLOCK_SHAPE = (2, 16, 1, 16)            # 1 KiB blocks: 1500 x 3 of them stay small


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


def _setup(gpu, seed):
    pool = random_pool((L, NB) + BLOCK_SHAPE, seed)
    dpool_new = to_bf16(pool, gpu)      # moved by kvc_swap_noalloc
    dpool_ref = to_bf16(pool, gpu)      # moved by kvc_swap_out / kvc_swap_in
    block_elems = int(np.prod(BLOCK_SHAPE))
    host_new = kvc.PinnedHostPool((NHB, L, block_elems), np.uint16)
    host_ref = kvc.PinnedHostPool((NHB, L, block_elems), np.uint16)
    fill = sentinel_pool(host_new.array.shape, seed + 1)
    host_new.array[...] = fill
    host_ref.array[...] = fill
    return pool, dpool_new, dpool_ref, host_new, host_ref


def _geometry():
    block_bytes = int(np.prod(BLOCK_SHAPE)) * 2
    return block_bytes, NB * block_bytes


def _noalloc(to_host, dpool, host, gpu_ids, host_ids, lb=0, le=L, stream=None):
    block_bytes, layer_stride = _geometry()
    return _lib.lib().kvc_swap_noalloc(int(to_host), dpool.data_ptr(), host.ptr, _ptr(gpu_ids), _ptr(host_ids),
                                       len(gpu_ids), L, layer_stride, block_bytes, NB, NHB, lb, le, stream)


def _existing(to_host, dpool, host, gpu_ids, host_ids, staging, lb=0, le=L):
    block_bytes, layer_stride = _geometry()
    lib = _lib.lib()
    n = len(gpu_ids)
    if to_host:
        return lib.kvc_swap_out(dpool.data_ptr(), host.ptr, _ptr(gpu_ids), _ptr(host_ids), n, L, layer_stride,
                                block_bytes, NB, NHB, lb, le, staging.data_ptr(), staging.numel(),
                                _lib.KVC_SWAP_DIRECT, None, None)
    return lib.kvc_swap_in(dpool.data_ptr(), host.ptr, _ptr(host_ids), _ptr(gpu_ids), n, L, layer_stride,
                           block_bytes, NB, NHB, lb, le, staging.data_ptr(), staging.numel(),
                           _lib.KVC_SWAP_DIRECT, None, None)


def test_noalloc_swap_equals_the_workspace_swap_on_calls_in_a_row(gpu):
    """Swap-out of 1000 blocks (three id packets), then of 37 with other ids (the
    static array still holds the first call's tail), then swap-in of 900 and of 5:
    after every call the host pool and the GPU pool equal those produced by
    kvc_swap_out / kvc_swap_in with a workspace, and the oracle's."""
    pool, dpool_new, dpool_ref, host_new, host_ref = _setup(gpu, 3)
    staging = torch.empty(1 << 16, dtype=torch.uint8, device=gpu)
    try:
        rng = np.random.default_rng(4)
        gpu_np = pool.reshape(L, NB, -1).copy()
        host_np = host_new.array.copy()
        for to_host, n in ((1, 1000), (1, 37), (0, 900), (0, 5)):
            gpu_ids = rng.permutation(NB)[:n].astype(np.int64)
            host_ids = rng.permutation(NHB)[:n].astype(np.int64)
            assert _noalloc(to_host, dpool_new, host_new, gpu_ids, host_ids) == _lib.KVC_OK, _lib.last_error()
            assert _existing(to_host, dpool_ref, host_ref, gpu_ids, host_ids, staging) == _lib.KVC_OK
            if to_host:
                orc.c_save_blocks_to_host(gpu_np, host_np, gpu_ids, host_ids)
            else:
                orc.c_load_blocks_from_host(gpu_np, host_np, host_ids, gpu_ids)
            torch.cuda.synchronize()
            assert np.array_equal(host_new.array, host_ref.array), (to_host, n)
            assert np.array_equal(host_new.array, host_np), (to_host, n)
            got = bits_of(dpool_new).reshape(L, NB, -1)
            assert np.array_equal(got, bits_of(dpool_ref).reshape(L, NB, -1)), (to_host, n)
            assert np.array_equal(got, gpu_np), (to_host, n)
    finally:
        torch.cuda.synchronize()
        host_new.close()
        host_ref.close()


def test_noalloc_swap_layer_ranges_streams_and_limits(gpu):
    """Layer ranges on a side stream; the size limit, out-of-range ids and bad
    ranges are refused with a message and launch nothing."""
    pool, dpool_new, dpool_ref, host_new, host_ref = _setup(gpu, 9)
    try:
        rng = np.random.default_rng(10)
        gpu_np = pool.reshape(L, NB, -1).copy()
        host_np = host_new.array.copy()
        n = 500
        gpu_ids = rng.permutation(NB)[:n].astype(np.int64)
        host_ids = rng.permutation(NHB)[:n].astype(np.int64)
        side = torch.cuda.Stream()
        for lb, le in ((1, 2), (2, 3), (0, 1)):
            assert _noalloc(1, dpool_new, host_new, gpu_ids, host_ids, lb, le, side.cuda_stream) == _lib.KVC_OK
            side.synchronize()
            orc.save_blocks_to_host_np(gpu_np, host_np, gpu_ids, host_ids, lb, le)
            assert np.array_equal(host_new.array, host_np), (lb, le)

        lib = _lib.lib()
        block_bytes, layer_stride = _geometry()
        big = np.zeros(_lib.KVC_NOALLOC_MAX_BLOCKS + 1, dtype=np.int64)
        rc = lib.kvc_swap_noalloc(1, dpool_new.data_ptr(), host_new.ptr, _ptr(big), _ptr(big), len(big), L,
                                  layer_stride, block_bytes, NB, NHB, 0, L, None)
        assert rc == _lib.KVC_ERR_UNSUPPORTED and str(_lib.KVC_NOALLOC_MAX_BLOCKS) in _lib.last_error()
        bad = np.asarray([0, NB], dtype=np.int64)
        ok = np.asarray([0, 1], dtype=np.int64)
        assert _noalloc(1, dpool_new, host_new, bad, ok) == _lib.KVC_ERR_OUT_OF_RANGE
        assert _noalloc(0, dpool_new, host_new, ok, np.asarray([NHB, 0], dtype=np.int64)) == _lib.KVC_ERR_OUT_OF_RANGE
        assert _noalloc(1, dpool_new, host_new, ok, ok, 2, 1) == _lib.KVC_ERR_INVALID_ARG
        assert _noalloc(1, dpool_new, host_new, ok[:0], ok[:0]) == _lib.KVC_OK       # nothing to move
        assert lib.kvc_swap_noalloc(1, None, host_new.ptr, _ptr(ok), _ptr(ok), 2, L, layer_stride, block_bytes,
                                    NB, NHB, 0, L, None) == _lib.KVC_ERR_INVALID_ARG
        torch.cuda.synchronize()
        assert np.array_equal(host_new.array, host_np)                                # the refusals moved nothing
        assert np.array_equal(bits_of(dpool_new).reshape(L, NB, -1), gpu_np)
    finally:
        torch.cuda.synchronize()
        host_new.close()
        host_ref.close()


def test_noalloc_swap_at_its_maximum_size(gpu):
    """KVC_NOALLOC_MAX_BLOCKS blocks in one call (19 id packets), then a small
    call: round trip through the host pool onto fresh blocks."""
    n = _lib.KVC_NOALLOC_MAX_BLOCKS
    nb = nhb = 2 * n
    block_elems = 64                                    # 128-byte blocks
    rng = np.random.default_rng(12)
    pool = rng.integers(0, 1 << 16, size=(2, nb, block_elems), dtype=np.uint16)
    dpool = to_bf16(pool, gpu)
    host = kvc.PinnedHostPool((nhb, 2, block_elems), np.uint16)
    try:
        host.array[...] = 0
        lib = _lib.lib()
        perm = rng.permutation(nb)
        old, new = perm[:n].astype(np.int64), perm[n:].astype(np.int64)
        hid = rng.permutation(nhb)[:n].astype(np.int64)
        args = (2, nb * block_elems * 2, block_elems * 2, nb, nhb, 0, 2, None)
        assert lib.kvc_swap_noalloc(1, dpool.data_ptr(), host.ptr, _ptr(old), _ptr(hid), n, *args) == _lib.KVC_OK
        assert lib.kvc_swap_noalloc(0, dpool.data_ptr(), host.ptr, _ptr(new), _ptr(hid), n, *args) == _lib.KVC_OK
        few_gpu, few_host = new[:3].copy(), hid[-3:].copy()
        assert lib.kvc_swap_noalloc(1, dpool.data_ptr(), host.ptr, _ptr(few_gpu), _ptr(few_host), 3, *args) == _lib.KVC_OK
        torch.cuda.synchronize()
        want = pool.copy()
        want_host = np.zeros_like(host.array)
        orc.save_blocks_to_host_np(want, want_host, old, hid)
        orc.load_blocks_from_host_np(want, want_host, hid, new)
        orc.save_blocks_to_host_np(want, want_host, few_gpu, few_host)
        assert np.array_equal(bits_of(dpool), want)
        assert np.array_equal(host.array, want_host)
        assert np.array_equal(want[:, new], pool[:, old])
    finally:
        torch.cuda.synchronize()
        host.close()


def test_noalloc_swap_leaves_device_memory_alone_and_replays_from_a_graph(gpu):
    """After one warm-up call (which looks up the static array's address), further
    calls change neither the free device memory nor torch's allocator; a call
    recorded into a hipGraph replays bit-exactly, twice, with eager work and a
    synchronisation between the replays."""
    pool, dpool_new, dpool_ref, host_new, host_ref = _setup(gpu, 21)
    staging = torch.empty(1 << 16, dtype=torch.uint8, device=gpu)
    try:
        rng = np.random.default_rng(22)
        one = np.zeros(1, dtype=np.int64)
        assert _noalloc(1, dpool_new, host_new, one, one) == _lib.KVC_OK          # warm-up, outside any capture
        assert _existing(1, dpool_ref, host_ref, one, one, staging) == _lib.KVC_OK
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info()
        reserved_before = torch.cuda.memory_reserved()
        for n in (700, 3, 1200):
            gpu_ids = rng.permutation(NB)[:n].astype(np.int64)
            host_ids = rng.permutation(NHB)[:n].astype(np.int64)
            assert _noalloc(1, dpool_new, host_new, gpu_ids, host_ids) == _lib.KVC_OK
            assert _noalloc(0, dpool_new, host_new, rng.permutation(NB)[:n].astype(np.int64), host_ids) == _lib.KVC_OK
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_reserved() == reserved_before

        # recorded into a graph: the ids travel as kernel arguments, so a replay moves the same blocks again
        dpool_new.copy_(dpool_ref)
        host_new.array[...] = host_ref.array
        n = 600
        gpu_ids = rng.permutation(NB)[:n].astype(np.int64)
        host_ids = rng.permutation(NHB)[:n].astype(np.int64)
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            assert _noalloc(1, dpool_new, host_new, gpu_ids, host_ids, stream=side.cuda_stream) == _lib.KVC_OK
        for rep in range(2):
            fresh = to_bf16(random_pool((L, NB) + BLOCK_SHAPE, 30 + rep), gpu)
            dpool_new.copy_(fresh)                                      # eager work between the replays
            dpool_ref.copy_(fresh)
            torch.cuda.synchronize()
            graph.replay()
            assert _existing(1, dpool_ref, host_ref, gpu_ids, host_ids, staging) == _lib.KVC_OK
            torch.cuda.synchronize()
            assert np.array_equal(host_new.array, host_ref.array), f"replay {rep}"
    finally:
        torch.cuda.synchronize()
        host_new.close()
        host_ref.close()

"""Seeded random geometries through every copy-path operator, against the oracle.

Covers what the fixed cases do not combine: block sizes that are not powers of
two, head sizes that force every vector width, strided K/V, int32 and int64
slots, one and several layers, all three storage widths."""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from oracle import kvc_oracle as orc

pytestmark = pytest.mark.gpu

WIDTHS = {2: (np.uint16, torch.bfloat16), 4: (np.uint32, torch.float32)}


def _dev(a, gpu, tdtype):
    signed = np.int16 if a.itemsize == 2 else np.int32
    return torch.from_numpy(a.view(signed).copy()).view(tdtype).to(gpu)


def _host(t, np_dtype):
    signed = torch.int16 if t.element_size() == 2 else torch.int32
    return t.cpu().contiguous().view(signed).numpy().view(np_dtype)


@pytest.mark.parametrize("seed", range(24))
def test_random_geometry_write_copy_swap(gpu, seed):
    rng = np.random.default_rng(1000 + seed)
    width = int(rng.choice([2, 2, 2, 4]))
    np_dtype, tdtype = WIDTHS[width]
    if width == 2 and seed % 3 == 0:
        tdtype = torch.float16
    L = int(rng.integers(1, 5))
    bs = int(rng.choice([1, 2, 3, 5, 8, 16, 32]))
    H = int(rng.integers(1, 6))
    D = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 40, 64, 96, 128]))
    nb = int(rng.integers(4, 40))
    hi = np.iinfo(np_dtype).max
    pool = rng.integers(0, hi, size=(L, nb, 2, bs, H, D), dtype=np_dtype)

    # ---- a step of mixed requests with tables drawn from the pool
    n_req = int(rng.integers(1, 5))
    filled = rng.integers(0, 2 * bs + 1, size=n_req).tolist()
    new = rng.integers(1, max(2, bs + 2), size=n_req).tolist()
    while sum((f + n + bs - 1) // bs for f, n in zip(filled, new)) > nb:
        filled = [f // 2 for f in filled]
        new = [max(1, n // 2) for n in new]
    shape = wl.KVShape("random", L, H, D, bs, width)
    w = wl._write_workload(shape, nb, filled, new, rng)
    idx = w.index
    T = w.num_tokens
    key = rng.integers(0, hi, size=(L, T, H, D), dtype=np_dtype)
    value = rng.integers(0, hi, size=(L, T, H, D), dtype=np_dtype)
    want = pool.copy()
    for l in range(L):
        orc.c_append_paged_kv_cache(key[l], value[l], idx.batch_indices, idx.positions, want[l],
                                    idx.kv_block_indices, idx.kv_block_indptrs)
    dev = kvc.to_device_one_launch(w.inputs, bs, gpu)
    assert np.array_equal(dev.slot_mapping.cpu().numpy(), idx.slot_mapping)

    # K/V as strided slices of a wider buffer in half of the cases
    dkey, dval = _dev(key, gpu, tdtype), _dev(value, gpu, tdtype)
    if seed % 2:
        wide = torch.zeros(L, T, 3, H, D, dtype=tdtype, device=gpu)
        wide[:, :, 1] = dkey
        wide[:, :, 2] = dval
        layer_k = [wide[l, :, 1] for l in range(L)]
        layer_v = [wide[l, :, 2] for l in range(L)]
    else:
        layer_k = [dkey[l] for l in range(L)]
        layer_v = [dval[l] for l in range(L)]
    slot_dtype = torch.int32 if seed % 4 < 2 else torch.int64

    a, b, c, d = (_dev(pool, gpu, tdtype) for _ in range(4))
    for l in range(L):
        kvc.append_paged_kv_cache(layer_k[l], layer_v[l], dev.batch_indices, dev.positions, a[l],
                                  dev.kv_block_indices, dev.kv_block_indptrs, dev.kv_last_block_lens)
        kvc.reshape_and_cache(layer_k[l], layer_v[l], b[l], dev.slot_mapping.to(slot_dtype))
    kvc.append_paged_kv_cache_layers(dkey, dval, dev.batch_indices, dev.positions, c,
                                     dev.kv_block_indices, dev.kv_block_indptrs, dev.kv_last_block_lens)
    kvc.reshape_and_cache_layers(dkey, dval, d, dev.slot_mapping.to(slot_dtype))
    torch.cuda.synchronize()
    for name, got in (("paged per layer", a), ("slot per layer", b), ("paged one launch", c),
                      ("slot one launch", d)):
        assert np.array_equal(_host(got, np_dtype), want), name

    # ---- copy_blocks on the written pool
    P = int(rng.integers(0, nb // 2 + 1))
    flat, pairs = wl.copy_on_write_pairs(nb, P, seed=seed)
    orc.c_copy_blocks(want, flat)
    kvc.copy_blocks(a, pairs, validate=True)
    torch.cuda.synchronize()
    assert np.array_equal(_host(a, np_dtype), want), "copy_blocks"

    # ---- swap out and back in, both modes, with a layer range in half of the cases
    nhb = int(rng.integers(2, 12))
    n = int(rng.integers(1, min(nhb, nb // 2) + 1))
    perm = rng.permutation(nb)
    old, new_ids = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
    host_ids = rng.permutation(nhb)[:n].astype(np.int64)
    lb, le = (0, L) if seed % 2 == 0 else (int(rng.integers(0, L)), L)
    for mode in ("direct", "staged"):
        worker = kvc.KVWorker(a, nhb, swap_mode=mode, staging_chunk_blocks=int(rng.integers(0, 3)))
        try:
            raw_host = worker.host_kv_caches.view(np_dtype)
            raw_host[...] = rng.integers(0, hi, size=raw_host.shape, dtype=np_dtype)
            want_host = raw_host.copy()
            gpu_np = want.reshape(L, nb, -1)
            orc.c_save_blocks_to_host(gpu_np, want_host, old, host_ids, lb, le)
            worker.save_kv_blocks_to_host_nowait(
                [kvc.BlockMapping.from_pairs(zip(old.tolist(), host_ids.tolist()))],
                layer_begin=lb, layer_end=le)
            worker.dtoh_stream.synchronize()
            assert np.array_equal(raw_host, want_host), f"swap-out {mode}"
            orc.c_load_blocks_from_host(gpu_np, want_host, host_ids, new_ids, lb, le)
            worker.load_kv_blocks_from_host_nowait(
                [kvc.BlockMapping.from_pairs(zip(host_ids.tolist(), new_ids.tolist()))],
                layer_begin=lb, layer_end=le)
            worker.htod_stream.synchronize()
            assert np.array_equal(_host(a, np_dtype), want), f"swap-in {mode}"
        finally:
            worker.close()


@pytest.mark.parametrize("seed", range(8))
def test_one_and_eight_byte_elements_write_copy_gather_swap(gpu, seed):
    """The storage widths the 16-bit cases do not reach: one byte per element (an
    8-bit KV cache) and eight. Same operators, same oracle, bit-exact."""
    rng = np.random.default_rng(3000 + seed)
    width = 1 if seed % 2 == 0 else 8
    np_dtype = np.uint8 if width == 1 else np.uint64
    tdtype = torch.uint8 if width == 1 else torch.float64

    def dev(a):
        if width == 1:
            return torch.from_numpy(a.copy()).to(gpu)
        return torch.from_numpy(a.view(np.int64).copy()).view(torch.float64).to(gpu)

    def host(t):
        if width == 1:
            return t.cpu().contiguous().numpy()
        return t.cpu().contiguous().view(torch.int64).numpy().view(np.uint64)

    L = int(rng.integers(1, 4))
    bs = int(rng.choice([1, 3, 4, 16]))
    H = int(rng.integers(1, 5))
    D = int(rng.choice([1, 3, 8, 16, 48, 128, 256]))
    nb = int(rng.integers(6, 30))
    hi = np.iinfo(np_dtype).max
    pool = rng.integers(0, hi, size=(L, nb, 2, bs, H, D), dtype=np_dtype)
    n_req = int(rng.integers(1, 4))
    filled = rng.integers(0, bs + 1, size=n_req).tolist()
    new = rng.integers(1, bs + 2, size=n_req).tolist()
    while sum((f + n + bs - 1) // bs for f, n in zip(filled, new)) > nb:
        filled = [f // 2 for f in filled]
        new = [max(1, n // 2) for n in new]
    w = wl._write_workload(wl.KVShape("random", L, H, D, bs, width), nb, filled, new, rng)
    idx, T = w.index, w.num_tokens
    key = rng.integers(0, hi, size=(L, T, H, D), dtype=np_dtype)
    value = rng.integers(0, hi, size=(L, T, H, D), dtype=np_dtype)
    want = pool.copy()
    for l in range(L):
        orc.c_append_paged_kv_cache(key[l], value[l], idx.batch_indices, idx.positions, want[l],
                                    idx.kv_block_indices, idx.kv_block_indptrs)
    d = kvc.to_device_one_launch(w.inputs, bs, gpu)
    dkey, dval = dev(key), dev(value)
    assert dkey.dtype == tdtype
    a, b, c = dev(pool), dev(pool), dev(pool)
    for l in range(L):
        kvc.append_paged_kv_cache(dkey[l], dval[l], d.batch_indices, d.positions, a[l],
                                  d.kv_block_indices, d.kv_block_indptrs, d.kv_last_block_lens)
        kvc.reshape_and_cache(dkey[l], dval[l], b[l], d.slot_mapping)
    kvc.reshape_and_cache_layers(dkey, dval, c, d.slot_mapping.to(torch.int32))
    torch.cuda.synchronize()
    for name, got in (("paged per layer", a), ("slot per layer", b), ("slot one launch", c)):
        assert np.array_equal(host(got), want), name

    P = int(rng.integers(1, nb // 2 + 1))
    flat, pairs = wl.copy_on_write_pairs(nb, P, seed=seed)
    orc.c_copy_blocks(want, flat)
    kvc.copy_blocks(a, pairs, validate=True)
    torch.cuda.synchronize()
    assert np.array_equal(host(a), want), "copy_blocks"

    # gather into the host layout, scatter back onto other blocks; the direct swap operators
    n = int(rng.integers(1, nb // 2 + 1))
    perm = rng.permutation(nb)
    old, new_ids = perm[:n].astype(np.int64), perm[n:2 * n].astype(np.int64)
    dense = kvc.gather_blocks(a, torch.from_numpy(old).to(gpu))
    torch.cuda.synchronize()
    assert np.array_equal(host(dense), want.reshape(L, nb, -1)[:, old].transpose(1, 0, 2))
    nhb = n + 3
    host_pool = torch.zeros(nhb, L, a[0][0].numel(), dtype=tdtype).pin_memory()
    host_ids = rng.permutation(nhb)[:n].astype(np.int64)
    want_host = host(host_pool).copy()
    gpu_np = want.reshape(L, nb, -1)
    orc.c_save_blocks_to_host(gpu_np, want_host, old, host_ids)
    kvc.swap_out(a, host_pool, old, host_ids)
    torch.cuda.synchronize()
    assert np.array_equal(host(host_pool), want_host), "swap_out"
    orc.c_load_blocks_from_host(gpu_np, want_host, host_ids, new_ids)
    kvc.swap_in(a, host_pool, host_ids, new_ids)
    kvc.scatter_blocks(b, torch.from_numpy(new_ids).to(gpu), dense)
    torch.cuda.synchronize()
    assert np.array_equal(host(a), want), "swap_in"
    assert np.array_equal(host(b).reshape(L, nb, -1)[:, new_ids], want.reshape(L, nb, -1)[:, new_ids]), "scatter"

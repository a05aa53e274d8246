"""The oracle's formulations against each other over random geometries.

Property tests (CPU): for random layer counts, block sizes, head shapes, item
sizes and index sets, the C loops, the NumPy statements, the element-by-element
Python loops and the torch-CPU one-liners must leave identical bytes. A slip
in one formulation's index arithmetic (a transposed stride, a dropped layer
offset) shows as a difference between them."""
import numpy as np
import torch
from hypothesis import given, settings, strategies as st

import workloads as wl
from oracle import kvc_oracle as orc
from oracle import torch_cpu

geom = st.tuples(st.integers(1, 3),            # layers
                 st.sampled_from([1, 2, 3, 4, 8]),   # block size
                 st.integers(1, 3),            # heads
                 st.sampled_from([1, 2, 4, 6]),      # head dim
                 st.integers(3, 12),           # blocks
                 st.sampled_from([np.uint16, np.uint32]),
                 st.integers(0, 2 ** 31 - 1))  # seed


@settings(max_examples=60, deadline=None)
@given(geom)
def test_write_formulations_agree(g):
    L, bs, H, D, nb, dt, seed = g
    rng = np.random.default_rng(seed)
    n_req = int(rng.integers(1, 4))
    filled = rng.integers(0, bs + 1, size=n_req).tolist()
    new = rng.integers(1, bs + 2, size=n_req).tolist()
    while sum((f + n + bs - 1) // bs for f, n in zip(filled, new)) > nb:
        filled = [f // 2 for f in filled]
        new = [max(1, n // 2) for n in new]
    shape = wl.KVShape("prop", L, H, D, bs, np.dtype(dt).itemsize)
    w = wl._write_workload(shape, nb, filled, new, rng)
    idx, T = w.index, w.num_tokens
    hi = np.iinfo(dt).max
    key = rng.integers(0, hi, size=(T, H, D), dtype=dt)
    value = rng.integers(0, hi, size=(T, H, D), dtype=dt)
    pool = rng.integers(0, hi, size=(nb, 2, bs, H, D), dtype=dt)
    outs = []
    for fn in (orc.c_append_paged_kv_cache, orc.append_paged_kv_cache_np, orc.append_paged_kv_cache_loops):
        p = pool.copy()
        fn(key, value, idx.batch_indices, idx.positions, p, idx.kv_block_indices, idx.kv_block_indptrs)
        outs.append(p)
    for fn in (orc.c_reshape_and_cache, orc.reshape_and_cache_np):
        p = pool.copy()
        fn(key, value, p, idx.slot_mapping)
        outs.append(p)
    signed = np.int16 if np.dtype(dt).itemsize == 2 else np.int32
    p = torch.from_numpy(pool.view(signed).copy())
    torch_cpu.reshape_and_cache_cpu(torch.from_numpy(key.view(signed).copy()),
                                    torch.from_numpy(value.view(signed).copy()), p,
                                    torch.from_numpy(idx.slot_mapping))
    outs.append(p.numpy().view(dt))
    for o in outs[1:]:
        assert np.array_equal(outs[0], o)
    # the index arrays themselves: closed forms of the two flashinfer helpers
    sl = orc.c_get_seq_lens(idx.kv_block_indptrs, idx.kv_last_block_lens, bs)
    assert np.array_equal(sl, orc.get_seq_lens_np(idx.kv_block_indptrs, idx.kv_last_block_lens, bs))
    for fn in (orc.get_batch_indices_positions_np, orc.c_get_batch_indices_positions):
        bi, pos = fn(idx.cu_seqlens_q, sl, T)
        assert np.array_equal(bi, idx.batch_indices) and np.array_equal(pos, idx.positions)


@settings(max_examples=60, deadline=None)
@given(geom)
def test_copy_and_swap_formulations_agree(g):
    L, bs, H, D, nb, dt, seed = g
    rng = np.random.default_rng(seed)
    hi = np.iinfo(dt).max
    E = 2 * bs * H * D
    pool = rng.integers(0, hi, size=(L, nb, E), dtype=dt)
    P = int(rng.integers(0, nb // 2 + 1))
    flat, _ = wl.copy_on_write_pairs(nb, P, seed=seed % 1000)
    a, b, c = pool.copy(), pool.copy(), pool.copy()
    orc.c_copy_blocks(a, flat)
    orc.copy_blocks_np(b, flat)
    orc.copy_blocks_loops(c, flat)
    signed = np.int16 if np.dtype(dt).itemsize == 2 else np.int32
    t = torch.from_numpy(pool.view(signed).copy())
    torch_cpu.copy_blocks_cpu(t, torch.from_numpy(flat[0::2].copy()), torch.from_numpy(flat[1::2].copy()))
    assert np.array_equal(a, b) and np.array_equal(a, c) and np.array_equal(a, t.numpy().view(dt))

    nhb = int(rng.integers(1, 8))
    n = int(rng.integers(1, min(nhb, nb) + 1))
    src = rng.permutation(nb)[:n].astype(np.int64)
    dst = rng.permutation(nhb)[:n].astype(np.int64)
    lb = int(rng.integers(0, L))
    le = int(rng.integers(lb + 1, L + 1))
    host = rng.integers(0, hi, size=(nhb, L, E), dtype=dt)
    h1, h2 = host.copy(), host.copy()
    orc.c_save_blocks_to_host(pool, h1, src, dst, lb, le)
    orc.save_blocks_to_host_np(pool, h2, src, dst, lb, le)
    assert np.array_equal(h1, h2)
    if (lb, le) == (0, L):
        h3 = host.copy()
        orc.save_blocks_to_host_loops(pool, h3, src, dst)
        assert np.array_equal(h1, h3)
    back = rng.permutation(nb)[:n].astype(np.int64)
    p1, p2 = pool.copy(), pool.copy()
    orc.c_load_blocks_from_host(p1, h1, dst, back, lb, le)
    orc.load_blocks_from_host_np(p2, h1, dst, back, lb, le)
    assert np.array_equal(p1, p2)
    # what was saved comes back: the payload survives the round trip
    assert np.array_equal(p1[lb:le][:, back], pool[lb:le][:, src])
    # and the disk legs: disk[dst] = host[src], host[dst] = disk[src]
    ndb = int(rng.integers(1, 6))
    m = int(rng.integers(1, min(ndb, nhb) + 1))
    hs, dd = rng.permutation(nhb)[:m], rng.permutation(ndb)[:m]
    d1 = np.zeros((ndb, L, E), dtype=dt)
    d2 = d1.copy()
    orc.save_blocks_to_disk_np(h1, d1, hs, dd)
    orc.save_blocks_to_disk_loops(h1, d2, hs, dd)
    assert np.array_equal(d1, d2) and np.array_equal(d1[dd], h1[hs])

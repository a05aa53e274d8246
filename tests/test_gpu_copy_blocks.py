"""GPU parity of copy_blocks against the CPU oracle (bit-exact, whole pool)."""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
from lmserve_amd import _lib
import workloads as wl
from oracle import kvc_oracle as orc
from tests.helpers import bits_of, random_pool, to_bf16

pytestmark = pytest.mark.gpu


def _run(gpu, shape, src_to_dst, seed=0, **kw):
    pool = random_pool(shape, seed)
    want = pool.copy()
    orc.c_copy_blocks(want, np.asarray(kvc.flatten_block_maps(src_to_dst), dtype=np.int64))
    dpool = to_bf16(pool, gpu)
    kvc.copy_blocks(dpool, src_to_dst, **kw)
    torch.cuda.synchronize()
    return bits_of(dpool), want, pool


@pytest.mark.parametrize("shape_name,L,nb,P", [
    ("llama-3-8b", 4, 256, 64),       # 64 KiB blocks
    ("llama-3.2-1b", 16, 128, 40),    # 32 KiB blocks, all 16 layers
    ("qwen2.5-7b", 3, 96, 17),
])
def test_copy_blocks_matches_oracle(gpu, shape_name, L, nb, P):
    s = {"llama-3-8b": wl.LLAMA_3_8B, "llama-3.2-1b": wl.LLAMA_3_2_1B,
         "qwen2.5-7b": wl.QWEN_2_5_7B}[shape_name]
    _, d = wl.copy_on_write_pairs(nb, P, seed=L)
    got, want, before = _run(gpu, (L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), d, seed=P)
    assert np.array_equal(got, want)
    assert not np.array_equal(got, before)


def test_copy_blocks_one_to_many_self_pair_and_empty(gpu):
    shape = (3, 32, 2, 16, 2, 64)
    got, want, before = _run(gpu, shape, {5: [0, 9, 31], 7: [7], 2: [3]}, seed=1)
    assert np.array_equal(got, want)
    for d in (0, 9, 31):
        assert np.array_equal(got[:, d], before[:, 5])
    got, want, before = _run(gpu, shape, {}, seed=2)
    assert np.array_equal(got, before)
    got, want, before = _run(gpu, shape, {4: []}, seed=3)
    assert np.array_equal(got, before)


@pytest.mark.parametrize("block_shape", [
    (2, 3, 1, 5),     # 60-byte blocks: 4-byte vectors
    (2, 1, 1, 3),     # 12-byte blocks
    (2, 1, 1, 1),     # 4-byte blocks
    (2, 16, 1, 72),   # 4608-byte blocks: a partial last chunk
    (2, 16, 8, 100),  # 51200-byte blocks, not a power of two
])
def test_copy_blocks_odd_block_sizes(gpu, block_shape):
    L, nb = 3, 24
    _, d = wl.copy_on_write_pairs(nb, 9, seed=5)
    got, want, _ = _run(gpu, (L, nb) + block_shape, d, seed=6)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("unroll", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("nt", [0, 1])
@pytest.mark.parametrize("max_wgs", [0, 7])
def test_copy_blocks_every_launch_shape(gpu, unroll, nt, max_wgs):
    """All unroll / load-store kind / grid-cap instantiations give the same bits."""
    s = wl.LLAMA_3_8B
    L, nb = 2, 64
    _, d = wl.copy_on_write_pairs(nb, 13, seed=unroll)
    _lib.set_tuning("copy_unroll", unroll)     # the autouse fixture puts the defaults back
    _lib.set_tuning("copy_nt", nt)
    _lib.set_tuning("copy_max_wgs", max_wgs)
    got, want, _ = _run(gpu, (L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), d, seed=8)
    ran = _lib.last_launch()
    assert ran["kernel"] == _lib.KVC_KERNEL_COPY_TILES and ran["per_lane"] == unroll
    assert ran["non_temporal"] == nt and ran["vec_bytes"] == 16
    assert ran["grid"] == (7 if max_wgs else 13 * L * (65536 // (256 * 16 * unroll)))
    assert np.array_equal(got, want)


def test_copy_blocks_accepts_a_device_pair_tensor_and_validates_on_request(gpu):
    s = wl.LLAMA_3_2_1B
    shape = (2, 40, 2, s.block_size, s.num_kv_heads, s.head_dim)
    flat, d = wl.copy_on_write_pairs(40, 10, seed=3)
    pool = random_pool(shape, 4)
    want = pool.copy()
    orc.copy_blocks_np(want, flat)
    dpool = to_bf16(pool, gpu)
    kvc.copy_blocks(dpool, torch.from_numpy(flat).to(gpu))
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)
    with pytest.raises(ValueError):
        kvc.copy_blocks(dpool, {1: [2], 2: [3]}, validate=True)
    with pytest.raises(IndexError):
        kvc.copy_blocks(dpool, {1: [40]}, validate=True)
    with pytest.raises(ValueError):
        kvc.copy_blocks(dpool, torch.zeros(3, dtype=torch.int64, device=gpu))


def test_copy_blocks_skips_out_of_range_ids_on_the_device(gpu):
    """Ids the host never saw (device tensor input) cannot fault: pairs with an
    id outside the pool are skipped."""
    shape = (2, 16, 2, 16, 1, 64)
    pool = random_pool(shape, 9)
    want = pool.copy()
    orc.copy_blocks_np(want, np.asarray([1, 2], dtype=np.int64))
    dpool = to_bf16(pool, gpu)
    maps = torch.tensor([1, 2, 3, 16, -1, 5, 99, 7], dtype=torch.int64, device=gpu)
    kvc.copy_blocks(dpool, maps)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)


@pytest.mark.parametrize("n", [1, 2, 4, 8, 16, 32, 100])
def test_every_launch_shape_the_size_rule_picks_matches_the_oracle(gpu, n):
    """Bytes per workgroup follow the launch size (1, 2, 4, 8 or 16 vectors per lane
    for small launches, 2 or 1 for large ones): copy, gather and scatter at sizes
    that reach each choice, Llama-3-8B block shape over 32 layers."""
    s = wl.LLAMA_3_8B
    L, nb = 32, 256
    pool = random_pool((L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim), seed=n)
    flat, pairs = wl.copy_on_write_pairs(nb, n, seed=n)
    want = pool.copy()
    orc.c_copy_blocks(want, flat)
    dpool = to_bf16(pool, gpu)
    assert _lib.lib().kvc_tuning_modified() == 0 and _lib.get_tuning("copy_unroll") == 0
    # vectors per lane the size rule must pick on a 256-CU part (2048 resident workgroups):
    # the smallest depth that fits n * 32 tiles of 64 KiB into 512 workgroups, a whole tile
    # per workgroup while that stays within 1024, else 2 (copy, scatter) or 1 (gather)
    small = {1: 1, 2: 2, 4: 4, 8: 8, 16: 16, 32: 16}
    kvc.copy_blocks(dpool, pairs)
    assert _lib.last_launch()["per_lane"] == small.get(n, 2)
    ids = torch.from_numpy(flat[1::2].copy()).to(gpu)               # the blocks just written
    dense = kvc.gather_blocks(dpool, ids)
    assert _lib.last_launch()["per_lane"] == small.get(n, 1)
    back = torch.from_numpy(flat[0::2].copy()).to(gpu)              # scatter them over their sources
    kvc.scatter_blocks(dpool, back, dense)
    assert _lib.last_launch()["per_lane"] == small.get(n, 2)
    torch.cuda.synchronize()
    view = want.reshape(L, nb, -1)
    want_dense = view[:, flat[1::2]].swapaxes(0, 1)
    assert np.array_equal(bits_of(dense), want_dense)
    view[:, flat[0::2]] = want_dense.swapaxes(0, 1)                 # a no-op by value: dst == src content
    assert np.array_equal(bits_of(dpool), want)

"""Writes the golden fixtures of tests/golden/*.npz.

The reference ships no tests, fixtures or golden vectors for its cache
operations, and its implementation of this path cannot run in a container
without a GPU, so these vectors are NOT reference outputs: they are produced by
the element-by-element pure-Python restatement in oracle/kvc_oracle.py (the most
literal reading of the reference's address arithmetic), from seeded inputs. The
faster oracles and the HIP library are then both held to them.

    python tests/golden/make_golden.py        # rewrites the .npz files in place
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from lmserve_amd.index_prep import InferInput, make_kv_index_inputs  # noqa: E402
from oracle import kvc_oracle as orc  # noqa: E402
from tests.helpers import bf16_bits, random_pool, sentinel_pool  # noqa: E402


def write_fixture():
    L, nb, bs, H, D = 2, 12, 4, 2, 16
    rng = np.random.default_rng(2024)
    perm = rng.permutation(nb).tolist()
    # a chunked-prefill continuation, a fresh prefill, and two decode tokens
    reqs = [
        InferInput(0, [0], 1, 6, 7, perm[0:2]),
        InferInput(1, [0] * 7, 7, 0, 7, perm[2:4]),
        InferInput(2, [0] * 5, 5, 8, 13, perm[4:8]),
        InferInput(3, [0], 1, 3, 4, perm[8:9]),
    ]
    idx = make_kv_index_inputs(reqs, bs)
    T = len(idx.slot_mapping)
    key, value = bf16_bits((L, T, H, D), 1), bf16_bits((L, T, H, D), 2)
    pool_before = sentinel_pool((L, nb, 2, bs, H, D), 3)
    pool_after = pool_before.copy()
    for l in range(L):
        orc.append_paged_kv_cache_loops(key[l], value[l], idx.batch_indices, idx.positions,
                                        pool_after[l], idx.kv_block_indices, idx.kv_block_indptrs)
    # packed caches through the flat-address kernel restatement
    kc_before = sentinel_pool((nb * bs, H, D), 4)
    vc_before = sentinel_pool((nb * bs, H, D), 5)
    kc_after, vc_after = kc_before.copy(), vc_before.copy()
    orc.fill_key_cache_loops(key[0], value[0], kc_after, vc_after, idx.slot_mapping)
    np.savez_compressed(
        os.path.join(HERE, "write.npz"), key=key, value=value, pool_before=pool_before,
        pool_after=pool_after, slot_mapping=idx.slot_mapping, batch_indices=idx.batch_indices,
        positions=idx.positions, kv_indices=idx.kv_block_indices, kv_indptr=idx.kv_block_indptrs,
        kv_last_page_len=idx.kv_last_block_lens, cu_seqlens_q=idx.cu_seqlens_q,
        kc_before=kc_before, vc_before=vc_before, kc_after=kc_after, vc_after=vc_after)


def copy_fixture():
    L, nb = 3, 10
    pool_before = random_pool((L, nb, 2, 4, 2, 8), 6)
    block_maps = np.asarray([7, 0, 7, 3, 2, 9, 5, 5, 4, 1], dtype=np.int64)  # {7:[0,3], 2:[9], 5:[5], 4:[1]}
    pool_after = pool_before.copy()
    orc.copy_blocks_loops(pool_after, block_maps)
    np.savez_compressed(os.path.join(HERE, "copy_blocks.npz"), pool_before=pool_before,
                        block_maps=block_maps, pool_after=pool_after)


def swap_fixture():
    L, nb, nhb, E = 3, 10, 6, 2 * 4 * 2 * 8
    gpu_before = random_pool((L, nb, E), 7)
    host_before = sentinel_pool((nhb, L, E), 8)
    out_src = np.asarray([8, 1, 5, 2], dtype=np.int64)
    out_dst = np.asarray([3, 4, 0, 5], dtype=np.int64)
    host_after = host_before.copy()
    orc.save_blocks_to_host_loops(gpu_before, host_after, out_src, out_dst)
    in_src = np.asarray([0, 5, 3], dtype=np.int64)
    in_dst = np.asarray([9, 6, 0], dtype=np.int64)
    gpu_after = gpu_before.copy()
    orc.load_blocks_from_host_loops(gpu_after, host_after, in_src, in_dst)
    np.savez_compressed(os.path.join(HERE, "swap.npz"), gpu_before=gpu_before,
                        host_before=host_before, out_src=out_src, out_dst=out_dst,
                        host_after=host_after, in_src=in_src, in_dst=in_dst, gpu_after=gpu_after)


if __name__ == "__main__":
    write_fixture()
    copy_fixture()
    swap_fixture()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")

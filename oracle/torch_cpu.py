"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

The torch-CPU statements of the same operations, multi-threaded through
torch's own CPU kernels. The reference has no CPU path for them (its wrapper
hard-codes device='cuda', ops/cache_ops.py:17-19, and swaps are driver
copies, kv_worker.py:207, :223), so these one-liners are what "the worker's
torch CPU path" amounts to. They are checked against the other oracles in
tests/ and timed by bench.py as the CPU baseline; lmserve_amd/ never imports
this module.

All tensors are CPU tensors; bf16 pools may be passed as bf16 or as int16 views.
"""
from __future__ import annotations

import torch


def fill_key_cache_cpu(key, value, key_cache, value_cache, slot_mapping) -> None:
    T = key.shape[0]
    row = key.shape[1] * key.shape[2]
    key_cache.view(-1, row).index_copy_(0, slot_mapping, key.reshape(T, row))
    value_cache.view(-1, row).index_copy_(0, slot_mapping, value.reshape(T, row))


def reshape_and_cache_cpu(key, value, kv_cache, slot_mapping) -> None:
    """kv_cache: one layer [nb, 2, bs, H, D]."""
    nb, _, bs, H, D = kv_cache.shape
    T = key.shape[0]
    flat = kv_cache.view(nb * 2 * bs, H * D)
    blk = torch.div(slot_mapping, bs, rounding_mode="floor")
    e = slot_mapping - blk * bs
    flat.index_copy_(0, blk * (2 * bs) + e, key.reshape(T, H * D))
    flat.index_copy_(0, blk * (2 * bs) + bs + e, value.reshape(T, H * D))


def reshape_and_cache_layers_cpu(key, value, kv_caches, slot_mapping) -> None:
    """key/value [L, T, H, D]; kv_caches [L, nb, 2, bs, H, D]."""
    for l in range(kv_caches.shape[0]):
        reshape_and_cache_cpu(key[l], value[l], kv_caches[l], slot_mapping)


def copy_blocks_cpu(kv_caches, src, dst) -> None:
    """kv_caches [L, nb, ...]; src, dst int64 [P]."""
    L, nb = kv_caches.shape[0], kv_caches.shape[1]
    pool = kv_caches.view(L, nb, -1)
    pool.index_copy_(1, dst, pool.index_select(1, src))


def swap_out_cpu(pool, host, src_ids, dst_ids) -> None:
    """pool [L, nb, E], host [nhb, L, E]: host[dst] = pool[:, src] transposed."""
    host[dst_ids] = pool.index_select(1, src_ids).transpose(0, 1)


def swap_in_cpu(pool, host, src_ids, dst_ids) -> None:
    pool.index_copy_(1, dst_ids, host[src_ids].transpose(0, 1))

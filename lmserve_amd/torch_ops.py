"""The write and copy operators registered as `torch.ops.kvcache.*`.

Importing this module defines
    torch.ops.kvcache.reshape_and_cache(key, value, kv_cache, slot_mapping)
    torch.ops.kvcache.append_paged_kv_cache(append_key, append_value, batch_indices, positions,
                                            paged_kv_cache, kv_indices, kv_indptr, kv_last_page_len)
    torch.ops.kvcache.copy_blocks(kv_caches, block_maps)        # block_maps: int64 [2P] on the device
    torch.ops.kvcache.swap_out(kv_caches, host_pool, src_ids, dst_ids)   # ids: int64 on the host
    torch.ops.kvcache.swap_in(kv_caches, host_pool, src_ids, dst_ids)
as custom ops that mutate their cache (or host pool) argument, for callers that need the
operators visible to the dispatcher (tracing, `torch.compile`). They run the
same HIP kernels as the plain functions in `cache_ops` / `paged`; the plain
functions are the cheaper way to call them from eager code.
"""
from __future__ import annotations

import torch

from . import cache_ops, paged


@torch.library.custom_op("kvcache::reshape_and_cache", mutates_args=("kv_cache",), device_types="cuda")
def reshape_and_cache(key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor,
                      slot_mapping: torch.Tensor) -> None:
    cache_ops.reshape_and_cache(key, value, kv_cache, slot_mapping)


@torch.library.custom_op("kvcache::append_paged_kv_cache", mutates_args=("paged_kv_cache",),
                         device_types="cuda")
def append_paged_kv_cache(append_key: torch.Tensor, append_value: torch.Tensor,
                          batch_indices: torch.Tensor, positions: torch.Tensor,
                          paged_kv_cache: torch.Tensor, kv_indices: torch.Tensor,
                          kv_indptr: torch.Tensor, kv_last_page_len: torch.Tensor) -> None:
    paged.append_paged_kv_cache(append_key, append_value, batch_indices, positions, paged_kv_cache,
                                kv_indices, kv_indptr, kv_last_page_len)


@torch.library.custom_op("kvcache::copy_blocks", mutates_args=("kv_caches",), device_types="cuda")
def copy_blocks(kv_caches: torch.Tensor, block_maps: torch.Tensor) -> None:
    cache_ops.copy_blocks(kv_caches, block_maps)


@torch.library.custom_op("kvcache::swap_out", mutates_args=("host_pool",))
def swap_out(kv_caches: torch.Tensor, host_pool: torch.Tensor, src_ids: torch.Tensor,
             dst_ids: torch.Tensor) -> None:
    cache_ops.swap_out(kv_caches, host_pool, src_ids, dst_ids)


@torch.library.custom_op("kvcache::swap_in", mutates_args=("kv_caches",))
def swap_in(kv_caches: torch.Tensor, host_pool: torch.Tensor, src_ids: torch.Tensor,
            dst_ids: torch.Tensor) -> None:
    cache_ops.swap_in(kv_caches, host_pool, src_ids, dst_ids)

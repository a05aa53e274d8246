"""KV-cache operators with the reference's Python signatures, on the HIP library.

Mirrors runtime/worker/llm_worker/ops/cache_ops.py of the reference:
`copy_blocks` (cache_ops.py:8-36) and `fill_key_cache` (cache_ops.py:39-59)
keep their names, argument order and in-place/return-None behaviour.
`reshape_and_cache` / `reshape_and_cache_layers` are the same write addressed
into the interleaved pool `[L, nb, 2, bs, H, D]`
(runtime/worker/llm_worker/model_worker.py:221-228) through a slot mapping
`slot = block_id * block_size + offset`.

All operators launch on `torch.cuda.current_stream()` of the cache's device
and never synchronise.
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Union

import torch

from . import _lib

_SLOT_DTYPES = {torch.int32: 4, torch.int64: 8}


def flatten_block_maps(src_to_dst: Dict[int, List[int]]) -> List[int]:
    """`{src: [dst, ...]}` -> `[src, dst, src, dst, ...]` in dict order
    (cache_ops.py:12-15 of the reference)."""
    block_maps: List[int] = []
    for src, dsts in src_to_dst.items():
        for dst in dsts:
            block_maps += [int(src), int(dst)]
    return block_maps


def check_block_maps(block_maps: Sequence[int], num_blocks: int) -> None:
    """Host-side validation of a flattened pair list: ids in range, dsts
    distinct, and no dst that is also a src. The reference performs none of
    these checks and its result is undefined when they fail
    (ops/triton/cache_kernels.py:28-36 has no ordering between pairs)."""
    srcs = block_maps[0::2]
    dsts = block_maps[1::2]
    for b in block_maps:
        if b < 0 or b >= num_blocks:
            raise IndexError(f"block id {b} outside [0, {num_blocks})")
    if len(set(dsts)) != len(dsts):
        raise ValueError("copy_blocks: duplicate destination block")
    overlap = set(dsts) & set(srcs)
    overlap = {d for s, d in zip(srcs, dsts) if d in overlap and s != d}
    if overlap:
        raise ValueError(f"copy_blocks: blocks {sorted(overlap)[:8]} are both source and destination")


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device}); "
                         "the KV-cache operators have no CPU path")


def _inner_contiguous(t: torch.Tensor) -> bool:
    """True when every slice `t[i]` is contiguous (dim 0 may have any stride)."""
    expected = 1
    shape, stride = t.shape, t.stride()
    for d in range(len(shape) - 1, 0, -1):
        if shape[d] != 1 and stride[d] != expected:
            return False
        expected *= shape[d]
    return True


def _stream_of(t: torch.Tensor) -> int:
    """Raw hipStream_t of torch's current stream on the tensor's device."""
    return torch._C._cuda_getCurrentRawStream(t.device.index)


class _on_device_of:
    """Make the tensor's device current for the launch; free when it already is
    (the common case), unlike `torch.cuda.device`, which always switches twice."""
    __slots__ = ("idx", "prev")

    def __init__(self, t: torch.Tensor):
        self.idx = t.device.index
        self.prev = -1

    def __enter__(self):
        cur = torch.cuda.current_device()
        if cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)
        return self

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


def copy_blocks(
    kv_caches: torch.Tensor,
    src_to_dst: Union[Dict[int, List[int]], torch.Tensor],
    validate: bool = False,
) -> None:
    """For every layer `l` and pair `(src, dst)`: `kv_caches[l, dst] = kv_caches[l, src]`.

    kv_caches: `[L, num_blocks, ...]` contiguous (the whole pool).
    src_to_dst: the reference's `Dict[int, List[int]]`; a device int64 tensor
      `[src0, dst0, src1, dst1, ...]` is also accepted so a caller can avoid
      the host-to-device copy of the pair list.
    validate: run `check_block_maps` on the host first (dict input only).
    """
    _require_gpu(kv_caches, "kv_caches")
    if kv_caches.dim() < 2 or not kv_caches.is_contiguous():
        raise ValueError("kv_caches must be a contiguous [L, num_blocks, ...] tensor")
    num_layers, num_blocks = kv_caches.shape[0], kv_caches.shape[1]
    if isinstance(src_to_dst, torch.Tensor):
        block_maps_tensor = src_to_dst
        if block_maps_tensor.dtype != torch.int64 or block_maps_tensor.device != kv_caches.device \
                or not block_maps_tensor.is_contiguous() or block_maps_tensor.numel() % 2:
            raise ValueError("block map tensor must be contiguous int64 [2P] on the cache's device")
    else:
        block_maps = flatten_block_maps(src_to_dst)
        if validate:
            check_block_maps(block_maps, num_blocks)
        if not block_maps:
            return
        block_maps_tensor = torch.tensor(block_maps, dtype=torch.long, device=kv_caches.device)
    num_pairs = block_maps_tensor.numel() // 2
    if num_pairs == 0 or num_layers == 0 or num_blocks == 0:
        return
    elem = kv_caches.element_size()
    numel_per_layer = kv_caches[0].numel()
    numel_per_block = numel_per_layer // num_blocks
    with _on_device_of(kv_caches):
        _lib.check(_lib.lib().kvc_copy_blocks(
            kv_caches.data_ptr(), block_maps_tensor.data_ptr(), num_pairs, num_layers,
            numel_per_layer * elem, numel_per_block * elem, num_blocks, _stream_of(kv_caches)))


def _rows(t: torch.Tensor, name: str):
    """Token-major `[T, H, D]` (or `[T, H*D]`) tensor -> (tensor, row_elems, token_stride)."""
    if t.dim() == 2:
        t = t.unsqueeze(1)
    if t.dim() != 3:
        raise ValueError(f"{name} must be [num_tokens, num_kv_heads, head_size]")
    T, H, D = t.shape
    if T > 0 and H * D > 0 and (t.stride(2) != 1 or (H > 1 and t.stride(1) != D)
                                or (T > 1 and t.stride(0) < H * D)):
        # rows that are not dense, or that overlap (an expanded or as_strided view)
        t = t.contiguous()
    stride = t.stride(0) if T > 1 else H * D
    return t, H * D, stride


def fill_key_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """`key_cache[slot_mapping[i]] = key[i]`, `value_cache[slot_mapping[i]] = value[i]`.

    key, value: `[T, H, D]`; key_cache, value_cache: contiguous, viewed as
    `[num_slots, H, D]` whatever their own shape (the reference addresses them
    flat, ops/triton/cache_kernels.py:49-51); slot_mapping: `[T]` int32/int64
    on the device.
    """
    for t, n in ((key, "key"), (value, "value"), (key_cache, "key_cache"),
                 (value_cache, "value_cache"), (slot_mapping, "slot_mapping")):
        _require_gpu(t, n)
    if key.dtype != key_cache.dtype or value.dtype != value_cache.dtype or key.dtype != value.dtype:
        raise TypeError("key/value and their caches must share one dtype")
    if not key_cache.is_contiguous() or not value_cache.is_contiguous():
        raise ValueError("key_cache and value_cache must be contiguous")
    key, row, k_stride = _rows(key, "key")
    value, row_v, v_stride = _rows(value, "value")
    if row != row_v or key.shape[0] != value.shape[0]:
        raise ValueError("key and value must have the same shape")
    num_tokens = len(slot_mapping)
    if num_tokens != key.shape[0]:
        raise ValueError("slot_mapping length differs from the number of tokens")
    if num_tokens == 0 or row == 0:
        return
    slot_bytes = _SLOT_DTYPES.get(slot_mapping.dtype)
    if slot_bytes is None:
        slot_mapping = slot_mapping.to(torch.int64)
        slot_bytes = 8
    if not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.contiguous()
    num_slots = min(key_cache.numel(), value_cache.numel()) // row
    with _on_device_of(key_cache):
        _lib.check(_lib.lib().kvc_reshape_and_cache(
            key.data_ptr(), value.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(),
            slot_mapping.data_ptr(), slot_bytes, num_tokens, row, k_stride, v_stride,
            1, row, row, num_slots, key.element_size(), _stream_of(key_cache)))


def _slot_args(slot_mapping: torch.Tensor):
    slot_bytes = _SLOT_DTYPES.get(slot_mapping.dtype)
    if slot_bytes is None:
        slot_mapping = slot_mapping.to(torch.int64)
        slot_bytes = 8
    if not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.contiguous()
    return slot_mapping, slot_bytes


def reshape_and_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    kv_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """Slot-mapped write into ONE layer of the interleaved pool.

    kv_cache: `[num_blocks, 2, block_size, H, D]` contiguous per block (a
    `kv_caches[l]` view); token `i` lands in block `slot // block_size`, entry
    `slot % block_size`: `kv_cache[blk, 0, e] = key[i]`, `kv_cache[blk, 1, e] = value[i]`.
    """
    if isinstance(kv_cache, torch.Tensor) and kv_cache.is_cuda:
        fast = _lib.fast_entry("reshape_and_cache")
        if fast is not None:
            # common layouts: checked and launched from C++ (1 = not one of them: fall through)
            dev = kv_cache.device.index
            rc = fast(key, value, kv_cache, slot_mapping, dev, torch._C._cuda_getCurrentRawStream(dev))
            if rc == 0:
                return
            if rc < 0:
                _lib.check(rc)
    for t, n in ((key, "key"), (value, "value"), (kv_cache, "kv_cache"),
                 (slot_mapping, "slot_mapping")):
        _require_gpu(t, n)
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2:
        raise ValueError("kv_cache must be [num_blocks, 2, block_size, H, D]")
    if key.dtype != kv_cache.dtype or value.dtype != kv_cache.dtype:
        raise TypeError("key/value and kv_cache must share one dtype")
    nb, _, bs, H, D = kv_cache.shape
    if not _inner_contiguous(kv_cache):
        raise ValueError("every block of kv_cache must be contiguous [2, block_size, H, D]")
    key, row, k_stride = _rows(key, "key")
    value, row_v, v_stride = _rows(value, "value")
    if row != H * D or row_v != H * D or key.shape[0] != value.shape[0]:
        raise ValueError("key/value rows do not match the cache's H*D")
    num_tokens = len(slot_mapping)
    if num_tokens != key.shape[0]:
        raise ValueError("slot_mapping length differs from the number of tokens")
    if num_tokens == 0 or row == 0 or nb == 0:
        return
    slot_mapping, slot_bytes = _slot_args(slot_mapping)
    elem = kv_cache.element_size()
    block_stride = kv_cache.stride(0) if nb > 1 else 2 * bs * row
    with _on_device_of(kv_cache):
        _lib.check(_lib.lib().kvc_reshape_and_cache(
            key.data_ptr(), value.data_ptr(), kv_cache.data_ptr(),
            kv_cache.data_ptr() + bs * row * elem, slot_mapping.data_ptr(), slot_bytes,
            num_tokens, row, k_stride, v_stride, bs, block_stride, row, nb, elem,
            _stream_of(kv_cache)))


def reshape_and_cache_layers(
    key: torch.Tensor,
    value: torch.Tensor,
    kv_caches: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """The write of `reshape_and_cache` for every layer in one launch.

    key, value: `[L, T, H, D]` contiguous; kv_caches: the whole pool
    `[L, num_blocks, 2, block_size, H, D]` contiguous; slot_mapping `[T]` is
    shared by all layers.
    """
    for t, n in ((key, "key"), (value, "value"), (kv_caches, "kv_caches"),
                 (slot_mapping, "slot_mapping")):
        _require_gpu(t, n)
    if kv_caches.dim() != 6 or kv_caches.shape[2] != 2 or not kv_caches.is_contiguous():
        raise ValueError("kv_caches must be contiguous [L, num_blocks, 2, block_size, H, D]")
    if key.dtype != kv_caches.dtype or value.dtype != kv_caches.dtype:
        raise TypeError("key/value and kv_caches must share one dtype")
    L, nb, _, bs, H, D = kv_caches.shape
    if key.dim() != 4 or key.shape != value.shape or key.shape[0] != L \
            or key.shape[2] * key.shape[3] != H * D:
        raise ValueError("key/value must be [L, T, H, D] matching the pool")
    key = key.contiguous()
    value = value.contiguous()
    num_tokens = key.shape[1]
    if len(slot_mapping) != num_tokens:
        raise ValueError("slot_mapping length differs from the number of tokens")
    row = H * D
    if num_tokens == 0 or row == 0 or nb == 0 or L == 0:
        return
    slot_mapping, slot_bytes = _slot_args(slot_mapping)
    elem = kv_caches.element_size()
    with _on_device_of(kv_caches):
        _lib.check(_lib.lib().kvc_reshape_and_cache_layers(
            key.data_ptr(), value.data_ptr(), kv_caches.data_ptr(),
            kv_caches.data_ptr() + bs * row * elem, slot_mapping.data_ptr(), slot_bytes,
            num_tokens, row, row, row, bs, 2 * bs * row, row, nb, L, num_tokens * row,
            num_tokens * row, nb * 2 * bs * row, elem, _stream_of(kv_caches)))


def _pool_geometry(kv_caches: torch.Tensor):
    _require_gpu(kv_caches, "kv_caches")
    if kv_caches.dim() < 3 or not kv_caches.is_contiguous():
        raise ValueError("kv_caches must be a contiguous [L, num_blocks, ...] tensor")
    L, nb = kv_caches.shape[0], kv_caches.shape[1]
    block_elems = kv_caches[0].numel() // nb if nb else 0
    elem = kv_caches.element_size()
    return L, nb, block_elems, block_elems * elem, nb * block_elems * elem


def _ids_on_device(block_ids: torch.Tensor, kv_caches: torch.Tensor) -> torch.Tensor:
    if block_ids.dtype != torch.int64 or block_ids.device != kv_caches.device or block_ids.dim() != 1:
        raise ValueError("block_ids must be a 1-D int64 tensor on the pool's device")
    return block_ids if block_ids.is_contiguous() else block_ids.contiguous()


def gather_blocks(kv_caches: torch.Tensor, block_ids: torch.Tensor, out: torch.Tensor = None,
                  layer_begin: int = 0, layer_end: int = None) -> torch.Tensor:
    """`out[i, l - layer_begin] = kv_caches[l, block_ids[i]]`: scattered pool
    blocks into a dense device buffer in host-pool layout `[n, layers, block_elems]`
    (the row order of the reference's host pool, kv_worker.py:123-127)."""
    L, nb, block_elems, block_bytes, layer_stride = _pool_geometry(kv_caches)
    block_ids = _ids_on_device(block_ids, kv_caches)
    layer_end = L if layer_end is None else layer_end
    n, nl = block_ids.numel(), layer_end - layer_begin
    if out is None:
        out = torch.empty(n, max(nl, 0), block_elems, dtype=kv_caches.dtype, device=kv_caches.device)
    elif out.dtype != kv_caches.dtype or out.device != kv_caches.device or not out.is_contiguous() \
            or out.numel() != n * nl * block_elems:
        raise ValueError("out must be a contiguous [n, layers, block_elems] tensor of the pool's dtype")
    with _on_device_of(kv_caches):
        _lib.check(_lib.lib().kvc_gather_blocks(
            kv_caches.data_ptr(), out.data_ptr(), block_ids.data_ptr(), n, L, layer_stride,
            block_bytes, nb, layer_begin, layer_end, _stream_of(kv_caches)))
    return out


def scatter_blocks(kv_caches: torch.Tensor, block_ids: torch.Tensor, buffer: torch.Tensor,
                   layer_begin: int = 0, layer_end: int = None) -> None:
    """`kv_caches[l, block_ids[i]] = buffer[i, l - layer_begin]`: the inverse of `gather_blocks`."""
    L, nb, block_elems, block_bytes, layer_stride = _pool_geometry(kv_caches)
    block_ids = _ids_on_device(block_ids, kv_caches)
    layer_end = L if layer_end is None else layer_end
    n, nl = block_ids.numel(), layer_end - layer_begin
    if buffer.dtype != kv_caches.dtype or buffer.device != kv_caches.device \
            or not buffer.is_contiguous() or buffer.numel() != n * nl * block_elems:
        raise ValueError("buffer must be a contiguous [n, layers, block_elems] tensor of the pool's dtype")
    with _on_device_of(kv_caches):
        _lib.check(_lib.lib().kvc_scatter_blocks(
            kv_caches.data_ptr(), buffer.data_ptr(), block_ids.data_ptr(), n, L, layer_stride,
            block_bytes, nb, layer_begin, layer_end, _stream_of(kv_caches)))


def _host_ids(ids, name: str):
    import numpy as np

    if isinstance(ids, torch.Tensor):
        if ids.is_cuda:
            raise ValueError(f"{name} must be host-resident (they are range-checked before the launch)")
        ids = ids.numpy()
    return np.ascontiguousarray(np.asarray(ids, dtype=np.int64).reshape(-1))


def _swap_direct(out: bool, kv_caches: torch.Tensor, host_pool: torch.Tensor, src_ids, dst_ids,
                 layer_begin: int, layer_end) -> None:
    L, nb, block_elems, block_bytes, layer_stride = _pool_geometry(kv_caches)
    if host_pool.is_cuda or not host_pool.is_pinned():
        raise ValueError("host_pool must be a pinned host tensor (the kernel addresses it over PCIe)")
    if host_pool.dtype.itemsize != kv_caches.dtype.itemsize or not host_pool.is_contiguous() \
            or host_pool.dim() != 3 or host_pool.shape[1] != L or host_pool.shape[2] != block_elems:
        raise ValueError("host_pool must be a contiguous [num_host_blocks, L, block_elems] tensor "
                         "with the pool's element width")
    src, dst = _host_ids(src_ids, "src_ids"), _host_ids(dst_ids, "dst_ids")
    if src.shape != dst.shape:
        raise ValueError("source and destination id lists differ in length")
    n = int(src.shape[0])
    layer_end = L if layer_end is None else layer_end
    if n == 0 or layer_end <= layer_begin:
        return
    lib = _lib.lib()
    need = lib.kvc_swap_staging_bytes(n, layer_end - layer_begin, block_bytes, _lib.KVC_SWAP_DIRECT, 0)
    with _on_device_of(kv_caches):
        ids_dev = torch.empty(int(need), dtype=torch.uint8, device=kv_caches.device)
        stream = _stream_of(kv_caches)
        fn = lib.kvc_swap_out if out else lib.kvc_swap_in
        _lib.check(fn(kv_caches.data_ptr(), host_pool.data_ptr(), src.ctypes.data, dst.ctypes.data, n,
                      L, layer_stride, block_bytes, nb, host_pool.shape[0], layer_begin, layer_end,
                      ids_dev.data_ptr(), ids_dev.numel(), _lib.KVC_SWAP_DIRECT, stream, stream))


def swap_out(kv_caches: torch.Tensor, host_pool: torch.Tensor, src_ids, dst_ids,
             layer_begin: int = 0, layer_end: int = None) -> None:
    """`host_pool[dst_ids[i], l] = kv_caches[l, src_ids[i]]` on the current stream
    (kv_worker.py:213-227 for every layer of the range): one kernel that stores
    into the pinned host pool. Asynchronous; the ids are host-resident lists,
    int64 tensors or arrays."""
    _swap_direct(True, kv_caches, host_pool, src_ids, dst_ids, layer_begin, layer_end)


def swap_in(kv_caches: torch.Tensor, host_pool: torch.Tensor, src_ids, dst_ids,
            layer_begin: int = 0, layer_end: int = None) -> None:
    """`kv_caches[l, dst_ids[i]] = host_pool[src_ids[i], l]` on the current stream
    (kv_worker.py:197-211 for every layer of the range)."""
    _swap_direct(False, kv_caches, host_pool, src_ids, dst_ids, layer_begin, layer_end)

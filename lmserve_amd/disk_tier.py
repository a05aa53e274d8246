"""Host <-> disk tier of the KV cache over the native block file.

Mirrors the disk half of the reference's KV worker
(runtime/worker/llm_worker/kv_worker.py:48-85 file handling, :229-247 row
copies, :297-322 thread pool): `DiskTier` owns the `.npy` block file of shape
`(num_disk_blocks, L, block_elems)` and moves whole blocks between it and a
host pool of the same row layout. A block is one contiguous extent on both
sides, so it travels as one positional read/write (several neighbours merged)
instead of L rows through a memory map; with `direct=True` the transfers
bypass the page cache when alignment allows.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence, Tuple

import numpy as np

from . import _lib


class DiskTier:
    """The block file `path`, created or reused as the reference does.

    shape: `(num_disk_blocks, num_layers, block_elems)`; dtype: the NumPy dtype
    of the host pool (bf16 lanes are carried as uint16, kv_worker.py:17-22).
    preallocate: a new file reserves all its blocks when it is made (the
    reference's memory map is sparse); first writes then run at the device's
    rate and cannot fail for lack of space.
    """

    def __init__(self, path: str, shape: Tuple[int, int, int], dtype, direct: bool = True,
                 threads: int = 8, preallocate: bool = False):
        if len(shape) != 3:
            raise ValueError("disk KV cache shape must be (num_disk_blocks, num_layers, block_elems)")
        self.path = str(path)
        self.shape = tuple(int(x) for x in shape)
        self.dtype = np.dtype(dtype)
        self.threads = int(threads)
        handle = ctypes.c_void_p()
        _lib.check(_lib.lib().kvc_disk_open(
            self.path.encode(), self.dtype.str.encode(), self.shape[0], self.shape[1], self.shape[2],
            self.dtype.itemsize,
            (_lib.KVC_DISK_DIRECT if direct else 0) | (_lib.KVC_DISK_PREALLOCATE if preallocate else 0),
            ctypes.byref(handle)))
        self._h: Optional[ctypes.c_void_p] = handle

    # ------------------------------------------------------------------ facts
    def _info(self, what: int) -> int:
        if self._h is None:
            raise ValueError("disk tier is closed")
        return int(_lib.lib().kvc_disk_info(self._h, what))

    @property
    def data_offset(self) -> int:
        return self._info(_lib.KVC_DISK_INFO_DATA_OFFSET)

    @property
    def is_direct(self) -> bool:
        return bool(self._info(_lib.KVC_DISK_INFO_DIRECT))

    @property
    def created(self) -> bool:
        return bool(self._info(_lib.KVC_DISK_INFO_CREATED))

    @property
    def last_transfer_staged(self) -> bool:
        """True if the last O_DIRECT transfer copied the host side through the
        aligned staging buffers (unaligned pool, or memory the kernel cannot pin)."""
        return bool(self._info(_lib.KVC_DISK_INFO_BOUNCED))

    @property
    def row_bytes(self) -> int:
        return self._info(_lib.KVC_DISK_INFO_ROW_BYTES)

    # ------------------------------------------------------------------ transfers
    def _check_pool(self, host_pool: np.ndarray, writable: bool) -> None:
        if not isinstance(host_pool, np.ndarray) or host_pool.ndim != 3:
            raise ValueError("host pool must be a [num_host_blocks, num_layers, block_elems] array")
        if host_pool.shape[1:] != self.shape[1:] or host_pool.dtype != self.dtype:
            raise ValueError(f"host pool rows {host_pool.shape[1:]} {host_pool.dtype} do not match the "
                             f"disk tier's {self.shape[1:]} {self.dtype}")
        if not host_pool.flags.c_contiguous:
            raise ValueError("host pool must be C-contiguous")
        if writable and not host_pool.flags.writeable:
            raise ValueError("host pool is read-only")

    @staticmethod
    def _ids(ids) -> np.ndarray:
        return np.ascontiguousarray(np.asarray(ids, dtype=np.int64).reshape(-1))

    def save_blocks(self, host_pool: np.ndarray, src_host_ids: Sequence[int],
                    dst_disk_ids: Sequence[int]) -> None:
        """disk[dst] = host[src] for every pair, all layers (kv_worker.py:239-247)."""
        self._check_pool(host_pool, writable=False)
        src, dst = self._ids(src_host_ids), self._ids(dst_disk_ids)
        if src.shape != dst.shape:
            raise ValueError("source and destination id lists differ in length")
        _lib.check(_lib.lib().kvc_disk_save_blocks(
            self._require(), host_pool.ctypes.data, host_pool.shape[0], src.ctypes.data,
            dst.ctypes.data, src.shape[0], self.threads))

    def load_blocks(self, host_pool: np.ndarray, src_disk_ids: Sequence[int],
                    dst_host_ids: Sequence[int]) -> None:
        """host[dst] = disk[src] for every pair, all layers (kv_worker.py:229-237)."""
        self._check_pool(host_pool, writable=True)
        src, dst = self._ids(src_disk_ids), self._ids(dst_host_ids)
        if src.shape != dst.shape:
            raise ValueError("source and destination id lists differ in length")
        _lib.check(_lib.lib().kvc_disk_load_blocks(
            self._require(), host_pool.ctypes.data, host_pool.shape[0], src.ctypes.data,
            dst.ctypes.data, src.shape[0], self.threads))

    def sync(self) -> None:
        _lib.check(_lib.lib().kvc_disk_sync(self._require()))

    def memmap(self, mode: str = "r") -> np.ndarray:
        """The file as a NumPy memory map (it is an ordinary `.npy` array)."""
        return np.load(self.path, mmap_mode=mode)

    def _require(self):
        if self._h is None:
            raise ValueError("disk tier is closed")
        return self._h

    def close(self) -> None:
        if self._h is not None:
            h, self._h = self._h, None
            _lib.check(_lib.lib().kvc_disk_close(h))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

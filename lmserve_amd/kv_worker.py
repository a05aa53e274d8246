"""Swap engine between the HBM block pool and a pinned host pool.

Mirrors the GPU<->Host part of runtime/worker/llm_worker/kv_worker.py of the
reference: the pools' layouts (kv_worker.py:104-130), the direction table
(kv_worker.py:190-195), `copy_kv(block_mappings, src, dst)` and its error
behaviour (kv_worker.py:336-346), and the per-entry semantics
  GPU->Host: host[dst_block_id, l] = gpu[l, src_block_id]   (kv_worker.py:213-227)
  Host->GPU: gpu[l, dst_block_id] = host[src_block_id, l]   (kv_worker.py:197-211)
Where the reference issues one driver memcpy per (layer, block), this engine
hands the whole mapping list to libkvcache (`kvc_swap_out` / `kvc_swap_in`):
a gather/scatter kernel plus large PCIe extents carried by the copy engines,
or one kernel that addresses the mapped host pool directly. Both legs of a
staged call run on the direction's own stream (the reference's two dedicated
streams, kv_worker.py:159-160): splitting kernel and copy over two streams
tied by events gained 1 % at best and lost up to three quarters of the rate
late in a busy process.

A copy that runs layer by layer (the reference's protocol with the model's
forward pass) flattens, checks and uploads its id lists once
(`kvc_swap_prepare`); each layer is then a single launch
(`kvc_swap_out_prepared` / `kvc_swap_in_prepared`).

When the layers of a copy travel one per call and the host blocks do not
neighbour each other (a layer's rows are then 64 KiB pieces a whole host block
apart: too small for the copy engines, and a kernel that stores them over PCIe
holds back the model's kernels), the PCIe leg of a layer is one copy between
the GPU and a dense pinned buffer and host threads move the rows between that
buffer and their places in the host pool (`kvc_host_copy_rows`).

The Host<->Disk legs (kv_worker.py:229-247) go through the native disk tier of
the same library (`disk_tier.DiskTier`: whole-block positional I/O on the
reference's `.npy` file); they involve no GPU work.
"""
from __future__ import annotations

import asyncio
import ctypes
import enum
import os
import queue
import time
import warnings
import weakref
from dataclasses import dataclass, field
from typing import Callable, Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib
from .disk_tier import DiskTier


class Device(enum.IntEnum):
    """proto/worker.proto:13-17 of the reference."""
    GPU = 0
    Host = 1
    Disk = 2


@dataclass
class BlockMappingEntry:
    """proto/worker.proto:78-81."""
    src_block_id: int
    dst_block_id: int


@dataclass
class BlockMapping:
    """proto/worker.proto:83-85: one mapping per sequence."""
    entries: List[BlockMappingEntry] = field(default_factory=list)

    @classmethod
    def from_pairs(cls, pairs: Iterable[Tuple[int, int]]) -> "BlockMapping":
        return cls([BlockMappingEntry(int(s), int(d)) for s, d in pairs])


# kv_worker.py:17-22: bf16 travels as uint16 on the host
dtype_map = {
    torch.float32: np.float32,
    torch.float16: np.float16,
    torch.bfloat16: np.uint16,
    torch.int32: np.int32,
}

SWAP_MODES = {"staged": _lib.KVC_SWAP_STAGED, "direct": _lib.KVC_SWAP_DIRECT, "auto": _lib.KVC_SWAP_AUTO}


def flatten_block_mappings(block_mappings: Sequence[BlockMapping]) -> Tuple[np.ndarray, np.ndarray]:
    """All entries of all mappings, in order, as (src_ids, dst_ids) int64 arrays.
    Accepts anything with `.entries[*].src_block_id/.dst_block_id` (the protobuf
    messages of the reference included)."""
    src: List[int] = []
    dst: List[int] = []
    for mapping in block_mappings:
        for entry in mapping.entries:
            src.append(entry.src_block_id)
            dst.append(entry.dst_block_id)
    return np.asarray(src, dtype=np.int64), np.asarray(dst, dtype=np.int64)


def check_distinct_destinations(dst_ids: np.ndarray, what: str) -> None:
    """Raise `ValueError` if a block id occurs twice among the destinations of one call."""
    if dst_ids.size > 1:
        ids, counts = np.unique(dst_ids, return_counts=True)
        if ids.size != dst_ids.size:
            twice = ids[counts > 1][:8].tolist()
            raise ValueError(f"{what}: destination block ids {twice} occur more than once in one call")


def order_by_host_id(gpu_ids: np.ndarray, host_ids: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """The pairs of one swap call in ascending order of their host block id
    (stable), so that host blocks which lie next to each other in the pool are
    next to each other in the call and leave as one PCIe extent. The result of a
    swap does not depend on the order of its pairs (the reference copies them
    one after the other, kv_worker.py:197-227, and they touch distinct blocks)."""
    if host_ids.size > 1 and bool(np.any(host_ids[1:] < host_ids[:-1])):
        order = np.argsort(host_ids, kind="stable")
        return gpu_ids[order], host_ids[order]
    return gpu_ids, host_ids


_warned_about_queues = False


def warn_if_few_hardware_queues(environ=os.environ) -> bool:
    """One warning per process when a KV worker is set up to copy beside a forward
    pass while the HIP runtime runs with its default of 4 hardware queues: the
    model's stream and the worker's stream can then share a queue and wait for
    each other (a forward pass of 15.6 ms took 33-36 ms beside a write-through
    on MI355X). `GPU_MAX_HW_QUEUES=8` in the environment, set before the process
    first touches the GPU, gives every stream involved a queue of its own. The
    reference runs the KV worker as a second process, which has its own queues.
    Returns whether it warned."""
    global _warned_about_queues
    try:
        queues = int(environ.get("GPU_MAX_HW_QUEUES", "4"))
    except ValueError:
        queues = 4
    if queues >= 8 or _warned_about_queues:
        return False
    _warned_about_queues = True
    warnings.warn("KVWorker with a layer-sync handle in a process with GPU_MAX_HW_QUEUES="
                  f"{environ.get('GPU_MAX_HW_QUEUES', 'unset (4)')}: copies beside a forward pass may share a "
                  "hardware queue with the model's stream and double its time; export GPU_MAX_HW_QUEUES=8 before "
                  "the process starts, or run the KV worker as its own process", RuntimeWarning, stacklevel=3)
    return True


def pick_streams_apart(count: int, avoid: Sequence, make_stream: Callable, share: Callable,
                       tries: int = 24) -> Tuple[list, bool]:
    """`count` streams of which none shares a hardware queue with another or with a
    stream of `avoid`, drawn with `make_stream()` and tested with
    `share(a, b) -> bool`. The runtime maps all streams of a process onto a few
    hardware queues and says nothing about which; streams that share one take
    turns, and a wait queued by one holds back the other. Returns
    `(streams, apart)`; after `tries` draws without success the remaining
    streams are taken as they come and `apart` is False."""
    chosen: list = []
    drawn = 0
    while len(chosen) < count and drawn < tries:
        s = make_stream()
        drawn += 1
        if any(share(s, o) for o in list(avoid) + chosen):
            continue
        chosen.append(s)
    apart = len(chosen) == count
    while len(chosen) < count:
        chosen.append(make_stream())
    return chosen, apart


_warned_about_shared_queue = False


def warn_streams_share_a_queue(environ=os.environ) -> bool:
    """One warning per process when a KV worker could not be given streams with
    hardware queues of their own. Returns whether it warned."""
    global _warned_about_shared_queue
    if _warned_about_shared_queue:
        return False
    _warned_about_shared_queue = True
    warnings.warn("KVWorker: no pair of streams with hardware queues of their own was found "
                  f"(GPU_MAX_HW_QUEUES={environ.get('GPU_MAX_HW_QUEUES', 'unset (4)')}): swap-out and swap-in issued "
                  "together will take turns (about 55 instead of 94 GB/s in sum) and copies beside a forward pass "
                  "may hold it back; export GPU_MAX_HW_QUEUES=8 before the process starts",
                  RuntimeWarning, stacklevel=3)
    return True


class PinnedHostPool:
    """`[num_host_blocks, L, block_elems]` page-locked, device-addressable host
    memory (replaces pycuda's `pagelocked_empty`, kv_worker.py:123-127)."""

    def __init__(self, shape: Tuple[int, int, int], np_dtype):
        self.shape = tuple(int(s) for s in shape)
        self.np_dtype = np.dtype(np_dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.np_dtype.itemsize
        self.ptr = _lib.lib().kvc_host_alloc_pinned(max(self.nbytes, 1))
        if not self.ptr:
            raise MemoryError(f"cannot pin {self.nbytes} bytes of host memory: {_lib.last_error()}")
        buf = (ctypes.c_char * max(self.nbytes, 1)).from_address(self.ptr)
        self.array = np.frombuffer(buf, dtype=self.np_dtype,
                                   count=self.nbytes // self.np_dtype.itemsize).reshape(self.shape)

    def close(self) -> None:
        if self.ptr:
            self.array = None
            _lib.check(_lib.lib().kvc_host_free_pinned(self.ptr))
            self.ptr = None


@dataclass
class PreparedSwap:
    """Id lists of one copy, already checked and resident on the device
    (`KVWorker.prepare_swap`)."""
    direction: str                 # "out" (GPU->Host) or "in" (Host->GPU)
    n: int
    host_ids: np.ndarray           # kept alive: the staged mode reads it per call
    staging: torch.Tensor          # head: [gpu_ids | host_ids] on the device
    stream: torch.cuda.Stream
    dense_ids: Optional[np.ndarray] = None   # 0..n-1, for calls that land in a dense bounce region


class HostBounce:
    """Dense pinned buffer of `slots` regions, each one layer of `n` blocks: what a
    one-layer PCIe copy lands in (or leaves from) when its rows are scattered over
    the host pool."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = _lib.lib().kvc_host_alloc_pinned(max(self.nbytes, 1))
        if not self.ptr:
            raise MemoryError(f"cannot pin {self.nbytes} bytes of host memory: {_lib.last_error()}")
        self.busy = False
        self.slots = 0
        self.slot_bytes = 0
        self.mover = None     # kvc_row_mover: its thread moves the rows of the regions

    def row_mover(self, threads: int, timeout: Optional[float] = None):
        if self.mover is None:
            mover = ctypes.c_void_p()
            _lib.check(_lib.lib().kvc_row_mover_create(int(threads), ctypes.byref(mover)))
            _lib.check(_lib.lib().kvc_row_mover_set_timeout_ms(mover, -1 if timeout is None else int(timeout * 1e3)))
            self.mover = mover
        return self.mover

    def shape(self, slots: int, slot_bytes: int) -> None:
        self.slots, self.slot_bytes = int(slots), int(slot_bytes)

    def slot_ptr(self, layer_idx: int) -> int:
        return self.ptr + (layer_idx % self.slots) * self.slot_bytes

    def close(self, cancel: bool = False) -> None:
        if self.mover is not None:
            if cancel:   # jobs that still wait for an event give up now instead of at their deadline
                _lib.check(_lib.lib().kvc_row_mover_cancel(self.mover))
            _lib.check(_lib.lib().kvc_row_mover_destroy(self.mover))   # after its queued jobs
            self.mover = None
        if self.ptr:
            _lib.check(_lib.lib().kvc_host_free_pinned(self.ptr))
            self.ptr = None


class KVWorker:
    """Owns the host pool and moves blocks between the tiers.

    gpu_kv_caches: the model worker's pool `[L, num_gpu_blocks, ...]`
      (`[L, nb, 2, bs, H, D]`), contiguous, on the GPU. The reference maps it
      from an IPC handle in a second process (kv_worker.py:104-108); here the
      tensor itself is passed.
    swap_mode: "staged": a short gather/scatter kernel between the pool and a
      device ring, the PCIe leg as DMA extents (runs of consecutive host ids);
      the copy engines carry the transfer, so a forward pass running on other
      streams keeps its speed, but every extent costs about 10 us beyond its
      transfer time: host blocks scattered over the pool, one layer per call,
      move at a ninth of the link rate. "direct": one kernel addresses the
      mapped host pool, no staging traffic, one launch per call and the link
      rate whatever the ids are; but while that kernel runs, kernels of other
      streams are held back (a stream of short GEMMs stands still beside a
      direct swap-out, measured on MI355X). "auto" (default): per call, staged
      when the call's extents are 1 MiB or more in the mean, else direct. The
      mappings of a call are sorted by host block id first (their order does not
      matter to the result), so a call's host blocks form the longest runs they
      can.
    kv_worker_handle: a `kv_pool.KVWorkerHandle`; when given, `copy_kv` between
      GPU and Host follows the reference's layer-pipelined protocol
      (kv_worker.py:249-295): a save waits for the model's doorbell and
      `post_events[l]` before touching layer l, a load records `pre_events[l]`
      and rings the model's doorbell after layer l. Without it the whole layer
      range moves in one call.
    disk_direct_io / disk_threads: the disk tier bypasses the page cache when
      alignment and the file system allow, and spreads block extents over this
      many threads (the reference copies rows through a memory map on 4);
      `disk_preallocate` reserves a new file's blocks when it is made.
    host_bounce_bytes / host_copy_threads: layer-by-layer copies (the protocol
      with a handle) whose host blocks are scattered so that a layer's PCIe
      extents would be under 1 MiB in the mean go through a dense pinned buffer
      of up to this many bytes (2 to `host_bounce_regions` regions of one layer
      of the copy's blocks; allocated on first use and kept) and this many host threads, in
      the "auto" and "staged" modes: the copy engines carry each layer as one
      copy and the model's kernels keep running. 0 turns it off ("auto" then
      takes the direct kernel for such copies). A copy too large for the buffer,
      or a second one of the same direction while the buffer is in use, goes
      the usual way. `host_bounce_always=True` sends every layer-by-layer copy
      that way, consecutive host blocks included: 5 % slower than the copy
      engines on the rows as they lie (their one-layer transfers are 2-D copies)
      while those are in their good state, and unaffected by the state they
      fall into for some seconds after the process has freed device memory
      (48 against 38 GB/s there).
    host_wait_timeout: seconds after which a host-side wait of the layer protocol
      gives up (`TimeoutError`): the doorbell of the model's next layer, the event
      a queued row copy waits for. `close()` returns within it whatever the other
      side does. None = no limit (the reference's behaviour).
    model_streams: the stream(s) the model's forward pass runs on, when that is not
      the stream that is current where the worker is made. The worker takes two
      streams that share a hardware queue neither with each other nor with these
      (`kvc_streams_share_hw_queue`; about 1 ms at construction). Whether it
      found them is `streams_have_own_queues`; if not it warns once: with the
      runtime's default of 4 hardware queues a process that already runs many
      streams may have none left, `GPU_MAX_HW_QUEUES=8` helps.
    own_queues: False takes the two streams as torch hands them out, as the
      reference does, without looking at their queues (for measurements).
    validate: check on the host that no block is the destination of two pairs of
      one GPU<->Host call (`ValueError`). The reference copies the pairs one
      after the other, so the later pair wins there (kv_worker.py:197-227);
      here the pairs of a call move concurrently and such a call has no defined
      result. Off by default: the scheduler hands out distinct blocks.
    """

    def __init__(
        self,
        gpu_kv_caches: torch.Tensor,
        num_host_blocks: int,
        num_disk_blocks: int = 0,
        disk_kv_cache_file: Optional[str] = None,
        swap_mode: str = "auto",
        staging_chunk_blocks: int = 0,
        kv_worker_handle=None,
        disk_direct_io: bool = True,
        disk_threads: int = 8,
        disk_preallocate: bool = False,
        validate: bool = False,
        host_bounce_bytes: int = 1 << 30,
        host_copy_threads: int = 4,
        host_bounce_regions: int = 4,
        host_bounce_always: bool = False,
        host_wait_timeout: Optional[float] = 30.0,
        model_streams: Optional[Sequence[torch.cuda.Stream]] = None,
        own_queues: bool = True,
    ):
        if not gpu_kv_caches.is_cuda:
            raise ValueError("gpu_kv_caches must live on the GPU")
        if gpu_kv_caches.dim() < 3 or not gpu_kv_caches.is_contiguous():
            raise ValueError("gpu_kv_caches must be a contiguous [L, num_gpu_blocks, ...] tensor")
        if swap_mode not in SWAP_MODES:
            raise ValueError(f"swap_mode must be one of {sorted(SWAP_MODES)}")
        np_dtype = dtype_map.get(gpu_kv_caches.dtype)
        if np_dtype is None:
            raise TypeError(f"Unsupported dtype: {gpu_kv_caches.dtype}")

        num_layers, num_gpu_blocks = gpu_kv_caches.shape[0], gpu_kv_caches.shape[1]
        self.gpu_kv_caches = gpu_kv_caches.view(num_layers, num_gpu_blocks, -1)
        block_elems = self.gpu_kv_caches.shape[2]
        self.device = gpu_kv_caches.device
        self.num_layers = num_layers
        self.num_gpu_blocks = num_gpu_blocks
        self.num_host_blocks = int(num_host_blocks)
        self.num_disk_blocks = int(num_disk_blocks)
        self.block_stride = block_elems * gpu_kv_caches.element_size()  # bytes, kv_worker.py:157
        self.layer_stride = num_gpu_blocks * self.block_stride
        self.swap_mode = swap_mode
        self.staging_chunk_blocks = int(staging_chunk_blocks)
        self.validate = bool(validate)
        self.host_bounce_bytes = int(host_bounce_bytes)
        self.host_copy_threads = int(host_copy_threads)
        self.host_bounce_regions = max(2, int(host_bounce_regions))
        self.host_bounce_always = bool(host_bounce_always)
        self.host_wait_timeout = None if host_wait_timeout is None else float(host_wait_timeout)
        self._bounce = {"out": None, "in": None}
        self.last_copy_went_through_host_bounce = False
        self.last_copy_swap_mode = -1    # KVC_SWAP_* the last layer-by-layer copy's calls ran in

        self._host_pool = PinnedHostPool((self.num_host_blocks, num_layers, block_elems), np_dtype)
        self.host_kv_caches = self._host_pool.array
        self.host_kv_caches_tensor = torch.from_numpy(self.host_kv_caches)

        # The block file of the disk tier (kv_worker.py:133-145). Transfers go through the
        # native tier; `disk_kv_caches` stays available as a read-only map of the same file.
        if self.num_disk_blocks > 0:
            if not disk_kv_cache_file:
                raise ValueError("disk_kv_cache_file is required when num_disk_blocks > 0")
            self.disk_tier = DiskTier(disk_kv_cache_file,
                                      (self.num_disk_blocks, num_layers, block_elems), np_dtype,
                                      direct=disk_direct_io, threads=disk_threads,
                                      preallocate=disk_preallocate)
            self.disk_kv_caches = self.disk_tier.memmap("r")
        else:
            self.disk_tier = None
            self.disk_kv_caches = None

        # Two streams as in the reference (kv_worker.py:159-160), chosen so that they share
        # a hardware queue neither with each other nor with the stream(s) the model runs
        # on (by default the stream that is current here): every swap call starts by
        # waiting for the caller's current stream, and a wait in a shared queue holds
        # back the other direction and the model's kernels as well.
        with torch.cuda.device(self.device):
            if model_streams is None:
                model_streams = [torch.cuda.current_stream(self.device)]
            if own_queues:
                (self.dtoh_stream, self.htod_stream), self.streams_have_own_queues = pick_streams_apart(
                    2, list(model_streams), torch.cuda.Stream,
                    lambda a, b: _lib.streams_share_hw_queue(a.cuda_stream, b.cuda_stream))
            else:
                self.dtoh_stream, self.htod_stream = torch.cuda.Stream(), torch.cuda.Stream()
                self.streams_have_own_queues = True    # not looked at: nothing to warn about
        self._staging = {}   # (direction, stream handle) -> [workspace, weak reference to its PreparedSwap]
        self.kv_worker_handle = kv_worker_handle
        if not self.streams_have_own_queues:
            warn_streams_share_a_queue()
            if kv_worker_handle is not None:
                warn_if_few_hardware_queues()

        self.COPY_KV_OP_MAP = {
            (Device.GPU, Device.Host): self._copy_kv_gpu_to_host,
            (Device.Host, Device.GPU): self._copy_kv_host_to_gpu,
            (Device.Host, Device.Disk): self._copy_kv_host_to_disk,
            (Device.Disk, Device.Host): self._copy_kv_disk_to_host,
        }

    # ------------------------------------------------------------------ GPU legs
    def _staging_for(self, direction: str, stream: torch.cuda.Stream, n: int,
                     *layers_per_call: int) -> Tuple[torch.Tensor, Optional[list]]:
        """Device workspace for calls of one direction on one stream that cover any
        of the given numbers of layers. Returns `(buffer, slot)`.

        The head of a workspace holds the id lists of the call that uses it, so a
        workspace serves one copy at a time. Each (direction, stream) keeps one
        that calls reuse (work of one stream runs in order, so the next call's
        upload comes after everything the previous call queued). While a
        `PreparedSwap` that was given this workspace is still alive (its layers
        may not all be queued yet), further calls get a buffer of their own:
        `slot` is None then. Otherwise `slot` is the kept workspace's record,
        whose owner a prepared swap sets to itself."""
        mode = SWAP_MODES[self.swap_mode]
        need = 0
        for nl in layers_per_call:
            b = _lib.lib().kvc_swap_staging_bytes(n, nl, self.block_stride, mode,
                                                  self.staging_chunk_blocks)
            if b < 0:
                raise ValueError("bad swap geometry")
            need = max(need, b)
        slot = self._staging.setdefault((direction, stream.cuda_stream), [None, None])
        owner = slot[1]() if slot[1] is not None else None
        if owner is not None:
            buf = torch.empty(int(need), dtype=torch.uint8, device=self.device)
            buf.record_stream(stream)
            return buf, None
        slot[1] = None
        if slot[0] is None or slot[0].numel() < need:
            slot[0] = torch.empty(int(need), dtype=torch.uint8, device=self.device)
        # the buffer may have been allocated with another stream current
        slot[0].record_stream(stream)
        return slot[0], slot

    def _swap(self, direction: str, src: np.ndarray, dst: np.ndarray, layer_begin: int,
              layer_end: int, stream: torch.cuda.Stream) -> None:
        n = int(src.shape[0])
        if n == 0 or layer_end <= layer_begin:
            return
        src = np.ascontiguousarray(src, dtype=np.int64)
        dst = np.ascontiguousarray(dst, dtype=np.int64)
        if self.validate:
            check_distinct_destinations(dst, "GPU->Host" if direction == "out" else "Host->GPU")
        if direction == "out":
            src, dst = order_by_host_id(src, dst)
        else:
            dst, src = order_by_host_id(dst, src)
        with torch.cuda.device(self.device):
            # whatever the caller's current stream has queued on the pool comes first
            stream.wait_stream(torch.cuda.current_stream(self.device))
            staging, _ = self._staging_for(direction, stream, n, layer_end - layer_begin)
            fn = _lib.lib().kvc_swap_out if direction == "out" else _lib.lib().kvc_swap_in
            _lib.check(fn(self.gpu_kv_caches.data_ptr(), self._host_pool.ptr,
                          src.ctypes.data, dst.ctypes.data, n, self.num_layers, self.layer_stride,
                          self.block_stride, self.num_gpu_blocks, self.num_host_blocks,
                          layer_begin, layer_end, staging.data_ptr(), staging.numel(),
                          SWAP_MODES[self.swap_mode], stream.cuda_stream, stream.cuda_stream))

    def save_kv_blocks_to_host_nowait(self, block_mappings: Sequence[BlockMapping],
                                      stream: Optional[torch.cuda.Stream] = None,
                                      layer_begin: int = 0, layer_end: Optional[int] = None) -> None:
        """Enqueue GPU->Host for layers [layer_begin, layer_end) on `stream`."""
        if len(block_mappings) == 0:
            return
        src, dst = flatten_block_mappings(block_mappings)
        self._swap("out", src, dst, layer_begin, self.num_layers if layer_end is None else layer_end,
                   stream or self.dtoh_stream)

    def load_kv_blocks_from_host_nowait(self, block_mappings: Sequence[BlockMapping],
                                        stream: Optional[torch.cuda.Stream] = None,
                                        layer_begin: int = 0, layer_end: Optional[int] = None) -> None:
        """Enqueue Host->GPU for layers [layer_begin, layer_end) on `stream`."""
        if len(block_mappings) == 0:
            return
        src, dst = flatten_block_mappings(block_mappings)
        self._swap("in", src, dst, layer_begin, self.num_layers if layer_end is None else layer_end,
                   stream or self.htod_stream)

    # ------------------------------------------------- layer by layer, ids uploaded once
    def prepare_swap(self, direction: str, block_mappings: Sequence[BlockMapping],
                     stream: Optional[torch.cuda.Stream] = None) -> Optional["PreparedSwap"]:
        """Flatten the mappings, range-check them and upload the id lists once, on
        `stream`; the result feeds `swap_prepared_layers` any number of times.
        direction: "out" (GPU->Host) or "in" (Host->GPU). None when there is
        nothing to move."""
        if direction not in ("out", "in"):
            raise ValueError("direction must be 'out' or 'in'")
        if len(block_mappings) == 0:
            return None
        src, dst = flatten_block_mappings(block_mappings)
        n = int(src.shape[0])
        if n == 0:
            return None
        if self.validate:
            check_distinct_destinations(dst, "GPU->Host" if direction == "out" else "Host->GPU")
        gpu_ids, host_ids = order_by_host_id(*((src, dst) if direction == "out" else (dst, src)))
        if stream is None:
            stream = self.dtoh_stream if direction == "out" else self.htod_stream
        with torch.cuda.device(self.device):
            stream.wait_stream(torch.cuda.current_stream(self.device))
            # room for one layer per call and for the whole range in one call
            staging, slot = self._staging_for(direction, stream, n, 1, self.num_layers)
            _lib.check(_lib.lib().kvc_swap_prepare(
                gpu_ids.ctypes.data, host_ids.ctypes.data, n, self.num_gpu_blocks,
                self.num_host_blocks, staging.data_ptr(), staging.numel(), stream.cuda_stream))
        prepared = PreparedSwap(direction, n, host_ids, staging, stream)
        if slot is not None:
            # the kept workspace is this copy's until the object goes away
            slot[1] = weakref.ref(prepared)
        return prepared

    def swap_prepared_layers(self, prepared: Optional["PreparedSwap"], layer_begin: int,
                             layer_end: int) -> None:
        """Enqueue layers [layer_begin, layer_end) of a prepared swap on its stream:
        one launch in direct mode, no id traffic, nothing to wait for on the host."""
        if prepared is None or layer_end <= layer_begin:
            return
        lib = _lib.lib()
        fn = lib.kvc_swap_out_prepared if prepared.direction == "out" else lib.kvc_swap_in_prepared
        with torch.cuda.device(self.device):
            _lib.check(fn(self.gpu_kv_caches.data_ptr(), self._host_pool.ptr,
                          prepared.host_ids.ctypes.data, prepared.n, self.num_layers,
                          self.layer_stride, self.block_stride, self.num_gpu_blocks,
                          self.num_host_blocks, layer_begin, layer_end, prepared.staging.data_ptr(),
                          prepared.staging.numel(), SWAP_MODES[self.swap_mode],
                          prepared.stream.cuda_stream, prepared.stream.cuda_stream))

    # ------------------------------- one layer per call, scattered host blocks
    def _bounce_for(self, prepared: Optional["PreparedSwap"]) -> Optional[HostBounce]:
        """The dense pinned buffer for the one-layer calls of `prepared`, marked
        busy, or None when they should go the usual way."""
        if prepared is None or self.swap_mode == "direct" or self.host_bounce_bytes <= 0:
            return None
        n, ids = prepared.n, prepared.host_ids
        runs = 1 + int(np.count_nonzero(ids[1:] != ids[:-1] + 1))
        if not self.host_bounce_always and \
                n * self.block_stride >= runs * _lib.get_tuning("auto_min_extent_bytes"):
            return None            # long extents: the copy engines take the rows as they lie
        slot_bytes = n * self.block_stride
        slots = min(self.host_bounce_regions, self.host_bounce_bytes // slot_bytes, self.num_layers)
        if slots < min(2, self.num_layers):
            return None
        bounce = self._bounce[prepared.direction]
        if bounce is not None and bounce.busy:
            return None
        if bounce is None or bounce.nbytes < slots * slot_bytes:
            if bounce is not None:
                with torch.cuda.device(self.device):
                    prepared.stream.synchronize()   # nothing of an earlier copy still lands in it
                bounce.close()
            bounce = self._bounce[prepared.direction] = HostBounce(slots * slot_bytes)
        bounce.shape(slots, slot_bytes)
        bounce.busy = True
        return bounce

    def _swap_layer_through_bounce(self, prepared: "PreparedSwap", layer_idx: int, slot_ptr: int) -> None:
        """Enqueue one layer of a prepared swap between the pool and a dense region
        of the bounce buffer: that region is the call's host pool (one layer, host
        ids 0..n-1), so the PCIe leg is one copy per staging chunk."""
        lib = _lib.lib()
        fn = lib.kvc_swap_out_prepared if prepared.direction == "out" else lib.kvc_swap_in_prepared
        if prepared.dense_ids is None:
            prepared.dense_ids = np.arange(prepared.n, dtype=np.int64)
        with torch.cuda.device(self.device):
            _lib.check(fn(self.gpu_kv_caches.data_ptr() + layer_idx * self.layer_stride, slot_ptr,
                          prepared.dense_ids.ctypes.data, prepared.n, 1, self.layer_stride,
                          self.block_stride, self.num_gpu_blocks, prepared.n, 0, 1,
                          prepared.staging.data_ptr(), prepared.staging.numel(), _lib.KVC_SWAP_STAGED,
                          prepared.stream.cuda_stream, prepared.stream.cuda_stream))

    def _submit_host_rows(self, bounce: HostBounce, prepared: "PreparedSwap", layer_idx: int,
                          to_pool: bool, after: Optional[torch.cuda.Event]) -> int:
        """Queue the rows of one layer between its bounce region and their host
        blocks (the mover's thread waits for `after` first); returns the ticket."""
        with torch.cuda.device(self.device):
            ticket = _lib.lib().kvc_row_mover_submit(
                bounce.row_mover(self.host_copy_threads, self.host_wait_timeout),
                after.cuda_event if after is not None else None,
                self._host_pool.ptr, self.num_host_blocks, self.num_layers * self.block_stride,
                layer_idx * self.block_stride, bounce.slot_ptr(layer_idx), prepared.host_ids.ctypes.data,
                prepared.n, self.block_stride, 1 if to_pool else 0)
        if ticket < 0:
            _lib.check(int(ticket))
        return int(ticket)

    async def _host_rows_done(self, bounce: HostBounce, ticket: int) -> None:
        """Return once the mover has finished `ticket` (and every job before it)."""
        lib = _lib.lib()
        if lib.kvc_row_mover_done(bounce.mover, ticket) == 1:
            _lib.check(lib.kvc_row_mover_wait(bounce.mover, ticket))       # returns at once: picks up errors
        else:
            _lib.check(await asyncio.to_thread(lib.kvc_row_mover_wait, bounce.mover, ticket))

    async def _doorbell(self, doorbell, layer_idx: int) -> None:
        """Take one token from `doorbell`, giving up after `host_wait_timeout`. A token
        that is there is taken at once. Otherwise the wait blocks on the queue in a
        helper thread, in slices of 50 ms so that a closing worker is not held up:
        the reference polls with `asyncio.sleep(1e-5)` (kv_worker.py:279-281), which
        an event loop on epoll rounds up to a millisecond per poll."""
        try:
            doorbell.get_nowait()
            return
        except queue.Empty:
            pass
        deadline = None if self.host_wait_timeout is None else time.monotonic() + self.host_wait_timeout

        def take() -> bool:
            while True:
                left = 0.05 if deadline is None else min(0.05, deadline - time.monotonic())
                if left <= 0:
                    return False
                try:
                    doorbell.get(True, left)
                    return True
                except queue.Empty:
                    if getattr(self, "_closing", False):
                        return False

        if not await asyncio.to_thread(take):
            raise TimeoutError(f"no doorbell for layer {layer_idx} within {self.host_wait_timeout} s: "
                               "the model side has stopped posting layers")

    async def save_kv_blocks_to_host(self, block_mappings: Sequence[BlockMapping],
                                     stream: torch.cuda.Stream) -> None:
        """GPU->Host (kv_worker.py:272-295). With a handle: per layer, wait for the
        model's doorbell, make `stream` wait for `post_events[layer]`, then save
        that layer of every mapped block. The mappings are flattened, checked and
        uploaded once, before the first layer."""
        handle = self.kv_worker_handle
        if handle is None:
            self.save_kv_blocks_to_host_nowait(block_mappings, stream)
        elif len(block_mappings) > 0:
            prepared = self.prepare_swap("out", block_mappings, stream)
            bounce = self._bounce_for(prepared)
            self.last_copy_went_through_host_bounce = bounce is not None
            if bounce is not None:
                self.last_copy_swap_mode = _lib.KVC_SWAP_STAGED     # one dense copy per layer
            tickets: List[int] = []                 # per layer: its rows' job in the mover
            landed: List[torch.cuda.Event] = []     # per layer: the layer sits in its bounce region
            try:
                for layer_idx in range(self.num_layers):
                    await self._doorbell(handle.kv_queue, layer_idx)
                    if handle.sync == "events":
                        stream.wait_event(handle.post_events[layer_idx])
                    # sync == "host": the token was sent after the layer's write had completed
                    if bounce is None:
                        self.swap_prepared_layers(prepared, layer_idx, layer_idx + 1)
                        self.last_copy_swap_mode = _lib.last_swap_mode()
                    else:
                        if layer_idx >= bounce.slots:       # the region's earlier rows must have left it
                            await self._host_rows_done(bounce, tickets[layer_idx - bounce.slots])
                        self._swap_layer_through_bounce(prepared, layer_idx, bounce.slot_ptr(layer_idx))
                        landed.append(torch.cuda.Event())
                        landed[-1].record(stream)
                        tickets.append(self._submit_host_rows(bounce, prepared, layer_idx, True, landed[-1]))
                    await asyncio.sleep(0)  # let other tasks of the loop run
            finally:
                if bounce is not None:
                    try:
                        if tickets:
                            await self._host_rows_done(bounce, tickets[-1])
                    finally:
                        bounce.busy = False
        await asyncio.to_thread(stream.synchronize)

    async def load_kv_blocks_from_host(self, block_mappings: Sequence[BlockMapping],
                                       stream: torch.cuda.Stream) -> None:
        """Host->GPU (kv_worker.py:249-270). With a handle: after each layer's
        copies are enqueued, record `pre_events[layer]` on `stream` and ring the
        model's doorbell."""
        handle = self.kv_worker_handle
        if handle is None:
            self.load_kv_blocks_from_host_nowait(block_mappings, stream)
        elif len(block_mappings) > 0:
            prepared = self.prepare_swap("in", block_mappings, stream)
            bounce = self._bounce_for(prepared)
            self.last_copy_went_through_host_bounce = bounce is not None
            if bounce is not None:
                self.last_copy_swap_mode = _lib.KVC_SWAP_STAGED
            tickets: List[int] = []                    # per layer: the job that fills its bounce region
            region_read: List[torch.cuda.Event] = []   # per layer: the GPU has taken the region's rows
            try:
                if bounce is not None:
                    # host threads fill the regions ahead of the GPU: the first ones now, region
                    # l % slots again for layer l + slots once the GPU has read layer l from it
                    for ahead in range(min(bounce.slots, self.num_layers)):
                        tickets.append(self._submit_host_rows(bounce, prepared, ahead, False, None))
                for layer_idx in range(self.num_layers):
                    if bounce is None:
                        self.swap_prepared_layers(prepared, layer_idx, layer_idx + 1)
                        self.last_copy_swap_mode = _lib.last_swap_mode()
                    else:
                        await self._host_rows_done(bounce, tickets[layer_idx])
                        self._swap_layer_through_bounce(prepared, layer_idx, bounce.slot_ptr(layer_idx))
                        region_read.append(torch.cuda.Event())
                        region_read[-1].record(stream)
                        if layer_idx + bounce.slots < self.num_layers:
                            tickets.append(self._submit_host_rows(bounce, prepared, layer_idx + bounce.slots,
                                                                  False, region_read[-1]))
                    await asyncio.sleep(0)
                    handle.pre_events[layer_idx].record(stream)
                    if handle.sync == "events":
                        handle.model_queue.put(b"")
                    else:
                        handle.ring_when_done(handle.pre_events[layer_idx], handle.model_queue)
            finally:
                if bounce is not None:
                    try:
                        if tickets:                      # after an error: let the queued jobs come to rest
                            await self._host_rows_done(bounce, tickets[-1])
                        if region_read:
                            await asyncio.to_thread(region_read[-1].synchronize)
                    finally:
                        bounce.busy = False
        await asyncio.to_thread(stream.synchronize)

    # ----------------------------------------------------------------- disk legs
    def _require_disk(self) -> None:
        if self.disk_tier is None:
            raise ValueError("no disk KV cache configured (num_disk_blocks == 0)")

    def load_kv_blocks_from_disk_sync(self, block_mappings: Sequence[BlockMapping]) -> None:
        """host[dst] = disk[src] for every layer (kv_worker.py:229-237)."""
        if len(block_mappings) == 0:
            return
        self._require_disk()
        src, dst = flatten_block_mappings(block_mappings)
        self.disk_tier.load_blocks(self.host_kv_caches, src, dst)

    def save_kv_blocks_to_disk_sync(self, block_mappings: Sequence[BlockMapping]) -> None:
        """disk[dst] = host[src] for every layer (kv_worker.py:239-247)."""
        if len(block_mappings) == 0:
            return
        self._require_disk()
        src, dst = flatten_block_mappings(block_mappings)
        self.disk_tier.save_blocks(self.host_kv_caches, src, dst)

    # ---------------------------------------------------------------- dispatcher
    async def _copy_kv_gpu_to_host(self, block_mappings):
        await self.save_kv_blocks_to_host(block_mappings, self.dtoh_stream)

    async def _copy_kv_host_to_gpu(self, block_mappings):
        await self.load_kv_blocks_from_host(block_mappings, self.htod_stream)

    async def _copy_kv_host_to_disk(self, block_mappings):
        await asyncio.to_thread(self.save_kv_blocks_to_disk_sync, block_mappings)

    async def _copy_kv_disk_to_host(self, block_mappings):
        await asyncio.to_thread(self.load_kv_blocks_from_disk_sync, block_mappings)

    async def copy_kv(self, block_mappings: Sequence[BlockMapping], src: Device, dst: Device) -> None:
        key = (src, dst)
        if key not in self.COPY_KV_OP_MAP:
            raise ValueError(f"Unsupported copy direction: {src} -> {dst}")
        await self.COPY_KV_OP_MAP[key](block_mappings)

    def copy_kv_sync(self, block_mappings: Sequence[BlockMapping], src: Device, dst: Device) -> None:
        """`copy_kv` for callers without an event loop; returns when the copy is complete."""
        key = (src, dst)
        if key not in self.COPY_KV_OP_MAP:
            raise ValueError(f"Unsupported copy direction: {src} -> {dst}")
        if key == (Device.GPU, Device.Host):
            self.save_kv_blocks_to_host_nowait(block_mappings)
            self.dtoh_stream.synchronize()
        elif key == (Device.Host, Device.GPU):
            self.load_kv_blocks_from_host_nowait(block_mappings)
            self.htod_stream.synchronize()
        elif key == (Device.Host, Device.Disk):
            self.save_kv_blocks_to_disk_sync(block_mappings)
        else:
            self.load_kv_blocks_from_disk_sync(block_mappings)

    def close(self) -> None:
        self._closing = True      # a doorbell wait in a helper thread ends at its next slice
        with torch.cuda.device(self.device):
            torch.cuda.synchronize()
        self.host_kv_caches_tensor = None
        self.host_kv_caches = None
        self.disk_kv_caches = None
        if self.disk_tier is not None:
            self.disk_tier.close()
            self.disk_tier = None
        for direction, bounce in self._bounce.items():   # first: its mover still writes into the pool
            if bounce is not None:
                bounce.close(cancel=True)     # a job still waiting for an event is given up, not waited for
                self._bounce[direction] = None
        self._host_pool.close()
        self._staging = {}
        # let go of the pool now: the direction table holds bound methods, so the
        # worker is part of a reference cycle and would otherwise keep tens of GiB
        # of HBM alive until the cycle collector runs
        self.gpu_kv_caches = None
        self.COPY_KV_OP_MAP = {}
        # events and id bounce buffers the library kept for this thread
        _lib.check(_lib.lib().kvc_thread_release())

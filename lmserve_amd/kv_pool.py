"""Pool sizing, the layer-sync handle and its hand-over to a second process.

Host-side mirrors of the pieces that decide what the data-movement kernels are
handed:

* `plan_cache` / `allocate_kv_caches` -- the pool arithmetic and layout of
  `ModelWorker.init_cache` (runtime/worker/llm_worker/model_worker.py:200-228,
  :278-281).
* `KVWorkerHandle` / `LayerSyncHooks` -- the per-layer event + queue protocol
  between the model's forward pass and the swap engine
  (model_worker.py:232-276, kv_worker.py:25-30), with `torch.cuda.Event`
  in place of pycuda events.
"""
from __future__ import annotations

import queue
from dataclasses import dataclass, field
from typing import Any, Iterable, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class CachePlan:
    kv_block_size: int      # bytes of K (or V) of one block of one layer
    num_gpu_blocks: int
    num_host_blocks: int
    num_disk_blocks: int


def plan_cache(gpu_cache_size: int, host_cache_size: int, disk_cache_size: int, num_layers: int,
               num_kv_heads: int, head_dim: int, block_size: int, dtype: torch.dtype) -> CachePlan:
    """Blocks per tier from byte budgets (model_worker.py:214-219, :278-281)."""
    dtype_byte = torch.finfo(dtype).bits // 8
    kv_block_size = block_size * num_kv_heads * head_dim * dtype_byte
    per_block = num_layers * 2 * kv_block_size
    return CachePlan(kv_block_size, int(gpu_cache_size) // per_block,
                     int(host_cache_size) // per_block, int(disk_cache_size) // per_block)


def allocate_kv_caches(num_layers: int, num_gpu_blocks: int, block_size: int, num_kv_heads: int,
                       head_dim: int, dtype: torch.dtype, device="cuda") -> torch.Tensor:
    """The pool `[L, num_gpu_blocks, 2, block_size, H, D]`, uninitialised
    (model_worker.py:221-228)."""
    return torch.empty(num_layers, num_gpu_blocks, 2, block_size, num_kv_heads, head_dim,
                       dtype=dtype, device=device)


@dataclass
class KVWorkerHandle:
    """Per-layer events and the two doorbell queues shared by the model's
    forward pass and the swap engine (kv_worker.py:25-30).

    pre_events[l]  recorded by the swap engine once layer l has been loaded
                   into the pool; the model waits on it before layer l.
    post_events[l] recorded by the model after layer l's attention (its K/V
                   write included); the swap engine waits on it before saving
                   layer l.
    A queue token accompanies every record, so the waiting side only looks at
    an event that has been recorded for this step.

    sync = "events" (the reference's protocol): both sides hold the SAME events
    (one process, or interprocess events opened from IPC handles) and order
    their streams with GPU-side event waits; a token only says "the event has
    been recorded".
    sync = "host": for two processes on machines whose HIP runtime cannot export
    event handles (it builds them on `hipHostRegister`). Events stay local to
    the process that records them; a token is sent only once the recorded work
    has COMPLETED (a notifier thread waits for the local event first), so
    receiving the token is the ordering and no cross-process event wait exists.
    `pre_events` / `post_events` are then this process's own events.
    """
    pre_events: List[Any]
    post_events: List[Any]
    model_queue: Any = field(default_factory=queue.Queue)
    kv_queue: Any = field(default_factory=queue.Queue)
    sync: str = "events"
    host_wait_timeout: Optional[float] = 30.0    # seconds a notifier thread waits for one event; None = forever
    _notifier: Any = field(default=None, repr=False, compare=False)

    @classmethod
    def create(cls, num_layers: int, interprocess: bool = False, mp_context=None,
               sync: str = "events") -> "KVWorkerHandle":
        """Events and doorbells for one process (threads: `queue.Queue`) or, with
        `interprocess=True`, for two (`multiprocessing` queues of `mp_context`,
        default the spawn context, model_worker.py:232-252). With sync="events"
        the events are created exportable as IPC handles; with sync="host" they
        are ordinary events of this process."""
        if sync not in ("events", "host"):
            raise ValueError("sync must be 'events' or 'host'")

        def events():
            return [torch.cuda.Event(enable_timing=False, interprocess=interprocess and sync == "events")
                    for _ in range(num_layers)]
        if not interprocess:
            return cls(events(), events(), sync=sync)
        import multiprocessing
        ctx = mp_context or multiprocessing.get_context("spawn")
        return cls(events(), events(), ctx.Queue(), ctx.Queue(), sync)

    def ring_when_done(self, event, doorbell) -> None:
        """sync="host": put a token on `doorbell` once `event` has completed, in
        the order of the calls (one notifier thread per handle and process).
        Raises `TimeoutError` once an earlier event was given up after
        `host_wait_timeout` seconds."""
        if self._notifier is None:
            self._notifier = _Notifier(self.host_wait_timeout)
        self._notifier.submit(event, doorbell)

    def close(self) -> None:
        if self._notifier is not None:
            self._notifier.stop()
            self._notifier = None


class _Notifier:
    """A thread that waits for events in submission order and rings a doorbell
    after each (host-signalled layer protocol). No wait is unbounded: an event
    that has not completed after `timeout` seconds is given up (its doorbell is
    NOT rung, so the other side's own timeout fires rather than a false "done"),
    the jobs queued behind it are dropped the same way, and `failed` says so.
    `stop()` abandons whatever is still waiting."""

    def __init__(self, timeout: Optional[float] = 30.0, poll: float = 2e-5):
        import threading
        self.jobs: "queue.Queue" = queue.Queue()
        self.timeout, self.poll = timeout, poll
        self.failed: Optional[str] = None
        self._stopping = threading.Event()
        self.thread = threading.Thread(target=self._run, name="kvc-layer-doorbell", daemon=True)
        self.thread.start()

    def submit(self, event, doorbell) -> None:
        if self.failed is not None:
            raise TimeoutError(self.failed)
        self.jobs.put((event, doorbell))

    def _wait(self, event) -> bool:
        import time
        deadline = None if self.timeout is None else time.monotonic() + self.timeout
        while not event.query():
            if self._stopping.is_set() or (deadline is not None and time.monotonic() > deadline):
                return False
            time.sleep(self.poll)
        return True

    def _run(self) -> None:
        while True:
            job = self.jobs.get()
            if job is None:
                return
            event, doorbell = job
            if self.failed is not None or self._stopping.is_set():
                continue                      # drained, not rung
            if self._wait(event):
                doorbell.put(b"")
            elif not self._stopping.is_set():
                self.failed = f"an event of the layer protocol was not reached within {self.timeout} s"

    def stop(self) -> None:
        self._stopping.set()
        self.jobs.put(None)
        self.thread.join(timeout=10)


class LayerSyncHooks:
    """Model-side half of the protocol (model_worker.py:254-276).

    `pre(i)` / `post(i)` are to be called around attention layer `i` on the
    stream the model runs on (`attach` registers them as forward hooks on a
    list of modules). The two flags mirror the RPC's `wait_before_execute` /
    `record_after_execute` (proto/worker.proto:49-54).
    """

    def __init__(self, handle: KVWorkerHandle):
        self.handle = handle
        self.enable_wait_before_execute = False
        self.enable_record_after_execute = False
        self.timeout: Optional[float] = None   # seconds to wait for a doorbell; None = forever

    def pre(self, layer_idx: int, stream: Optional[torch.cuda.Stream] = None) -> None:
        if self.enable_wait_before_execute:
            self.handle.model_queue.get(timeout=self.timeout)
            if self.handle.sync == "events":
                (stream or torch.cuda.current_stream()).wait_event(self.handle.pre_events[layer_idx])
            # sync == "host": the token was sent after the layer's load had completed

    def post(self, layer_idx: int, stream: Optional[torch.cuda.Stream] = None) -> None:
        if self.enable_record_after_execute:
            event = self.handle.post_events[layer_idx]
            event.record(stream or torch.cuda.current_stream())
            if self.handle.sync == "events":
                self.handle.kv_queue.put(b"")   # doorbell: layer's K/V may be saved
            else:
                self.handle.ring_when_done(event, self.handle.kv_queue)

    def attach(self, attention_layers: Iterable[torch.nn.Module]) -> None:
        for i, layer in enumerate(attention_layers):
            layer.register_forward_pre_hook(lambda mod, inp, i=i: self.pre(i))
            layer.register_forward_hook(lambda mod, inp, out, i=i: self.post(i))


@dataclass
class KVWorkerParams:
    """What the model worker hands to the KV-worker process it starts: the pool
    as an IPC storage handle, its geometry, the per-layer events as IPC handles
    and the two doorbell queues (kv_worker.py:33-45 of the reference; built at
    model_worker.py:278-306, consumed at kv_worker.py:97-153). Picklable, so it
    travels as an argument of `multiprocessing.Process` (spawn start method, as
    cli.py:115-121 and :282 of the reference use)."""
    kv_cache_metadata: Tuple[Any, ...]
    num_layers: int
    num_gpu_blocks: int
    num_host_blocks: int
    num_disk_blocks: int
    disk_kv_cache_file: str
    dtype: torch.dtype
    pre_event_handles: List[bytes]
    post_event_handles: List[bytes]
    model_queue: Any
    kv_queue: Any
    sync: str = "events"   # "host": no event handles travel (see KVWorkerHandle)


IPC_SEGMENT_LIMIT = 2 << 30


def allocator_segment_bytes(tensor: torch.Tensor, snapshot=None) -> Optional[int]:
    """Size of the caching-allocator segment that holds `tensor`'s storage, or None
    when the snapshot does not list it. An IPC handle of a tensor covers its whole
    segment, not just the tensor."""
    address = tensor.untyped_storage().data_ptr()
    for segment in (snapshot if snapshot is not None else torch.cuda.memory_snapshot()):
        if segment["address"] <= address < segment["address"] + segment["total_size"]:
            return int(segment["total_size"])
    return None


def check_ipc_segment(kv_caches: torch.Tensor, snapshot=None, limit: int = IPC_SEGMENT_LIMIT) -> None:
    """Refuse to export a pool whose allocator segment is `limit` bytes or more:
    opening such a handle in another process does not return on this platform.
    Pools of that size are served by a `KVWorker` in the model's own process."""
    size = allocator_segment_bytes(kv_caches, snapshot)
    if size is None:
        size = kv_caches.untyped_storage().nbytes()
    if size >= limit:
        raise ValueError(
            f"the pool sits in an allocator segment of {size} bytes; a shared allocation must stay under "
            f"{limit} bytes on this platform. Give the pool a segment of its own below that size "
            "(torch.cuda.empty_cache() before allocating it), or run the KV worker in this process "
            "(KVWorker(kv_caches, ...)) instead of exporting the pool")


def make_kv_worker_params(kv_caches: torch.Tensor, handle: KVWorkerHandle, num_host_blocks: int,
                          num_disk_blocks: int = 0, disk_kv_cache_file: str = "") -> KVWorkerParams:
    """Export the pool and the handle's events for another process on the same GPU
    (model_worker.py:278-306). `handle` must hold interprocess events and queues
    that cross processes (`multiprocessing` queues). The pool tensor must stay
    alive in this process for as long as the other process maps it."""
    if not kv_caches.is_cuda or not kv_caches.is_contiguous() or kv_caches.dim() < 3:
        raise ValueError("kv_caches must be a contiguous [L, num_gpu_blocks, ...] tensor on the GPU")
    if kv_caches.storage_offset() != 0 or \
            kv_caches.untyped_storage().nbytes() != kv_caches.numel() * kv_caches.element_size():
        raise ValueError("kv_caches must own its storage (the other process maps the whole storage)")
    check_ipc_segment(kv_caches)
    return KVWorkerParams(
        kv_cache_metadata=kv_caches.untyped_storage()._share_cuda_(),
        num_layers=kv_caches.shape[0], num_gpu_blocks=kv_caches.shape[1],
        num_host_blocks=int(num_host_blocks), num_disk_blocks=int(num_disk_blocks),
        disk_kv_cache_file=disk_kv_cache_file, dtype=kv_caches.dtype,
        pre_event_handles=[e.ipc_handle() for e in handle.pre_events] if handle.sync == "events" else [],
        post_event_handles=[e.ipc_handle() for e in handle.post_events] if handle.sync == "events" else [],
        model_queue=handle.model_queue, kv_queue=handle.kv_queue, sync=handle.sync)


def open_kv_worker_params(params: KVWorkerParams, device: int = 0):
    """The receiving side (kv_worker.py:104-108, :140-153): map the pool from its
    IPC handle as `[L, num_gpu_blocks, block_elems]` and open the events. Returns
    `(gpu_kv_caches, KVWorkerHandle)`."""
    device = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
    with torch.cuda.device(device):
        storage = torch.UntypedStorage._new_shared_cuda(*params.kv_cache_metadata)
        gpu_kv_caches = torch.empty(0, dtype=params.dtype, device=device)
        gpu_kv_caches.set_(storage)
        gpu_kv_caches = gpu_kv_caches.view(params.num_layers, params.num_gpu_blocks, -1)
        if params.sync == "events":
            pre = [torch.cuda.Event.from_ipc_handle(device, h) for h in params.pre_event_handles]
            post = [torch.cuda.Event.from_ipc_handle(device, h) for h in params.post_event_handles]
        else:   # host-signalled: this process records events of its own
            pre = [torch.cuda.Event(enable_timing=False) for _ in range(params.num_layers)]
            post = [torch.cuda.Event(enable_timing=False) for _ in range(params.num_layers)]
    return gpu_kv_caches, KVWorkerHandle(pre, post, params.model_queue, params.kv_queue, params.sync)

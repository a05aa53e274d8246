"""Pool sizing and the layer-sync handle.

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
from typing import Any, Iterable, List, Optional

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
    """
    pre_events: List[Any]
    post_events: List[Any]
    model_queue: Any = field(default_factory=queue.Queue)
    kv_queue: Any = field(default_factory=queue.Queue)

    @classmethod
    def create(cls, num_layers: int, interprocess: bool = False) -> "KVWorkerHandle":
        def events():
            return [torch.cuda.Event(enable_timing=False, interprocess=interprocess)
                    for _ in range(num_layers)]
        return cls(events(), events())


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
            (stream or torch.cuda.current_stream()).wait_event(self.handle.pre_events[layer_idx])

    def post(self, layer_idx: int, stream: Optional[torch.cuda.Stream] = None) -> None:
        if self.enable_record_after_execute:
            self.handle.post_events[layer_idx].record(stream or torch.cuda.current_stream())
            self.handle.kv_queue.put(b"")   # doorbell: layer's K/V may be saved

    def attach(self, attention_layers: Iterable[torch.nn.Module]) -> None:
        for i, layer in enumerate(attention_layers):
            layer.register_forward_pre_hook(lambda mod, inp, i=i: self.pre(i))
            layer.register_forward_hook(lambda mod, inp, out, i=i: self.post(i))

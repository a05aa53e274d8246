"""A whole step's K/V write as ONE recordable sequence: index build + every layer.

The reference rebuilds its index tensors on the host for every step and uploads
them piecewise (`ModelWorker._make_inputs`,
runtime/worker/llm_worker/model_worker.py:310-455), then issues one write per
attention layer (models/llama.py:236-242, models/layers/attention.py:76-85).
Each of those launches moves a few MiB and is bound by launch latency, not by
HBM; what removes that cost is recording the step once into a hipGraph and
replaying it. For a recording to serve the NEXT step too, nothing in it may
depend on a host scalar of the step it was recorded for:

* the per-request scalars and the block tables live in device buffers of fixed
  CAPACITY (`max_requests`, `max_block_ids`); only their contents change;
* `kvc_build_write_index` is launched for the capacities and reads the step's
  own sizes on the device (padding requests have no new tokens; per-token
  entries beyond the step's tokens are -1);
* the per-layer writes run through a plan over those buffers that addresses
  the cache by the slot mapping the index build writes, sized for
  `max_tokens`; tokens with slot -1 are skipped.

`KVWriteStep` owns those buffers and plans. `set_requests` (or `set_arrays`)
packs a step on the host and uploads it with one copy; `build_index` and
`append` / `rotate_and_append` are the launches, eager or under stream capture.
"""
from __future__ import annotations

import struct
from typing import Optional, Sequence

import numpy as np
import torch

from .index_prep import InferInput
from .paged import BlockRuns, PagedKVWritePlan, build_write_index, max_block_runs
from .rotary import PagedRotaryWritePlan


class KVWriteStep:
    """Fixed-capacity index buffers of a step and the plans that write through them.

    num_kv_heads, head_dim, page_size, dtype: geometry of one layer of the pool
      `[num_pages, 2, page_size, H, D]`.
    max_requests, max_tokens, max_block_ids: capacities of a step (requests, new
      tokens over all requests, block-table entries over all requests).
    cos_sin_cache, num_heads: when given, `rotate_and_append` is available (the
      rotation fused with the write, one launch per layer).
    with_runs: also have the index build emit the step's block runs (`self.runs`).
    """

    def __init__(self, num_kv_heads: int, head_dim: int, page_size: int, dtype: torch.dtype, device,
                 max_requests: int, max_tokens: int, max_block_ids: int,
                 cos_sin_cache: Optional[torch.Tensor] = None, num_heads: int = 0,
                 with_runs: bool = False):
        self.device = torch.device(device)
        self.page_size = int(page_size)
        self.max_requests, self.max_tokens, self.max_block_ids = int(max_requests), int(max_tokens), int(max_block_ids)
        if min(self.max_requests, self.max_tokens, self.max_block_ids) < 1:
            raise ValueError("capacities must be positive")
        B, T, N = self.max_requests, self.max_tokens, self.max_block_ids
        # one device buffer and one pinned mirror: [input_lens | context_lens | num_blocks | kv_indices]
        self._packed = torch.zeros(3 * B + N, dtype=torch.int32, device=self.device)
        self._host = torch.zeros(3 * B + N, dtype=torch.int32, pin_memory=True)
        self._host_np = self._host.numpy()
        self._uploaded = torch.cuda.Event()
        self._upload_pending = False
        self.input_lens = self._packed[0:B]
        self.context_lens = self._packed[B:2 * B]
        self.num_blocks = self._packed[2 * B:3 * B]
        self.kv_indices = self._packed[3 * B:]
        i32 = dict(dtype=torch.int32, device=self.device)
        self.cu_seqlens_q = torch.zeros(B + 1, **i32)
        self.kv_indptr = torch.zeros(B + 1, **i32)
        self.kv_last_page_len = torch.zeros(B, **i32)
        # -1 = "no token here": valid content before the first index build
        self.batch_indices = torch.full((T,), -1, **i32)
        self.positions = torch.full((T,), -1, **i32)
        self.slot_mapping = torch.full((T,), -1, dtype=torch.int64, device=self.device)
        self.runs: Optional[BlockRuns] = None
        if with_runs:
            cap = max_block_runs(T, B, self.page_size)
            self.runs = BlockRuns(torch.zeros(cap, 4, **i32), torch.zeros(1, **i32), torch.zeros(B + 1, **i32))
        self._out = (self.cu_seqlens_q, self.kv_indptr, self.kv_last_page_len, self.batch_indices,
                     self.positions, self.slot_mapping) + ((self.runs,) if with_runs else ())
        self.plan = PagedKVWritePlan(self.batch_indices, self.positions, self.kv_indices, self.kv_indptr,
                                     self.kv_last_page_len, num_kv_heads, head_dim, page_size, dtype,
                                     slots=self.slot_mapping)
        self.rotary_plan = None
        if cos_sin_cache is not None:
            self.rotary_plan = PagedRotaryWritePlan(self.batch_indices, self.positions, self.kv_indices,
                                                    self.kv_indptr, self.kv_last_page_len, cos_sin_cache,
                                                    num_heads, num_kv_heads, head_dim, page_size,
                                                    slots=self.slot_mapping)
        self.num_tokens = 0       # of the step last packed (host-side knowledge)
        self.num_requests = 0

    # ------------------------------------------------------------------ host side
    def set_arrays(self, input_lens, context_lens, num_blocks, kv_indices) -> None:
        """Pack a step from per-request arrays in batch order (the caller has
        sorted them, model_worker.py:326-328) and the concatenated block tables,
        and upload it with one copy on the current stream. Raises `ValueError`
        when the step exceeds a capacity; nothing is uploaded then."""
        input_lens = np.asarray(input_lens, dtype=np.int32)
        context_lens = np.asarray(context_lens, dtype=np.int32)
        num_blocks = np.asarray(num_blocks, dtype=np.int32)
        kv_indices = np.asarray(kv_indices, dtype=np.int32)
        b = int(input_lens.shape[0])
        if context_lens.shape[0] != b or num_blocks.shape[0] != b:
            raise ValueError("input_lens, context_lens and num_blocks must have one entry per request")
        B, N = self.max_requests, self.max_block_ids
        tokens = int(input_lens.sum()) if b else 0
        if b > B or tokens > self.max_tokens or kv_indices.shape[0] > N:
            raise ValueError(f"step of {b} requests, {tokens} tokens, {kv_indices.shape[0]} block ids exceeds the "
                             f"capacities ({B}, {self.max_tokens}, {N})")
        if int(num_blocks.sum()) != kv_indices.shape[0]:
            raise ValueError("kv_indices must be the concatenation of the block tables")
        if self._upload_pending:
            self._uploaded.synchronize()      # the previous upload has read the pinned mirror
        h = self._host_np
        h[0:b] = input_lens
        h[b:B] = 0                            # padding requests: no new tokens
        h[B:B + b] = context_lens
        h[B + b:2 * B] = 0
        h[2 * B:2 * B + b] = num_blocks
        h[2 * B + b:3 * B] = 0
        h[3 * B:3 * B + kv_indices.shape[0]] = kv_indices
        with torch.cuda.device(self.device):
            self._packed.copy_(self._host, non_blocking=True)
            self._uploaded.record()
        self._upload_pending = True
        self.num_tokens, self.num_requests = tokens, b

    def set_requests(self, inputs: Sequence[InferInput]) -> list:
        """`set_arrays` from the scheduler's requests (proto/worker.proto:40-47),
        ordered by decreasing new-token count as the reference orders them
        (model_worker.py:326-328). Returns that order (indices into `inputs`)."""
        order = sorted(range(len(inputs)), key=lambda i: -inputs[i].input_len)
        reqs = [inputs[i] for i in order]
        tables: list = []
        for r in reqs:
            tables += r.block_ids
        tables_np = np.frombuffer(struct.pack(f"{len(tables)}i", *tables), dtype=np.int32) if tables \
            else np.empty(0, dtype=np.int32)
        self.set_arrays([r.input_len for r in reqs], [r.context_len for r in reqs],
                        [len(r.block_ids) for r in reqs], tables_np)
        return order

    # ------------------------------------------------------------------ launches
    def build_index(self) -> None:
        """One launch on the current stream: every index tensor of the step that
        the buffers hold, written in place."""
        build_write_index(self.input_lens, self.context_lens, self.num_blocks, self.kv_indices,
                          self.page_size, self.max_tokens, out=self._out)

    def append(self, key: torch.Tensor, value: torch.Tensor, paged_kv_cache: torch.Tensor) -> None:
        """One layer's write; `key` / `value` hold `max_tokens` rows, of which the
        step's first `num_tokens` are written."""
        self.plan.append(key, value, paged_kv_cache)

    def rotate_and_append(self, query, key, value, paged_kv_cache, query_out=None, key_out=None):
        if self.rotary_plan is None:
            raise ValueError("this step was made without a cos/sin table")
        return self.rotary_plan.run(query, key, value, paged_kv_cache, query_out=query_out, key_out=key_out)

    def capture(self, keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                caches: Sequence[torch.Tensor], queries: Optional[Sequence[torch.Tensor]] = None,
                query_outs: Optional[Sequence[torch.Tensor]] = None) -> "torch.cuda.CUDAGraph":
        """Record `build_index` and one write per layer into a hipGraph. The tensors
        are the fixed buffers the model writes its projections into before every
        replay (`max_tokens` rows each). With `queries` the fused rotation runs in
        place of the plain write. One eager pass runs first (outside the capture)."""
        def body():
            self.build_index()
            for l, (k, v, c) in enumerate(zip(keys, values, caches)):
                if queries is None:
                    self.append(k, v, c)
                else:
                    self.rotate_and_append(queries[l], k, v, c,
                                           query_out=query_outs[l] if query_outs is not None else None)
        with torch.cuda.device(self.device):
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                body()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # thread-local capture: a KV worker's threads (row mover, notifier) may
            # query events and enqueue copies on their own streams meanwhile
            with torch.cuda.graph(graph, capture_error_mode="thread_local"):
                body()
        return graph

"""Host-side construction of the index tensors the K/V write consumes.

Mirrors the part of `ModelWorker._make_inputs`
(runtime/worker/llm_worker/model_worker.py:310-455) that decides WHERE each new
token's K/V lands, and the slot rule of the Rust side
(runtime/src/llm_engine/scheduler.rs:453-541 with
runtime/src/llm_engine/block_manager.rs:241-273):

    block_ids covers tokens [0, context_len); the new tokens of a request sit
    at positions [filled_token_len, context_len);
    slot(pos) = block_ids[pos // block_size] * block_size + pos % block_size.

The list building is pure Python/NumPy and runs without a GPU; `to_device`
moves the results to the GPU and finishes with the device-side
`get_seq_lens` / `get_batch_indices_positions` calls.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch


@dataclass
class InferInput:
    """proto/worker.proto:40-47 of the reference."""
    seq_id: int
    input_ids: List[int]
    input_len: int
    filled_token_len: int
    context_len: int
    block_ids: List[int] = field(default_factory=list)


@dataclass
class KVIndexInputs:
    """Host copies (NumPy int32) of what `_make_inputs` uploads, plus the
    per-token slot mapping derived from them."""
    position_ids: np.ndarray          # [nnz]   model_worker.py:346
    cu_seqlens_q: np.ndarray          # [B+1]   model_worker.py:362-365
    prefill_input_len: int            #         model_worker.py:335-337
    kv_block_indices: np.ndarray      # [sum blocks] model_worker.py:404
    kv_block_indptrs: np.ndarray      # [B+1]   model_worker.py:410-413
    kv_last_block_lens: np.ndarray    # [B]     model_worker.py:406-407
    batch_indices: np.ndarray         # [nnz]   closed form of get_batch_indices_positions
    positions: np.ndarray             # [nnz]
    slot_mapping: np.ndarray          # [nnz] int64
    order: List[int]                  # request order after the sort (indices into the input list)


def make_kv_index_inputs(inputs: Sequence[InferInput], page_size: int) -> KVIndexInputs:
    """Build the index arrays for one step.

    Requests are ordered by decreasing `input_len` with a stable sort, so
    prefill chunks come before decode tokens (model_worker.py:326-328).
    """
    order = sorted(range(len(inputs)), key=lambda i: -inputs[i].input_len)
    position_ids: List[int] = []
    seqlens_q: List[int] = []
    prefill_input_len = 0
    kv_block_indices: List[int] = []
    num_blocks_per_seq: List[int] = []
    kv_last_block_lens: List[int] = []
    batch_indices: List[int] = []
    slots: List[int] = []
    for b, i in enumerate(order):
        data = inputs[i]
        seqlen_q = int(data.input_len)
        if seqlen_q > 1:
            prefill_input_len += seqlen_q
        seqlen_k = int(data.context_len)
        new_positions = list(range(int(data.filled_token_len), seqlen_k))
        if len(new_positions) != seqlen_q:
            raise ValueError(
                f"request {data.seq_id}: context_len - filled_token_len = {len(new_positions)} "
                f"differs from input_len = {seqlen_q}")
        need_blocks = (seqlen_k + page_size - 1) // page_size
        if len(data.block_ids) < need_blocks:
            raise ValueError(
                f"request {data.seq_id}: {len(data.block_ids)} blocks cannot hold "
                f"{seqlen_k} tokens of {page_size}")
        position_ids += new_positions
        seqlens_q.append(seqlen_q)
        kv_block_indices += [int(x) for x in data.block_ids]
        num_blocks_per_seq.append(len(data.block_ids))
        kv_last_block_lens.append((seqlen_k - 1) % page_size + 1)
        batch_indices += [b] * seqlen_q
        slots += [int(data.block_ids[p // page_size]) * page_size + p % page_size
                  for p in new_positions]
    i32 = np.int32
    return KVIndexInputs(
        position_ids=np.asarray(position_ids, dtype=i32),
        cu_seqlens_q=np.cumsum([0] + seqlens_q).astype(i32),
        prefill_input_len=prefill_input_len,
        kv_block_indices=np.asarray(kv_block_indices, dtype=i32),
        kv_block_indptrs=np.cumsum([0] + num_blocks_per_seq).astype(i32),
        kv_last_block_lens=np.asarray(kv_last_block_lens, dtype=i32),
        batch_indices=np.asarray(batch_indices, dtype=i32),
        positions=np.asarray(position_ids, dtype=i32),
        slot_mapping=np.asarray(slots, dtype=np.int64),
        order=order,
    )


@dataclass
class DeviceKVIndexInputs:
    """Device tensors in the shape of the reference's `InputParams`
    (runtime/worker/llm_worker/models/input_params.py:9-23), write-related fields only."""
    position_ids: torch.Tensor
    cu_seqlens_q: torch.Tensor
    prefill_input_len: int
    batch_indices: torch.Tensor
    positions: torch.Tensor
    kv_block_indices: torch.Tensor
    kv_block_indptrs: torch.Tensor
    kv_last_block_lens: torch.Tensor
    slot_mapping: Optional[torch.Tensor] = None


def to_device(host: KVIndexInputs, page_size: int, device="cuda",
              with_slot_mapping: bool = True) -> DeviceKVIndexInputs:
    """Upload the index arrays and derive `batch_indices` / `positions` ON the
    device from `cu_seqlens_q` and the page table, the way the reference does
    (model_worker.py:425-433)."""
    from .paged import get_batch_indices_positions, get_seq_lens

    def up(a: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(np.ascontiguousarray(a)).to(device, non_blocking=True)

    cu = up(host.cu_seqlens_q)
    indptr = up(host.kv_block_indptrs)
    last = up(host.kv_last_block_lens)
    nnz = int(host.cu_seqlens_q[-1]) if len(host.cu_seqlens_q) else 0
    batch_indices, positions = get_batch_indices_positions(
        cu, get_seq_lens(indptr, last, page_size), nnz)
    return DeviceKVIndexInputs(
        position_ids=up(host.position_ids),
        cu_seqlens_q=cu,
        prefill_input_len=host.prefill_input_len,
        batch_indices=batch_indices,
        positions=positions,
        kv_block_indices=up(host.kv_block_indices),
        kv_block_indptrs=indptr,
        kv_last_block_lens=last,
        slot_mapping=up(host.slot_mapping) if with_slot_mapping else None,
    )


def to_device_one_launch(inputs: Sequence[InferInput], page_size: int, device="cuda",
                         with_slot_mapping: bool = True) -> DeviceKVIndexInputs:
    """The same device tensors as `to_device(make_kv_index_inputs(...))`, but the
    host only packs four small arrays (new-token count, context length and
    block-table length per request, and the concatenated block tables); prefix
    sums, positions, request indices and slots are computed on the device in a
    single launch. Requests are ordered as `make_kv_index_inputs` orders them."""
    from .paged import build_write_index

    order = sorted(range(len(inputs)), key=lambda i: -inputs[i].input_len)
    reqs = [inputs[i] for i in order]
    packed = np.empty((3, len(reqs)), dtype=np.int32)
    tables: List[int] = []
    prefill_input_len = 0
    for b, r in enumerate(reqs):
        packed[0, b] = r.input_len
        packed[1, b] = r.context_len
        packed[2, b] = len(r.block_ids)
        tables += r.block_ids
        if r.input_len > 1:
            prefill_input_len += int(r.input_len)
    nnz = int(packed[0].sum()) if len(reqs) else 0
    dev_packed = torch.from_numpy(packed).to(device, non_blocking=True)
    # a Python list of tens of thousands of ints converts about three times faster
    # through struct.pack than through np.asarray
    tables_np = np.frombuffer(struct.pack(f"{len(tables)}i", *tables), dtype=np.int32) if tables \
        else np.empty(0, dtype=np.int32)
    kv_indices = torch.from_numpy(tables_np.copy()).to(device, non_blocking=True)
    cu, indptr, last, batch_indices, positions, slots = build_write_index(
        dev_packed[0], dev_packed[1], dev_packed[2], kv_indices, page_size, nnz, with_slot_mapping)
    return DeviceKVIndexInputs(position_ids=positions, cu_seqlens_q=cu,
                               prefill_input_len=prefill_input_len, batch_indices=batch_indices,
                               positions=positions, kv_block_indices=kv_indices,
                               kv_block_indptrs=indptr, kv_last_block_lens=last, slot_mapping=slots)

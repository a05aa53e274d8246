"""Page-table addressed K/V write and its index preparation.

Drop-in for the three third-party calls on the reference's live write path
(flashinfer-python 0.3.1.post1, pinned in runtime/worker/uv.lock:148-149):
`append_paged_kv_cache` as called at
runtime/worker/llm_worker/models/layers/attention.py:76-85, and
`get_seq_lens` / `get_batch_indices_positions` as called at
runtime/worker/llm_worker/model_worker.py:425-433. Names, argument order and
tensor layouts are those calls'; the "NHD" single-tensor cache
`[num_pages, 2, page_size, H, D]` is the only layout the reference uses
(model_worker.py:65-66) and the only one served here.
"""
from __future__ import annotations

import ctypes
from typing import Tuple

import torch

from . import _lib
from .cache_ops import _inner_contiguous, _on_device_of, _require_gpu, _rows, _stream_of


_raw_stream = torch._C._cuda_getCurrentRawStream
_fast_entry = _lib.fast_entry


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    _require_gpu(t, name)
    if t.dtype != torch.int32:
        raise TypeError(f"{name} must be int32 (got {t.dtype})")
    return t if t.is_contiguous() else t.contiguous()


def get_seq_lens(kv_indptr: torch.Tensor, kv_last_page_len: torch.Tensor,
                 page_size: int) -> torch.Tensor:
    """`seq_lens[b] = max(kv_indptr[b+1]-kv_indptr[b]-1, 0)*page_size + kv_last_page_len[b]`."""
    kv_indptr = _i32(kv_indptr, "kv_indptr")
    kv_last_page_len = _i32(kv_last_page_len, "kv_last_page_len")
    batch_size = kv_last_page_len.numel()
    if kv_indptr.numel() != batch_size + 1:
        raise ValueError("kv_indptr must have batch_size + 1 entries")
    seq_lens = torch.empty(batch_size, dtype=torch.int32, device=kv_indptr.device)
    with _on_device_of(kv_indptr):
        _lib.check(_lib.lib().kvc_get_seq_lens(
            kv_indptr.data_ptr(), kv_last_page_len.data_ptr(), batch_size, int(page_size),
            seq_lens.data_ptr(), _stream_of(kv_indptr)))
    return seq_lens


def get_batch_indices_positions(append_indptr: torch.Tensor, seq_lens: torch.Tensor,
                                nnz: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per appended token: the request it belongs to and its absolute position.

    For request `b` with `n_b = append_indptr[b+1]-append_indptr[b]` new tokens
    the j-th of them gets `batch_indices = b`, `positions = seq_lens[b] - n_b + j`.
    With the reference's inputs `seq_lens[b]` is the request's context length,
    so `positions` equals its `position_ids` (model_worker.py:346).
    """
    append_indptr = _i32(append_indptr, "append_indptr")
    seq_lens = _i32(seq_lens, "seq_lens")
    batch_size = seq_lens.numel()
    if append_indptr.numel() != batch_size + 1:
        raise ValueError("append_indptr must have batch_size + 1 entries")
    batch_indices = torch.empty(int(nnz), dtype=torch.int32, device=append_indptr.device)
    positions = torch.empty(int(nnz), dtype=torch.int32, device=append_indptr.device)
    with _on_device_of(append_indptr):
        _lib.check(_lib.lib().kvc_get_batch_indices_positions(
            append_indptr.data_ptr(), seq_lens.data_ptr(), batch_size, int(nnz),
            batch_indices.data_ptr(), positions.data_ptr(), _stream_of(append_indptr)))
    return batch_indices, positions


def _paged_common(append_key, append_value, batch_indices, positions, kv_indices, kv_indptr,
                  kv_last_page_len, kv_layout):
    if kv_layout != "NHD":
        raise ValueError(f"kv_layout {kv_layout!r} is not supported (the reference uses 'NHD')")
    batch_indices = _i32(batch_indices, "batch_indices")
    positions = _i32(positions, "positions")
    kv_indices = _i32(kv_indices, "kv_indices")
    kv_indptr = _i32(kv_indptr, "kv_indptr")
    kv_last_page_len = _i32(kv_last_page_len, "kv_last_page_len")
    if batch_indices.numel() != positions.numel():
        raise ValueError("batch_indices and positions differ in length")
    return batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len


def append_paged_kv_cache(
    append_key: torch.Tensor,
    append_value: torch.Tensor,
    batch_indices: torch.Tensor,
    positions: torch.Tensor,
    paged_kv_cache: torch.Tensor,
    kv_indices: torch.Tensor,
    kv_indptr: torch.Tensor,
    kv_last_page_len: torch.Tensor,
    kv_layout: str = "NHD",
) -> None:
    """Write token `i` to page `kv_indices[kv_indptr[b] + p // page_size]`, entry
    `p % page_size`, with `b = batch_indices[i]`, `p = positions[i]`.

    append_key, append_value: `[nnz, H, D]`; paged_kv_cache:
    `[num_pages, 2, page_size, H, D]` (one layer of the pool); index tensors
    int32 on the device. In place; returns None.
    """
    if isinstance(paged_kv_cache, (tuple, list)):
        raise ValueError("only the single-tensor NHD paged cache is supported")
    if kv_layout == "NHD" and isinstance(paged_kv_cache, torch.Tensor) and paged_kv_cache.is_cuda:
        fast = _fast_entry("append_paged")
        if fast is not None:
            # the common layouts are checked and launched from C++; 1 = not one of them:
            # the checks below then name what is wrong, or handle the rare layout
            dev = paged_kv_cache.device.index
            rc = fast(append_key, append_value, batch_indices, positions, paged_kv_cache, kv_indices,
                      kv_indptr, kv_last_page_len, dev, _raw_stream(dev))
            if rc == 0:
                return
            if rc < 0:
                _lib.check(rc)
    for t, n in ((append_key, "append_key"), (append_value, "append_value"),
                 (paged_kv_cache, "paged_kv_cache")):
        _require_gpu(t, n)
    batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len = _paged_common(
        append_key, append_value, batch_indices, positions, kv_indices, kv_indptr,
        kv_last_page_len, kv_layout)
    if paged_kv_cache.dim() != 5 or paged_kv_cache.shape[1] != 2:
        raise ValueError("paged_kv_cache must be [num_pages, 2, page_size, H, D]")
    if append_key.dtype != paged_kv_cache.dtype or append_value.dtype != paged_kv_cache.dtype:
        raise TypeError("append_key/append_value and paged_kv_cache must share one dtype")
    num_pages, _, page_size, H, D = paged_kv_cache.shape
    if not _inner_contiguous(paged_kv_cache):
        raise ValueError("every page of paged_kv_cache must be contiguous [2, page_size, H, D]")
    append_key, row, k_stride = _rows(append_key, "append_key")
    append_value, row_v, v_stride = _rows(append_value, "append_value")
    if row != H * D or row_v != H * D:
        raise ValueError("append_key/append_value rows do not match the cache's H*D")
    nnz = batch_indices.numel()
    if append_key.shape[0] < nnz or append_value.shape[0] < nnz:
        raise ValueError("fewer key/value rows than index entries")
    if nnz == 0 or row == 0 or num_pages == 0:
        return
    page_stride = paged_kv_cache.stride(0) if num_pages > 1 else 2 * page_size * row
    with _on_device_of(paged_kv_cache):
        _lib.check(_lib.lib().kvc_append_paged_kv_cache(
            append_key.data_ptr(), append_value.data_ptr(), batch_indices.data_ptr(),
            positions.data_ptr(), paged_kv_cache.data_ptr(), kv_indices.data_ptr(),
            kv_indptr.data_ptr(), kv_last_page_len.data_ptr(), nnz, kv_indptr.numel() - 1,
            kv_indices.numel(), H, D, page_size, k_stride, v_stride, page_stride, num_pages,
            paged_kv_cache.element_size(), _stream_of(paged_kv_cache)))


def append_paged_kv_cache_layers(
    append_key: torch.Tensor,
    append_value: torch.Tensor,
    batch_indices: torch.Tensor,
    positions: torch.Tensor,
    kv_caches: torch.Tensor,
    kv_indices: torch.Tensor,
    kv_indptr: torch.Tensor,
    kv_last_page_len: torch.Tensor,
    kv_layout: str = "NHD",
) -> None:
    """`append_paged_kv_cache` for every layer of the pool in one launch.

    append_key, append_value: `[L, nnz, H, D]` contiguous; kv_caches:
    `[L, num_pages, 2, page_size, H, D]` contiguous; one page table for all layers.
    """
    for t, n in ((append_key, "append_key"), (append_value, "append_value"),
                 (kv_caches, "kv_caches")):
        _require_gpu(t, n)
    batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len = _paged_common(
        append_key, append_value, batch_indices, positions, kv_indices, kv_indptr,
        kv_last_page_len, kv_layout)
    if kv_caches.dim() != 6 or kv_caches.shape[2] != 2 or not kv_caches.is_contiguous():
        raise ValueError("kv_caches must be contiguous [L, num_pages, 2, page_size, H, D]")
    if append_key.dtype != kv_caches.dtype or append_value.dtype != kv_caches.dtype:
        raise TypeError("append_key/append_value and kv_caches must share one dtype")
    L, num_pages, _, page_size, H, D = kv_caches.shape
    row = H * D
    if append_key.dim() != 4 or append_key.shape != append_value.shape \
            or append_key.shape[0] != L or append_key.shape[2] * append_key.shape[3] != row:
        raise ValueError("append_key/append_value must be [L, nnz, H, D] matching the pool")
    append_key = append_key.contiguous()
    append_value = append_value.contiguous()
    nnz = batch_indices.numel()
    tokens = append_key.shape[1]
    if tokens < nnz:
        raise ValueError("fewer key/value rows than index entries")
    if nnz == 0 or row == 0 or num_pages == 0 or L == 0:
        return
    with _on_device_of(kv_caches):
        _lib.check(_lib.lib().kvc_append_paged_kv_cache_layers(
            append_key.data_ptr(), append_value.data_ptr(), batch_indices.data_ptr(),
            positions.data_ptr(), kv_caches.data_ptr(), kv_indices.data_ptr(),
            kv_indptr.data_ptr(), kv_last_page_len.data_ptr(), nnz, kv_indptr.numel() - 1,
            kv_indices.numel(), H, D, page_size, row, row, 2 * page_size * row, num_pages,
            L, tokens * row, tokens * row, num_pages * 2 * page_size * row,
            kv_caches.element_size(), _stream_of(kv_caches)))


class PagedKVWritePlan:
    """The page-table write with its per-step arguments handed over ONCE.

    A forward pass calls `append_paged_kv_cache` once per layer with the same
    five index tensors (runtime/worker/llm_worker/models/layers/attention.py:76-85
    inside the layer loop of models/llama.py:236-242). A plan is built per step
    (where the reference builds `InputParams`, model_worker.py:435-446): the
    library keeps the index arguments (`kvc_write_plan_create`), and
    `plan.append(key, value, kv_caches[i])` per layer marshals only the layer's
    three pointers, their strides and the stream (`kvc_write_plan_append`).

    With `resolve_slots=True` the page table is walked once, at construction (one
    small launch on the current stream, `kvc_write_plan_resolve_slots`), and every
    layer's launch addresses the cache through the resulting slot per token: its
    chain of three dependent index loads is gone. Same results; the appends must
    run on that stream or be ordered after it. `slots=` hands over slots that
    already exist on the device (the slot mapping of `build_write_index`)
    instead: no launch, and a plan over fixed-capacity index buffers stays valid
    for every later step written into them.

    The plan keeps references to the index tensors, so their memory stays valid
    for as long as the plan lives.
    """

    def __init__(self, batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len,
                 num_kv_heads: int, head_dim: int, page_size: int, dtype: torch.dtype,
                 kv_layout: str = "NHD", resolve_slots: bool = False, slots: torch.Tensor = None):
        (self.batch_indices, self.positions, self.kv_indices, self.kv_indptr,
         self.kv_last_page_len) = _paged_common(None, None, batch_indices, positions, kv_indices,
                                                kv_indptr, kv_last_page_len, kv_layout)
        self.device = self.batch_indices.device
        self.dtype = dtype
        self.H, self.D, self.page_size = int(num_kv_heads), int(head_dim), int(page_size)
        self.row = self.H * self.D
        self.nnz = self.batch_indices.numel()
        self.elem = torch.empty(0, dtype=dtype).element_size()
        lib = _lib.lib()
        handle = ctypes.c_void_p()
        _lib.check(lib.kvc_write_plan_create(
            self.batch_indices.data_ptr(), self.positions.data_ptr(), self.kv_indices.data_ptr(),
            self.kv_indptr.data_ptr(), self.kv_last_page_len.data_ptr(), self.nnz,
            self.kv_indptr.numel() - 1, self.kv_indices.numel(), self.H, self.D, self.page_size,
            self.elem, ctypes.byref(handle)))
        self._plan = handle.value
        self.slots = None
        if slots is not None:
            # slots the caller already has (the index build's slot_mapping): nothing to launch
            _require_gpu(slots, "slots")
            if slots.dtype != torch.int64 or not slots.is_contiguous() or slots.numel() != self.nnz:
                raise TypeError("slots must be contiguous int64 [nnz]")
            self.slots = slots
            _lib.check(lib.kvc_write_plan_set_slots(self._plan, slots.data_ptr()))
        elif resolve_slots and self.nnz:
            self.slots = torch.empty(self.nnz, dtype=torch.int64, device=self.device)
            with _on_device_of(self.batch_indices):
                _lib.check(lib.kvc_write_plan_resolve_slots(self._plan, self.slots.data_ptr(),
                                                            _stream_of(self.batch_indices)))
        fast = _lib.fast()
        self._fast_append = fast.write_plan_append if fast else None
        self._dtype_code = fast.scalar_type_code(torch.empty(0, dtype=dtype)) if fast else -1
        self._append = lib.kvc_write_plan_append
        self._destroy = lib.kvc_write_plan_destroy
        self._cache_shape_tail = torch.Size((2, self.page_size, self.H, self.D))
        self._k_plane = self.page_size * self.row
        self._dense_page = 2 * self.page_size * self.row
        self._dev_index = self.device.index
        self._get_stream = torch._C._cuda_getCurrentRawStream

    def __del__(self):
        plan, self._plan = getattr(self, "_plan", None), None
        if plan:
            self._destroy(plan)

    def _row_stride(self, t: torch.Tensor, name: str) -> int:
        """Token stride of `[nnz, H, D]` / `[nnz, H*D]` rows that are dense inside a
        token; raises with the reason when the tensor does not qualify."""
        if t.dtype != self.dtype or t.device != self.device:
            raise TypeError(f"{name} must have the plan's dtype and device")
        st = t.stride()
        if t.dim() == 3:
            ok = st[2] == 1 and (st[1] == self.D or self.H == 1) and t.shape[1] * t.shape[2] == self.row
        else:
            ok = t.dim() == 2 and st[1] == 1 and t.shape[1] == self.row
        if not ok or t.shape[0] < self.nnz:
            raise ValueError(f"{name} must be [nnz, H, D] (or [nnz, H*D]) with dense rows")
        if self.nnz > 1 and st[0] < self.row:
            raise ValueError(f"{name} rows overlap (token stride {st[0]} < {self.row})")
        return st[0] if self.nnz > 1 else self.row

    def append(self, append_key: torch.Tensor, append_value: torch.Tensor,
               paged_kv_cache: torch.Tensor) -> None:
        """`append_paged_kv_cache` for one layer. Requirements (checked): key/value
        `[nnz, H, D]` (or `[nnz, H*D]`) of the plan's dtype on its device with dense
        rows (any token stride: slices of a fused QKV projection are read in
        place), `paged_kv_cache` `[num_pages, 2, page_size, H, D]` with contiguous
        pages. Launches on the current stream of the plan's device, which must be
        the current device."""
        nnz = self.nnz
        if nnz == 0:
            return
        fast = self._fast_append
        if fast is not None:
            # layouts checked and pointers read in C++; 1 = not a layout it knows: fall through
            # to the checks below, which name what is wrong (or handle the rare case)
            rc = fast(self._plan, nnz, self.H, self.D, self.page_size, self._dtype_code,
                      self._dev_index, append_key, append_value, paged_kv_cache,
                      self._get_stream(self._dev_index))
            if rc == 0:
                return
            if rc < 0:
                _lib.check(rc)
        row = self.row
        k_stride = append_key.stride(0)
        v_stride = append_value.stride(0)
        dt, dev = self.dtype, self.device
        if not (append_key.dtype is dt and append_value.dtype is dt and append_key.device == dev
                and append_value.device == dev and append_key.is_contiguous()
                and append_value.is_contiguous() and k_stride == row and v_stride == row
                and append_key.shape[0] >= nnz and append_value.shape[0] >= nnz):
            k_stride = self._row_stride(append_key, "append_key")
            v_stride = self._row_stride(append_value, "append_value")
        shape = paged_kv_cache.shape
        num_pages = shape[0]
        if num_pages == 0:
            return
        if paged_kv_cache.dtype is not dt or paged_kv_cache.device != dev:
            raise TypeError("paged_kv_cache must have the plan's dtype and device")
        st = paged_kv_cache.stride()
        if shape[1:] != self._cache_shape_tail or st[4] != 1 or st[3] != self.D \
                or st[2] != row or st[1] != self._k_plane:
            raise ValueError("paged_kv_cache must be [num_pages, 2, page_size, H, D] with contiguous pages")
        rc = self._append(self._plan, append_key.data_ptr(), append_value.data_ptr(), k_stride,
                          v_stride, paged_kv_cache.data_ptr(),
                          st[0] if num_pages > 1 else self._dense_page, num_pages,
                          self._get_stream(self._dev_index))
        if rc:
            _lib.check(rc)


class BlockRuns:
    """Block-run descriptors of a step on the device: `runs` int32 `[max_runs, 4]`
    (first token, block id, first entry, token count), `num_runs` int32 `[1]`,
    and, when they come from the index build, `run_indptr` int32 `[B + 1]`."""

    def __init__(self, runs: torch.Tensor, num_runs: torch.Tensor, run_indptr=None):
        self.runs, self.num_runs, self.run_indptr = runs, num_runs, run_indptr

    @property
    def max_runs(self) -> int:
        return int(self.runs.shape[0])

    def tolist(self):
        """The step's descriptors as a list of 4-tuples (synchronises)."""
        n = int(self.num_runs.item())
        return [tuple(r) for r in self.runs[:n].cpu().tolist()]


def max_block_runs(nnz: int, batch_size: int, page_size: int) -> int:
    """Upper bound of the block runs `nnz` new tokens of `batch_size` requests form."""
    return max(1, min(int(nnz), int(nnz) // int(page_size) + 2 * int(batch_size)))


def build_write_index(input_lens: torch.Tensor, context_lens: torch.Tensor,
                      num_blocks: torch.Tensor, kv_indices: torch.Tensor, page_size: int,
                      nnz: int, with_slot_mapping: bool = True, with_runs: bool = False, out=None):
    """All index tensors of a step from the per-request scalars, in one launch.

    input_lens, context_lens, num_blocks: int32 `[B]` on the device (new tokens,
    context length and block-table length of every request, in batch order);
    kv_indices: int32 concatenation of the block tables. Returns
    `(cu_seqlens_q, kv_indptr, kv_last_page_len, batch_indices, positions, slot_mapping)`
    -- what `ModelWorker._make_inputs` builds on the host and uploads piecewise
    (model_worker.py:346, :362-365, :399-433), plus the slot mapping; with
    `with_runs=True` a seventh element, the step's `BlockRuns`.

    `B`, `nnz` and `kv_indices.numel()` are capacities: requests with
    `input_lens[b] == 0` pad the batch and per-token outputs beyond the step's
    token count are -1 (skipped by every write). `out` takes the outputs of an
    earlier call to be written again (fixed addresses, for a recorded launch).
    """
    input_lens = _i32(input_lens, "input_lens")
    context_lens = _i32(context_lens, "context_lens")
    num_blocks = _i32(num_blocks, "num_blocks")
    kv_indices = _i32(kv_indices, "kv_indices")
    B = input_lens.numel()
    if context_lens.numel() != B or num_blocks.numel() != B:
        raise ValueError("input_lens, context_lens and num_blocks must have one entry per request")
    dev = input_lens.device
    nnz = int(nnz)
    if out is not None:
        cu, indptr, last, batch_indices, positions, slots = out[:6]
        runs = out[6] if len(out) > 6 else None
        if cu.numel() != B + 1 or indptr.numel() != B + 1 or last.numel() != B \
                or batch_indices.numel() != nnz or positions.numel() != nnz \
                or (slots is not None and slots.numel() != nnz):
            raise ValueError("`out` does not match the sizes of this call")
    else:
        cu = torch.empty(B + 1, dtype=torch.int32, device=dev)
        indptr = torch.empty(B + 1, dtype=torch.int32, device=dev)
        last = torch.empty(B, dtype=torch.int32, device=dev)
        batch_indices = torch.empty(nnz, dtype=torch.int32, device=dev)
        positions = torch.empty(nnz, dtype=torch.int32, device=dev)
        slots = torch.empty(nnz, dtype=torch.int64, device=dev) if with_slot_mapping else None
        runs = None
        if with_runs:
            cap = max_block_runs(nnz, B, page_size)
            runs = BlockRuns(torch.empty(cap, 4, dtype=torch.int32, device=dev),
                             torch.zeros(1, dtype=torch.int32, device=dev),
                             torch.empty(B + 1, dtype=torch.int32, device=dev))
    with _on_device_of(input_lens):
        _lib.check(_lib.lib().kvc_build_write_index(
            input_lens.data_ptr(), context_lens.data_ptr(), num_blocks.data_ptr(),
            kv_indices.data_ptr(), B, kv_indices.numel(), int(page_size), nnz, cu.data_ptr(),
            indptr.data_ptr(), last.data_ptr(), batch_indices.data_ptr(), positions.data_ptr(),
            slots.data_ptr() if slots is not None else None,
            runs.run_indptr.data_ptr() if runs is not None else None,
            runs.runs.data_ptr() if runs is not None else None,
            runs.num_runs.data_ptr() if runs is not None else None,
            runs.max_runs if runs is not None else 0, _stream_of(input_lens)))
    if runs is not None:
        return cu, indptr, last, batch_indices, positions, slots, runs
    return cu, indptr, last, batch_indices, positions, slots


def slot_block_runs(slot_mapping: torch.Tensor, block_size: int) -> BlockRuns:
    """Block runs of any slot mapping on the device (one small launch): token t
    opens a run when its slot is valid and is not the successor of token t-1's
    slot inside the same block."""
    _require_gpu(slot_mapping, "slot_mapping")
    if slot_mapping.dtype not in (torch.int32, torch.int64) or slot_mapping.dim() != 1:
        raise TypeError("slot_mapping must be a 1-D int32 or int64 tensor")
    slot_mapping = slot_mapping.contiguous()
    T = slot_mapping.numel()
    dev = slot_mapping.device
    runs = BlockRuns(torch.empty(max(T, 1), 4, dtype=torch.int32, device=dev),
                     torch.zeros(1, dtype=torch.int32, device=dev))
    with _on_device_of(slot_mapping):
        _lib.check(_lib.lib().kvc_slot_runs(slot_mapping.data_ptr(), slot_mapping.element_size(), T,
                                            int(block_size), runs.runs.data_ptr(), runs.num_runs.data_ptr(),
                                            runs.max_runs, _stream_of(slot_mapping)))
    return runs


def write_block_runs_layers(key: torch.Tensor, value: torch.Tensor, kv_caches: torch.Tensor,
                            runs: BlockRuns) -> None:
    """`reshape_and_cache_layers` on the slot mapping `runs` describes, as tile
    copies: every (run, layer, K|V) moves as one contiguous piece.

    key, value: `[L, T, H, D]` contiguous; kv_caches `[L, nb, 2, bs, H, D]` contiguous.
    """
    for t, n in ((key, "key"), (value, "value"), (kv_caches, "kv_caches")):
        _require_gpu(t, n)
    if kv_caches.dim() != 6 or kv_caches.shape[2] != 2 or not kv_caches.is_contiguous():
        raise ValueError("kv_caches must be contiguous [L, num_blocks, 2, block_size, H, D]")
    if key.dtype != kv_caches.dtype or value.dtype != kv_caches.dtype:
        raise TypeError("key/value and kv_caches must share one dtype")
    L, nb, _, bs, H, D = kv_caches.shape
    row = H * D
    if key.dim() != 4 or key.shape != value.shape or key.shape[0] != L or key.shape[2] * key.shape[3] != row:
        raise ValueError("key/value must be [L, T, H, D] matching the pool")
    key, value = key.contiguous(), value.contiguous()
    T = key.shape[1]
    if T == 0 or row == 0 or nb == 0 or L == 0:
        return
    with _on_device_of(kv_caches):
        _lib.check(_lib.lib().kvc_write_runs_layers(
            key.data_ptr(), value.data_ptr(), kv_caches.data_ptr(),
            kv_caches.data_ptr() + bs * row * kv_caches.element_size(), runs.runs.data_ptr(),
            runs.num_runs.data_ptr(), runs.max_runs, T, row, row, row, bs, 2 * bs * row, row, nb, L,
            T * row, T * row, nb * 2 * bs * row, kv_caches.element_size(), _stream_of(kv_caches)))

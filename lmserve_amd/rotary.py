"""Rotary position embedding, alone or fused with the K/V write.

Mirrors runtime/worker/llm_worker/ops/rotary_embedding_ops.py:8-35
(`rotary_pos_emb`) and the cos/sin table of
runtime/worker/llm_worker/models/layers/rotary_embedding.py:11-70
(`RotaryEmbedding`, llama3 frequency scaling included). The fused forms add the
cache write that follows the rotation in the reference's attention layer
(runtime/worker/llm_worker/models/llama.py:156-167,
 runtime/worker/llm_worker/models/layers/attention.py:76-85), so K is read
once and the write costs no launch of its own.

Arithmetic: fp32 with one rounding to the tensors' dtype.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple

import torch

from . import _lib
from .cache_ops import _SLOT_DTYPES, _inner_contiguous, _on_device_of, _require_gpu, _stream_of

_DTYPES = {torch.bfloat16: _lib.KVC_DTYPE_BF16, torch.float16: _lib.KVC_DTYPE_F16,
           torch.float32: _lib.KVC_DTYPE_F32}


def make_cos_sin_cache(rotary_dim: int, max_position_embeddings: int, base: float = 10000.0,
                       rope_scaling: Optional[dict] = None, dtype: torch.dtype = torch.bfloat16,
                       device=None) -> torch.Tensor:
    """`[max_position, 2*rotary_dim]` = cos(emb) | sin(emb), emb = cat(freqs, freqs),
    freqs[p, i] = p * inv_freq[i]; computed in fp32 and cast to `dtype`
    (rotary_embedding.py:27-70). `rope_scaling` is the llama3 dict with keys
    factor, low_freq_factor, high_freq_factor, original_max_position_embeddings."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.int64).float() / rotary_dim))
    if rope_scaling is not None:
        factor = rope_scaling["factor"]
        low_freq_factor = rope_scaling["low_freq_factor"]
        high_freq_factor = rope_scaling["high_freq_factor"]
        old_context_len = rope_scaling["original_max_position_embeddings"]
        low_freq_wavelen = old_context_len / low_freq_factor
        high_freq_wavelen = old_context_len / high_freq_factor
        wavelen = 2 * math.pi / inv_freq
        scaled = torch.where(wavelen > low_freq_wavelen, inv_freq / factor, inv_freq)
        smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        smoothed = (1 - smooth) * scaled / factor + smooth * scaled
        is_medium = ~(wavelen < high_freq_wavelen) & ~(wavelen > low_freq_wavelen)
        inv_freq = torch.where(is_medium, smoothed, scaled)
    t = torch.arange(max_position_embeddings).float()
    freqs = torch.einsum("i,j->ij", t, inv_freq.float())
    emb = torch.cat((freqs, freqs), dim=-1)
    cos_sin = torch.cat((emb.cos().to(dtype), emb.sin().to(dtype)), dim=-1)
    return cos_sin.to(device) if device is not None else cos_sin


_raw_stream = torch._C._cuda_getCurrentRawStream
_fast_entry = _lib.fast_entry


def _prep(query, key, positions, cos_sin_cache, head_dim):
    for t, n in ((query, "query"), (key, "key"), (positions, "positions"),
                 (cos_sin_cache, "cos_sin_cache")):
        _require_gpu(t, n)
    kd = _DTYPES.get(query.dtype)
    if kd is None:
        raise TypeError(f"Unsupported dtype: {query.dtype}")
    if key.dtype != query.dtype or cos_sin_cache.dtype != query.dtype:
        raise TypeError("query, key and cos_sin_cache must share one dtype")
    num_tokens = positions.shape[0]
    q2 = query.reshape(num_tokens, -1)
    k2 = key.reshape(num_tokens, -1)
    if q2.stride(-1) != 1:
        q2 = q2.contiguous()
    if k2.stride(-1) != 1:
        k2 = k2.contiguous()
    if q2.shape[1] % head_dim or k2.shape[1] % head_dim:
        raise ValueError("query/key width is not a multiple of head_dim")
    pos_bytes = _SLOT_DTYPES.get(positions.dtype)
    if pos_bytes is None:
        raise TypeError("positions must be int32 or int64")
    if not positions.is_contiguous():
        positions = positions.contiguous()
    if cos_sin_cache.dim() != 2 or cos_sin_cache.shape[1] % 2 or not cos_sin_cache.is_contiguous():
        raise ValueError("cos_sin_cache must be contiguous [max_position, 2*rotary_dim]")
    return q2, k2, positions, pos_bytes, kd, num_tokens


def _tok_stride(t2):
    return t2.stride(0) if t2.shape[0] > 1 else t2.shape[1]


def rotary_pos_emb(query: torch.Tensor, key: torch.Tensor, positions: torch.Tensor,
                   cos_sin_cache: torch.Tensor, head_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rotate `query [T, Hq*D]` and `key [T, Hkv*D]`; returns new tensors of the
    inputs' shapes (rotary_embedding_ops.py:8-35)."""
    fast = _fast_entry("rotary_pos_emb")
    if fast is not None and isinstance(query, torch.Tensor) and query.is_cuda and query.dim() in (2, 3) \
            and isinstance(key, torch.Tensor) and key.dim() in (2, 3):
        # common layouts: checked and launched from C++ (1 = not one of them: fall through)
        dev = query.device.index
        q_out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        k_out = torch.empty(key.shape, dtype=key.dtype, device=key.device)
        rc = fast(query, key, positions, cos_sin_cache, head_dim, q_out, k_out, dev, _raw_stream(dev))
        if rc == 0:
            return q_out, k_out
        if rc < 0:
            _lib.check(rc)
    q2, k2, positions, pos_bytes, kd, T = _prep(query, key, positions, cos_sin_cache, head_dim)
    q_out = torch.empty_like(q2, memory_format=torch.contiguous_format)
    k_out = torch.empty_like(k2, memory_format=torch.contiguous_format)
    if T > 0:
        with _on_device_of(q2):
            _lib.check(_lib.lib().kvc_rotary_pos_emb(
                q2.data_ptr(), k2.data_ptr(), positions.data_ptr(), pos_bytes,
                cos_sin_cache.data_ptr(), cos_sin_cache.shape[0], T, q2.shape[1] // head_dim,
                k2.shape[1] // head_dim, head_dim, cos_sin_cache.shape[1] // 2, _tok_stride(q2),
                _tok_stride(k2), q_out.data_ptr(), k_out.data_ptr(), q_out.shape[1], k_out.shape[1],
                kd, _stream_of(q2)))
    return q_out.view(query.shape), k_out.view(key.shape)


def rotary_pos_emb_and_cache(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                             positions: torch.Tensor, cos_sin_cache: torch.Tensor, head_dim: int,
                             kv_cache: torch.Tensor, slot_mapping: torch.Tensor,
                             return_key: bool = True):
    """`rotary_pos_emb` plus the slot-mapped write of the rotated key and the
    value into one layer of the pool, `kv_cache [num_blocks, 2, block_size, H, D]`.
    Returns `(q_out, k_out)`; `k_out` is None with `return_key=False`."""
    q2, k2, positions, pos_bytes, kd, T = _prep(query, key, positions, cos_sin_cache, head_dim)
    for t, n in ((value, "value"), (kv_cache, "kv_cache"), (slot_mapping, "slot_mapping")):
        _require_gpu(t, n)
    if value.dtype != query.dtype or kv_cache.dtype != query.dtype:
        raise TypeError("value and kv_cache must have the query's dtype")
    if kv_cache.dim() != 5 or kv_cache.shape[1] != 2 or not _inner_contiguous(kv_cache):
        raise ValueError("kv_cache must be [num_blocks, 2, block_size, H, D] with contiguous blocks")
    nb, _, bs, H, D = kv_cache.shape
    v2 = value.reshape(T, -1)
    if v2.stride(-1) != 1:
        v2 = v2.contiguous()
    if D != head_dim or k2.shape[1] != H * D or v2.shape[1] != H * D:
        raise ValueError("key/value rows do not match the cache's H*D")
    if slot_mapping.shape[0] != T:
        raise ValueError("slot_mapping length differs from the number of tokens")
    slot_bytes = _SLOT_DTYPES.get(slot_mapping.dtype)
    if slot_bytes is None:
        slot_mapping, slot_bytes = slot_mapping.to(torch.int64), 8
    if not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.contiguous()
    q_out = torch.empty_like(q2, memory_format=torch.contiguous_format)
    k_out = torch.empty_like(k2, memory_format=torch.contiguous_format) if return_key else None
    if T > 0 and nb > 0:
        elem = kv_cache.element_size()
        row = H * D
        with _on_device_of(q2):
            _lib.check(_lib.lib().kvc_rotary_pos_emb_and_cache(
                q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), positions.data_ptr(), pos_bytes,
                cos_sin_cache.data_ptr(), cos_sin_cache.shape[0], T, q2.shape[1] // head_dim, H,
                head_dim, cos_sin_cache.shape[1] // 2, _tok_stride(q2), _tok_stride(k2),
                _tok_stride(v2), q_out.data_ptr(), k_out.data_ptr() if return_key else None,
                q_out.shape[1], row, kv_cache.data_ptr(), kv_cache.data_ptr() + bs * row * elem,
                slot_mapping.data_ptr(), slot_bytes, bs,
                kv_cache.stride(0) if nb > 1 else 2 * bs * row, row, nb, kd, _stream_of(q2)))
    return q_out.view(query.shape), (k_out.view(key.shape) if return_key else None)


def rotary_pos_emb_and_append_paged(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                    batch_indices: torch.Tensor, positions: torch.Tensor,
                                    cos_sin_cache: torch.Tensor, head_dim: int,
                                    paged_kv_cache: torch.Tensor, kv_indices: torch.Tensor,
                                    kv_indptr: torch.Tensor, kv_last_page_len: torch.Tensor,
                                    return_key: bool = True):
    """`rotary_pos_emb` plus `append_paged_kv_cache` of the rotated key and the
    value in one launch; `positions` (int32) is both the rotation position and
    the KV position of each token, as in the reference."""
    fast = _fast_entry("rotary_append_paged")
    if fast is not None and isinstance(query, torch.Tensor) and query.is_cuda and query.dim() in (2, 3) \
            and isinstance(key, torch.Tensor) and key.dim() in (2, 3):
        dev = query.device.index
        q_out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
        k_out = torch.empty(key.shape, dtype=key.dtype, device=key.device) if return_key else None
        rc = fast(query, key, value, batch_indices, positions, cos_sin_cache, head_dim, paged_kv_cache,
                  kv_indices, kv_indptr, kv_last_page_len, q_out, k_out, dev, _raw_stream(dev))
        if rc == 0:
            return q_out, k_out
        if rc < 0:
            _lib.check(rc)
    q2, k2, positions, pos_bytes, kd, T = _prep(query, key, positions, cos_sin_cache, head_dim)
    if pos_bytes != 4:
        raise TypeError("positions must be int32 for page-table addressing")
    for t, n in ((value, "value"), (paged_kv_cache, "paged_kv_cache")):
        _require_gpu(t, n)
    for t, n in ((batch_indices, "batch_indices"), (kv_indices, "kv_indices"),
                 (kv_indptr, "kv_indptr"), (kv_last_page_len, "kv_last_page_len")):
        _require_gpu(t, n)
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise TypeError(f"{n} must be contiguous int32")
    if value.dtype != query.dtype or paged_kv_cache.dtype != query.dtype:
        raise TypeError("value and paged_kv_cache must have the query's dtype")
    if paged_kv_cache.dim() != 5 or paged_kv_cache.shape[1] != 2 or \
            not _inner_contiguous(paged_kv_cache):
        raise ValueError("paged_kv_cache must be [num_pages, 2, page_size, H, D] with contiguous pages")
    num_pages, _, page_size, H, D = paged_kv_cache.shape
    v2 = value.reshape(T, -1)
    if v2.stride(-1) != 1:
        v2 = v2.contiguous()
    if D != head_dim or k2.shape[1] != H * D or v2.shape[1] != H * D:
        raise ValueError("key/value rows do not match the cache's H*D")
    if batch_indices.numel() != T:
        raise ValueError("batch_indices and positions differ in length")
    q_out = torch.empty_like(q2, memory_format=torch.contiguous_format)
    k_out = torch.empty_like(k2, memory_format=torch.contiguous_format) if return_key else None
    if T > 0 and num_pages > 0:
        row = H * D
        with _on_device_of(q2):
            _lib.check(_lib.lib().kvc_rotary_pos_emb_and_append_paged(
                q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), batch_indices.data_ptr(),
                positions.data_ptr(), cos_sin_cache.data_ptr(), cos_sin_cache.shape[0], T,
                q2.shape[1] // head_dim, H, head_dim, cos_sin_cache.shape[1] // 2, _tok_stride(q2),
                _tok_stride(k2), _tok_stride(v2), q_out.data_ptr(),
                k_out.data_ptr() if return_key else None, q_out.shape[1], row,
                paged_kv_cache.data_ptr(), kv_indices.data_ptr(), kv_indptr.data_ptr(),
                kv_indptr.numel() - 1, kv_indices.numel(), page_size,
                paged_kv_cache.stride(0) if num_pages > 1 else 2 * page_size * row, num_pages, kd,
                _stream_of(q2)))
    return q_out.view(query.shape), (k_out.view(key.shape) if return_key else None)


class PagedRotaryWritePlan:
    """`rotary_pos_emb_and_append_paged` with its per-step arguments checked ONCE.

    The rotation and the append run once per layer with the same positions,
    index tensors and cos/sin table (models/llama.py:156-167 and
    models/layers/attention.py:76-85 inside the layer loop of llama.py:236-242).
    A plan built per step (where the reference builds `InputParams`,
    model_worker.py:435-446) leaves the layer loop with a handful of pointer
    reads and the library call; `query_out` / `key_out` may be caller-owned
    buffers reused across layers, so that nothing is allocated either.

    `resolve_slots=True` walks the page table once, at construction (one small
    launch on the current stream); the per-layer launches then read one slot per
    token. Same results; the runs must be ordered after the construction.
    `slots=` hands over slots that already exist on the device (the slot mapping
    of `build_write_index`) instead: no launch, and a plan over fixed-capacity
    index buffers stays valid for every later step written into them.

    The plan keeps references to its tensors for as long as it lives.
    """

    def __init__(self, batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len,
                 cos_sin_cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                 page_size: int, resolve_slots: bool = False, slots: torch.Tensor = None):
        for t, n in ((batch_indices, "batch_indices"), (positions, "positions"),
                     (kv_indices, "kv_indices"), (kv_indptr, "kv_indptr"),
                     (kv_last_page_len, "kv_last_page_len")):
            _require_gpu(t, n)
            if t.dtype != torch.int32 or not t.is_contiguous():
                raise TypeError(f"{n} must be contiguous int32")
        _require_gpu(cos_sin_cache, "cos_sin_cache")
        self.kd = _DTYPES.get(cos_sin_cache.dtype)
        if self.kd is None:
            raise TypeError(f"Unsupported dtype: {cos_sin_cache.dtype}")
        if cos_sin_cache.dim() != 2 or cos_sin_cache.shape[1] % 2 or not cos_sin_cache.is_contiguous():
            raise ValueError("cos_sin_cache must be contiguous [max_position, 2*rotary_dim]")
        if batch_indices.numel() != positions.numel():
            raise ValueError("batch_indices and positions differ in length")
        self._keep = (batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len, cos_sin_cache)
        self.device, self.dtype = cos_sin_cache.device, cos_sin_cache.dtype
        self.Hq, self.H, self.D, self.page_size = int(num_heads), int(num_kv_heads), int(head_dim), int(page_size)
        self.nnz = positions.numel()
        self.q_row, self.kv_row = self.Hq * self.D, self.H * self.D
        lib = _lib.lib()
        handle = ctypes.c_void_p()
        _lib.check(lib.kvc_rotary_plan_create(
            batch_indices.data_ptr(), positions.data_ptr(), cos_sin_cache.data_ptr(),
            cos_sin_cache.shape[0], self.nnz, self.Hq, self.H, self.D, cos_sin_cache.shape[1] // 2,
            kv_indices.data_ptr(), kv_indptr.data_ptr(), kv_indptr.numel() - 1, kv_indices.numel(),
            self.page_size, self.kd, ctypes.byref(handle)))
        self._plan = handle.value
        self.slots = None
        if slots is not None:
            # slots the caller already has (the index build's slot_mapping): nothing to launch
            _require_gpu(slots, "slots")
            if slots.dtype != torch.int64 or not slots.is_contiguous() or slots.numel() != self.nnz:
                raise TypeError("slots must be contiguous int64 [nnz]")
            self.slots = slots
            _lib.check(lib.kvc_rotary_plan_set_slots(self._plan, slots.data_ptr()))
        elif resolve_slots and self.nnz:
            # the page table is walked once, here; every layer's launch reads one slot per token
            self.slots = torch.empty(self.nnz, dtype=torch.int64, device=self.device)
            with torch.cuda.device(self.device):
                _lib.check(lib.kvc_rotary_plan_resolve_slots(
                    self._plan, self.slots.data_ptr(),
                    torch._C._cuda_getCurrentRawStream(self.device.index)))
        fast = _lib.fast()
        self._fast_run = fast.rotary_plan_run if fast else None
        self._dtype_code = fast.scalar_type_code(cos_sin_cache) if fast else -1
        self._run = lib.kvc_rotary_plan_run
        self._destroy = lib.kvc_rotary_plan_destroy
        self._cache_shape_tail = torch.Size((2, self.page_size, self.H, self.D))
        self._k_plane = self.page_size * self.kv_row
        self._dense_page = 2 * self.page_size * self.kv_row
        self._dev_index = self.device.index
        self._get_stream = torch._C._cuda_getCurrentRawStream

    def __del__(self):
        plan, self._plan = getattr(self, "_plan", None), None
        if plan:
            self._destroy(plan)

    def _rows(self, t: torch.Tensor, width: int, name: str, dense: bool = False) -> int:
        """Token stride (elements) of a `[nnz, width]` / `[nnz, heads, D]` tensor with dense rows."""
        if t.dtype != self.dtype or t.device != self.device:
            raise TypeError(f"{name} must have the plan's dtype and device")
        st = t.stride()
        if t.shape[0] != self.nnz or t.numel() != self.nnz * width:
            raise ValueError(f"{name} must hold [nnz, {width}] elements")
        if st[-1] != 1 or (t.dim() == 3 and st[1] != t.shape[2]):
            raise ValueError(f"{name} rows must be dense")
        stride = st[0] if self.nnz > 1 else width
        if stride < width or (dense and stride != width):
            raise ValueError(f"{name} must have {'contiguous' if dense else 'non-overlapping'} rows")
        return stride

    def run(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
            paged_kv_cache: torch.Tensor, query_out: torch.Tensor = None,
            key_out: torch.Tensor = None, return_key: bool = False):
        """One layer: rotates `query` and `key`, writes the rotated key and `value`
        into the pages. Returns `(query_out, key_out)`; `key_out` is None unless a
        buffer is given or `return_key` is set. Token-strided inputs (slices of a
        fused QKV projection) are read in place; the output buffers are contiguous.
        Launches on the current stream of the plan's device, which must be the
        current device."""
        if query_out is None:
            query_out = torch.empty((self.nnz, self.q_row), dtype=self.dtype, device=self.device)
        if key_out is None and return_key:
            key_out = torch.empty((self.nnz, self.kv_row), dtype=self.dtype, device=self.device)
        if self.nnz == 0:
            return query_out, key_out
        fast = self._fast_run
        if fast is not None:
            # layouts checked and pointers read in C++; 1 = not a layout it knows: fall through
            # to the checks below, which name what is wrong (or handle the rare case)
            rc = fast(self._plan, self.nnz, self.Hq, self.H, self.D, self.page_size, self._dtype_code,
                      self._dev_index, query, key, value, query_out, key_out, paged_kv_cache,
                      self._get_stream(self._dev_index))
            if rc == 0:
                return query_out, key_out
            if rc < 0:
                _lib.check(rc)
        dt, dev, nnz = self.dtype, self.device, self.nnz
        if paged_kv_cache.dtype is not dt or paged_kv_cache.device != dev:
            raise TypeError("paged_kv_cache must have the plan's dtype and device")
        shape, st = paged_kv_cache.shape, paged_kv_cache.stride()
        if shape[1:] != self._cache_shape_tail or st[4] != 1 or st[3] != self.D \
                or st[2] != self.kv_row or st[1] != self._k_plane:
            raise ValueError("paged_kv_cache must be [num_pages, 2, page_size, H, D] with contiguous pages")
        num_pages = shape[0]
        if num_pages == 0:
            raise ValueError("paged_kv_cache has no pages")
        q_row, kv_row = self.q_row, self.kv_row
        # the common case in one pass: 2-D [nnz, width] views with unit inner stride (the
        # slices of a fused projection); anything else goes through the checks that name
        # what is wrong
        qs, ks, vs = query.stride(), key.stride(), value.stride()
        if (query.dtype is dt and key.dtype is dt and value.dtype is dt and len(qs) == 2 and len(ks) == 2
                and len(vs) == 2 and qs[1] == 1 and ks[1] == 1 and vs[1] == 1
                and query.shape == (nnz, q_row) and key.shape == (nnz, kv_row)
                and value.shape == (nnz, kv_row) and qs[0] >= q_row and ks[0] >= kv_row
                and vs[0] >= kv_row and query.device == dev and key.device == dev
                and value.device == dev):
            q_stride, k_stride, v_stride = qs[0], ks[0], vs[0]
        else:
            q_stride = self._rows(query, q_row, "query")
            k_stride = self._rows(key, kv_row, "key")
            v_stride = self._rows(value, kv_row, "value")
        if not (query_out.dtype is dt and query_out.is_contiguous() and query_out.device == dev
                and query_out.numel() == nnz * q_row):
            self._rows(query_out, q_row, "query_out", dense=True)
        ko_ptr = None
        if key_out is not None:
            if not (key_out.dtype is dt and key_out.is_contiguous() and key_out.device == dev
                    and key_out.numel() == nnz * kv_row):
                self._rows(key_out, kv_row, "key_out", dense=True)
            ko_ptr = key_out.data_ptr()
        rc = self._run(self._plan, query.data_ptr(), key.data_ptr(), value.data_ptr(), q_stride,
                       k_stride, v_stride, query_out.data_ptr(), ko_ptr, paged_kv_cache.data_ptr(),
                       st[0] if num_pages > 1 else self._dense_page, num_pages,
                       self._get_stream(self._dev_index))
        if rc:
            _lib.check(rc)
        return query_out, key_out


class RotaryEmbedding(torch.nn.Module):
    """`RotaryEmbedding` of the reference (rotary_embedding.py:11-80): builds the
    cos/sin table from a HF-style config and rotates `(query, key)` in `forward`."""

    def __init__(self, config, base: int = 10000) -> None:
        super().__init__()
        base = getattr(config, "rope_theta", base)
        partial_rotary_factor = getattr(config, "partial_rotary_factor", 1.0)
        head_dim = getattr(config, "head_dim", None) or \
            config.hidden_size // config.num_attention_heads
        self.rotary_dim = int(head_dim * partial_rotary_factor)
        self.max_position_embeddings = config.max_position_embeddings
        self.head_dim = head_dim
        cos_sin = make_cos_sin_cache(self.rotary_dim, self.max_position_embeddings, base,
                                     getattr(config, "rope_scaling", None),
                                     getattr(config, "torch_dtype", torch.bfloat16))
        self.register_buffer("cos_sin_cached", cos_sin, persistent=False)

    def forward(self, query: torch.Tensor, key: torch.Tensor,
                positions: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        return rotary_pos_emb(query, key, positions, self.cos_sin_cached, self.head_dim)

"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

CPU restatements of the reference's paged KV-cache data movement, used only as
the checker for the HIP library (tests/, the smoke check, bench.py's
cpu_baseline leg). Nothing under lmserve_amd/ may import this module.

Three independent formulations live here so that they can be checked against
each other and against closed forms:

  *_np     vectorised NumPy (fancy indexing on shaped views)
  c_*      the plain-C loops of oracle/kvc_oracle.c through ctypes
  *_loops  element-by-element pure Python following the reference kernels'
           flat address arithmetic; only for tiny inputs

All operate IN PLACE on NumPy arrays of any item size (bf16 is carried as
uint16, as the reference's host pool does: kv_worker.py:17-22). Citations are
paths under the reference's runtime/worker/llm_worker/. Pinning status is listed
in the header of kvc_oracle.c; parity of the three page-table functions with
the third-party flashinfer binary itself is UNPINNED. The block-run functions
(`block_runs_loops`, `slot_runs_loops`, `runs_to_slots`, `write_runs_np`) are
pinned in tests/test_oracle_pinning.py: a step written out by hand, the runs
expanded back to slots against the independently pinned slot mapping, maximality
of the runs, and the slice write against the pinned slot-mapped write. The two functions that
exist only here, `build_write_index_*` and `paged_write_slots_np`, are pinned in
tests/test_host_logic.py: a step written out by hand, NumPy against loops, the
pinned page-table functions, and (for the slots) the property that a slot-mapped
write through them equals the page-table write.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import numpy as np

ORACLE_DIR = os.path.dirname(os.path.abspath(__file__))
C_LIB_PATH = os.path.join(ORACLE_DIR, "libkvc_oracle.so")

# --------------------------------------------------------------------------- NumPy


def fill_key_cache_np(key, value, key_cache, value_cache, slot_mapping) -> None:
    """ops/cache_ops.py:39-59 + ops/triton/cache_kernels.py:39-58: caches are
    addressed flat as [num_slots, H*D]."""
    T = len(slot_mapping)
    row = key.shape[1] * key.shape[2]
    slots = np.asarray(slot_mapping, dtype=np.int64)
    key_cache.reshape(-1, row)[slots] = key.reshape(T, row)
    value_cache.reshape(-1, row)[slots] = value.reshape(T, row)


def reshape_and_cache_np(key, value, kv_cache, slot_mapping) -> None:
    """One layer of the pool [nb, 2, bs, H, D] (model_worker.py:221-228);
    slot = blk*bs + e."""
    bs = kv_cache.shape[2]
    slots = np.asarray(slot_mapping, dtype=np.int64)
    kv_cache[slots // bs, 0, slots % bs] = key
    kv_cache[slots // bs, 1, slots % bs] = value


def append_paged_kv_cache_np(append_key, append_value, batch_indices, positions, paged_kv_cache,
                             kv_indices, kv_indptr, kv_last_page_len=None) -> None:
    """The flashinfer call at models/layers/attention.py:76-85, NHD layout."""
    page_size = paged_kv_cache.shape[2]
    b = np.asarray(batch_indices, dtype=np.int64)
    p = np.asarray(positions, dtype=np.int64)
    pages = np.asarray(kv_indices, dtype=np.int64)[np.asarray(kv_indptr, dtype=np.int64)[b]
                                                   + p // page_size]
    paged_kv_cache[pages, 0, p % page_size] = append_key[:len(b)]
    paged_kv_cache[pages, 1, p % page_size] = append_value[:len(b)]


def get_seq_lens_np(kv_indptr, kv_last_page_len, page_size) -> np.ndarray:
    """The flashinfer call at model_worker.py:427-431."""
    kv_indptr = np.asarray(kv_indptr, dtype=np.int64)
    full = np.maximum(kv_indptr[1:] - kv_indptr[:-1] - 1, 0)
    return (full * page_size + np.asarray(kv_last_page_len, dtype=np.int64)).astype(np.int32)


def get_batch_indices_positions_np(append_indptr, seq_lens, nnz) -> Tuple[np.ndarray, np.ndarray]:
    """The flashinfer call at model_worker.py:425-433."""
    append_indptr = np.asarray(append_indptr, dtype=np.int64)
    n_new = append_indptr[1:] - append_indptr[:-1]
    batch = np.repeat(np.arange(len(n_new), dtype=np.int64), n_new)
    within = np.arange(int(append_indptr[-1]), dtype=np.int64) - append_indptr[:-1][batch]
    pos = np.asarray(seq_lens, dtype=np.int64)[batch] - n_new[batch] + within
    assert len(batch) <= nnz
    return batch.astype(np.int32), pos.astype(np.int32)


def build_write_index_np(input_lens, context_lens, num_blocks, kv_indices, page_size):
    """The whole index of a step from the per-request scalars the scheduler sends
    (proto/worker.proto:40-47), as `ModelWorker._make_inputs` builds it piecewise
    on the host (model_worker.py:346 position_ids, :362-365 cu_seqlens_q, :399-423
    page table and last-page fill), the two flashinfer calls derive it
    (model_worker.py:425-433) and the scheduler's slot rule places it
    (scheduler.rs:453-541, block_manager.rs:241-273):
        cu_seqlens_q = [0, cumsum(input_lens)], kv_indptr = [0, cumsum(num_blocks)],
        last_page_len[b] = (context_lens[b] - 1) % page_size + 1,
        for the j-th new token of request b:
            batch_indices = b, position = context_lens[b] - input_lens[b] + j,
            slot = kv_indices[kv_indptr[b] + position // page_size] * page_size + position % page_size
    A position outside its request's own table yields slot -1. Requests are taken in
    the order given (the caller has sorted them, model_worker.py:326-328). Returns
    (cu_seqlens_q, kv_indptr, last_page_len, batch_indices, positions, slot_mapping):
    int32 except the int64 slot mapping."""
    q = np.asarray(input_lens, dtype=np.int64)
    ctx = np.asarray(context_lens, dtype=np.int64)
    nblk = np.asarray(num_blocks, dtype=np.int64)
    table = np.asarray(kv_indices, dtype=np.int64)
    cu = np.concatenate([[0], np.cumsum(q)])
    indptr = np.concatenate([[0], np.cumsum(nblk)])
    last = np.where(ctx > 0, (ctx - 1) % page_size + 1, 0)
    batch = np.repeat(np.arange(len(q), dtype=np.int64), q)
    within = np.arange(int(cu[-1]), dtype=np.int64) - cu[:-1][batch]
    pos = ctx[batch] - q[batch] + within
    entry = indptr[:-1][batch] + pos // page_size
    ok = (pos >= 0) & (entry >= 0) & (entry < np.minimum(indptr[1:][batch], len(table)))
    slots = np.full(len(batch), -1, dtype=np.int64)
    slots[ok] = table[entry[ok]] * page_size + pos[ok] % page_size
    i32 = np.int32
    return (cu.astype(i32), indptr.astype(i32), last.astype(i32), batch.astype(i32), pos.astype(i32), slots)


def build_write_index_loops(input_lens, context_lens, num_blocks, kv_indices, page_size):
    """`build_write_index_np` request by request and token by token."""
    cu, indptr, last, batch, pos, slots = [0], [0], [], [], [], []
    for b, (q, ctx, nblk) in enumerate(zip(input_lens, context_lens, num_blocks)):
        q, ctx, nblk = int(q), int(ctx), int(nblk)
        table = [int(x) for x in kv_indices[indptr[-1]:indptr[-1] + nblk]]
        cu.append(cu[-1] + q)
        indptr.append(indptr[-1] + nblk)
        last.append((ctx - 1) % page_size + 1 if ctx > 0 else 0)
        for j in range(q):
            p = ctx - q + j
            batch.append(b)
            pos.append(p)
            page = p // page_size
            slots.append(table[page] * page_size + p % page_size if p >= 0 and page < len(table) else -1)
    i32 = np.int32
    return (np.asarray(cu, dtype=i32), np.asarray(indptr, dtype=i32), np.asarray(last, dtype=i32),
            np.asarray(batch, dtype=i32), np.asarray(pos, dtype=i32), np.asarray(slots, dtype=np.int64))


def pad_write_index(index, nnz):
    """`build_write_index_*` output with its per-token arrays padded to the
    capacity `nnz` the way a capacity-bound launch leaves them: -1 in
    batch_indices, positions and slot_mapping beyond the step's tokens (entries a
    write skips: models/layers/attention.py:76-85 is never given them)."""
    cu, indptr, last, batch, pos, slots = index
    t = len(batch)
    assert t <= nnz

    def pad(a):
        out = np.full(nnz, -1, dtype=a.dtype)
        out[:t] = a
        return out
    return cu, indptr, last, pad(batch), pad(pos), pad(slots)


def block_runs_loops(input_lens, context_lens, num_blocks, kv_indices, page_size):
    """Block runs of a step, request by request: the new tokens of request b sit
    at positions [ctx - q, ctx) (scheduler.rs:453-541) and each block they touch
    takes one run -- consecutive tokens on the source side, consecutive entries
    of one block on the cache side (scheduler.rs:466-512: a chunk fills whole
    blocks). Returns (run_indptr int32 [B+1], runs int32 [n, 4]) with
    runs[r] = (first token, block id or -1 outside the table, first entry, count)."""
    run_indptr, runs = [0], []
    token, table_at = 0, 0
    for q, ctx, nblk in zip(input_lens, context_lens, num_blocks):
        q, ctx, nblk = int(q), int(ctx), int(nblk)
        table = [int(x) for x in kv_indices[table_at:table_at + nblk]]
        table_at += nblk
        pos = ctx - q
        if q > 0 and pos >= 0:
            while pos < ctx:
                page, entry = pos // page_size, pos % page_size
                count = min(page_size - entry, ctx - pos)
                runs.append((token + pos - (ctx - q), table[page] if page < len(table) else -1, entry, count))
                pos += count
        token += q
        run_indptr.append(len(runs))
    return np.asarray(run_indptr, dtype=np.int32), np.asarray(runs, dtype=np.int32).reshape(-1, 4)


def slot_runs_loops(slot_mapping, block_size):
    """Block runs of any slot mapping, token by token: a token with a valid slot
    continues the current run when its slot follows the previous token's inside
    the same block, and opens a new one otherwise. int32 [n, 4]."""
    runs = []
    prev = None
    for t, s in enumerate(int(x) for x in slot_mapping):
        if s < 0:
            prev = None
            continue
        if prev is not None and s == prev + 1 and s % block_size != 0:
            runs[-1][3] += 1
        else:
            runs.append([t, s // block_size, s % block_size, 1])
        prev = s
    return np.asarray(runs, dtype=np.int32).reshape(-1, 4)


def runs_to_slots(runs, num_tokens, block_size):
    """Slot of every token the runs cover (-1 for tokens they do not cover, and
    for runs outside the table)."""
    slots = np.full(num_tokens, -1, dtype=np.int64)
    for t0, blk, e, c in np.asarray(runs, dtype=np.int64).reshape(-1, 4):
        if blk >= 0:
            slots[t0:t0 + c] = blk * block_size + e + np.arange(c)
    return slots


def write_runs_np(key, value, kv_caches, runs) -> None:
    """The write the run descriptors stand for, as slice copies: for every layer,
    `kv_caches[l, blk, 0, e:e+c] = key[l, t0:t0+c]`, likewise value into plane 1.
    key/value [L, T, H, D], kv_caches [L, nb, 2, bs, H, D]."""
    nb = kv_caches.shape[1]
    for t0, blk, e, c in np.asarray(runs, dtype=np.int64).reshape(-1, 4):
        if 0 <= blk < nb and c > 0:
            kv_caches[:, blk, 0, e:e + c] = key[:, t0:t0 + c]
            kv_caches[:, blk, 1, e:e + c] = value[:, t0:t0 + c]


def paged_write_slots_np(batch_indices, positions, kv_indices, kv_indptr, page_size) -> np.ndarray:
    """Slot of every token of a page-table write (the addressing of
    `append_paged_kv_cache`, models/layers/attention.py:76-85, restated as the
    slot rule of scheduler.rs:453-541): for token i with b = batch_indices[i],
    p = positions[i]: `kv_indices[kv_indptr[b] + p // page_size] * page_size +
    p % page_size`; -1 where the write skips the token (no such request, negative
    position, a page outside the request's own table or outside the array, a
    negative page id). int64."""
    bi = np.asarray(batch_indices, dtype=np.int64)
    pos = np.asarray(positions, dtype=np.int64)
    table = np.asarray(kv_indices, dtype=np.int64)
    indptr = np.asarray(kv_indptr, dtype=np.int64)
    batch_size = len(indptr) - 1
    slots = np.full(len(bi), -1, dtype=np.int64)
    for i in range(len(bi)):
        b, p = int(bi[i]), int(pos[i])
        if b < 0 or b >= batch_size or p < 0:
            continue
        entry = int(indptr[b]) + p // page_size
        if entry < 0 or entry >= int(indptr[b + 1]) or entry >= len(table):
            continue
        page = int(table[entry])
        if page >= 0:
            slots[i] = page * page_size + p % page_size
    return slots


def copy_blocks_np(kv_caches, block_maps) -> None:
    """ops/cache_ops.py:8-36 + ops/triton/cache_kernels.py:5-36 on the pool
    viewed as [L, nb, block_elems]; NumPy evaluates the right-hand side first,
    i.e. snapshot semantics."""
    L, nb = kv_caches.shape[0], kv_caches.shape[1]
    pool = kv_caches.reshape(L, nb, -1)
    maps = np.asarray(block_maps, dtype=np.int64)
    src, dst = maps[0::2], maps[1::2]
    pool[:, dst] = pool[:, src]


def save_blocks_to_host_np(gpu, host, src_ids, dst_ids, layer_begin=0, layer_end=None) -> None:
    """kv_worker.py:213-227: host[dst, l] = gpu[l, src]; gpu [L, nb, E], host [nhb, L, E]."""
    layer_end = gpu.shape[0] if layer_end is None else layer_end
    src = np.asarray(src_ids, dtype=np.int64)
    dst = np.asarray(dst_ids, dtype=np.int64)
    host[dst, layer_begin:layer_end] = gpu[layer_begin:layer_end][:, src].swapaxes(0, 1)


def load_blocks_from_host_np(gpu, host, src_ids, dst_ids, layer_begin=0, layer_end=None) -> None:
    """kv_worker.py:197-211: gpu[l, dst] = host[src, l]."""
    layer_end = gpu.shape[0] if layer_end is None else layer_end
    src = np.asarray(src_ids, dtype=np.int64)
    dst = np.asarray(dst_ids, dtype=np.int64)
    gpu[layer_begin:layer_end][:, dst] = host[src, layer_begin:layer_end].swapaxes(0, 1)


def save_blocks_to_disk_np(host, disk, src_ids, dst_ids) -> None:
    """kv_worker.py:239-247 over all layers (:311-322): disk[dst, l] = host[src, l];
    host [nhb, L, E], disk [ndb, L, E]."""
    disk[np.asarray(dst_ids, dtype=np.int64)] = host[np.asarray(src_ids, dtype=np.int64)]


def load_blocks_from_disk_np(host, disk, src_ids, dst_ids) -> None:
    """kv_worker.py:229-237 over all layers (:297-309): host[dst, l] = disk[src, l]."""
    host[np.asarray(dst_ids, dtype=np.int64)] = disk[np.asarray(src_ids, dtype=np.int64)]


# ----------------------------------------------------------------- pure-Python loops


def fill_key_cache_loops(key, value, key_cache, value_cache, slot_mapping) -> None:
    """Element-by-element flat addressing of cache_kernels.py:39-58."""
    H, D = key.shape[1], key.shape[2]
    kf, vf = key.reshape(-1), value.reshape(-1)
    kcf, vcf = key_cache.reshape(-1), value_cache.reshape(-1)
    for i in range(len(slot_mapping)):
        start = i * H * D
        cache_start = int(slot_mapping[i]) * H * D
        for off in range(H * D):
            kcf[cache_start + off] = kf[start + off]
            vcf[cache_start + off] = vf[start + off]


def copy_blocks_loops(kv_caches, block_maps) -> None:
    """Element-by-element flat addressing of cache_kernels.py:13-36."""
    flat = kv_caches.reshape(-1)
    L = kv_caches.shape[0]
    numel_per_layer = kv_caches[0].size
    numel_per_block = kv_caches[0][0].size
    for j in range(len(block_maps) // 2):
        src, dst = int(block_maps[2 * j]), int(block_maps[2 * j + 1])
        for l in range(L):
            base = l * numel_per_layer
            for k in range(numel_per_block):
                flat[base + dst * numel_per_block + k] = flat[base + src * numel_per_block + k]


def append_paged_kv_cache_loops(append_key, append_value, batch_indices, positions,
                                paged_kv_cache, kv_indices, kv_indptr) -> None:
    page_size, H, D = paged_kv_cache.shape[2:]
    for i in range(len(batch_indices)):
        b, p = int(batch_indices[i]), int(positions[i])
        page = int(kv_indices[int(kv_indptr[b]) + p // page_size])
        e = p % page_size
        for h in range(H):
            for d in range(D):
                paged_kv_cache[page, 0, e, h, d] = append_key[i, h, d]
                paged_kv_cache[page, 1, e, h, d] = append_value[i, h, d]


def save_blocks_to_host_loops(gpu, host, src_ids, dst_ids) -> None:
    for l in range(gpu.shape[0]):
        for s, d in zip(src_ids, dst_ids):
            for k in range(gpu.shape[2]):
                host[int(d), l, k] = gpu[l, int(s), k]


def load_blocks_from_host_loops(gpu, host, src_ids, dst_ids) -> None:
    for l in range(gpu.shape[0]):
        for s, d in zip(src_ids, dst_ids):
            for k in range(gpu.shape[2]):
                gpu[l, int(d), k] = host[int(s), l, k]


def save_blocks_to_disk_loops(host, disk, src_ids, dst_ids) -> None:
    """The reference's own order: one pass per layer, one row per entry."""
    for l in range(host.shape[1]):
        for s, d in zip(src_ids, dst_ids):
            disk[int(d)][l] = host[int(s)][l]


def load_blocks_from_disk_loops(host, disk, src_ids, dst_ids) -> None:
    for l in range(host.shape[1]):
        for s, d in zip(src_ids, dst_ids):
            host[int(d)][l] = disk[int(s)][l]


# ----------------------------------------------------------------------- C via ctypes

_clib: Optional[ctypes.CDLL] = None


def build_c_oracle() -> str:
    """Compile oracle/kvc_oracle.c with the Makefile beside it."""
    subprocess.run(["make", "-s", "-B", "-C", ORACLE_DIR, "libkvc_oracle.so"], check=True)
    return C_LIB_PATH


def c_lib() -> ctypes.CDLL:
    global _clib
    if _clib is None:
        if not os.path.exists(C_LIB_PATH):
            build_c_oracle()
        _clib = ctypes.CDLL(C_LIB_PATH)
    return _clib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return ctypes.c_void_p(a.ctypes.data)


def _i64(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int64)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


_L = ctypes.c_int64


def c_fill_key_cache(key, value, key_cache, value_cache, slot_mapping) -> None:
    slots = _i64(slot_mapping)
    c_lib().oracle_fill_key_cache(_p(key), _p(value), _p(key_cache), _p(value_cache), _p(slots),
                                  _L(len(slots)), _L(key.shape[1]), _L(key.shape[2]),
                                  _L(key.itemsize))


def c_reshape_and_cache(key, value, kv_cache, slot_mapping) -> None:
    slots = _i64(slot_mapping)
    _, _, bs, H, D = kv_cache.shape
    c_lib().oracle_reshape_and_cache(_p(key), _p(value), _p(kv_cache), _p(slots), _L(len(slots)),
                                     _L(bs), _L(H), _L(D), _L(key.itemsize))


def c_append_paged_kv_cache(append_key, append_value, batch_indices, positions, paged_kv_cache,
                            kv_indices, kv_indptr, kv_last_page_len=None) -> None:
    bi, pos, ind, ptr = _i32(batch_indices), _i32(positions), _i32(kv_indices), _i32(kv_indptr)
    _, _, page_size, H, D = paged_kv_cache.shape
    c_lib().oracle_append_paged_kv_cache(_p(append_key), _p(append_value), _p(bi), _p(pos),
                                         _p(paged_kv_cache), _p(ind), _p(ptr), _L(len(bi)), _L(H),
                                         _L(D), _L(page_size), _L(append_key.itemsize))


def c_get_seq_lens(kv_indptr, kv_last_page_len, page_size) -> np.ndarray:
    ptr, last = _i32(kv_indptr), _i32(kv_last_page_len)
    out = np.zeros(len(last), dtype=np.int32)
    c_lib().oracle_get_seq_lens(_p(ptr), _p(last), _L(len(last)), ctypes.c_int32(page_size), _p(out))
    return out


def c_get_batch_indices_positions(append_indptr, seq_lens, nnz) -> Tuple[np.ndarray, np.ndarray]:
    ptr, sl = _i32(append_indptr), _i32(seq_lens)
    bi = np.zeros(nnz, dtype=np.int32)
    pos = np.zeros(nnz, dtype=np.int32)
    c_lib().oracle_get_batch_indices_positions(_p(ptr), _p(sl), _L(len(sl)), _p(bi), _p(pos))
    return bi, pos


def c_copy_blocks(kv_caches, block_maps) -> None:
    maps = _i64(block_maps)
    c_lib().oracle_copy_blocks(_p(kv_caches), _p(maps), _L(len(maps) // 2), _L(kv_caches.shape[0]),
                               _L(kv_caches[0].size), _L(kv_caches[0][0].size),
                               _L(kv_caches.itemsize))


def c_save_blocks_to_host(gpu, host, src_ids, dst_ids, layer_begin=0, layer_end=None) -> None:
    src, dst = _i64(src_ids), _i64(dst_ids)
    L, nb = gpu.shape[0], gpu.shape[1]
    block_bytes = gpu[0][0].size * gpu.itemsize
    c_lib().oracle_save_blocks_to_host(_p(gpu), _p(host), _p(src), _p(dst), _L(len(src)), _L(L),
                                       _L(nb), _L(block_bytes), _L(layer_begin),
                                       _L(L if layer_end is None else layer_end))


def c_load_blocks_from_host(gpu, host, src_ids, dst_ids, layer_begin=0, layer_end=None) -> None:
    src, dst = _i64(src_ids), _i64(dst_ids)
    L, nb = gpu.shape[0], gpu.shape[1]
    block_bytes = gpu[0][0].size * gpu.itemsize
    c_lib().oracle_load_blocks_from_host(_p(gpu), _p(host), _p(src), _p(dst), _L(len(src)), _L(L),
                                         _L(nb), _L(block_bytes), _L(layer_begin),
                                         _L(L if layer_end is None else layer_end))

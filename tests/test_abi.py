"""The C-ABI library loads and exports every symbol include/*.h declares.

No kernel is launched here: only symbol lookup and entry points that return
before their first HIP call (argument validation, pure host arithmetic).
"""
import ctypes
import os
import re

import numpy as np
import pytest

from lmserve_amd import _lib

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "kvcache.h")
EXPERIMENTAL_HEADER = os.path.join(REPO, "include", "kvcache_experimental.h")


def header_text(*paths):
    return "\n".join(re.sub(r"/\*.*?\*/", "", open(p).read(), flags=re.S) for p in paths)


def declared_functions(*paths):
    text = header_text(*(paths or (HEADER, EXPERIMENTAL_HEADER)))
    return sorted(set(re.findall(r"\b(kvc_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions(HEADER)     # the stable header alone
    for must in ("kvc_reshape_and_cache", "kvc_reshape_and_cache_layers",
                 "kvc_append_paged_kv_cache", "kvc_append_paged_kv_cache_layers",
                 "kvc_get_seq_lens", "kvc_get_batch_indices_positions", "kvc_copy_blocks",
                 "kvc_swap_out", "kvc_swap_in", "kvc_swap_staging_bytes",
                 "kvc_host_alloc_pinned", "kvc_host_free_pinned", "kvc_last_error_string",
                 "kvc_abi_version"):
        assert must in names
    # knobs, launch introspection and the host-side row mover are not part of the stable surface
    for name in names:
        assert not name.startswith(("kvc_set_tuning", "kvc_get_tuning", "kvc_last_launch_info", "kvc_row_mover")), name
    assert "kvc_row_mover_cancel" in declared_functions(EXPERIMENTAL_HEADER)


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(handle, name), f"{name} is declared in kvcache.h but not exported"


def test_python_binding_types_every_declared_symbol():
    for name in declared_functions():
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature in lmserve_amd/_lib.py"


def test_binding_arity_matches_the_header():
    text = header_text(HEADER, EXPERIMENTAL_HEADER)
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", text, flags=re.S)
        if m is None:
            continue  # tuning hook: exported, not part of the public header
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else len(params.split(","))
        assert n == len(argtypes), f"{name}: header has {n} parameters, binding {len(argtypes)}"


def test_abi_version():
    assert _lib.lib().kvc_abi_version() == _lib.KVC_ABI_VERSION


def test_argument_validation_returns_codes_not_crashes():
    L = _lib.lib()
    assert L.kvc_copy_blocks(None, None, -1, 1, 1, 1, 1, None) == _lib.KVC_ERR_INVALID_ARG
    assert "negative" in _lib.last_error()
    # empty work is OK even with null pointers
    assert L.kvc_copy_blocks(None, None, 0, 32, 1 << 32, 65536, 65536, None) == _lib.KVC_OK
    assert L.kvc_reshape_and_cache(None, None, None, None, None, 8, 0, 1024, 1024, 1024, 16,
                                   32768, 1024, 64, 2, None) == _lib.KVC_OK
    # unsupported element width / slot width
    assert L.kvc_reshape_and_cache(1, 1, 1, 1, 1, 8, 4, 1024, 1024, 1024, 16, 32768, 1024, 64, 3,
                                   None) == _lib.KVC_ERR_UNSUPPORTED
    assert L.kvc_reshape_and_cache(256, 256, 256, 256, 256, 2, 4, 1024, 1024, 1024, 16, 32768,
                                   1024, 64, 2, None) == _lib.KVC_ERR_UNSUPPORTED
    # token stride smaller than a row
    assert L.kvc_reshape_and_cache(256, 256, 256, 256, 256, 8, 4, 1024, 512, 1024, 16, 32768,
                                   1024, 64, 2, None) == _lib.KVC_ERR_INVALID_ARG
    with pytest.raises(ValueError):
        _lib.check(_lib.KVC_ERR_INVALID_ARG)
    with pytest.raises(TypeError):
        _lib.check(_lib.KVC_ERR_UNSUPPORTED)
    with pytest.raises(IndexError):
        _lib.check(_lib.KVC_ERR_OUT_OF_RANGE)


def test_swap_rejects_out_of_range_host_lists_before_touching_the_gpu():
    L = _lib.lib()
    src = np.asarray([0, 5, 99], dtype=np.int64)
    dst = np.asarray([0, 1, 2], dtype=np.int64)
    rc = L.kvc_swap_out(4096, 4096, src.ctypes.data, dst.ctypes.data, 3, 2, 64 * 1024, 1024, 64, 8,
                        0, 2, 4096, 1 << 20, _lib.KVC_SWAP_STAGED, None, None)
    assert rc == _lib.KVC_ERR_OUT_OF_RANGE and "99" in _lib.last_error()
    rc = L.kvc_swap_in(4096, 4096, dst.ctypes.data, src.ctypes.data, 3, 2, 64 * 1024, 1024, 64, 8,
                       0, 2, 4096, 1 << 20, _lib.KVC_SWAP_STAGED, None, None)
    assert rc == _lib.KVC_ERR_OUT_OF_RANGE
    # bad layer range, unknown mode, staging too small
    ok = np.asarray([0, 1, 2], dtype=np.int64)
    assert L.kvc_swap_out(4096, 4096, ok.ctypes.data, ok.ctypes.data, 3, 2, 64 * 1024, 1024, 64, 8,
                          1, 3, 4096, 1 << 20, 0, None, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_swap_out(4096, 4096, ok.ctypes.data, ok.ctypes.data, 3, 2, 64 * 1024, 1024, 64, 8,
                          0, 2, 4096, 1 << 20, 7, None, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_swap_out(4096, 4096, ok.ctypes.data, ok.ctypes.data, 3, 2, 64 * 1024, 1024, 64, 8,
                          0, 2, 4096, 512, 0, None, None) == _lib.KVC_ERR_STAGING


def test_staging_size_arithmetic():
    L = _lib.lib()
    blk, nl = 65536, 80
    ids = 2 * 8192 * 8
    # default ring slot: as many whole blocks as fit 64 MiB, more when that would cut the call
    # into more than 128 chunks
    per_block = nl * blk
    chunk = (64 << 20) // per_block
    assert chunk == 12
    assert L.kvc_swap_staging_bytes(1024, nl, blk, _lib.KVC_SWAP_STAGED, 0) == 2 * 1024 * 8 + 2 * chunk * per_block
    assert L.kvc_swap_staging_bytes(8192, nl, blk, _lib.KVC_SWAP_STAGED, 0) == ids + 2 * 64 * per_block
    assert L.kvc_swap_staging_bytes(8192, 1, blk, _lib.KVC_SWAP_STAGED, 0) == ids + 2 * 1024 * blk
    assert L.kvc_swap_staging_bytes(8192, nl, blk, _lib.KVC_SWAP_STAGED, 4) == ids + 8 * per_block
    assert L.kvc_swap_staging_bytes(3, nl, blk, _lib.KVC_SWAP_STAGED, 100) == 256 + 6 * per_block
    assert L.kvc_swap_staging_bytes(8192, nl, blk, _lib.KVC_SWAP_DIRECT, 0) == ids
    # the per-call choice wants room for the staged path
    assert (L.kvc_swap_staging_bytes(8192, nl, blk, _lib.KVC_SWAP_AUTO, 0)
            == L.kvc_swap_staging_bytes(8192, nl, blk, _lib.KVC_SWAP_STAGED, 0))
    assert L.kvc_swap_staging_bytes(8192, nl, blk, 3, 0) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_swap_staging_bytes(-1, nl, blk, 0, 0) < 0


def test_rope_and_index_build_validate_their_arguments():
    L = _lib.lib()
    f = L.kvc_rotary_pos_emb
    #  q, k, pos, pos_bytes, cs, max_pos, T, Hq, Hkv, D, rd, qs, ks, qo, ko, qos, kos, dtype, stream
    ok = [256, 256, 256, 4, 256, 100, 4, 8, 2, 64, 64, 512, 128, 256, 256, 512, 128, _lib.KVC_DTYPE_BF16, None]

    def call(**kw):
        names = ["q", "k", "pos", "pos_bytes", "cs", "max_pos", "T", "Hq", "Hkv", "D", "rd", "qs", "ks",
                 "qo", "ko", "qos", "kos", "dtype", "stream"]
        a = list(ok)
        for k, v in kw.items():
            a[names.index(k)] = v
        return f(*a)

    assert call(T=0) == _lib.KVC_OK                         # nothing to do, nothing launched
    assert call(dtype=7) == _lib.KVC_ERR_UNSUPPORTED
    assert call(rd=65) == _lib.KVC_ERR_INVALID_ARG          # odd
    assert call(rd=128) == _lib.KVC_ERR_INVALID_ARG         # beyond head_dim
    assert call(D=1024, rd=1024, qs=8192, ks=2048, qos=8192, kos=2048) == _lib.KVC_ERR_UNSUPPORTED
    assert call(pos_bytes=2) == _lib.KVC_ERR_UNSUPPORTED
    assert call(q=None) == _lib.KVC_ERR_INVALID_ARG
    assert call(ko=None) == _lib.KVC_ERR_INVALID_ARG        # no cache and no key_out: nowhere to put K
    assert call(qs=100) == _lib.KVC_ERR_INVALID_ARG         # stride smaller than the row
    g = L.kvc_build_write_index
    no_runs = (None, None, None, 0, None)
    assert g(None, None, None, None, -1, 0, 16, 0, 1, 1, 1, 1, 1, 1, *no_runs) == _lib.KVC_ERR_INVALID_ARG
    assert g(None, None, None, None, 2, 0, 16, 4, 1, 1, 1, 1, 1, 1, *no_runs) == _lib.KVC_ERR_INVALID_ARG
    assert g(1, 1, 1, 1, 2, 4, 0, 4, 1, 1, 1, 1, 1, 1, *no_runs) == _lib.KVC_ERR_INVALID_ARG   # page_size 0
    # a run list needs its prefix sums and its count, 16-byte alignment and room for every run
    assert g(1, 1, 1, 1, 2, 4, 16, 64, 1, 1, 1, 1, 1, 1, None, 16, 1, 64, None) == _lib.KVC_ERR_INVALID_ARG
    assert g(1, 1, 1, 1, 2, 4, 16, 64, 1, 1, 1, 1, 1, 1, 1, 24, 1, 64, None) == _lib.KVC_ERR_INVALID_ARG
    assert g(1, 1, 1, 1, 2, 4, 16, 64, 1, 1, 1, 1, 1, 1, 1, 16, 1, 7, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_set_tuning(b"no_such_knob", 1) == _lib.KVC_ERR_INVALID_ARG


def test_tuning_knobs_read_back_and_reset():
    L = _lib.lib()
    assert L.kvc_tuning_modified() == 0
    defaults = {"copy_unroll": 0, "gather_unroll": 0, "copy_nt": 1, "copy_max_wgs": 0, "copy_order": 0,
                "write_vpt": 0, "write_nt": 3, "write_order": 0, "write_threads": 0, "write_planes": 1,
                "write_planes_vpt": 0, "write_planes_min_bytes": 256 << 10, "write_planes_max_vpr": 256, "write_planes_threads": 0,
                "write_pipe": -1, "direct_max_wgs": 96, "auto_min_extent_bytes": 1 << 20, "rope_threads": 0, "disk_bounce_mib": 4,
                "runs_unroll": 0, "runs_order": 1, "runs_nt": 1, "rope_nt": 0, "host_rows_nt": 1, "direct_max_wgs_in": 16}
    for key, value in defaults.items():
        assert _lib.get_tuning(key) == value, key
    for i, key in enumerate(defaults):
        _lib.set_tuning(key, 100 + i)
        assert _lib.get_tuning(key) == 100 + i
        assert L.kvc_tuning_modified() == i + 1
    _lib.reset_tuning()
    assert L.kvc_tuning_modified() == 0
    for key, value in defaults.items():
        assert _lib.get_tuning(key) == value, key
    out = ctypes.c_int(0)
    assert L.kvc_get_tuning(b"no_such_knob", ctypes.byref(out)) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_get_tuning(b"copy_nt", None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_last_launch_info(99) == _lib.KVC_ERR_INVALID_ARG
    import torch
    if not torch.cuda.is_available():       # nothing can have been launched in this process
        assert _lib.last_launch()["kernel"] == _lib.KVC_KERNEL_NONE


def test_plans_and_prepared_swap_validate_before_touching_the_gpu():
    L = _lib.lib()
    h = ctypes.c_void_p()
    create = L.kvc_write_plan_create
    assert create(1, 1, 1, 1, 1, 4, 2, 8, 8, 128, 16, 2, ctypes.byref(h)) == _lib.KVC_OK and h.value
    # a null key pointer is caught by the write's own checks, before any launch
    assert L.kvc_write_plan_append(h, None, 1, 1024, 1024, 1, 32768, 4, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_write_plan_append(h, 1, 1, 512, 1024, 1, 32768, 4, None) == _lib.KVC_ERR_INVALID_ARG
    assert "stride" in _lib.last_error()
    assert L.kvc_write_plan_resolve_slots(h, None, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_write_plan_resolve_slots(None, 1, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_write_plan_destroy(h) == _lib.KVC_OK
    assert L.kvc_write_plan_destroy(None) == _lib.KVC_OK
    assert create(1, 1, 1, 1, 1, 4, 2, 8, 8, 128, 0, 2, ctypes.byref(h)) == _lib.KVC_ERR_INVALID_ARG
    assert h.value is None
    assert create(1, 1, 1, 1, 1, 4, 2, 8, 8, 128, 16, 3, ctypes.byref(h)) == _lib.KVC_ERR_UNSUPPORTED
    assert create(None, 1, 1, 1, 1, 4, 2, 8, 8, 128, 16, 2, ctypes.byref(h)) == _lib.KVC_ERR_INVALID_ARG
    assert create(1, 1, 1, 1, 1, 4, 2, 8, 8, 128, 16, 2, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_write_plan_append(None, 1, 1, 1, 1, 1, 1, 1, None) == _lib.KVC_ERR_INVALID_ARG

    rcreate = L.kvc_rotary_plan_create
    #        bi pos cs max nnz Hq Hkv D rd idx ptr B nidx ps dtype out
    assert rcreate(1, 1, 1, 100, 4, 8, 2, 64, 64, 1, 1, 2, 8, 16, 0, ctypes.byref(h)) == _lib.KVC_OK
    assert L.kvc_rotary_plan_run(h, None, 1, 1, 512, 128, 128, 1, None, 1, 4096, 4, None) == \
        _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_rotary_plan_resolve_slots(h, None, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_rotary_plan_resolve_slots(None, 1, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_rotary_plan_destroy(h) == _lib.KVC_OK
    assert rcreate(1, 1, 1, 100, 4, 8, 2, 64, 63, 1, 1, 2, 8, 16, 0, ctypes.byref(h)) == _lib.KVC_ERR_INVALID_ARG
    assert rcreate(1, 1, 1, 100, 4, 8, 2, 64, 64, 1, 1, 2, 8, 16, 9, ctypes.byref(h)) == _lib.KVC_ERR_UNSUPPORTED
    assert rcreate(1, 1, None, 100, 4, 8, 2, 64, 64, 1, 1, 2, 8, 16, 0, ctypes.byref(h)) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_rotary_plan_run(None, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, None) == _lib.KVC_ERR_INVALID_ARG

    ids = np.asarray([0, 5, 63], dtype=np.int64)
    bad = np.asarray([0, 64, 1], dtype=np.int64)
    prep = L.kvc_swap_prepare
    assert prep(None, None, 0, 64, 8, None, 0, None) == _lib.KVC_OK            # nothing to prepare
    assert prep(bad.ctypes.data, ids.ctypes.data, 3, 64, 64, 4096, 4096, None) == _lib.KVC_ERR_OUT_OF_RANGE
    assert "gpu block id 64" in _lib.last_error()
    assert prep(ids.ctypes.data, bad.ctypes.data, 3, 64, 64, 4096, 4096, None) == _lib.KVC_ERR_OUT_OF_RANGE
    assert prep(ids.ctypes.data, None, 3, 64, 64, 4096, 4096, None) == _lib.KVC_ERR_INVALID_ARG
    assert prep(ids.ctypes.data, ids.ctypes.data, 3, 64, 64, None, 4096, None) == _lib.KVC_ERR_STAGING
    assert prep(ids.ctypes.data, ids.ctypes.data, 3, 64, 64, 4096 + 8, 4096, None) == _lib.KVC_ERR_STAGING
    assert prep(ids.ctypes.data, ids.ctypes.data, 3, 64, 64, 4096, 16, None) == _lib.KVC_ERR_STAGING
    out = L.kvc_swap_out_prepared
    #  pool host host_ids n L layer_stride block nb nhb lb le staging bytes mode ks cs
    assert out(4096, 4096, None, 3, 2, 65536, 1024, 64, 64, 0, 2, 4096, 4096, _lib.KVC_SWAP_STAGED,
               None, None) == _lib.KVC_ERR_INVALID_ARG                          # staged needs the host ids
    assert out(4096, 4096, None, 3, 2, 65536, 1024, 64, 64, 1, 3, 4096, 4096, _lib.KVC_SWAP_DIRECT,
               None, None) == _lib.KVC_ERR_INVALID_ARG                          # layer range
    assert out(4096, 4096, None, 3, 2, 65536, 1024, 64, 64, 0, 2, 4096, 16, _lib.KVC_SWAP_DIRECT,
               None, None) == _lib.KVC_ERR_STAGING
    assert out(4096, 4096, None, 0, 2, 65536, 1024, 64, 64, 0, 2, None, 0, _lib.KVC_SWAP_DIRECT,
               None, None) == _lib.KVC_OK
    assert out(4096, 4096, None, 0, 2, 65536, 1024, 64, 64, 0, 2, None, 0, _lib.KVC_SWAP_AUTO,
               None, None) == _lib.KVC_OK                                        # nothing to move
    assert out(4096, 4096, None, 3, 2, 65536, 1024, 64, 64, 0, 2, 4096, 4096, 3,
               None, None) == _lib.KVC_ERR_INVALID_ARG                          # no such mode
    assert L.kvc_swap_in_prepared(None, 4096, None, 3, 2, 65536, 1024, 64, 64, 0, 2, 4096, 4096,
                                  _lib.KVC_SWAP_DIRECT, None, None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_thread_release() == _lib.KVC_OK       # nothing held by this thread: a no-op


def test_pairs_are_ordered_by_host_block_id_like_a_stable_sort():
    L = _lib.lib()
    rng = np.random.default_rng(3)
    for n in (0, 1, 2, 7, 1000):
        gpu = rng.integers(0, 1 << 20, size=n).astype(np.int64)
        host = rng.integers(0, max(1, n // 3), size=n).astype(np.int64)      # many ties
        order = np.argsort(host, kind="stable")
        g, h = gpu.copy(), host.copy()
        assert L.kvc_order_pairs_by_host_id(g.ctypes.data, h.ctypes.data, n) == _lib.KVC_OK
        assert np.array_equal(h, host[order]) and np.array_equal(g, gpu[order])
    asc = np.asarray([0, 0, 3, 9], dtype=np.int64)
    g = np.asarray([5, 4, 3, 2], dtype=np.int64)
    assert L.kvc_order_pairs_by_host_id(g.ctypes.data, asc.ctypes.data, 4) == _lib.KVC_OK
    assert g.tolist() == [5, 4, 3, 2] and asc.tolist() == [0, 0, 3, 9]       # already ascending: untouched
    assert L.kvc_order_pairs_by_host_id(None, None, 0) == _lib.KVC_OK
    assert L.kvc_order_pairs_by_host_id(None, asc.ctypes.data, 4) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_order_pairs_by_host_id(g.ctypes.data, asc.ctypes.data, -1) == _lib.KVC_ERR_INVALID_ARG


@pytest.mark.parametrize("threads", [1, 3, 8])
def test_host_rows_between_a_dense_buffer_and_scattered_host_blocks(threads):
    """kvc_host_copy_rows runs on the host alone: rows of one layer to and from
    scattered blocks of a [num_host_blocks, L, block] pool, against NumPy indexing,
    the rest of the pool untouched; then the argument checks."""
    L_fn = _lib.lib().kvc_host_copy_rows
    rng = np.random.default_rng(7 + threads)
    nhb, layers, row = 97, 3, 40 << 10          # 120 KiB host blocks, 40 KiB rows
    pool = rng.integers(0, 255, size=(nhb, layers, row), dtype=np.uint8)
    for n in (1, 8, 61):                        # below one MiB (inline) and above (threads)
        ids = rng.permutation(nhb)[:n].astype(np.int64)
        for layer in (0, layers - 1):
            dense = rng.integers(0, 255, size=(n, row), dtype=np.uint8)
            want = pool.copy()
            want[ids, layer] = dense
            assert L_fn(pool.ctypes.data, nhb, layers * row, layer * row, dense.ctypes.data,
                        ids.ctypes.data, n, row, 1, threads) == 0
            assert np.array_equal(pool, want)
            back = np.zeros_like(dense)
            assert L_fn(pool.ctypes.data, nhb, layers * row, layer * row, back.ctypes.data,
                        ids.ctypes.data, n, row, 0, threads) == 0
            assert np.array_equal(back, dense) and np.array_equal(pool, want)
    ids = np.asarray([0, nhb], dtype=np.int64)
    dense = np.zeros((2, row), dtype=np.uint8)
    before = pool.copy()
    assert L_fn(pool.ctypes.data, nhb, layers * row, 0, dense.ctypes.data, ids.ctypes.data, 2, row, 1,
                threads) == _lib.KVC_ERR_OUT_OF_RANGE
    assert "host block id" in _lib.last_error()
    assert L_fn(pool.ctypes.data, nhb, layers * row, 2 * row + 1, dense.ctypes.data, ids.ctypes.data, 1, row,
                1, threads) == _lib.KVC_ERR_INVALID_ARG
    assert L_fn(None, nhb, layers * row, 0, dense.ctypes.data, ids.ctypes.data, 1, row, 1, threads) \
        == _lib.KVC_ERR_INVALID_ARG
    assert L_fn(pool.ctypes.data, nhb, layers * row, 0, dense.ctypes.data, ids.ctypes.data, 0, row, 1,
                threads) == 0
    assert np.array_equal(pool, before)


def test_row_mover_runs_its_jobs_in_order_and_reports_errors():
    """The queue form of the host row copies, without events (so on the CPU): jobs
    finish in the order of their tickets, a wait covers everything before it, the
    id list may go away after the submit, bad arguments fail at the submit."""
    L = _lib.lib()
    mover = ctypes.c_void_p()
    assert L.kvc_row_mover_create(3, ctypes.byref(mover)) == 0
    try:
        rng = np.random.default_rng(11)
        nhb, layers, row, n = 64, 4, 48 << 10, 40
        pool = rng.integers(0, 255, size=(nhb, layers, row), dtype=np.uint8)
        want = pool.copy()
        dense = [rng.integers(0, 255, size=(n, row), dtype=np.uint8) for _ in range(layers)]
        tickets = []
        for layer in range(layers):
            ids = rng.permutation(nhb)[:n].astype(np.int64)
            want[ids, layer] = dense[layer]
            tickets.append(L.kvc_row_mover_submit(mover, None, pool.ctypes.data, nhb, layers * row, layer * row,
                                                  dense[layer].ctypes.data, ids.ctypes.data, n, row, 1))
            ids[:] = -1                     # the mover keeps its own copy of the list
        assert tickets == [0, 1, 2, 3]
        assert L.kvc_row_mover_wait(mover, tickets[-1]) == 0
        assert all(L.kvc_row_mover_done(mover, t) == 1 for t in tickets)
        assert np.array_equal(pool, want)
        # out of the pool again, one job reading what the job before it wrote
        ids = rng.permutation(nhb)[:n].astype(np.int64)
        back = np.zeros((n, row), dtype=np.uint8)
        t1 = L.kvc_row_mover_submit(mover, None, pool.ctypes.data, nhb, layers * row, 2 * row,
                                    dense[0].ctypes.data, ids.ctypes.data, n, row, 1)
        t2 = L.kvc_row_mover_submit(mover, None, pool.ctypes.data, nhb, layers * row, 2 * row,
                                    back.ctypes.data, ids.ctypes.data, n, row, 0)
        assert (t1, t2) == (4, 5)
        assert L.kvc_row_mover_wait(mover, t2) == 0
        assert np.array_equal(back, dense[0])
        bad = np.asarray([nhb], dtype=np.int64)
        assert L.kvc_row_mover_submit(mover, None, pool.ctypes.data, nhb, layers * row, 0, back.ctypes.data,
                                      bad.ctypes.data, 1, row, 1) == _lib.KVC_ERR_OUT_OF_RANGE
        assert L.kvc_row_mover_wait(mover, 99) == _lib.KVC_ERR_INVALID_ARG
        assert L.kvc_row_mover_submit(mover, None, pool.ctypes.data, nhb, layers * row, 0, back.ctypes.data,
                                      bad.ctypes.data, 0, row, 1) == 6          # an empty job is a job
        assert L.kvc_row_mover_wait(mover, 6) == 0
    finally:
        assert L.kvc_row_mover_destroy(mover) == 0
    assert L.kvc_row_mover_destroy(None) == 0
    assert L.kvc_row_mover_submit(None, None, None, 0, 0, 0, None, None, 0, 0, 0) == _lib.KVC_ERR_INVALID_ARG


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """include/kvcache.h compiles as C99 with no extensions, and a C translation
    unit that only knows the header links against libkvcache.so and runs the
    entry points that need no GPU."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "kvcache.h"\n'
        "int main(void) {\n"
        "  if (kvc_abi_version() != KVC_ABI_VERSION) return 1;\n"
        "  if (kvc_copy_blocks(0, 0, -1, 1, 1, 1, 1, 0) != KVC_ERR_INVALID_ARG) return 2;\n"
        '  if (!strstr(kvc_last_error_string(), "negative")) return 3;\n'
        "  if (kvc_swap_staging_bytes(3, 80, 65536, KVC_SWAP_DIRECT, 0) != 256) return 4;\n"
        "  if (kvc_disk_close(0) != KVC_OK) return 5;\n"
        '  puts("c ok");\n  return 0;\n}\n')
    exe = tmp_path / "use"
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", os.path.join(REPO, "include"),
                    str(src), "-L", lib_dir, "-lkvcache", f"-Wl,-rpath,{lib_dir}", "-o", str(exe)],
                   check=True, capture_output=True, text=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and "c ok" in out.stdout, out.stdout + out.stderr


def test_call_extension_is_built_and_binds_the_same_library():
    """`_kvc_fast` (the CPython entry of the per-layer calls) sits next to the library,
    reports the library's ABI version and exposes one function per call it serves."""
    if os.environ.get("KVC_DISABLE_CALL_EXTENSION"):
        pytest.skip("switched off in the environment")
    mod = _lib.fast()
    assert mod is not None, "lmserve_amd/_kvc_fast.so is missing: run python -m lmserve_amd.build"
    assert mod.abi_version == _lib.KVC_ABI_VERSION and mod.NOT_FAST == 1
    for name in ("write_plan_append", "rotary_plan_run", "append_paged", "reshape_and_cache",
                 "rotary_pos_emb", "rotary_append_paged", "scalar_type_code"):
        assert callable(getattr(mod, name)), name
        assert _lib.fast_entry(name) is getattr(mod, name)
    # not tensors: every entry hands the call back to Python (1), it never guesses
    assert mod.append_paged(*([None] * 8), 0, None) == 1
    assert mod.reshape_and_cache(None, None, None, None, 0, None) == 1
    with pytest.raises(TypeError):
        mod.append_paged(None)


def test_operators_fail_loudly_without_the_library(monkeypatch, tmp_path):
    """No CPU fallback: with the shared library absent every entry into the
    binding raises, and so do the operators that sit on it."""
    import torch

    import lmserve_amd as kvc

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libkvcache.so"))
    with pytest.raises(_lib.KVCacheLibraryError, match="no CPU fallback"):
        _lib.lib()
    with pytest.raises(_lib.KVCacheLibraryError):
        kvc.DiskTier(str(tmp_path / "x.npy"), (2, 1, 8), np.uint16)
    # the device operators refuse CPU tensors before they even reach the library
    pool = torch.zeros(1, 4, 2, 2, 1, 4, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        kvc.copy_blocks(pool, {0: [1]})
    with pytest.raises(ValueError):
        kvc.reshape_and_cache(torch.zeros(1, 1, 4, dtype=torch.bfloat16),
                              torch.zeros(1, 1, 4, dtype=torch.bfloat16), pool[0],
                              torch.zeros(1, dtype=torch.int64))


# ------------------------------------------------------------------ no host-side wait is unbounded
def _mover_fixture(n=6, row=64, layers=2, nhb=8):
    rng = np.random.default_rng(3)
    pool = np.zeros((nhb, layers, row), dtype=np.uint8)
    dense = rng.integers(0, 255, size=(n, row), dtype=np.uint8)
    ids = rng.permutation(nhb)[:n].astype(np.int64)
    return pool, dense, ids


def test_row_mover_job_starts_when_its_host_flag_is_set():
    import threading
    import time
    L = _lib.lib()
    mover = ctypes.c_void_p()
    assert L.kvc_row_mover_create(2, ctypes.byref(mover)) == 0
    pool, dense, ids = _mover_fixture()
    flag = np.zeros(1, dtype=np.int32)
    try:
        t = L.kvc_row_mover_submit_after_flag(mover, flag.ctypes.data, pool.ctypes.data, 8, 2 * 64, 64,
                                              dense.ctypes.data, ids.ctypes.data, 6, 64, 1)
        assert t == 0
        time.sleep(0.05)
        assert L.kvc_row_mover_done(mover, t) == 0 and not pool.any()       # still waiting, nothing moved
        threading.Timer(0.05, lambda: flag.__setitem__(0, 1)).start()
        assert L.kvc_row_mover_wait(mover, t) == 0
        assert np.array_equal(pool[ids, 1], dense)
    finally:
        assert L.kvc_row_mover_destroy(mover) == 0


def test_row_mover_gives_up_at_its_deadline_and_drains_what_was_queued_behind():
    """A job whose flag is never set (the stand-in for an event that never
    completes) fails with KVC_ERR_TIMEOUT after the mover's deadline, the jobs
    already queued behind it complete at once without copying, a job submitted
    afterwards runs normally, and destroy returns."""
    import time
    L = _lib.lib()
    mover = ctypes.c_void_p()
    assert L.kvc_row_mover_create(2, ctypes.byref(mover)) == 0
    assert L.kvc_row_mover_set_timeout_ms(mover, 150) == 0
    pool, dense, ids = _mover_fixture()
    never = np.zeros(1, dtype=np.int32)
    t0 = time.monotonic()
    stuck = L.kvc_row_mover_submit_after_flag(mover, never.ctypes.data, pool.ctypes.data, 8, 2 * 64, 0,
                                              dense.ctypes.data, ids.ctypes.data, 6, 64, 1)
    behind = [L.kvc_row_mover_submit(mover, None, pool.ctypes.data, 8, 2 * 64, 64, dense.ctypes.data,
                                     ids.ctypes.data, 6, 64, 1) for _ in range(3)]
    assert stuck == 0 and behind == [1, 2, 3]
    assert L.kvc_row_mover_wait(mover, behind[-1]) == _lib.KVC_ERR_TIMEOUT
    waited = time.monotonic() - t0
    assert 0.14 <= waited < 2.0, waited
    assert "not reached" in _lib.last_error()
    assert not pool.any()                                   # neither the stuck job nor the ones behind it copied
    assert L.kvc_row_mover_done(mover, behind[-1]) == 1
    # the error has been collected: the mover works again
    later = L.kvc_row_mover_submit(mover, None, pool.ctypes.data, 8, 2 * 64, 64, dense.ctypes.data,
                                   ids.ctypes.data, 6, 64, 1)
    assert later == 4 and L.kvc_row_mover_wait(mover, later) == 0
    assert np.array_equal(pool[ids, 1], dense)
    assert L.kvc_row_mover_destroy(mover) == 0


def test_row_mover_cancel_and_destroy_do_not_wait_for_a_stuck_job():
    import time
    L = _lib.lib()
    mover = ctypes.c_void_p()
    assert L.kvc_row_mover_create(1, ctypes.byref(mover)) == 0
    assert L.kvc_row_mover_set_timeout_ms(mover, -1) == 0           # no deadline at all
    pool, dense, ids = _mover_fixture()
    never = np.zeros(1, dtype=np.int32)
    stuck = L.kvc_row_mover_submit_after_flag(mover, never.ctypes.data, pool.ctypes.data, 8, 2 * 64, 0,
                                              dense.ctypes.data, ids.ctypes.data, 6, 64, 1)
    behind = L.kvc_row_mover_submit(mover, None, pool.ctypes.data, 8, 2 * 64, 0, dense.ctypes.data,
                                    ids.ctypes.data, 6, 64, 1)
    time.sleep(0.05)
    assert L.kvc_row_mover_done(mover, stuck) == 0
    t0 = time.monotonic()
    assert L.kvc_row_mover_cancel(mover) == 0
    assert L.kvc_row_mover_wait(mover, behind) == _lib.KVC_ERR_CANCELLED
    assert not pool.any()
    assert L.kvc_row_mover_destroy(mover) == 0
    assert time.monotonic() - t0 < 1.0
    # destroy alone, with a deadline: returns within one deadline of the call
    mover = ctypes.c_void_p()
    assert L.kvc_row_mover_create(1, ctypes.byref(mover)) == 0
    assert L.kvc_row_mover_set_timeout_ms(mover, 100) == 0
    for _ in range(4):
        L.kvc_row_mover_submit_after_flag(mover, never.ctypes.data, pool.ctypes.data, 8, 2 * 64, 0,
                                          dense.ctypes.data, ids.ctypes.data, 6, 64, 1)
    t0 = time.monotonic()
    assert L.kvc_row_mover_destroy(mover) == 0
    assert time.monotonic() - t0 < 1.0                      # one deadline, not four
    assert L.kvc_row_mover_cancel(None) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_row_mover_set_timeout_ms(None, 5) == _lib.KVC_ERR_INVALID_ARG


def test_swap_mode_can_be_asked_before_the_call():
    L = _lib.lib()
    MiB = 1 << 20
    consecutive = np.arange(64, dtype=np.int64)
    scattered = np.arange(0, 128, 2, dtype=np.int64)
    big = L.kvc_swap_staging_bytes(64, 1, 64 << 10, _lib.KVC_SWAP_STAGED, 0)
    # one layer of 64 consecutive 64 KiB blocks is one 4 MiB extent: the copy engines
    assert L.kvc_swap_resolve_mode(consecutive.ctypes.data, 64, 1, 64 << 10, big) == _lib.KVC_SWAP_STAGED
    # every second host block: 64 KiB extents, the direct kernel
    assert L.kvc_swap_resolve_mode(scattered.ctypes.data, 64, 1, 64 << 10, big) == _lib.KVC_SWAP_DIRECT
    # all 80 layers of a scattered block travel as one 5 MiB extent
    assert L.kvc_swap_resolve_mode(scattered.ctypes.data, 64, 80, 64 << 10, 64 * MiB) == _lib.KVC_SWAP_STAGED
    # no ring in the staging buffer: only the direct kernel can run
    assert L.kvc_swap_resolve_mode(consecutive.ctypes.data, 64, 1, 64 << 10, 1024) == _lib.KVC_SWAP_DIRECT
    assert L.kvc_swap_resolve_mode(None, 64, 1, 64 << 10, big) == _lib.KVC_SWAP_DIRECT
    assert L.kvc_swap_resolve_mode(consecutive.ctypes.data, -1, 1, 64 << 10, big) == _lib.KVC_ERR_INVALID_ARG
    assert L.kvc_swap_last_mode() in (-1, _lib.KVC_SWAP_STAGED, _lib.KVC_SWAP_DIRECT)


def test_queue_sharing_query_without_a_launch():
    """The same stream twice shares its queue with itself: answered without
    touching the GPU; a null result pointer is refused."""
    L = _lib.lib()
    out = ctypes.c_int(0)
    assert L.kvc_streams_share_hw_queue(None, None, ctypes.byref(out)) == _lib.KVC_OK and out.value == 1
    assert L.kvc_streams_share_hw_queue(None, None, None) == _lib.KVC_ERR_INVALID_ARG
    assert _lib.streams_share_hw_queue(0, 0) is True

"""ctypes binding of libkvcache.so (the C ABI in include/kvcache.h and
include/kvcache_experimental.h).

There is no fallback: if the library is missing, `lib()` raises. Every
operator in this package goes through the handles defined here.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p
from typing import Optional

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libkvcache.so")

KVC_OK = 0
KVC_ERR_INVALID_ARG = -1
KVC_ERR_UNSUPPORTED = -2
KVC_ERR_OUT_OF_RANGE = -3
KVC_ERR_STAGING = -4
KVC_ERR_HIP = -5
KVC_ERR_IO = -6
KVC_ERR_TIMEOUT = -7
KVC_ERR_CANCELLED = -8

KVC_DISK_DIRECT = 1
KVC_DISK_PREALLOCATE = 2
KVC_DISK_INFO_DATA_OFFSET = 0
KVC_DISK_INFO_DIRECT = 1
KVC_DISK_INFO_CREATED = 2
KVC_DISK_INFO_ROW_BYTES = 3
KVC_DISK_INFO_NUM_BLOCKS = 4
KVC_DISK_INFO_BOUNCED = 5

KVC_SWAP_STAGED = 0
KVC_SWAP_DIRECT = 1
KVC_SWAP_AUTO = 2

KVC_KERNEL_NONE = 0
KVC_KERNEL_WRITE_ROWS = 1
KVC_KERNEL_COPY_TILES = 2
KVC_KERNEL_WRITE_PLANES = 3
KVC_KERNEL_WRITE_RUNS = 4
KVC_LAUNCH_KERNEL = 0
KVC_LAUNCH_VEC_BYTES = 1
KVC_LAUNCH_PER_LANE = 2
KVC_LAUNCH_THREADS = 3
KVC_LAUNCH_GRID = 4
KVC_LAUNCH_NON_TEMPORAL = 5
KVC_LAUNCH_PIPE = 6
KVC_LAUNCH_SWAP_MODE = 7

KVC_ABI_VERSION = 6
KVC_NOALLOC_MAX_BLOCKS = 8192

KVC_DTYPE_BF16 = 0
KVC_DTYPE_F16 = 1
KVC_DTYPE_F32 = 2

_I64 = c_int64
_P = c_void_p

# name -> (restype, argtypes); mirrors include/kvcache.h declaration by declaration
SIGNATURES = {
    "kvc_abi_version": (c_int, []),
    "kvc_last_error_string": (c_char_p, []),
    "kvc_set_tuning": (c_int, [c_char_p, c_int]),
    "kvc_get_tuning": (c_int, [c_char_p, ctypes.POINTER(c_int)]),
    "kvc_reset_tuning": (c_int, []),
    "kvc_tuning_modified": (c_int, []),
    "kvc_last_launch_info": (_I64, [c_int]),
    "kvc_write_plan_create": (c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, c_int,
                                      ctypes.POINTER(_P)]),
    "kvc_write_plan_append": (c_int, [_P, _P, _P, _I64, _I64, _P, _I64, _I64, _P]),
    "kvc_write_plan_destroy": (c_int, [_P]),
    "kvc_write_plan_resolve_slots": (c_int, [_P, _P, _P]),
    "kvc_rotary_plan_create": (c_int, [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _P, _P, _I64,
                                       _I64, _I64, c_int, ctypes.POINTER(_P)]),
    "kvc_rotary_plan_run": (c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _P, _P, _P, _I64, _I64, _P]),
    "kvc_rotary_plan_destroy": (c_int, [_P]),
    "kvc_rotary_plan_resolve_slots": (c_int, [_P, _P, _P]),
    "kvc_order_pairs_by_host_id": (c_int, [_P, _P, _I64]),
    "kvc_swap_prepare": (c_int, [_P, _P, _I64, _I64, _I64, _P, _I64, _P]),
    "kvc_swap_out_prepared": (c_int, [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P,
                                      _I64, c_int, _P, _P]),
    "kvc_swap_in_prepared": (c_int, [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P,
                                     _I64, c_int, _P, _P]),
    "kvc_thread_release": (c_int, []),
    "kvc_swap_noalloc": (c_int, [c_int, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                 _P]),
    "kvc_reshape_and_cache": (c_int, [_P, _P, _P, _P, _P, c_int, _I64, _I64, _I64, _I64, _I64,
                                      _I64, _I64, _I64, c_int, _P]),
    "kvc_reshape_and_cache_layers": (c_int, [_P, _P, _P, _P, _P, c_int, _I64, _I64, _I64, _I64,
                                             _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                             c_int, _P]),
    "kvc_append_paged_kv_cache": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64,
                                          _I64, _I64, _I64, _I64, _I64, _I64, c_int, _P]),
    "kvc_append_paged_kv_cache_layers": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64,
                                                 _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                                 _I64, _I64, _I64, c_int, _P]),
    "kvc_get_seq_lens": (c_int, [_P, _P, _I64, _I64, _P, _P]),
    "kvc_get_batch_indices_positions": (c_int, [_P, _P, _I64, _I64, _P, _P, _P]),
    "kvc_build_write_index": (c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I64, _P, _P, _P, _P, _P, _P,
                                      _P, _P, _P, _I64, _P]),
    "kvc_slot_runs": (c_int, [_P, c_int, _I64, _I64, _P, _P, _I64, _P]),
    "kvc_streams_share_hw_queue": (c_int, [_P, _P, _P]),
    "kvc_write_runs_layers": (c_int, [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                      _I64, _I64, _I64, _I64, _I64, _I64, c_int, _P]),
    "kvc_write_plan_set_slots": (c_int, [_P, _P]),
    "kvc_rotary_plan_set_slots": (c_int, [_P, _P]),
    "kvc_swap_resolve_mode": (c_int, [_P, _I64, _I64, _I64, _I64]),
    "kvc_swap_last_mode": (c_int, []),
    "kvc_row_mover_submit_after_flag": (_I64, [_P, _P, _P, _I64, _I64, _I64, _P, _P, _I64, _I64, c_int]),
    "kvc_row_mover_set_timeout_ms": (c_int, [_P, _I64]),
    "kvc_row_mover_cancel": (c_int, [_P]),
    "kvc_rotary_pos_emb": (c_int, [_P, _P, _P, c_int, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                                   _I64, _P, _P, _I64, _I64, c_int, _P]),
    "kvc_rotary_pos_emb_and_cache": (c_int, [_P, _P, _P, _P, c_int, _P, _I64, _I64, _I64, _I64, _I64,
                                             _I64, _I64, _I64, _I64, _P, _P, _I64, _I64, _P, _P, _P,
                                             c_int, _I64, _I64, _I64, _I64, c_int, _P]),
    "kvc_rotary_pos_emb_and_append_paged": (c_int, [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64,
                                                    _I64, _I64, _I64, _I64, _I64, _P, _P, _I64, _I64,
                                                    _P, _P, _P, _I64, _I64, _I64, _I64, _I64, c_int,
                                                    _P]),
    "kvc_copy_blocks": (c_int, [_P, _P, _I64, _I64, _I64, _I64, _I64, _P]),
    "kvc_gather_blocks": (c_int, [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    "kvc_scatter_blocks": (c_int, [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P]),
    "kvc_swap_staging_bytes": (_I64, [_I64, _I64, _I64, c_int, _I64]),
    "kvc_swap_out": (c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P,
                             _I64, c_int, _P, _P]),
    "kvc_swap_in": (c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P,
                            _I64, c_int, _P, _P]),
    "kvc_disk_open": (c_int, [c_char_p, c_char_p, _I64, _I64, _I64, c_int, c_int, ctypes.POINTER(_P)]),
    "kvc_disk_close": (c_int, [_P]),
    "kvc_disk_sync": (c_int, [_P]),
    "kvc_disk_info": (_I64, [_P, c_int]),
    "kvc_disk_save_blocks": (c_int, [_P, _P, _I64, _P, _P, _I64, c_int]),
    "kvc_disk_load_blocks": (c_int, [_P, _P, _I64, _P, _P, _I64, c_int]),
    "kvc_host_copy_rows": (c_int, [_P, _I64, _I64, _I64, _P, _P, _I64, _I64, c_int, c_int]),
    "kvc_row_mover_create": (c_int, [c_int, ctypes.POINTER(_P)]),
    "kvc_row_mover_submit": (_I64, [_P, _P, _P, _I64, _I64, _I64, _P, _P, _I64, _I64, c_int]),
    "kvc_row_mover_done": (c_int, [_P, _I64]),
    "kvc_row_mover_wait": (c_int, [_P, _I64]),
    "kvc_row_mover_destroy": (c_int, [_P]),
    "kvc_host_alloc_pinned": (_P, [c_size_t]),
    "kvc_host_free_pinned": (c_int, [_P]),
}

_lib: Optional[ctypes.CDLL] = None


class KVCacheLibraryError(RuntimeError):
    """libkvcache.so is missing, or a HIP runtime call inside it failed."""


def lib() -> ctypes.CDLL:
    """Load libkvcache.so once and type its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KVCacheLibraryError(
            f"{LIB_PATH} is not built; run `python -m lmserve_amd.build` (needs hipcc). "
            "There is no CPU fallback for the KV-cache operators.")
    handle = ctypes.CDLL(LIB_PATH)
    handle.kvc_abi_version.restype = c_int
    if handle.kvc_abi_version() != KVC_ABI_VERSION:
        raise KVCacheLibraryError(
            f"{LIB_PATH} has ABI version {handle.kvc_abi_version()}, this package needs "
            f"{KVC_ABI_VERSION}: rebuild it with `python -m lmserve_amd.build`")
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = handle
    return handle


_fast = None


def fast():
    """The `_kvc_fast` extension module (METH_FASTCALL wrappers of the per-layer
    calls), or None when it is not built or `KVC_DISABLE_CALL_EXTENSION` is set in
    the environment; callers then go through ctypes to the same entry points."""
    global _fast
    if _fast is None:
        lib()   # the shared library first: the extension binds to the same instance
        if os.environ.get("KVC_DISABLE_CALL_EXTENSION"):
            _fast = False   # everything through ctypes (same entry points, more host time per call)
            return None
        try:
            from . import _kvc_fast
            _fast = _kvc_fast if _kvc_fast.abi_version == KVC_ABI_VERSION else False
        except ImportError:
            _fast = False
    return _fast or None


_fast_entries: dict = {}


def fast_entry(name: str):
    """A function of the `_kvc_fast` extension by name, or None when the extension
    is not built (looked up once per name)."""
    try:
        return _fast_entries[name]
    except KeyError:
        mod = fast()
        fn = _fast_entries[name] = getattr(mod, name, None) if mod else None
        return fn


def last_error() -> str:
    return lib().kvc_last_error_string().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Turn a kvc_status into the Python exception the reference surface uses."""
    if rc == KVC_OK:
        return
    msg = last_error()
    if rc == KVC_ERR_UNSUPPORTED:
        raise TypeError(msg)
    if rc in (KVC_ERR_INVALID_ARG, KVC_ERR_STAGING):
        raise ValueError(msg)
    if rc == KVC_ERR_OUT_OF_RANGE:
        raise IndexError(msg)
    if rc == KVC_ERR_IO:
        raise OSError(msg)
    if rc == KVC_ERR_TIMEOUT:
        raise TimeoutError(msg)
    raise KVCacheLibraryError(msg)


def set_tuning(key: str, value: int) -> None:
    check(lib().kvc_set_tuning(key.encode(), int(value)))


def get_tuning(key: str) -> int:
    out = c_int(0)
    check(lib().kvc_get_tuning(key.encode(), ctypes.byref(out)))
    return out.value


def reset_tuning() -> None:
    check(lib().kvc_reset_tuning())


def streams_share_hw_queue(stream_x: int, stream_y: int) -> bool:
    """Whether two streams (raw handles) feed the same hardware queue, found out
    by holding one for 200 us and watching an empty kernel on the other."""
    out = ctypes.c_int(1)
    check(lib().kvc_streams_share_hw_queue(stream_x, stream_y, ctypes.byref(out)))
    return bool(out.value)


def last_swap_mode() -> int:
    """The KVC_SWAP_* mode the calling thread's most recent swap call ran in
    (what KVC_SWAP_AUTO chose); -1 before the first."""
    return int(lib().kvc_swap_last_mode())


def last_launch() -> dict:
    """Shape of the calling thread's most recent kernel launch."""
    L = lib()
    return {"kernel": L.kvc_last_launch_info(KVC_LAUNCH_KERNEL),
            "vec_bytes": L.kvc_last_launch_info(KVC_LAUNCH_VEC_BYTES),
            "per_lane": L.kvc_last_launch_info(KVC_LAUNCH_PER_LANE),
            "threads": L.kvc_last_launch_info(KVC_LAUNCH_THREADS),
            "grid": L.kvc_last_launch_info(KVC_LAUNCH_GRID),
            "non_temporal": L.kvc_last_launch_info(KVC_LAUNCH_NON_TEMPORAL),
            "pipe": L.kvc_last_launch_info(KVC_LAUNCH_PIPE)}

"""The KV worker as a process of its own.

The reference starts the swap engine in a second process on the same GPU
(`init_kv_cache`, runtime/worker/llm_worker/cli.py:232-272, started at
cli.py:115-121): it maps the model worker's pool from an IPC handle, opens the
per-layer events and serves `CopyKV` requests (cli.py:150-163) while the model
worker runs the forward pass. `serve_kv_worker` is that process body with the
gRPC transport (out of scope here) replaced by a pair of `multiprocessing`
queues; everything the data path needs is the same: `KVWorkerParams` in,
`KVWorker.copy_kv` per request, the layer doorbells and events across the
process boundary.

Requests (tuples):
    ("copy_kv", [[(src, dst), ...], ...], src_device, dst_device)   -> ("ok",) | ("error", text)
    ("read_host", [block ids])                                      -> ("host", ndarray [n, L, block_elems])
    ("write_host", [block ids], ndarray)                            -> ("ok",)
    ("stop",)                                                       -> ("stopped",)
"""
from __future__ import annotations

import asyncio
import traceback

import numpy as np
import torch

from .kv_pool import KVWorkerParams, open_kv_worker_params
from .kv_worker import BlockMapping, Device, KVWorker


def serve_kv_worker(params: KVWorkerParams, device: int, requests, replies,
                    swap_mode: str = "auto") -> None:
    """Process entry point (target of `multiprocessing.Process`, spawn context)."""
    torch.cuda.set_device(device)
    try:
        gpu_kv_caches, handle = open_kv_worker_params(params, device)
        worker = KVWorker(gpu_kv_caches, params.num_host_blocks, params.num_disk_blocks,
                          params.disk_kv_cache_file or None, swap_mode=swap_mode,
                          kv_worker_handle=handle)
    except Exception:
        replies.put(("error", traceback.format_exc()))
        return
    replies.put(("ready", tuple(gpu_kv_caches.shape)))
    try:
        while True:
            req = requests.get()
            kind = req[0]
            try:
                if kind == "stop":
                    break
                if kind == "copy_kv":
                    maps = [BlockMapping.from_pairs(pairs) for pairs in req[1]]
                    asyncio.run(worker.copy_kv(maps, Device(req[2]), Device(req[3])))
                    replies.put(("ok",))
                elif kind == "read_host":
                    replies.put(("host", worker.host_kv_caches[np.asarray(req[1], dtype=np.int64)].copy()))
                elif kind == "write_host":
                    worker.host_kv_caches[np.asarray(req[1], dtype=np.int64)] = req[2]
                    replies.put(("ok",))
                else:
                    replies.put(("error", f"unknown request {kind!r}"))
            except Exception:
                replies.put(("error", traceback.format_exc()))
    finally:
        worker.close()
        handle.close()
        del worker, gpu_kv_caches, handle
        replies.put(("stopped",))

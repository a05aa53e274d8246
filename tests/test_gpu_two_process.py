"""The reference's two-process shape on one GPU: the model worker owns the pool,
a KV-worker process maps it from an IPC handle and moves blocks layer by layer,
ordered against the model's stream layer by layer through queue doorbells
(runtime/worker/llm_worker/model_worker.py:232-306, kv_worker.py:97-160, :249-295,
cli.py:115-121). The child is a fresh process (spawn); the pool is a few MiB in a
segment of its own.

The reference orders the two processes with interprocess events. HIP builds an
exported event on `hipHostRegister` of a shared-memory page, and the machines
these tests run on refuse `hipHostRegister` (recording such an event fails with
"invalid argument"), so the handle runs in its host-signalled mode here: a
doorbell is rung only after the recorded work has completed."""
import gc
import multiprocessing as mp
import queue
import time

import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from oracle import kvc_oracle as orc
from tests.helpers import bf16_bits, bits_of, random_pool, to_bf16

pytestmark = pytest.mark.gpu

WAIT_S = 60.0


def _get(replies, what):
    try:
        msg = replies.get(timeout=WAIT_S)
    except queue.Empty:
        pytest.fail(f"the KV-worker process did not answer within {WAIT_S:.0f} s ({what})")
    assert msg[0] != "error", f"KV-worker process failed ({what}):\n{msg[1]}"
    return msg


def _wait_stream(stream, what):
    """Synchronise with a time limit: a cross-process wait that never fires must
    fail the test, not hang it."""
    done = torch.cuda.Event()
    done.record(stream)
    t_end = time.monotonic() + WAIT_S
    while not done.query():
        assert time.monotonic() < t_end, f"stream did not drain within {WAIT_S:.0f} s ({what})"
        time.sleep(0.001)


def _segment_bytes(t: torch.Tensor) -> int:
    """Size of the allocator segment that holds the tensor: what an IPC handle of
    its storage exports."""
    p = t.data_ptr()
    for seg in torch.cuda.memory_snapshot():
        if seg["address"] <= p < seg["address"] + seg["total_size"]:
            return seg["total_size"]
    raise AssertionError("tensor not found in the allocator's segments")


def test_kv_worker_in_a_second_process_follows_the_layer_protocol(gpu):
    s = wl.LLAMA_3_2_1B
    L, nb, nhb, bs, H, D = 6, 96, 40, s.block_size, s.num_kv_heads, s.head_dim
    gc.collect()
    torch.cuda.empty_cache()                       # the pool gets a segment of its own
    pool_np = random_pool((L, nb, 2, bs, H, D), 41)
    pool = to_bf16(pool_np, gpu)
    assert _segment_bytes(pool) < (1 << 30), "the shared segment must stay far below 2 GiB"

    ctx = mp.get_context("spawn")
    handle = kvc.KVWorkerHandle.create(L, interprocess=True, mp_context=ctx, sync="host")
    params = kvc.make_kv_worker_params(pool, handle, nhb)
    requests, replies = ctx.Queue(), ctx.Queue()
    child = ctx.Process(target=kvc.serve_kv_worker, args=(params, gpu.index or 0, requests, replies),
                        daemon=True)
    child.start()
    try:
        ready = _get(replies, "start-up")
        assert ready == ("ready", (L, nb, 2 * bs * H * D))

        hooks = kvc.LayerSyncHooks(handle)
        hooks.timeout = WAIT_S
        model_stream = torch.cuda.Stream()
        rng = np.random.default_rng(42)

        # ---- write-through: the model writes layer l, then the worker saves layer l -----
        w = wl._write_workload(s, nb, [3, 30, 0, 17], [13, 2, 16, 1], rng)
        T = w.num_tokens
        key, value = bf16_bits((L, T, H, D), 43), bf16_bits((L, T, H, D), 44)
        dkey, dval = to_bf16(key, gpu), to_bf16(value, gpu)
        idx = kvc.to_device(w.index, bs, gpu)
        touched = np.unique(w.index.slot_mapping // bs).astype(np.int64)   # blocks the step writes into
        others = np.setdiff1d(np.arange(nb), touched)[:5].astype(np.int64)
        src = np.concatenate([touched, others])
        host_ids = rng.permutation(nhb)[:len(src)].astype(np.int64)
        want_pool = pool_np.copy()
        for l in range(L):
            orc.c_append_paged_kv_cache(key[l], value[l], w.index.batch_indices, w.index.positions,
                                        want_pool[l], w.index.kv_block_indices, w.index.kv_block_indptrs)
        want_host = np.zeros((nhb, L, 2 * bs * H * D), dtype=np.uint16)
        orc.c_save_blocks_to_host(want_pool.reshape(L, nb, -1), want_host, src, host_ids)

        requests.put(("copy_kv", [list(zip(src[:7].tolist(), host_ids[:7].tolist())),
                                  list(zip(src[7:].tolist(), host_ids[7:].tolist()))],
                      int(kvc.Device.GPU), int(kvc.Device.Host)))
        hooks.enable_record_after_execute = True
        torch.cuda.synchronize()
        with torch.cuda.stream(model_stream):
            for l in range(L):
                # the layer's write sits behind ~10 ms of other work on the model's stream:
                # a worker that did not wait for the layer's completion would save the old rows
                torch.cuda._sleep(20_000_000)
                kvc.append_paged_kv_cache(dkey[l], dval[l], idx.batch_indices, idx.positions, pool[l],
                                          idx.kv_block_indices, idx.kv_block_indptrs,
                                          idx.kv_last_block_lens)
                hooks.post(l)
        hooks.enable_record_after_execute = False
        assert _get(replies, "GPU->Host copy_kv") == ("ok",)
        requests.put(("read_host", host_ids.tolist()))
        got = _get(replies, "read_host")[1]
        assert np.array_equal(got, want_host[host_ids]), "host pool differs from the oracle"
        _wait_stream(model_stream, "model stream after the write-through")
        assert np.array_equal(bits_of(pool), want_pool)

        # ---- fetch: the worker loads layer l, then the model reads layer l ---------------
        new = np.setdiff1d(np.arange(nb), src)[:len(src)].astype(np.int64)
        fresh = rng.integers(0, 1 << 16, size=(len(src), L, 2 * bs * H * D), dtype=np.uint16)
        requests.put(("write_host", host_ids.tolist(), fresh))
        assert _get(replies, "write_host") == ("ok",)
        orc.c_load_blocks_from_host(want_pool.reshape(L, nb, -1), _as_host(fresh, host_ids, nhb), host_ids, new)
        requests.put(("copy_kv", [list(zip(host_ids.tolist(), new.tolist()))],
                      int(kvc.Device.Host), int(kvc.Device.GPU)))
        hooks.enable_wait_before_execute = True
        seen = torch.empty(L, len(new), 2 * bs * H * D, dtype=torch.bfloat16, device=gpu)
        pool3 = pool.view(L, nb, -1)
        new_dev = torch.from_numpy(new).to(gpu)
        with torch.cuda.stream(model_stream):
            for l in range(L):
                hooks.pre(l)                           # the doorbell says: layer l has landed
                torch.index_select(pool3[l], 0, new_dev, out=seen[l])
        hooks.enable_wait_before_execute = False
        assert _get(replies, "Host->GPU copy_kv") == ("ok",)
        _wait_stream(model_stream, "model stream after the fetch")
        want_seen = want_pool.reshape(L, nb, -1)[:, new]
        assert np.array_equal(bits_of(seen), want_seen), "a layer was read before its fetch had landed"
        assert np.array_equal(bits_of(pool), want_pool)
        assert handle.model_queue.empty() and handle.kv_queue.empty()
    finally:
        handle.close()
        requests.put(("stop",))
        child.join(timeout=30)
        if child.is_alive():
            child.kill()
            child.join(timeout=10)
    assert child.exitcode == 0


def _as_host(rows, host_ids, nhb):
    """A host pool image holding `rows[i]` at `host_ids[i]`."""
    host = np.zeros((nhb,) + rows.shape[1:], dtype=rows.dtype)
    host[host_ids] = rows
    return host

"""The KV worker's two streams get hardware queues of their own.

The runtime maps the streams of a process onto a few hardware queues. Streams
that share one take turns, and a wait queued by one (a kernel behind a
copy-engine transfer, the event of another stream) holds back the other: with
its streams in one queue -- or one of them in the caller's queue, because every
swap call first waits for the caller's stream -- swap-out and swap-in issued
together move 55 GB/s in sum instead of 94. Which streams share a queue changes
with what the process has done before (a recorded graph shifts it), so the
worker finds out at construction (`kvc_streams_share_hw_queue`) and draws
streams until two are apart from each other and from the model's stream.
"""
import os
import time

import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from lmserve_amd import _lib
from lmserve_amd.step_graph import KVWriteStep

pytestmark = pytest.mark.gpu

HW_QUEUES = int(os.environ.get("GPU_MAX_HW_QUEUES", "4") or 4)      # the runtime's default is 4


def test_a_stream_shares_its_queue_with_itself_and_the_answer_is_stable(gpu):
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    assert _lib.streams_share_hw_queue(a.cuda_stream, a.cuda_stream) is True
    first = _lib.streams_share_hw_queue(a.cuda_stream, b.cuda_stream)
    for _ in range(3):      # the mapping of a stream does not change once it has been used
        assert _lib.streams_share_hw_queue(a.cuda_stream, b.cuda_stream) is first
        assert _lib.streams_share_hw_queue(b.cuda_stream, a.cuda_stream) is first
    # among the streams torch hands out, some pair shares a queue (there are more streams than queues)
    streams = [torch.cuda.Stream() for _ in range(12)]
    shares = [_lib.streams_share_hw_queue(streams[0].cuda_stream, s.cuda_stream) for s in streams[1:]]
    if HW_QUEUES < 12:
        assert any(shares)
    if HW_QUEUES > 1:
        assert not all(shares)
    # not while a stream is being captured
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=a):
        with pytest.raises(ValueError):
            _lib.streams_share_hw_queue(a.cuda_stream, b.cuda_stream)
        torch.zeros(4, device=gpu).add_(1)


def test_both_swap_directions_overlap_for_every_worker_made_after_a_graph_ran(gpu):
    """Workers made one after another, after a recorded step has been replayed (the
    state in which a worker's streams used to land in one queue every other
    time): each has streams apart from each other and from the current stream,
    and swap-out beside swap-in takes clearly less than the two in turn."""
    if HW_QUEUES < 3:
        pytest.skip("needs three hardware queues: the caller's and one per direction")
    s8 = wl.LLAMA_3_8B
    L8, B, nb8 = 4, 64, 512
    pool8 = torch.zeros(L8, nb8, 2, 16, 8, 128, dtype=torch.bfloat16, device=gpu)
    w = wl.decode_step(s8, num_blocks=nb8, batch=B, max_context=200, seed=1)
    step = KVWriteStep(8, 128, 16, torch.bfloat16, gpu, max_requests=B, max_tokens=B, max_block_ids=B * 16)
    step.set_requests(w.inputs)
    k = torch.zeros(L8, B, 8, 128, dtype=torch.bfloat16, device=gpu)
    graph = step.capture([k[l] for l in range(L8)], [k[l] for l in range(L8)], [pool8[l] for l in range(L8)])
    for _ in range(20):
        graph.replay()
    torch.cuda.synchronize()

    s70 = wl.LLAMA_3_1_70B
    nb, n = 2048, 1024                                   # 2.5 GiB each way
    pool = torch.zeros(s70.num_layers, nb, 2, 16, 8, 128, dtype=torch.bfloat16, device=gpu)
    old, _, new = wl.swap_round_trip(nb, n, seed=0)
    out = [kvc.BlockMapping.from_pairs(zip(old[:n // 2].tolist(), range(n // 2)))]
    inn = [kvc.BlockMapping.from_pairs(zip(range(n // 2, n), new[n // 2:].tolist()))]
    current = torch.cuda.current_stream()
    for number in range(4):
        worker = kvc.KVWorker(pool, n, swap_mode="staged")
        try:
            assert worker.streams_have_own_queues
            a, b = worker.dtoh_stream, worker.htod_stream
            assert not _lib.streams_share_hw_queue(a.cuda_stream, b.cuda_stream)
            assert not _lib.streams_share_hw_queue(current.cuda_stream, a.cuda_stream)
            assert not _lib.streams_share_hw_queue(current.cuda_stream, b.cuda_stream)

            def run(do_out, do_in):
                if do_out:
                    worker.save_kv_blocks_to_host_nowait(out)
                if do_in:
                    worker.load_kv_blocks_from_host_nowait(inn)
                a.synchronize()
                b.synchronize()

            def timed(do_out, do_in):
                run(do_out, do_in)
                ts = []
                for _ in range(3):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    run(do_out, do_in)
                    ts.append(time.perf_counter() - t0)
                return sorted(ts)[1]

            t_out, t_in, t_both = timed(True, False), timed(False, True), timed(True, True)
            assert t_both < 0.8 * (t_out + t_in), \
                f"worker {number}: out {t_out * 1e3:.1f} ms, in {t_in * 1e3:.1f} ms, both {t_both * 1e3:.1f} ms"
        finally:
            worker.close()

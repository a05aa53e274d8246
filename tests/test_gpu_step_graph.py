"""A whole step -- index build included -- recorded ONCE into a hipGraph and
replayed for the steps that follow it (bit-exact against the CPU oracle).

Every replay is a NEW step: contexts have advanced, sequences have crossed into
new blocks, a request has been replaced, the chunk has another size. Between
replays the program does eager work and synchronises, and every replay is
compared with the oracle over the whole pool.
"""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from lmserve_amd.step_graph import KVWriteStep
from oracle import kvc_oracle as orc
from tests.helpers import FifoBlockIds, bf16_bits, bits_of, sentinel_pool, to_bf16

pytestmark = pytest.mark.gpu


class Seq:
    def __init__(self, seq_id, context, ids):
        self.seq_id, self.context, self.blocks = seq_id, context, ids


def _oracle_index(reqs, bs, cap):
    """The oracle's index of the step, padded to the capacity the launch was recorded for."""
    order = sorted(range(len(reqs)), key=lambda i: -reqs[i].input_len)
    rs = [reqs[i] for i in order]
    index = orc.build_write_index_np([r.input_len for r in rs], [r.context_len for r in rs],
                                     [len(r.block_ids) for r in rs],
                                     [b for r in rs for b in r.block_ids], bs)
    return rs, index, orc.pad_write_index(index, cap)


def _check_index(step, rs, index, padded):
    b = len(rs)
    cu, indptr, last, batch, pos, slots = padded
    assert np.array_equal(step.cu_seqlens_q.cpu().numpy()[:b + 1], cu)
    assert np.all(step.cu_seqlens_q.cpu().numpy()[b:] == cu[-1])          # padding requests add nothing
    assert np.array_equal(step.kv_indptr.cpu().numpy()[:b + 1], indptr)
    assert np.array_equal(step.kv_last_page_len.cpu().numpy()[:b], last)
    assert np.array_equal(step.batch_indices.cpu().numpy(), batch)
    assert np.array_equal(step.positions.cpu().numpy(), pos)
    assert np.array_equal(step.slot_mapping.cpu().numpy(), slots)


def test_decode_steps_replay_from_one_graph_with_the_index_build_inside(gpu):
    """Benchmark configuration 2's shape (256 sequences x 1 token, 32 layers, 8 KV
    heads x 128, 16-token blocks) on a reduced pool. One graph = the index build +
    32 per-layer writes, recorded for the first step; five replays serve five
    consecutive decode steps: every context grows by one, sequences cross into
    freshly allocated blocks, and each step one request is replaced by another."""
    s = wl.LLAMA_3_8B
    L, nb, bs, B = s.num_layers, 1024, s.block_size, 256
    H, D = s.num_kv_heads, s.head_dim
    rng = np.random.default_rng(7)
    ids = FifoBlockIds(nb)
    seqs = []
    for i in range(B):
        ctx = int(rng.integers(1, 40))          # tokens held before this step
        seqs.append(Seq(i, ctx, ids.take((ctx + 1 + bs - 1) // bs)))
    # churn the allocator so that tables are not runs of consecutive ids
    for i in rng.permutation(B)[:64]:
        ids.give_back(seqs[i].blocks)
        ctx = int(rng.integers(1, 40))
        seqs[i] = Seq(1000 + int(i), ctx, ids.take((ctx + 1 + bs - 1) // bs))
    pool_np = sentinel_pool((L, nb, 2, bs, H, D), 3)
    dpool = to_bf16(pool_np, gpu)
    want = pool_np.copy()
    step = KVWriteStep(H, D, bs, torch.bfloat16, gpu, max_requests=B, max_tokens=B,
                       max_block_ids=B * 8)
    static_k = torch.zeros(L, B, H, D, dtype=torch.bfloat16, device=gpu)
    static_v = torch.zeros_like(static_k)
    graph = None
    crossed = replaced = 0
    for rep in range(6):
        # the step: one new token per sequence at position `context`
        reqs = [kvc.InferInput(q.seq_id, [0], 1, q.context, q.context + 1, list(q.blocks)) for q in seqs]
        rs, index, padded = _oracle_index(reqs, bs, B)
        key, value = bf16_bits((L, B, H, D), 100 + rep), bf16_bits((L, B, H, D), 200 + rep)
        static_k.copy_(to_bf16(key, gpu))
        static_v.copy_(to_bf16(value, gpu))
        step.set_requests(reqs)
        if graph is None:
            graph = step.capture([static_k[l] for l in range(L)], [static_v[l] for l in range(L)],
                                 [dpool[l] for l in range(L)])
            dpool.copy_(to_bf16(pool_np, gpu))        # the recording's eager pass wrote step 0: start over
            torch.cuda.synchronize()
        (torch.ones(1 << 20, device=gpu) * 2).sum().item()       # eager work + a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        _check_index(step, rs, index, padded)
        for l in range(L):
            orc.c_append_paged_kv_cache(key[l], value[l], index[3], index[4], want[l],
                                        [b for r in rs for b in r.block_ids], index[1])
        assert np.array_equal(bits_of(dpool), want), f"decode step {rep} differs from the oracle"
        # the next step: every context one longer, new blocks where a sequence fills its last one
        for q in seqs:
            q.context += 1
            if (q.context + 1 + bs - 1) // bs > len(q.blocks):
                q.blocks += ids.take(1)
                crossed += 1
        out = int(rng.integers(0, B))
        ids.give_back(seqs[out].blocks)
        ctx = int(rng.integers(1, 40))
        seqs[out] = Seq(2000 + rep, ctx, ids.take((ctx + 1 + bs - 1) // bs))
        replaced += 1
    assert crossed >= 20 and replaced == 6


def test_chunks_of_other_sizes_replay_from_a_graph_recorded_for_the_largest(gpu):
    """A graph recorded for a 2048-token chunk of 4 sequences (configuration 3's
    shape, reduced pool and layers) also serves smaller steps: a 3-sequence chunk,
    a mixed step of a chunk and decode tokens, an empty step. The launches are
    sized for the capacities; the step's sizes are read on the device. The block
    runs the index build emits feed the run write in the same graph."""
    s = wl.QWEN_2_5_7B
    L, nb, bs = 6, 2048, s.block_size
    H, D = s.num_kv_heads, s.head_dim
    T_cap, B_cap = 2048, 8
    pool_np = sentinel_pool((L, nb, 2, bs, H, D), 5)
    d_token = to_bf16(pool_np, gpu)       # written by the per-layer token writes
    d_runs = to_bf16(pool_np, gpu)        # written by the run write (all layers in one launch)
    want = pool_np.copy()
    step = KVWriteStep(H, D, bs, torch.bfloat16, gpu, max_requests=B_cap, max_tokens=T_cap,
                       max_block_ids=4096, with_runs=True)
    static_k = torch.zeros(L, T_cap, H, D, dtype=torch.bfloat16, device=gpu)
    static_v = torch.zeros_like(static_k)

    def body():
        step.build_index()
        for l in range(L):
            step.append(static_k[l], static_v[l], d_token[l])
        kvc.write_block_runs_layers(static_k, static_v, d_runs, step.runs)

    rng = np.random.default_rng(11)
    steps = [
        ([500, 37, 1000, 60], [512, 512, 512, 512]),        # recorded: a full 2048-token chunk
        ([33, 700, 15], [300, 129, 16]),                     # fewer sequences, fewer tokens
        ([0, 48, 200, 31, 77, 5], [640, 1, 1, 1, 1, 1]),     # a chunk and decode tokens
        ([], []),                                            # nothing to write
        ([1, 17], [1023, 1025]),                             # back to the full capacity
    ]
    graph = None
    for rep, (filled, new) in enumerate(steps):
        w = wl._write_workload(s, nb, filled, new, rng)
        rs, index, padded = _oracle_index(w.inputs, bs, T_cap)
        T = int(sum(new))
        key, value = bf16_bits((L, T_cap, H, D), 300 + rep), bf16_bits((L, T_cap, H, D), 400 + rep)
        static_k.copy_(to_bf16(key, gpu))
        static_v.copy_(to_bf16(value, gpu))
        step.set_requests(w.inputs)
        if graph is None:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                body()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                body()
            d_token.copy_(to_bf16(pool_np, gpu))
            d_runs.copy_(to_bf16(pool_np, gpu))
            torch.cuda.synchronize()
        (torch.ones(1 << 20, device=gpu) * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        _check_index(step, rs, index, padded)
        # the runs against the oracle's, request by request
        want_indptr, want_runs = orc.block_runs_loops([r.input_len for r in rs], [r.context_len for r in rs],
                                                      [len(r.block_ids) for r in rs],
                                                      [b for r in rs for b in r.block_ids], bs)
        n_runs = int(step.runs.num_runs.item())
        assert n_runs == len(want_runs)
        assert np.array_equal(step.runs.runs.cpu().numpy()[:n_runs], want_runs)
        assert np.all(step.runs.runs.cpu().numpy()[n_runs:, 1] == -1)          # the rest is marked empty
        assert np.array_equal(step.runs.run_indptr.cpu().numpy()[:len(rs) + 1], want_indptr)
        for l in range(L):
            if T:
                orc.c_reshape_and_cache(key[l, :T], value[l, :T], want[l], index[5])
        assert np.array_equal(bits_of(d_token), want), f"step {rep}: per-layer writes differ from the oracle"
        assert np.array_equal(bits_of(d_runs), want), f"step {rep}: the run write differs from the oracle"


def test_rotation_fused_steps_replay_from_one_graph(gpu):
    """The same with the rotation fused into every layer's launch: replays of the
    recorded step equal the eager operator on the same inputs, bit for bit, for
    three consecutive decode steps (positions, hence cos/sin rows, change)."""
    s = wl.LLAMA_3_8B
    L, nb, bs, B = 4, 512, s.block_size, 64
    H, D, Hq = s.num_kv_heads, s.head_dim, 32
    cs = kvc.make_cos_sin_cache(D, 4096, 500000.0, dtype=torch.bfloat16).to(gpu)
    step = KVWriteStep(H, D, bs, torch.bfloat16, gpu, max_requests=B, max_tokens=B, max_block_ids=B * 8,
                       cos_sin_cache=cs, num_heads=Hq)
    d_graph = torch.zeros(L, nb, 2, bs, H, D, dtype=torch.bfloat16, device=gpu)
    d_eager = torch.zeros_like(d_graph)
    g = torch.Generator(device="cpu").manual_seed(5)
    q = [torch.zeros(B, Hq * D, dtype=torch.bfloat16, device=gpu) for _ in range(L)]
    k = [torch.zeros(B, H * D, dtype=torch.bfloat16, device=gpu) for _ in range(L)]
    v = [torch.zeros(B, H * D, dtype=torch.bfloat16, device=gpu) for _ in range(L)]
    q_out = [torch.zeros(B, Hq * D, dtype=torch.bfloat16, device=gpu) for _ in range(L)]
    graph = None
    for rep in range(3):
        w = wl.decode_step(s, num_blocks=nb, batch=B - rep, max_context=100, seed=40 + rep)
        for t in q + k + v:
            t.copy_(torch.randn(t.shape, generator=g).to(torch.bfloat16))
        step.set_requests(w.inputs)
        if graph is None:
            graph = step.capture(k, v, [d_graph[l] for l in range(L)], queries=q, query_outs=q_out)
            d_graph.zero_()
            torch.cuda.synchronize()
        (torch.ones(1 << 20, device=gpu) * 2).sum().item()
        graph.replay()
        torch.cuda.synchronize()
        idx = kvc.to_device(w.index, bs, gpu)
        T = w.num_tokens
        for l in range(L):
            want_q, _ = kvc.rotary_pos_emb_and_append_paged(
                q[l][:T], k[l][:T], v[l][:T], idx.batch_indices, idx.positions, cs, D, d_eager[l],
                idx.kv_block_indices, idx.kv_block_indptrs, idx.kv_last_block_lens)
            assert torch.equal(q_out[l][:T], want_q), f"step {rep}, layer {l}: rotated query differs"
        torch.cuda.synchronize()
        assert torch.equal(d_graph, d_eager), f"step {rep}: cache differs from the eager operator"


def test_a_step_beyond_the_capacities_is_refused_before_any_upload(gpu):
    step = KVWriteStep(2, 8, 4, torch.bfloat16, gpu, max_requests=2, max_tokens=8, max_block_ids=6)
    with pytest.raises(ValueError):
        step.set_arrays([1, 1, 1], [3, 3, 3], [1, 1, 1], [0, 1, 2])          # three requests
    with pytest.raises(ValueError):
        step.set_arrays([9], [9], [3], [0, 1, 2])                            # nine tokens
    with pytest.raises(ValueError):
        step.set_arrays([1], [30], [8], list(range(8)))                      # eight block ids
    with pytest.raises(ValueError):
        step.set_arrays([1], [3], [2], [0])                                  # table shorter than it says
    assert step.num_tokens == 0
    step.set_arrays([2], [6], [2], [4, 1])
    step.build_index()
    torch.cuda.synchronize()
    assert step.slot_mapping.cpu().tolist() == [1 * 4 + 0, 1 * 4 + 1, -1, -1, -1, -1, -1, -1]


def test_a_step_is_recorded_while_another_thread_works_on_its_own_stream(gpu):
    """The recording is thread-local: a second thread (what a KV worker's mover and
    notifier threads are in a serving process) keeps launching copies, recording
    and querying events on its own stream while the step is captured; the capture
    succeeds and its replay is bit-exact."""
    import threading

    s = wl.LLAMA_3_8B
    L, nb, bs, B = 4, 256, s.block_size, 32
    H, D = s.num_kv_heads, s.head_dim
    rng = np.random.default_rng(21)
    ids = FifoBlockIds(nb)
    reqs = []
    for i in range(B):
        ctx = int(rng.integers(1, 50))
        reqs.append(kvc.InferInput(i, [0], 1, ctx, ctx + 1, ids.take((ctx + 1 + bs - 1) // bs)))
    rs, index, padded = _oracle_index(reqs, bs, B)
    pool_np = sentinel_pool((L, nb, 2, bs, H, D), 5)
    dpool = to_bf16(pool_np, gpu)
    other_pool = torch.zeros(2, 64, 2, bs, H, D, dtype=torch.bfloat16, device=gpu)
    key, value = bf16_bits((L, B, H, D), 31), bf16_bits((L, B, H, D), 32)
    dk, dv = to_bf16(key, gpu), to_bf16(value, gpu)
    step = KVWriteStep(H, D, bs, torch.bfloat16, gpu, max_requests=B, max_tokens=B, max_block_ids=B * 8)
    step.set_requests(reqs)
    stop, failures, rounds = threading.Event(), [], [0]

    def busy():
        try:
            torch.cuda.set_device(gpu)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                while not stop.is_set():
                    kvc.copy_blocks(other_pool, {0: [1, 2], 3: [4]})
                    done = torch.cuda.Event()
                    done.record(stream)
                    while not done.query():
                        pass
                    rounds[0] += 1
        except Exception as exc:      # noqa: BLE001 - reported by the assertion below
            failures.append(repr(exc))

    worker = threading.Thread(target=busy)
    worker.start()
    try:
        while rounds[0] < 3 and worker.is_alive():
            pass
        graph = step.capture([dk[l] for l in range(L)], [dv[l] for l in range(L)], [dpool[l] for l in range(L)])
        before = rounds[0]
        dpool.copy_(to_bf16(pool_np, gpu))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        while rounds[0] < before + 3 and worker.is_alive():
            pass
    finally:
        stop.set()
        worker.join(30)
    assert not failures and not worker.is_alive(), failures
    want = pool_np.copy()
    for l in range(L):
        orc.c_append_paged_kv_cache(key[l], value[l], index[3], index[4], want[l],
                                    [b for r in rs for b in r.block_ids], index[1])
    assert np.array_equal(bits_of(dpool), want)
    _check_index(step, rs, index, padded)

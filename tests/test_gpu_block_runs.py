"""GPU parity of the block-run write (`kvc_write_runs_layers`) and of the run
descriptors (`kvc_slot_runs`, `kvc_build_write_index`) against the CPU oracle,
bit-exact over the whole pool."""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from lmserve_amd import _lib
from oracle import kvc_oracle as orc
from tests.helpers import bf16_bits, bits_of, sentinel_pool, to_bf16

pytestmark = pytest.mark.gpu


def _run_case(gpu, L, nb, bs, H, D, slots, seed):
    T = len(slots)
    key, value = bf16_bits((L, T, H, D), seed), bf16_bits((L, T, H, D), seed + 1)
    pool = sentinel_pool((L, nb, 2, bs, H, D), seed)
    want = pool.copy()
    ok = slots >= 0
    for l in range(L):
        orc.c_reshape_and_cache(np.ascontiguousarray(key[l][ok]), np.ascontiguousarray(value[l][ok]),
                                want[l], slots[ok])
    dslots = torch.from_numpy(slots).to(gpu)
    runs = kvc.slot_block_runs(dslots, bs)
    torch.cuda.synchronize()
    want_runs = orc.slot_runs_loops(slots, bs)
    assert int(runs.num_runs.item()) == len(want_runs)
    assert np.array_equal(runs.runs.cpu().numpy()[:len(want_runs)], want_runs)
    dpool = to_bf16(pool, gpu)
    kvc.write_block_runs_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool, runs)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)
    return want_runs


@pytest.mark.parametrize("unroll,order", [(0, 0), (1, 1), (2, 0), (4, 1)])
def test_prefill_chunk_block_runs_every_launch_shape(gpu, unroll, order):
    """Configuration 3's shape on a reduced pool: runs of 16 tokens with a partial
    run at either end of every sequence."""
    s = wl.QWEN_2_5_7B
    L, nb = 5, 1024
    w = wl.chunked_prefill(s, num_blocks=nb, num_seqs=4, chunk_tokens=512, min_context=3, max_context=900, seed=2)
    _lib.set_tuning("runs_unroll", unroll)
    _lib.set_tuning("runs_order", order)
    runs = _run_case(gpu, L, nb, s.block_size, s.num_kv_heads, s.head_dim, w.index.slot_mapping, 30)
    ran = _lib.last_launch()
    assert ran["kernel"] == _lib.KVC_KERNEL_WRITE_RUNS and ran["vec_bytes"] == 16
    # by default one vector per lane: 512 descriptors x 10 planes x 4 chunks exceed a resident set
    assert ran["per_lane"] == (unroll or 1)
    assert len(runs) >= 4 * (512 // 16 // 4)


@pytest.mark.parametrize("H,D,bs", [(8, 128, 16), (1, 128, 16), (3, 5, 4), (1, 6, 8), (2, 64, 1), (4, 128, 32)])
def test_block_runs_of_random_slot_mappings(gpu, H, D, bs):
    """Rows from 10 bytes to 2 KiB (vector widths 2 to 16 bytes), block sizes 1 to
    32, slot mappings that mix long runs, single tokens, skipped tokens (-1) and
    runs that stop inside a block."""
    rng = np.random.default_rng(H * 100 + D + bs)
    L, nb = 3, 96
    free = rng.permutation(nb).tolist()
    slots = []
    while len(slots) < 300 and free:
        kind = rng.integers(0, 4)
        blk = free.pop()
        if kind == 0:                                  # a whole block
            slots += [blk * bs + e for e in range(bs)]
        elif kind == 1:                                # a piece of a block
            a = int(rng.integers(0, bs))
            b = int(rng.integers(a, bs)) + 1
            slots += [blk * bs + e for e in range(a, b)]
        elif kind == 2:                                # one token, then a token that is skipped
            slots += [blk * bs + int(rng.integers(0, bs)), -1]
        else:                                          # entries of one block out of order: runs of one
            es = rng.permutation(bs)[:3].tolist()
            slots += [blk * bs + e for e in es]
    _run_case(gpu, L, nb, bs, H, D, np.asarray(slots, dtype=np.int64), 50)


def test_runs_outside_the_pool_or_the_tokens_are_skipped(gpu):
    L, nb, bs, H, D, T = 2, 8, 4, 2, 8, 12
    key, value = bf16_bits((L, T, H, D), 1), bf16_bits((L, T, H, D), 2)
    pool = sentinel_pool((L, nb, 2, bs, H, D), 3)
    runs_np = np.asarray([[0, 3, 0, 4],      # good
                          [4, 8, 0, 2],      # block id beyond the pool
                          [4, -1, 0, 2],     # marked as outside its table
                          [6, 2, 3, 2],      # runs past the end of its block
                          [10, 5, 0, 4],     # tokens past the end of the sources
                          [8, 6, 1, 2],      # good
                          [0, 0, 0, 0]],     # empty
                         dtype=np.int32)
    want = pool.copy()
    orc.write_runs_np(key, value, want, runs_np[[0, 5]])
    druns = kvc.paged.BlockRuns(torch.from_numpy(runs_np).to(gpu), torch.tensor([7], dtype=torch.int32, device=gpu))
    dpool = to_bf16(pool, gpu)
    kvc.write_block_runs_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool, druns)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)
    # only the first *num_runs descriptors count
    druns.num_runs.fill_(1)
    want = pool.copy()
    orc.write_runs_np(key, value, want, runs_np[[0]])
    dpool = to_bf16(pool, gpu)
    kvc.write_block_runs_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool, druns)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)


def test_launch_rule_of_the_run_write(gpu):
    """Two vectors per lane while the grid fits one resident set of workgroups (one
    layer of a chunk), one beyond it (all layers)."""
    s = wl.QWEN_2_5_7B
    nb, T = 2048, 2048
    w = wl.chunked_prefill(s, num_blocks=nb, min_context=16, max_context=4000, seed=1)
    order = sorted(range(len(w.inputs)), key=lambda i: -w.inputs[i].input_len)
    rs = [w.inputs[i] for i in order]
    up = lambda a: torch.tensor(a, dtype=torch.int32, device=gpu)
    out = kvc.build_write_index(up([r.input_len for r in rs]), up([r.context_len for r in rs]),
                                up([len(r.block_ids) for r in rs]), up([b for r in rs for b in r.block_ids]),
                                s.block_size, T, with_runs=True)
    runs = out[6]
    assert runs.max_runs == T // s.block_size + 2 * len(rs)
    for L, want in ((1, 2), (28, 1)):
        pool = torch.zeros(L, nb, 2, s.block_size, s.num_kv_heads, s.head_dim, dtype=torch.bfloat16, device=gpu)
        k = torch.zeros(L, T, s.num_kv_heads, s.head_dim, dtype=torch.bfloat16, device=gpu)
        kvc.write_block_runs_layers(k, k, pool, runs)
        ran = _lib.last_launch()
        assert ran["kernel"] == _lib.KVC_KERNEL_WRITE_RUNS and ran["per_lane"] == want
        assert ran["grid"] == runs.max_runs * 2 * L * (4 // want)
    torch.cuda.synchronize()


def test_index_build_emits_the_oracles_runs(gpu):
    s = wl.QWEN_2_5_7B
    w = wl.chunked_prefill(s, num_blocks=16384, seed=4)
    order = sorted(range(len(w.inputs)), key=lambda i: -w.inputs[i].input_len)
    rs = [w.inputs[i] for i in order]
    q, ctx, nblk = [r.input_len for r in rs], [r.context_len for r in rs], [len(r.block_ids) for r in rs]
    table = [b for r in rs for b in r.block_ids]
    up = lambda a: torch.tensor(a, dtype=torch.int32, device=gpu)
    out = kvc.build_write_index(up(q), up(ctx), up(nblk), up(table), s.block_size, sum(q), with_runs=True)
    torch.cuda.synchronize()
    want_indptr, want_runs = orc.block_runs_loops(q, ctx, nblk, table, s.block_size)
    runs = out[6]
    assert runs.max_runs >= len(want_runs)
    assert int(runs.num_runs.item()) == len(want_runs)
    assert np.array_equal(runs.runs.cpu().numpy()[:len(want_runs)], want_runs)
    assert np.array_equal(runs.run_indptr.cpu().numpy(), want_indptr)
    assert np.array_equal(out[5].cpu().numpy(), orc.runs_to_slots(want_runs, sum(q), s.block_size))
    # a capacity below the bound is refused before anything is launched
    small = kvc.paged.BlockRuns(torch.zeros(8, 4, dtype=torch.int32, device=gpu),
                                torch.zeros(1, dtype=torch.int32, device=gpu),
                                torch.zeros(len(q) + 1, dtype=torch.int32, device=gpu))
    with pytest.raises(ValueError):
        kvc.build_write_index(up(q), up(ctx), up(nblk), up(table), s.block_size, sum(q),
                              out=tuple(out[:6]) + (small,))

"""Pins the CPU oracles before anything is checked against them.

The reference holds no tests, fixtures or golden vectors for its cache
operations, so every oracle function is pinned by what the mathematics fixes:
special cases that reduce to a library routine (a dense copy, np.take,
np.swapaxes), a census of which elements may change, relations between
operations (round trips, idempotence), the reference's OWN index construction
for the page-table functions, and element-by-element brute force on tiny
inputs. Each check is written without the oracle's formula, so a dropped
term, a wrong index or swapped K/V operands fails at least one of them.

Every check runs on all three formulations (NumPy, C, pure-Python loops where
one exists).
"""
import numpy as np
import pytest

from oracle import kvc_oracle as orc
from tests.helpers import SENTINEL_BASE, bf16_bits, random_pool, sentinel_pool

FILL_IMPLS = [orc.fill_key_cache_np, orc.c_fill_key_cache, orc.fill_key_cache_loops]
RESHAPE_IMPLS = [orc.reshape_and_cache_np, orc.c_reshape_and_cache]
PAGED_IMPLS = [orc.append_paged_kv_cache_np, orc.c_append_paged_kv_cache,
               orc.append_paged_kv_cache_loops]
COPY_IMPLS = [orc.copy_blocks_np, orc.c_copy_blocks, orc.copy_blocks_loops]
SAVE_IMPLS = [orc.save_blocks_to_host_np, orc.c_save_blocks_to_host, orc.save_blocks_to_host_loops]
LOAD_IMPLS = [orc.load_blocks_from_host_np, orc.c_load_blocks_from_host,
              orc.load_blocks_from_host_loops]


def _ids(impls):
    return [f.__name__ for f in impls]


# ------------------------------------------------------------------ fill_key_cache

@pytest.mark.parametrize("fill", FILL_IMPLS, ids=_ids(FILL_IMPLS))
def test_fill_identity_slots_is_a_dense_copy(fill):
    T, H, D, slots = 12, 2, 8, 40
    key, value = bf16_bits((T, H, D), 1), bf16_bits((T, H, D), 2)
    kc, vc = sentinel_pool((slots, H, D), 3), sentinel_pool((slots, H, D), 4)
    kc0, vc0 = kc.copy(), vc.copy()
    fill(key, value, kc, vc, np.arange(T, dtype=np.int64))
    n = T * H * D
    assert np.array_equal(kc.reshape(-1)[:n], key.reshape(-1))
    assert np.array_equal(vc.reshape(-1)[:n], value.reshape(-1))
    assert np.array_equal(kc.reshape(-1)[n:], kc0.reshape(-1)[n:])
    assert np.array_equal(vc.reshape(-1)[n:], vc0.reshape(-1)[n:])


@pytest.mark.parametrize("fill", FILL_IMPLS, ids=_ids(FILL_IMPLS))
def test_fill_permutation_slots_is_np_take(fill):
    T, H, D = 16, 2, 4
    rng = np.random.default_rng(5)
    perm = rng.permutation(T).astype(np.int64)
    key, value = bf16_bits((T, H, D), 6), bf16_bits((T, H, D), 7)
    kc, vc = sentinel_pool((T, H, D), 8), sentinel_pool((T, H, D), 9)
    fill(key, value, kc, vc, perm)
    inv = np.argsort(perm)  # cache row r holds the token whose slot is r
    assert np.array_equal(kc, np.take(key, inv, axis=0))
    assert np.array_equal(vc, np.take(value, inv, axis=0))


@pytest.mark.parametrize("fill", FILL_IMPLS, ids=_ids(FILL_IMPLS))
def test_fill_census_and_blocked_view(fill):
    """Exactly the rows named by the slots change; read back through the
    [num_blocks, block_size, H, D] view with slot = blk*bs + e."""
    T, H, D, nb, bs = 20, 2, 4, 8, 4
    rng = np.random.default_rng(10)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((T, H, D), 11), bf16_bits((T, H, D), 12)
    kc, vc = sentinel_pool((nb, bs, H, D), 13), sentinel_pool((nb, bs, H, D), 14)
    kc0, vc0 = kc.copy(), vc.copy()
    fill(key, value, kc, vc, slots)
    assert (key < SENTINEL_BASE).all() and (value < SENTINEL_BASE).all()
    for cache, cache0, new in ((kc, kc0, key), (vc, vc0, value)):
        changed_rows = np.flatnonzero((cache != cache0).reshape(nb * bs, -1).any(axis=1))
        assert sorted(changed_rows.tolist()) == sorted(slots.tolist())
        assert int((cache < SENTINEL_BASE).sum()) == T * H * D  # every written element, no more
        for i, s in enumerate(slots.tolist()):
            for h in range(H):
                for d in range(D):
                    assert cache[s // bs, s % bs, h, d] == new[i, h, d]


@pytest.mark.parametrize("fill", FILL_IMPLS, ids=_ids(FILL_IMPLS))
def test_fill_empty(fill):
    H, D = 2, 4
    kc, vc = sentinel_pool((6, H, D), 1), sentinel_pool((6, H, D), 2)
    kc0, vc0 = kc.copy(), vc.copy()
    fill(np.zeros((0, H, D), np.uint16), np.zeros((0, H, D), np.uint16), kc, vc,
         np.zeros(0, np.int64))
    assert np.array_equal(kc, kc0) and np.array_equal(vc, vc0)


# ------------------------------------------------------- interleaved pool, one layer

@pytest.mark.parametrize("reshape", RESHAPE_IMPLS, ids=_ids(RESHAPE_IMPLS))
def test_reshape_and_cache_matches_packed_fill_and_keeps_k_v_apart(reshape):
    """The K half and the V half of the interleaved layer [nb, 2, bs, H, D]
    must equal the packed caches that the (independently pinned) fill produces."""
    T, H, D, nb, bs = 24, 2, 4, 10, 4
    rng = np.random.default_rng(20)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((T, H, D), 21), bf16_bits((T, H, D), 22)
    pool = sentinel_pool((nb, 2, bs, H, D), 23)
    kc = pool[:, 0].copy()
    vc = pool[:, 1].copy()
    reshape(key, value, pool, slots)
    orc.fill_key_cache_loops(key, value, kc, vc, slots)
    assert np.array_equal(pool[:, 0], kc)
    assert np.array_equal(pool[:, 1], vc)
    assert not np.array_equal(key, value)


# ---------------------------------------------------------------- page-table write

def _requests(rng, nb, bs, filled, new):
    """(block tables, per-token request index, per-token position, per-token slot)
    by the rule of the reference's scheduler: new tokens of a request sit at
    positions [filled, filled+new) and slot(pos) = table[pos // bs]*bs + pos % bs."""
    perm = rng.permutation(nb)
    tables, at = [], 0
    for f, n in zip(filled, new):
        need = (f + n + bs - 1) // bs
        tables.append(perm[at:at + need].tolist())
        at += need
    req, pos, slot = [], [], []
    for b, (f, n) in enumerate(zip(filled, new)):
        for p in range(f, f + n):
            req.append(b)
            pos.append(p)
            slot.append(tables[b][p // bs] * bs + p % bs)
    return tables, req, pos, slot


@pytest.mark.parametrize("impl", ["np", "c"])
def test_index_prep_reproduces_the_references_own_position_ids(impl):
    """With the inputs the reference builds (last_page_len = (ctx-1) % bs + 1,
    one page-table row per request covering [0, ctx)), seq_lens must be the
    context length and positions must equal range(filled, ctx)."""
    bs = 4
    filled = [0, 3, 4, 9, 16, 1]
    new = [5, 1, 4, 7, 1, 1]
    ctx = [f + n for f, n in zip(filled, new)]
    nblocks = [(c + bs - 1) // bs for c in ctx]
    kv_indptr = np.cumsum([0] + nblocks).astype(np.int32)
    last = np.asarray([(c - 1) % bs + 1 for c in ctx], dtype=np.int32)
    append_indptr = np.cumsum([0] + new).astype(np.int32)
    get_sl = orc.get_seq_lens_np if impl == "np" else orc.c_get_seq_lens
    get_bp = orc.get_batch_indices_positions_np if impl == "np" else orc.c_get_batch_indices_positions
    seq_lens = get_sl(kv_indptr, last, bs)
    assert seq_lens.tolist() == ctx
    bi, pos = get_bp(append_indptr, seq_lens, sum(new))
    want_pos = [p for f, c in zip(filled, ctx) for p in range(f, c)]
    want_bi = [b for b, n in enumerate(new) for _ in range(n)]
    assert pos.tolist() == want_pos
    assert bi.tolist() == want_bi


def test_seq_lens_of_an_empty_page_table_row_is_clamped():
    # a request with no pages: max(0 - 1, 0) * bs + last
    out_np = orc.get_seq_lens_np([0, 0, 2], [0, 3], 4)
    out_c = orc.c_get_seq_lens([0, 0, 2], [0, 3], 4)
    assert out_np.tolist() == [0, 7] and out_c.tolist() == [0, 7]


@pytest.mark.parametrize("paged", PAGED_IMPLS, ids=_ids(PAGED_IMPLS))
def test_append_paged_equals_slot_write_under_the_scheduler_rule(paged):
    H, D, nb, bs = 2, 4, 16, 4
    rng = np.random.default_rng(30)
    filled = [0, 5, 8, 2]
    new = [6, 1, 3, 1]
    tables, req, pos, slot = _requests(rng, nb, bs, filled, new)
    T = sum(new)
    key, value = bf16_bits((T, H, D), 31), bf16_bits((T, H, D), 32)
    pool_a = sentinel_pool((nb, 2, bs, H, D), 33)
    pool_b = pool_a.copy()
    kv_indices = np.asarray([b for t in tables for b in t], dtype=np.int32)
    kv_indptr = np.cumsum([0] + [len(t) for t in tables]).astype(np.int32)
    paged(key, value, np.asarray(req, np.int32), np.asarray(pos, np.int32), pool_a, kv_indices,
          kv_indptr)
    # independent statement: explicit 5-D element placement from the slot rule
    for i, s in enumerate(slot):
        pool_b[s // bs, 0, s % bs] = key[i]
        pool_b[s // bs, 1, s % bs] = value[i]
    assert np.array_equal(pool_a, pool_b)
    assert int((pool_a < SENTINEL_BASE).sum()) == 2 * T * H * D


# ---------------------------------------------------------------------- copy_blocks

@pytest.mark.parametrize("copy", COPY_IMPLS, ids=_ids(COPY_IMPLS))
def test_copy_blocks_is_np_take_on_disjoint_pairs(copy):
    L, nb, bs, H, D, P = 3, 12, 2, 1, 4, 4
    rng = np.random.default_rng(40)
    perm = rng.permutation(nb)
    src, dst = perm[:P], perm[P:2 * P]
    maps = np.stack([src, dst], axis=1).reshape(-1).astype(np.int64)
    pool = random_pool((L, nb, 2, bs, H, D), 41)
    before = pool.copy()
    copy(pool, maps)
    assert np.array_equal(np.take(pool, dst, axis=1), np.take(before, src, axis=1))
    untouched = np.setdiff1d(np.arange(nb), dst)
    assert np.array_equal(pool[:, untouched], before[:, untouched])
    # idempotent
    again = pool.copy()
    copy(again, maps)
    assert np.array_equal(again, pool)


@pytest.mark.parametrize("copy", COPY_IMPLS, ids=_ids(COPY_IMPLS))
def test_copy_blocks_self_pair_one_to_many_and_empty(copy):
    L, nb = 2, 8
    pool = random_pool((L, nb, 2, 2, 1, 4), 42)
    before = pool.copy()
    copy(pool, np.asarray([3, 3, 5, 5], dtype=np.int64))
    assert np.array_equal(pool, before)
    copy(pool, np.zeros(0, dtype=np.int64))
    assert np.array_equal(pool, before)
    copy(pool, np.asarray([1, 0, 1, 6, 1, 7], dtype=np.int64))  # {1: [0, 6, 7]}
    for d in (0, 6, 7):
        assert np.array_equal(pool[:, d], before[:, 1])
    for keep in (1, 2, 3, 4, 5):
        assert np.array_equal(pool[:, keep], before[:, keep])


@pytest.mark.parametrize("copy", COPY_IMPLS, ids=_ids(COPY_IMPLS))
def test_copy_blocks_layers_are_independent(copy):
    """Running the operation on each layer alone (as a 1-layer pool) gives the same pool."""
    L, nb = 4, 6
    pool = random_pool((L, nb, 2, 2, 2, 2), 43)
    maps = np.asarray([0, 4, 2, 5], dtype=np.int64)
    whole = pool.copy()
    copy(whole, maps)
    for l in range(L):
        single = pool[l:l + 1].copy()
        copy(single, maps)
        assert np.array_equal(whole[l], single[0])


# ----------------------------------------------------------------------------- swap

@pytest.mark.parametrize("save", SAVE_IMPLS, ids=_ids(SAVE_IMPLS))
def test_save_contiguous_ids_is_swapaxes(save):
    L, nb, E, n, a = 3, 10, 8, 4, 5
    gpu = random_pool((L, nb, E), 50)
    host = sentinel_pool((6, L, E), 51)
    host0 = host.copy()
    save(gpu, host, np.arange(a, a + n), np.arange(n))
    assert np.array_equal(host[:n], np.swapaxes(gpu[:, a:a + n], 0, 1))
    assert np.array_equal(host[n:], host0[n:])


@pytest.mark.parametrize("save,load", list(zip(SAVE_IMPLS, LOAD_IMPLS)), ids=_ids(SAVE_IMPLS))
def test_swap_round_trip_is_the_identity_on_the_payload(save, load):
    L, nb, E, n = 3, 16, 8, 5
    rng = np.random.default_rng(52)
    perm = rng.permutation(nb)
    old, new = perm[:n], perm[n:2 * n]
    host_ids = rng.permutation(7)[:n]
    gpu = random_pool((L, nb, E), 53)
    before = gpu.copy()
    host = sentinel_pool((7, L, E), 54)
    save(gpu, host, old, host_ids)
    assert np.array_equal(gpu, before)  # swap-out never writes the pool
    host_after_save = host.copy()
    load(gpu, host, host_ids, new)
    assert np.array_equal(host, host_after_save)  # swap-in never writes the host pool
    assert np.array_equal(gpu[:, new], before[:, old])
    rest = np.setdiff1d(np.arange(nb), new)
    assert np.array_equal(gpu[:, rest], before[:, rest])
    # per-element statement of the direction semantics
    for i in range(n):
        for l in range(L):
            assert np.array_equal(host[host_ids[i], l], before[l, old[i]])


@pytest.mark.parametrize("save,load", list(zip(SAVE_IMPLS[:2], LOAD_IMPLS[:2])),
                         ids=_ids(SAVE_IMPLS[:2]))
def test_swap_layer_range_touches_only_its_layers(save, load):
    L, nb, E = 5, 8, 4
    gpu = random_pool((L, nb, E), 55)
    host = sentinel_pool((4, L, E), 56)
    host0 = host.copy()
    save(gpu, host, [1, 6], [3, 0], 1, 3)
    assert np.array_equal(host[[3, 0], 1:3], np.swapaxes(gpu[1:3][:, [1, 6]], 0, 1))
    mask = np.ones_like(host, dtype=bool)
    mask[[3, 0], 1:3] = False
    assert np.array_equal(host[mask], host0[mask])
    gpu2 = sentinel_pool((L, nb, E), 57)
    gpu20 = gpu2.copy()
    load(gpu2, host, [3, 0], [2, 7], 1, 3)
    assert np.array_equal(gpu2[1:3][:, [2, 7]], np.swapaxes(host[[3, 0], 1:3], 0, 1))
    mask = np.ones_like(gpu2, dtype=bool)
    mask[1:3, [2, 7]] = False
    assert np.array_equal(gpu2[mask], gpu20[mask])


# ----------------------------------------------------- the three formulations agree

def test_all_formulations_agree_on_a_mid_size_case():
    T, H, D, nb, bs, L = 64, 4, 16, 32, 8, 3
    rng = np.random.default_rng(60)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((T, H, D), 61), bf16_bits((T, H, D), 62)
    a, b = sentinel_pool((nb, 2, bs, H, D), 63), sentinel_pool((nb, 2, bs, H, D), 63)
    orc.reshape_and_cache_np(key, value, a, slots)
    orc.c_reshape_and_cache(key, value, b, slots)
    assert np.array_equal(a, b)
    pool = random_pool((L, nb, 2, bs, H, D), 64)
    perm = rng.permutation(nb)
    maps = np.stack([perm[:8], perm[8:16]], axis=1).reshape(-1).astype(np.int64)
    p1, p2 = pool.copy(), pool.copy()
    orc.copy_blocks_np(p1, maps)
    orc.c_copy_blocks(p2, maps)
    assert np.array_equal(p1, p2)


# ------------------------------------------------------------------ block runs
def test_block_runs_of_a_step_written_out_by_hand():
    """Two requests, page size 4. Request 0: 6 new tokens at positions 3..8 of
    table [7, 2, 9] -> blocks 7 (entry 3, 1 token), 2 (entries 0..3), 9 (entry 0, 1
    token). Request 1: 2 new tokens at positions 1..2 of table [5] -> one run."""
    indptr, runs = orc.block_runs_loops([6, 2], [9, 3], [3, 1], [7, 2, 9, 5], 4)
    assert indptr.tolist() == [0, 3, 4]
    assert runs.tolist() == [[0, 7, 3, 1], [1, 2, 0, 4], [5, 9, 0, 1], [6, 5, 1, 2]]
    # a request whose table is too short: the run exists, its block is -1
    _, runs = orc.block_runs_loops([5], [8], [1], [6], 4)
    assert runs.tolist() == [[0, 6, 3, 1], [1, -1, 0, 4]]
    # padding requests (no new tokens) add nothing
    indptr, runs = orc.block_runs_loops([0, 1, 0], [0, 5, 0], [0, 2, 0], [3, 4], 4)
    assert indptr.tolist() == [0, 0, 1, 1] and runs.tolist() == [[0, 4, 0, 1]]


@pytest.mark.parametrize("seed", range(6))
def test_block_runs_expand_to_the_pinned_slot_mapping_and_are_maximal(seed):
    """Independent of the run construction: expanded token by token, the runs give
    exactly the slot mapping that `build_write_index_np` derives (pinned against a
    hand case and against the page-table write), they cover the tokens in order
    without gaps, and no two neighbouring runs could be one."""
    rng = np.random.default_rng(seed)
    bs = int(rng.choice([1, 2, 4, 16]))
    B = int(rng.integers(1, 9))
    q = rng.integers(0, 40, size=B)
    filled = rng.integers(0, 50, size=B)
    ctx = np.where(q > 0, filled + q, rng.integers(0, 3, size=B))
    nblk = (ctx + bs - 1) // bs
    table = rng.permutation(int(nblk.sum()) + 5)[:int(nblk.sum())]
    index = orc.build_write_index_np(q, ctx, nblk, table, bs)
    slots = index[5]
    indptr, runs = orc.block_runs_loops(q, ctx, nblk, table, bs)
    T = int(q.sum())
    assert np.array_equal(orc.runs_to_slots(runs, T, bs), slots)
    assert int(runs[:, 3].sum()) == T and np.all(runs[:, 3] >= 1)
    assert np.array_equal(runs[:, 0], np.concatenate([[0], np.cumsum(runs[:, 3])[:-1]]))   # in order, no gaps
    assert np.all(runs[:, 2] + runs[:, 3] <= bs)
    cu = index[0]
    for r in range(1, len(runs)):
        same_request = np.searchsorted(cu, runs[r, 0], side="right") == np.searchsorted(cu, runs[r - 1, 0], side="right")
        if same_request:       # inside a request a new run starts at the head of a block
            assert runs[r, 2] == 0 and runs[r - 1, 2] + runs[r - 1, 3] == bs
    assert indptr[-1] == len(runs)
    # the runs of an arbitrary slot mapping: the same descriptors, found token by token
    assert np.array_equal(orc.slot_runs_loops(slots, bs), runs)


def test_slot_runs_split_at_gaps_blocks_and_invalid_slots():
    runs = orc.slot_runs_loops([4, 5, 6, 7, 8, 20, 19, -1, 30, 31, 33], 4)
    assert runs.tolist() == [[0, 1, 0, 4], [4, 2, 0, 1], [5, 5, 0, 1], [6, 4, 3, 1], [8, 7, 2, 2], [10, 8, 1, 1]]
    assert orc.slot_runs_loops([], 4).shape == (0, 4)
    assert orc.runs_to_slots(runs, 11, 4).tolist() == [4, 5, 6, 7, 8, 20, 19, -1, 30, 31, 33]


@pytest.mark.parametrize("seed", range(3))
def test_run_write_equals_the_pinned_slot_mapped_write(seed):
    rng = np.random.default_rng(seed)
    L, nb, bs, H, D = 3, 12, 4, 2, 4
    q = rng.integers(1, 12, size=3)
    ctx = q + rng.integers(0, 6, size=3)
    nblk = (ctx + bs - 1) // bs
    table = rng.permutation(nb)[:int(nblk.sum())]
    slots = orc.build_write_index_np(q, ctx, nblk, table, bs)[5]
    _, runs = orc.block_runs_loops(q, ctx, nblk, table, bs)
    T = int(q.sum())
    key = rng.integers(0, 1 << 16, size=(L, T, H, D), dtype=np.uint16)
    value = rng.integers(0, 1 << 16, size=(L, T, H, D), dtype=np.uint16)
    pool = rng.integers(0, 1 << 16, size=(L, nb, 2, bs, H, D), dtype=np.uint16)
    want = pool.copy()
    for l in range(L):
        orc.reshape_and_cache_np(key[l], value[l], want[l], slots)
    orc.write_runs_np(key, value, pool, runs)
    assert np.array_equal(pool, want)


def test_padded_index_marks_the_entries_beyond_the_step():
    index = orc.build_write_index_np([2, 1], [5, 9], [2, 3], [1, 2, 3, 4, 5], 4)
    cu, indptr, last, batch, pos, slots = orc.pad_write_index(index, 6)
    assert batch.tolist() == [0, 0, 1, -1, -1, -1] and pos.tolist() == [3, 4, 8, -1, -1, -1]
    assert slots.tolist()[3:] == [-1, -1, -1] and slots.tolist()[:3] == index[5].tolist()

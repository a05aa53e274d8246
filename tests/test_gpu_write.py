"""GPU parity of the K/V write entry points against the CPU oracle (bit-exact).

Every comparison is over the WHOLE destination pool, so stray writes show.
"""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
from lmserve_amd import _lib
import workloads as wl
from oracle import kvc_oracle as orc
from tests.helpers import bf16_bits, bits_of, sentinel_pool, to_bf16

pytestmark = pytest.mark.gpu


def _dev(a, dev, dtype=torch.bfloat16):
    """NumPy bit patterns -> device tensor of a same-width dtype."""
    if dtype == torch.bfloat16 or dtype == torch.float16:
        return torch.from_numpy(a.view(np.int16).copy()).view(dtype).to(dev)
    return torch.from_numpy(a.view(np.int32).copy()).view(dtype).to(dev)


def _host(t):
    t = t.detach().cpu().contiguous()
    if t.element_size() == 2:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.view(torch.int32).numpy().view(np.uint32)


def _bits(shape, seed, width):
    if width == 2:
        return bf16_bits(shape, seed)
    rng = np.random.default_rng(seed)
    return rng.integers(0, 1 << 32, size=shape, dtype=np.uint32)


def _pool(shape, seed, width):
    if width == 2:
        return sentinel_pool(shape, seed)
    rng = np.random.default_rng(seed + 1000)
    return rng.integers(0, 1 << 32, size=shape, dtype=np.uint32)


FILL_CASES = [
    # T, H, D, num_slots, dtype, slot dtype
    (256, 8, 64, 64 * 16, torch.bfloat16, torch.int64),    # config-1 rows, reduced pool
    (256, 8, 128, 96 * 16, torch.bfloat16, torch.int64),   # Llama-3-8B rows
    (77, 4, 128, 200, torch.float16, torch.int32),
    (33, 3, 5, 64, torch.bfloat16, torch.int64),           # 30-byte rows: 2-byte vectors
    (19, 1, 6, 40, torch.bfloat16, torch.int64),           # 12-byte rows: 4-byte vectors
    (21, 1, 4, 40, torch.bfloat16, torch.int32),           # 8-byte rows
    (50, 2, 64, 128, torch.float32, torch.int64),
    (1, 8, 128, 16, torch.bfloat16, torch.int64),
    (0, 8, 128, 16, torch.bfloat16, torch.int64),
]


@pytest.mark.parametrize("T,H,D,num_slots,dtype,slot_dtype", FILL_CASES)
def test_fill_key_cache_matches_oracle(gpu, T, H, D, num_slots, dtype, slot_dtype):
    width = torch.empty(0, dtype=dtype).element_size()
    rng = np.random.default_rng(T * 131 + H)
    slots = rng.permutation(num_slots)[:T].astype(np.int64)
    key, value = _bits((T, H, D), 1, width), _bits((T, H, D), 2, width)
    kc, vc = _pool((num_slots, H, D), 3, width), _pool((num_slots, H, D), 4, width)
    want_k, want_v = kc.copy(), vc.copy()
    orc.c_fill_key_cache(key, value, want_k, want_v, slots)
    dk, dv = _dev(kc, gpu, dtype), _dev(vc, gpu, dtype)
    kvc.fill_key_cache(_dev(key, gpu, dtype), _dev(value, gpu, dtype), dk, dv,
                       torch.from_numpy(slots).to(gpu).to(slot_dtype))
    torch.cuda.synchronize()
    assert np.array_equal(_host(dk), want_k)
    assert np.array_equal(_host(dv), want_v)


@pytest.mark.parametrize("vpt", [1, 2, 4, 8])
@pytest.mark.parametrize("nt", [0, 1, 2, 3])
@pytest.mark.parametrize("threads", [0, 64, 128])
def test_write_rows_every_launch_shape(gpu, vpt, nt, threads):
    """All vectors-per-lane / load-store kind / workgroup-size instantiations give
    the same bits, and the instantiation asked for is the one that ran (8 layers
    in one launch, so a token has 2048 vectors and every depth fits)."""
    T, L, H, D, bs, nb = 301, 8, 8, 128, 16, 32
    rng = np.random.default_rng(7)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((L, T, H, D), 1), bf16_bits((L, T, H, D), 2)
    pool = sentinel_pool((L, nb, 2, bs, H, D), 3)
    want = pool.copy()
    for l in range(L):
        orc.c_reshape_and_cache(key[l], value[l], want[l], slots)
    dpool = to_bf16(pool, gpu)
    _lib.set_tuning("write_planes", 0)    # the token kernel, whatever the size
    _lib.set_tuning("write_vpt", vpt)     # the autouse fixture puts the defaults back
    _lib.set_tuning("write_nt", nt)
    _lib.set_tuning("write_threads", threads)
    _lib.set_tuning("write_pipe", nt & 1)  # both load orders over the sweep
    kvc.reshape_and_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool,
                                 torch.from_numpy(slots).to(gpu))
    torch.cuda.synchronize()
    ran = _lib.last_launch()
    assert ran["kernel"] == _lib.KVC_KERNEL_WRITE_ROWS and ran["non_temporal"] == nt
    assert ran["per_lane"] == vpt and ran["threads"] == (threads or 256) and ran["vec_bytes"] == 16
    assert np.array_equal(bits_of(dpool), want)


NARROW_CASES = [
    # T, H, D, layers, narrow_vpt   (rows of 16 * H*D/8 ... bytes, all under 1 KiB)
    (256, 1, 128, 80, 0),    # one KV head of Llama-3.1-70B at tp=8: 256-byte rows
    (256, 1, 128, 80, 1),
    (256, 1, 128, 80, 2),
    (256, 1, 128, 80, 4),
    (256, 1, 128, 80, 8),
    (77, 2, 128, 5, 0),      # 512-byte rows, odd token and layer counts
    (77, 2, 128, 5, 8),
    (3, 1, 64, 3, 0),        # 128-byte rows, fewer tokens than a wavefront covers
    (300, 1, 32, 7, 4),      # 64-byte rows
    (1000, 1, 8, 2, 0),      # 16-byte rows: one vector per row
    (1, 1, 128, 1, 0),
    (70, 8, 128, 6, 4),      # 2 KiB rows (Llama-3-8B): two tokens per 256-lane workgroup
    (70, 8, 128, 6, 8),
    (33, 16, 128, 3, 2),     # 4 KiB rows: one token per workgroup, the widest the kernel takes
    (90, 4, 128, 9, 0),      # 1 KiB rows (Qwen2.5-7B), depth by rule
]


@pytest.mark.parametrize("T,H,D,L,vpt", NARROW_CASES)
@pytest.mark.parametrize("paged", [False, True])
def test_narrow_rows_take_the_plane_kernel_and_match_the_oracle(gpu, T, H, D, L, vpt, paged):
    """Rows under 1 KiB (a tensor-parallel shard's head slice) run the kernel whose
    lanes walk the tokens of one (layer, K|V) plane; every planes-per-lane
    instantiation, both addressing modes, whole pool compared."""
    bs, nb = 16, 96
    rng = np.random.default_rng(T * 7 + D)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((L, T, H, D), 1), bf16_bits((L, T, H, D), 2)
    pool = sentinel_pool((L, nb, 2, bs, H, D), 3)
    want = pool.copy()
    for l in range(L):
        orc.c_reshape_and_cache(key[l], value[l], want[l], slots)
    dpool = to_bf16(pool, gpu)
    _lib.set_tuning("write_planes_vpt", vpt)
    _lib.set_tuning("write_planes", 2)          # whatever the launch size
    # workgroup size and load order vary over the cases (both are by rule otherwise)
    _lib.set_tuning("write_planes_threads", (0, 256, 512, 1024)[(T + L) % 4])
    _lib.set_tuning("write_pipe", (-1, 0, 1)[(T + vpt) % 3])
    nt = (3, 1, 2, 0)[(T + vpt + L + int(paged)) % 4]       # every load/store kind over the cases
    _lib.set_tuning("write_nt", nt)
    if paged:
        # requests of up to three tokens, each token on a page of its own:
        # page = slot // bs at table entry j, position = j * bs + slot % bs
        sizes = []
        while sum(sizes) < T:
            sizes.append(min(int(rng.integers(1, 4)), T - sum(sizes)))
        bi = np.repeat(np.arange(len(sizes)), sizes).astype(np.int32)
        j = np.concatenate([np.arange(n) for n in sizes])
        pos = (j * bs + slots % bs).astype(np.int32)
        indptr = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
        indices = (slots // bs).astype(np.int32)
        last = np.ones(len(sizes), dtype=np.int32)
        bi, pos, indices, indptr, last = (torch.from_numpy(a).to(gpu) for a in (bi, pos, indices, indptr, last))
        kvc.append_paged_kv_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), bi, pos, dpool,
                                         indices, indptr, last)
    else:
        kvc.reshape_and_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool,
                                     torch.from_numpy(slots).to(gpu))
    torch.cuda.synchronize()
    ran = _lib.last_launch()
    assert ran["kernel"] == _lib.KVC_KERNEL_WRITE_PLANES and ran["vec_bytes"] == 16
    # non-temporal loads are taken for rows of 1 KiB or more only
    assert ran["non_temporal"] == ((nt & 1) | (nt & 2 if H * D * 2 >= 1024 else 0))
    if vpt:
        assert ran["per_lane"] == min(vpt, 1 << (2 * L - 1).bit_length())
    assert np.array_equal(bits_of(dpool), want)


def test_narrow_kernel_switch_and_strided_sources(gpu):
    """`write_planes = 0` sends narrow rows through the token-per-workgroup kernel,
    `2` through the plane kernel whatever the size; both agree with the oracle on
    token-strided sources (slices of a wider projection), where the source side
    is no longer one run. By default the launch size decides."""
    T, H, D, bs, nb = 130, 1, 128, 16, 40
    rng = np.random.default_rng(5)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    wide_k, wide_v = bf16_bits((T, 3 * H * D), 1), bf16_bits((T, 3 * H * D), 2)
    key, value = wide_k[:, H * D:2 * H * D], wide_v[:, 2 * H * D:]
    pool = sentinel_pool((nb, 2, bs, H, D), 3)
    want = pool.copy()
    orc.c_reshape_and_cache(np.ascontiguousarray(key).reshape(T, H, D),
                            np.ascontiguousarray(value).reshape(T, H, D), want, slots)
    dk = to_bf16(wide_k, gpu)[:, H * D:2 * H * D].view(T, H, D)
    dv = to_bf16(wide_v, gpu)[:, 2 * H * D:].view(T, H, D)
    assert not dk.is_contiguous()
    for narrow, kernel in ((2, _lib.KVC_KERNEL_WRITE_PLANES), (0, _lib.KVC_KERNEL_WRITE_ROWS)):
        _lib.set_tuning("write_planes", narrow)
        dpool = to_bf16(pool, gpu)
        kvc.reshape_and_cache(dk, dv, dpool, torch.from_numpy(slots).to(gpu))
        torch.cuda.synchronize()
        assert _lib.last_launch()["kernel"] == kernel
        assert np.array_equal(bits_of(dpool), want)
    _lib.reset_tuning()
    # by size: 130 tokens x 2 planes x 256 bytes stay with the token kernel, 16 layers of
    # 512 tokens (4 MiB of source rows) take the plane kernel
    kvc.reshape_and_cache(dk, dv, to_bf16(pool, gpu), torch.from_numpy(slots).to(gpu))
    assert _lib.last_launch()["kernel"] == _lib.KVC_KERNEL_WRITE_ROWS
    Lb, Tb = 16, 512
    big_slots = np.random.default_rng(6).permutation(nb * bs)[:Tb].astype(np.int64)
    bk, bv = bf16_bits((Lb, Tb, H, D), 7), bf16_bits((Lb, Tb, H, D), 8)
    big_pool = sentinel_pool((Lb, nb, 2, bs, H, D), 9)
    big_want = big_pool.copy()
    for l in range(Lb):
        orc.c_reshape_and_cache(bk[l], bv[l], big_want[l], big_slots)
    dbig = to_bf16(big_pool, gpu)
    kvc.reshape_and_cache_layers(to_bf16(bk, gpu), to_bf16(bv, gpu), dbig, torch.from_numpy(big_slots).to(gpu))
    torch.cuda.synchronize()
    assert _lib.last_launch()["kernel"] == _lib.KVC_KERNEL_WRITE_PLANES
    assert np.array_equal(bits_of(dbig), big_want)


def test_config1_llama_1b_write_all_layers(gpu):
    """Configuration 1 (Llama-3.2-1B) at its full size: 16 layers, pool of 1024 blocks, 256
    tokens on seeded random distinct free slots; per-layer op and the one-launch
    form must both equal the oracle on the whole 512 MiB pool."""
    s = wl.LLAMA_3_2_1B
    nb, T = 1024, 256
    slots = wl.random_free_slots(s, nb, T, seed=0)
    L, H, D, bs = s.num_layers, s.num_kv_heads, s.head_dim, s.block_size
    key, value = bf16_bits((L, T, H, D), 10), bf16_bits((L, T, H, D), 11)
    pool = sentinel_pool((L, nb, 2, bs, H, D), 12)
    want = pool.copy()
    for l in range(L):
        orc.c_reshape_and_cache(key[l], value[l], want[l], slots)
    dkey, dval = to_bf16(key, gpu), to_bf16(value, gpu)
    dslots = torch.from_numpy(slots).to(gpu)

    per_layer = to_bf16(pool, gpu)
    for l in range(L):
        kvc.reshape_and_cache(dkey[l], dval[l], per_layer[l], dslots)
    fused = to_bf16(pool, gpu)
    kvc.reshape_and_cache_layers(dkey, dval, fused, dslots)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(per_layer), want)
    assert np.array_equal(bits_of(fused), want)


def test_reshape_and_cache_strided_tokens_and_guarded_slots(gpu):
    """K/V rows taken as slices of a fused projection (token stride > row), and
    slots that are negative or beyond the pool are skipped, not written."""
    T, H, D, nb, bs = 40, 2, 64, 8, 16
    rng = np.random.default_rng(3)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    fused = bf16_bits((T, 3 * H * D), 5)
    key = np.ascontiguousarray(fused[:, H * D:2 * H * D]).reshape(T, H, D)
    value = np.ascontiguousarray(fused[:, 2 * H * D:]).reshape(T, H, D)
    bad = slots.copy()
    bad[3] = -1
    bad[17] = nb * bs
    bad[29] = nb * bs + 5
    keep = np.asarray([i for i in range(T) if i not in (3, 17, 29)])
    pool = sentinel_pool((nb, 2, bs, H, D), 6)
    want = pool.copy()
    orc.c_reshape_and_cache(np.ascontiguousarray(key[keep]), np.ascontiguousarray(value[keep]),
                            want, slots[keep])
    dfused = to_bf16(fused, gpu)
    dk = dfused[:, H * D:2 * H * D].view(T, H, D)
    dv = dfused[:, 2 * H * D:].view(T, H, D)
    assert not dk.is_contiguous()
    dpool = to_bf16(pool, gpu)
    kvc.reshape_and_cache(dk, dv, dpool, torch.from_numpy(bad).to(gpu))
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)


def _paged_case(gpu, workload, L, seed):
    s = workload.shape
    nb, bs, H, D = workload.num_blocks, s.block_size, s.num_kv_heads, s.head_dim
    idx = workload.index
    T = workload.num_tokens
    key, value = bf16_bits((L, T, H, D), seed), bf16_bits((L, T, H, D), seed + 1)
    pool = sentinel_pool((L, nb, 2, bs, H, D), seed + 2)
    want = pool.copy()
    for l in range(L):
        orc.c_append_paged_kv_cache(key[l], value[l], idx.batch_indices, idx.positions, want[l],
                                    idx.kv_block_indices, idx.kv_block_indptrs)
    # the slot-mapped oracle must agree (scheduler rule), before the GPU is involved
    want2 = pool.copy()
    for l in range(L):
        orc.reshape_and_cache_np(key[l], value[l], want2[l], idx.slot_mapping)
    assert np.array_equal(want, want2)
    dev = kvc.to_device(idx, bs, gpu)
    dkey, dval = to_bf16(key, gpu), to_bf16(value, gpu)
    return pool, want, dev, dkey, dval


@pytest.mark.parametrize("kind", ["decode", "chunked_prefill", "mixed"])
def test_append_paged_kv_cache_matches_oracle(gpu, kind):
    if kind == "decode":
        w = wl.decode_step(wl.LLAMA_3_8B, num_blocks=512, batch=48, max_context=150, seed=1)
    elif kind == "chunked_prefill":
        w = wl.chunked_prefill(wl.QWEN_2_5_7B, num_blocks=512, num_seqs=4, chunk_tokens=256,
                               min_context=100, max_context=1500, seed=2)
    else:
        rng = np.random.default_rng(9)
        filled = [0, 37, 5, 64, 200, 16, 15]
        new = [70, 1, 1, 33, 1, 16, 2]
        w = wl._write_workload(wl.LLAMA_3_2_1B, 256, filled, new, rng)
    L = 3
    pool, want, dev, dkey, dval = _paged_case(gpu, w, L, 40)
    # device-side index prep must reproduce the host arrays
    assert np.array_equal(dev.batch_indices.cpu().numpy(), w.index.batch_indices)
    assert np.array_equal(dev.positions.cpu().numpy(), w.index.positions)

    per_layer = to_bf16(pool, gpu)
    for l in range(L):
        kvc.append_paged_kv_cache(dkey[l], dval[l], dev.batch_indices, dev.positions, per_layer[l],
                                  dev.kv_block_indices, dev.kv_block_indptrs, dev.kv_last_block_lens)
    fused = to_bf16(pool, gpu)
    kvc.append_paged_kv_cache_layers(dkey, dval, dev.batch_indices, dev.positions, fused,
                                     dev.kv_block_indices, dev.kv_block_indptrs,
                                     dev.kv_last_block_lens)
    slotted = to_bf16(pool, gpu)
    kvc.reshape_and_cache_layers(dkey, dval, slotted, dev.slot_mapping)
    planned = to_bf16(pool, gpu)
    s = w.shape
    plan = kvc.PagedKVWritePlan(dev.batch_indices, dev.positions, dev.kv_block_indices,
                                dev.kv_block_indptrs, dev.kv_last_block_lens, s.num_kv_heads,
                                s.head_dim, s.block_size, torch.bfloat16)
    for l in range(L):
        plan.append(dkey[l], dval[l], planned[l])
    # the same plan with the page table walked once: slots against the scheduler's rule,
    # then the per-layer launches through them
    resolved = to_bf16(pool, gpu)
    plan_r = kvc.PagedKVWritePlan(dev.batch_indices, dev.positions, dev.kv_block_indices,
                                  dev.kv_block_indptrs, dev.kv_last_block_lens, s.num_kv_heads,
                                  s.head_dim, s.block_size, torch.bfloat16, resolve_slots=True)
    for l in range(L):
        plan_r.append(dkey[l], dval[l], resolved[l])
    torch.cuda.synchronize()
    assert np.array_equal(plan_r.slots.cpu().numpy(),
                          orc.paged_write_slots_np(w.index.batch_indices, w.index.positions,
                                                   w.index.kv_block_indices, w.index.kv_block_indptrs,
                                                   s.block_size))
    assert np.array_equal(bits_of(per_layer), want)
    assert np.array_equal(bits_of(fused), want)
    assert np.array_equal(bits_of(slotted), want)
    assert np.array_equal(bits_of(planned), want)
    assert np.array_equal(bits_of(resolved), want)
    with pytest.raises(TypeError):
        plan.append(dkey[0].float(), dval[0], planned[0])
    with pytest.raises(ValueError):
        plan.append(dkey[0], dval[0], planned[0][:, :, :8])


def test_write_plan_reads_token_strided_rows_and_outlives_nothing(gpu):
    """`kvc_write_plan_*` through `PagedKVWritePlan`: K and V read in place from
    slices of one fused `[T, 3*H*D]` projection (token stride 3 rows), 2-D and 3-D
    views, against the oracle; overlapping rows and short inputs are refused; a
    plan of zero tokens does nothing."""
    rng = np.random.default_rng(3)
    s = wl.LLAMA_3_2_1B
    w = wl._write_workload(s, 96, [5, 0, 31, 16], [3, 20, 1, 16], rng)
    T, H, D, bs, nb = w.num_tokens, s.num_kv_heads, s.head_dim, s.block_size, w.num_blocks
    row = H * D
    fused = bf16_bits((T, 3 * row), 4)
    pool = sentinel_pool((nb, 2, bs, H, D), 5)
    want = pool.copy()
    orc.c_append_paged_kv_cache(np.ascontiguousarray(fused[:, row:2 * row]).reshape(T, H, D),
                                np.ascontiguousarray(fused[:, 2 * row:]).reshape(T, H, D),
                                w.index.batch_indices, w.index.positions, want,
                                w.index.kv_block_indices, w.index.kv_block_indptrs)
    dev = kvc.to_device(w.index, bs, gpu)
    plan = kvc.PagedKVWritePlan(dev.batch_indices, dev.positions, dev.kv_block_indices,
                                dev.kv_block_indptrs, dev.kv_last_block_lens, H, D, bs, torch.bfloat16)
    dfused = to_bf16(fused, gpu)
    k2, v2 = dfused[:, row:2 * row], dfused[:, 2 * row:]
    for k, v in ((k2, v2), (k2.view(T, H, D), v2.view(T, H, D))):
        assert not k.is_contiguous()
        dpool = to_bf16(pool, gpu)
        plan.append(k, v, dpool)
        torch.cuda.synchronize()
        assert np.array_equal(bits_of(dpool), want)
    dpool = to_bf16(pool, gpu)
    with pytest.raises(ValueError):
        plan.append(k2[:1].expand(T, row), v2, dpool)          # every token reads the same row
    with pytest.raises(ValueError):
        plan.append(k2[:-1], v2, dpool)
    with pytest.raises(ValueError):
        plan.append(k2, v2, dpool.transpose(1, 2))
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), pool)
    empty = torch.empty(0, dtype=torch.int32, device=gpu)
    nothing = kvc.PagedKVWritePlan(empty, empty, dev.kv_block_indices, dev.kv_block_indptrs,
                                   dev.kv_last_block_lens, H, D, bs, torch.bfloat16)
    nothing.append(k2, v2, dpool)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), pool)


def test_append_paged_skips_tokens_with_bad_indices(gpu):
    w = wl.decode_step(wl.LLAMA_3_2_1B, num_blocks=64, batch=8, max_context=60, seed=4)
    s = w.shape
    idx = w.index
    T, H, D, bs, nb = w.num_tokens, s.num_kv_heads, s.head_dim, s.block_size, w.num_blocks
    key, value = bf16_bits((T, H, D), 1), bf16_bits((T, H, D), 2)
    pool = sentinel_pool((nb, 2, bs, H, D), 3)
    bi = idx.batch_indices.copy()
    pos = idx.positions.copy()
    bi[2] = -1          # no such request
    bi[5] = 8           # beyond the batch
    pos[6] = 1 << 20    # beyond the page table
    # beyond its own request's table, yet inside the array: would land in the next request's page
    own_pages = int(idx.kv_block_indptrs[bi[4] + 1] - idx.kv_block_indptrs[bi[4]])
    assert bi[4] + 1 < 8
    pos[4] = own_pages * bs + 3
    keep = np.asarray([0, 1, 3, 7])
    want = pool.copy()
    orc.c_append_paged_kv_cache(np.ascontiguousarray(key[keep]), np.ascontiguousarray(value[keep]),
                                bi[keep], pos[keep], want, idx.kv_block_indices,
                                idx.kv_block_indptrs)
    dpool = to_bf16(pool, gpu)

    def up(a):
        return torch.from_numpy(a).to(gpu)

    kvc.append_paged_kv_cache(to_bf16(key, gpu), to_bf16(value, gpu), up(bi), up(pos), dpool,
                              up(idx.kv_block_indices), up(idx.kv_block_indptrs),
                              up(idx.kv_last_block_lens))
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(dpool), want)
    # a plan with resolved slots skips the same tokens (their slot is -1) ...
    neg = idx.kv_block_indices.copy()
    plan = kvc.PagedKVWritePlan(up(bi), up(pos), up(neg), up(idx.kv_block_indptrs),
                                up(idx.kv_last_block_lens), H, D, bs, torch.bfloat16,
                                resolve_slots=True)
    dpool2 = to_bf16(pool, gpu)
    plan.append(to_bf16(key, gpu), to_bf16(value, gpu), dpool2)
    torch.cuda.synchronize()
    slots = plan.slots.cpu().numpy()
    assert np.array_equal(slots, orc.paged_write_slots_np(bi, pos, neg, idx.kv_block_indptrs, bs))
    assert (slots[[2, 4, 5, 6]] == -1).all() and (slots[keep] >= 0).all()
    assert np.array_equal(bits_of(dpool2), want)
    # ... and a negative page id or a page beyond the layer's pool is skipped too
    first = int(idx.kv_block_indptrs[bi[0]]) + int(pos[0]) // bs
    neg[first] = -3
    plan = kvc.PagedKVWritePlan(up(bi), up(pos), up(neg), up(idx.kv_block_indptrs),
                                up(idx.kv_last_block_lens), H, D, bs, torch.bfloat16,
                                resolve_slots=True)
    want3 = pool.copy()
    orc.c_append_paged_kv_cache(np.ascontiguousarray(key[keep[1:]]), np.ascontiguousarray(value[keep[1:]]),
                                bi[keep[1:]], pos[keep[1:]], want3, idx.kv_block_indices,
                                idx.kv_block_indptrs)
    dpool3 = to_bf16(pool, gpu)
    plan.append(to_bf16(key, gpu), to_bf16(value, gpu), dpool3)
    torch.cuda.synchronize()
    assert np.array_equal(plan.slots.cpu().numpy(),
                          orc.paged_write_slots_np(bi, pos, neg, idx.kv_block_indptrs, bs))
    assert plan.slots.cpu().numpy()[0] == -1
    assert np.array_equal(bits_of(dpool3), want3)
    half = to_bf16(pool, gpu)[:nb // 2]
    want4 = pool[:nb // 2].copy()
    small = kvc.PagedKVWritePlan(up(idx.batch_indices), up(idx.positions), up(idx.kv_block_indices),
                                 up(idx.kv_block_indptrs), up(idx.kv_last_block_lens), H, D, bs,
                                 torch.bfloat16, resolve_slots=True)
    small.append(to_bf16(key, gpu), to_bf16(value, gpu), half)
    torch.cuda.synchronize()
    pages = idx.slot_mapping // bs
    inside = np.flatnonzero(pages < nb // 2)
    assert 0 < len(inside) < T
    orc.reshape_and_cache_np(np.ascontiguousarray(key[inside]), np.ascontiguousarray(value[inside]),
                             want4, idx.slot_mapping[inside])
    assert np.array_equal(bits_of(half), want4)


def test_drop_in_writes_agree_with_and_without_the_call_extension(gpu, monkeypatch):
    """`append_paged_kv_cache` and `reshape_and_cache` check and launch the common
    layouts from the `_kvc_fast` extension; without it (or for a layout it does not
    take) the Python checks and ctypes do the same work. Both routes, same bits."""
    if _lib.fast() is None:
        pytest.skip("the call extension is switched off or not built")
    w = wl._write_workload(wl.LLAMA_3_2_1B, 128, [5, 0, 31, 16], [3, 20, 1, 16], np.random.default_rng(5))
    s = w.shape
    pool, want, dev, dkey, dval = _paged_case(gpu, w, 1, 60)
    routes = {}
    for route in ("extension", "python"):
        if route == "python":
            monkeypatch.setattr(_lib, "_fast_entries", {"append_paged": None, "reshape_and_cache": None})
        a, b, c = to_bf16(pool, gpu), to_bf16(pool, gpu), to_bf16(pool, gpu)
        kvc.append_paged_kv_cache(dkey[0], dval[0], dev.batch_indices, dev.positions, a[0],
                                  dev.kv_block_indices, dev.kv_block_indptrs, dev.kv_last_block_lens)
        kvc.reshape_and_cache(dkey[0], dval[0], b[0], dev.slot_mapping)
        kvc.reshape_and_cache(dkey[0], dval[0], c[0], dev.slot_mapping.int())       # int32 slots
        torch.cuda.synchronize()
        routes[route] = [bits_of(x) for x in (a, b, c)]
        for got in routes[route]:
            assert np.array_equal(got, want), route
    # a layout the extension leaves to Python: index arrays that are strided views
    strided = torch.stack([dev.batch_indices, dev.batch_indices], dim=1)[:, 0]
    assert not strided.is_contiguous() or strided.numel() <= 1
    monkeypatch.undo()
    d = to_bf16(pool, gpu)
    kvc.append_paged_kv_cache(dkey[0], dval[0], strided, dev.positions, d[0], dev.kv_block_indices,
                              dev.kv_block_indptrs, dev.kv_last_block_lens)
    torch.cuda.synchronize()
    assert np.array_equal(bits_of(d), want)
    # errors keep their Python types on both routes
    with pytest.raises(TypeError):
        kvc.append_paged_kv_cache(dkey[0], dval[0], dev.batch_indices.long(), dev.positions, d[0],
                                  dev.kv_block_indices, dev.kv_block_indptrs, dev.kv_last_block_lens)
    with pytest.raises(ValueError):
        kvc.reshape_and_cache(dkey[0][:-1], dval[0], d[0], dev.slot_mapping)


def test_write_runs_on_the_current_stream(gpu):
    """The op is enqueued on torch's current stream: a copy of the pool taken on
    the same side stream right after the call must already see the write."""
    T, H, D, nb, bs = 64, 8, 128, 32, 16
    rng = np.random.default_rng(2)
    slots = rng.permutation(nb * bs)[:T].astype(np.int64)
    key, value = bf16_bits((T, H, D), 1), bf16_bits((T, H, D), 2)
    pool = sentinel_pool((nb, 2, bs, H, D), 3)
    want = pool.copy()
    orc.reshape_and_cache_np(key, value, want, slots)
    dk, dv, dpool, ds = to_bf16(key, gpu), to_bf16(value, gpu), to_bf16(pool, gpu), \
        torch.from_numpy(slots).to(gpu)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        kvc.reshape_and_cache(dk, dv, dpool, ds)
        snap = dpool.clone()
    side.synchronize()
    assert np.array_equal(bits_of(snap), want)


def test_dtype_mismatch_raises(gpu):
    k = torch.zeros(2, 1, 8, dtype=torch.float16, device=gpu)
    pool = torch.zeros(4, 2, 4, 1, 8, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(TypeError):
        kvc.reshape_and_cache(k, k, pool, torch.zeros(2, dtype=torch.int64, device=gpu))
    with pytest.raises(TypeError):
        kvc.append_paged_kv_cache(k.bfloat16(), k.bfloat16(),
                                  torch.zeros(2, dtype=torch.int64, device=gpu),
                                  torch.zeros(2, dtype=torch.int32, device=gpu), pool,
                                  torch.zeros(2, dtype=torch.int32, device=gpu),
                                  torch.zeros(2, dtype=torch.int32, device=gpu),
                                  torch.zeros(1, dtype=torch.int32, device=gpu))


# token count -> what the launch rule must pick on a 256-CU part for 32 layers of 2 KiB rows:
# (kernel, planes or vectors per lane, lanes per workgroup, lanes wait per load) slot-mapped /
# page-table addressed. fill = lanes of the launch / lanes the GPU holds at once.
_TOKEN, _PLANE = _lib.KVC_KERNEL_WRITE_ROWS, _lib.KVC_KERNEL_WRITE_PLANES
SIZE_RULE = {
    12: ((_TOKEN, 1, 256, 0), (_TOKEN, 1, 256, 0)),     # latency-bound: token kernel
    16: ((_TOKEN, 1, 256, 0), (_PLANE, 2, 256, 0)),     # fill 1/4 at one plane per lane: page-table launches switch
    32: ((_PLANE, 1, 256, 0), (_PLANE, 2, 256, 0)),     # fill 1/2: slot-mapped launches switch
    40: ((_PLANE, 2, 256, 0), (_PLANE, 2, 256, 0)),     # fewest planes per lane that leave the GPU half full
    64: ((_PLANE, 2, 256, 0), (_PLANE, 2, 256, 0)),
    100: ((_PLANE, 4, 256, 0), (_PLANE, 4, 256, 0)),
    128: ((_PLANE, 4, 256, 0), (_PLANE, 4, 256, 0)),
    200: ((_PLANE, 4, 512, 1), (_PLANE, 4, 256, 0)),    # over half full at 4: one resident set, lanes wait per load
    256: ((_PLANE, 4, 512, 1), (_PLANE, 4, 256, 0)),    # the decode step of the benchmark
    300: ((_PLANE, 8, 512, 1), (_PLANE, 8, 256, 0)),
    600: ((_TOKEN, 1, 256, 0), (_TOKEN, 1, 256, 0)),    # no depth fits one set: stream through the token kernel
}


@pytest.mark.parametrize("T", sorted(SIZE_RULE))
@pytest.mark.parametrize("paged", [False, True])
def test_one_launch_write_through_every_shape_the_size_rule_picks(gpu, T, paged):
    """32 layers of the Llama-3-8B row in one launch, at token counts on both sides
    of each switch of the launch-shape rule (token kernel for latency-bound
    launches; plane kernel with the fewest planes per lane that leave the GPU half
    full, else that fit one resident set; token kernel again beyond), slot-mapped
    and page-table addressed; the shape that ran is asserted as well as the bits."""
    s = wl.LLAMA_3_8B
    L, nb, bs = 32, 96, s.block_size
    w = wl.decode_step(s, num_blocks=nb, batch=T, max_context=4, seed=T) if T <= nb else \
        wl.chunked_prefill(s, num_blocks=nb, num_seqs=4, chunk_tokens=T - T % 4, min_context=1,
                           max_context=40, seed=T)
    idx = w.index
    n = w.num_tokens
    key, value = bf16_bits((L, n, s.num_kv_heads, s.head_dim), T), bf16_bits((L, n, s.num_kv_heads, s.head_dim), T + 1)
    pool = sentinel_pool((L, nb, 2, bs, s.num_kv_heads, s.head_dim), T + 2)
    want = pool.copy()
    for l in range(L):
        orc.c_reshape_and_cache(key[l], value[l], want[l], idx.slot_mapping)
    dev = kvc.to_device(idx, bs, gpu)
    dpool = to_bf16(pool, gpu)
    if paged:
        kvc.append_paged_kv_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dev.batch_indices,
                                         dev.positions, dpool, dev.kv_block_indices,
                                         dev.kv_block_indptrs, dev.kv_last_block_lens)
    else:
        kvc.reshape_and_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool, dev.slot_mapping)
    torch.cuda.synchronize()
    ran = _lib.last_launch()
    assert _lib.lib().kvc_tuning_modified() == 0
    assert (ran["kernel"], ran["per_lane"], ran["threads"], ran["pipe"]) == SIZE_RULE[T][1 if paged else 0]
    assert np.array_equal(bits_of(dpool), want)


# (shape, layers, tokens) -> launch slot-mapped / page-table addressed, for the corners of the
# rule that 32 layers of wide rows do not reach
_S8 = wl.LLAMA_3_1_70B.shard(8)          # one KV head: 256-byte rows
RULE_CORNERS = {
    "one layer, 1 KiB rows, one resident set at 2 planes per lane":
        (wl.QWEN_2_5_7B, 1, 8192, (_PLANE, 2, 256, 1), (_PLANE, 2, 256, 0)),
    "one layer, 1 KiB rows, beyond one set: few planes keep page-table launches on the plane kernel":
        (wl.QWEN_2_5_7B, 1, 12288, (_TOKEN, 1, 128, 0), (_PLANE, 2, 256, 0)),
    "256-byte rows, 160 KiB of source rows": (_S8, 80, 4, (_TOKEN, 1, 256, 0), (_TOKEN, 1, 256, 0)),
    "256-byte rows, 320 KiB of source rows": (_S8, 80, 8, (_PLANE, 1, 128, 0), (_PLANE, 2, 128, 0)),
    "256-byte rows, over half full at 1 plane per lane": (_S8, 80, 160, (_PLANE, 2, 256, 0), (_PLANE, 2, 256, 0)),
    "256-byte rows, beyond one set": (_S8, 80, 2048, (_PLANE, 1, 256, 0), (_PLANE, 2, 256, 0)),
}


@pytest.mark.parametrize("case", sorted(RULE_CORNERS))
@pytest.mark.parametrize("paged", [False, True])
def test_corners_of_the_launch_rule(gpu, case, paged):
    s, L, T, want_slot, want_paged = RULE_CORNERS[case]
    bs = s.block_size
    nb = T // bs + 16
    w = wl.chunked_prefill(s, num_blocks=nb, num_seqs=4, chunk_tokens=T, min_context=1, max_context=40, seed=7)
    idx = w.index
    n = w.num_tokens
    assert n == T
    key, value = bf16_bits((L, n, s.num_kv_heads, s.head_dim), 3), bf16_bits((L, n, s.num_kv_heads, s.head_dim), 4)
    pool = sentinel_pool((L, nb, 2, bs, s.num_kv_heads, s.head_dim), 5)
    want = pool.copy()
    for l in range(L):
        orc.c_reshape_and_cache(key[l], value[l], want[l], idx.slot_mapping)
    dev = kvc.to_device(idx, bs, gpu)
    dpool = to_bf16(pool, gpu)
    if paged:
        kvc.append_paged_kv_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dev.batch_indices,
                                         dev.positions, dpool, dev.kv_block_indices,
                                         dev.kv_block_indptrs, dev.kv_last_block_lens)
    else:
        kvc.reshape_and_cache_layers(to_bf16(key, gpu), to_bf16(value, gpu), dpool, dev.slot_mapping)
    torch.cuda.synchronize()
    ran = _lib.last_launch()
    assert _lib.lib().kvc_tuning_modified() == 0
    assert (ran["kernel"], ran["per_lane"], ran["threads"], ran["pipe"]) == (want_paged if paged else want_slot)
    assert np.array_equal(bits_of(dpool), want)

"""The native host <-> disk tier against the closed form disk[dst] = host[src].

Runs without a GPU: the tier is file I/O. The oracle is the NumPy statement of
runtime/worker/llm_worker/kv_worker.py:229-247 (and its per-layer loop form);
the file format is checked by NumPy's own reader and writer."""
import mmap
import os

import numpy as np
import pytest

from lmserve_amd import DiskTier, _lib
from oracle import kvc_oracle as orc


def _aligned(shape, dtype):
    """A page-aligned array (what a pinned host pool is), so O_DIRECT can apply."""
    n = int(np.prod(shape)) * np.dtype(dtype).itemsize
    buf = mmap.mmap(-1, max(n, 1))
    return np.frombuffer(buf, dtype=dtype, count=int(np.prod(shape))).reshape(shape)


def _fill(a, rng):
    a[...] = rng.integers(0, np.iinfo(a.dtype).max, size=a.shape, dtype=a.dtype)


def test_oracle_forms_agree_and_match_a_hand_case():
    rng = np.random.default_rng(0)
    host = rng.integers(0, 1 << 16, size=(5, 3, 4), dtype=np.uint16)
    disk = np.zeros((6, 3, 4), dtype=np.uint16)
    a, b = disk.copy(), disk.copy()
    orc.save_blocks_to_disk_np(host, a, [4, 0], [1, 5])
    orc.save_blocks_to_disk_loops(host, b, [4, 0], [1, 5])
    assert np.array_equal(a, b)
    assert np.array_equal(a[1], host[4]) and np.array_equal(a[5], host[0])
    assert not a[[0, 2, 3, 4]].any()                      # nothing else touched
    h1, h2 = host.copy(), host.copy()
    orc.load_blocks_from_disk_np(h1, a, [5, 1], [2, 3])
    orc.load_blocks_from_disk_loops(h2, a, [5, 1], [2, 3])
    assert np.array_equal(h1, h2)
    assert np.array_equal(h1[2], host[0]) and np.array_equal(h1[3], host[4])


def test_new_file_is_a_numpy_array_with_page_aligned_data(tmp_path):
    path = str(tmp_path / "disk-kv-cache-0.npy")
    with DiskTier(path, (7, 3, 2048), np.uint16) as d:
        assert d.created and d.data_offset == 4096 and d.row_bytes == 3 * 2048 * 2
    a = np.load(path, mmap_mode="r")
    assert a.shape == (7, 3, 2048) and a.dtype == np.uint16 and a.offset == 4096
    assert not np.asarray(a).any()                         # sparse file reads as zeros
    assert os.path.getsize(path) == 4096 + 7 * 3 * 2048 * 2
    with DiskTier(path, (7, 3, 2048), np.uint16) as d:     # reopened, not recreated
        assert not d.created


@pytest.mark.parametrize("shape,dtype,threads,direct", [
    ((24, 4, 1024), np.uint16, 8, True),      # 8 KiB rows: aligned
    ((24, 4, 1024), np.uint16, 1, False),
    ((17, 3, 100), np.uint16, 4, True),       # 600-byte rows: never aligned, buffered path
    ((9, 2, 512), np.float32, 3, True),
    ((12, 5, 333), np.float16, 8, True),
])
def test_save_and_load_match_the_closed_form(tmp_path, shape, dtype, threads, direct):
    rng = np.random.default_rng(shape[0] * 7 + threads)
    ndb, L, E = shape
    nhb = ndb + 5
    host = _aligned((nhb, L, E), np.dtype(dtype).str.replace("f", "u"))   # payload is opaque bits
    host = host.view(dtype)
    raw = host.view(np.dtype(f"u{host.itemsize}"))
    _fill(raw, rng)
    path = str(tmp_path / "cache.npy")
    with DiskTier(path, shape, dtype, direct=direct, threads=threads) as d:
        want_disk = np.zeros(shape, dtype=raw.dtype)
        for step in range(3):
            n = int(rng.integers(1, ndb + 1))
            src = rng.permutation(nhb)[:n]
            dst = rng.permutation(ndb)[:n]
            if step == 1:                                   # runs of consecutive pairs merge
                src = np.arange(2, 2 + n) % nhb
                dst = np.arange(n)
            d.save_blocks(host, src, dst)
            orc.save_blocks_to_disk_np(raw, want_disk, src, dst)
            got = np.load(path, mmap_mode="r")
            assert np.array_equal(np.asarray(got).view(raw.dtype), want_disk), f"save step {step}"
            del got
        for step in range(3):
            n = int(rng.integers(1, min(ndb, nhb) + 1))
            src = rng.permutation(ndb)[:n]
            dst = rng.permutation(nhb)[:n]
            want_host = raw.copy()
            orc.load_blocks_from_disk_np(want_host, want_disk, src, dst)
            d.load_blocks(host, src, dst)
            assert np.array_equal(raw, want_host), f"load step {step}"
        d.sync()
        # empty lists are no-ops (kv_worker.py:255)
        d.save_blocks(host, [], [])
        d.load_blocks(host, [], [])


def test_direct_io_is_used_when_alignment_allows_and_gives_the_same_bytes(tmp_path):
    rng = np.random.default_rng(5)
    host = _aligned((10, 2, 4096), np.uint16)              # 16 KiB rows
    _fill(host, rng)
    path = str(tmp_path / "direct.npy")
    with DiskTier(path, (8, 2, 4096), np.uint16, direct=True) as d:
        used_direct = d.is_direct                           # the file system may refuse O_DIRECT
        d.save_blocks(host, [9, 1, 2, 3], [0, 4, 5, 6])
        assert not d.last_transfer_staged                   # aligned ordinary memory goes in place
        d.sync()
        back = _aligned((10, 2, 4096), np.uint16)
        d.load_blocks(back, [0, 4, 5, 6], [0, 1, 2, 3])
    got = np.load(path, mmap_mode="r")
    assert np.array_equal(got[0], host[9]) and np.array_equal(got[4:7], host[1:4])
    assert np.array_equal(back[0], host[9]) and np.array_equal(back[1:4], host[1:4])
    with DiskTier(path, (8, 2, 4096), np.uint16, direct=False) as d:
        assert not d.is_direct
    print("O_DIRECT in use:", used_direct)


def test_unaligned_host_pool_is_staged_through_aligned_buffers(tmp_path):
    rng = np.random.default_rng(6)
    backing = np.zeros(10 * 2 * 4096 + 8, dtype=np.uint16)
    host = backing[1:1 + 10 * 2 * 4096].reshape(10, 2, 4096)   # 2 bytes off any alignment
    _fill(host, rng)
    with DiskTier(str(tmp_path / "u.npy"), (4, 2, 4096), np.uint16, direct=True) as d:
        d.save_blocks(host, [7, 8], [3, 0])
        assert d.last_transfer_staged == d.is_direct
        out = np.zeros_like(host)
        d.load_blocks(out, [3, 0], [1, 2])
    assert np.array_equal(out[1], host[7]) and np.array_equal(out[2], host[8])


def test_long_runs_are_split_across_threads(tmp_path):
    """80 consecutive 1 MiB blocks: one run, cut into extents of at most 64 MiB."""
    rng = np.random.default_rng(7)
    host = _aligned((80, 1, 1 << 19), np.uint16)
    host[...] = rng.integers(0, 1 << 16, size=(80, 1, 1), dtype=np.uint16)   # one value per block
    host[:, 0, -1] = np.arange(80)
    path = str(tmp_path / "runs.npy")
    with DiskTier(path, (80, 1, 1 << 19), np.uint16, threads=4) as d:
        d.save_blocks(host, np.arange(80), np.arange(80))
        back = _aligned((80, 1, 1 << 19), np.uint16)
        d.load_blocks(back, np.arange(80), np.arange(80)[::-1].copy())
    assert np.array_equal(np.load(path, mmap_mode="r"), host)
    assert np.array_equal(back[::-1], host)


def test_save_and_load_may_run_concurrently_on_disjoint_blocks(tmp_path):
    """The KV worker's dispatcher can have a Host->Disk and a Disk->Host copy in
    flight at once (both legs run in threads)."""
    import threading
    rng = np.random.default_rng(11)
    host = _aligned((32, 2, 8192), np.uint16)
    _fill(host, rng)
    with DiskTier(str(tmp_path / "c.npy"), (32, 2, 8192), np.uint16, threads=4) as d:
        d.save_blocks(host, np.arange(16), np.arange(16))              # disk 0..15 = host 0..15
        want = host.copy()
        want[16:24] = host[0:8]
        errors = []

        def saver():
            try:
                for _ in range(10):
                    d.save_blocks(host, np.arange(24, 32), np.arange(16, 24))   # disk 16..23 = host 24..31
            except Exception as exc:   # pragma: no cover
                errors.append(exc)

        def loader():
            try:
                for _ in range(10):
                    d.load_blocks(host, np.arange(0, 8), np.arange(16, 24))     # host 16..23 = disk 0..7
            except Exception as exc:   # pragma: no cover
                errors.append(exc)

        ts = [threading.Thread(target=saver), threading.Thread(target=loader)]
        [t.start() for t in ts]
        [t.join() for t in ts]
        assert not errors
        assert np.array_equal(host, want)
    disk = np.load(str(tmp_path / "c.npy"), mmap_mode="r")
    assert np.array_equal(disk[16:24], want[24:32]) and np.array_equal(disk[:16], want[:16])


def test_preallocation_reserves_the_blocks_of_a_new_file(tmp_path):
    sparse, full = str(tmp_path / "sparse.npy"), str(tmp_path / "full.npy")
    shape = (64, 2, 8192)                                   # 2 MiB of payload
    with DiskTier(sparse, shape, np.uint16) as a, DiskTier(full, shape, np.uint16, preallocate=True) as b:
        assert a.created and b.created
    payload = 64 * 2 * 8192 * 2
    assert os.stat(full).st_blocks * 512 >= payload         # reserved on disk
    assert os.stat(sparse).st_blocks * 512 < payload        # holes, like the reference's memory map
    assert os.path.getsize(full) == os.path.getsize(sparse) == 4096 + payload
    assert not np.asarray(np.load(full, mmap_mode="r")).any()


def test_staging_buffers_are_reused_across_calls(tmp_path):
    """Staged transfers (here: an unaligned pool) keep their aligned buffers with
    the handle; many calls in a row give the same bytes as the closed form."""
    rng = np.random.default_rng(13)
    backing = np.zeros(12 * 2 * 4096 + 8, dtype=np.uint16)
    host = backing[1:1 + 12 * 2 * 4096].reshape(12, 2, 4096)
    _fill(host, rng)
    want_disk = np.zeros((10, 2, 4096), dtype=np.uint16)
    path = str(tmp_path / "reuse.npy")
    with DiskTier(path, (10, 2, 4096), np.uint16, threads=3) as d:
        for step in range(8):
            src = rng.permutation(12)[:5]
            dst = rng.permutation(10)[:5]
            d.save_blocks(host, src, dst)
            orc.save_blocks_to_disk_np(host, want_disk, src, dst)
            back = rng.permutation(12)[:4]
            frm = rng.permutation(10)[:4]
            want_host = host.copy()
            orc.load_blocks_from_disk_np(want_host, want_disk, frm, back)
            d.load_blocks(host, frm, back)
            assert np.array_equal(host, want_host), step
    assert np.array_equal(np.load(path, mmap_mode="r"), want_disk)


def test_a_numpy_made_file_is_reused_in_place(tmp_path):
    """The reference creates the file with np.lib.format.open_memmap (kv_worker.py:78-82):
    data starts at byte 128 there, so the tier uses buffered I/O on it."""
    path = str(tmp_path / "ref-made.npy")
    rng = np.random.default_rng(8)
    mm = np.lib.format.open_memmap(path, mode="w+", dtype=np.uint16, shape=(6, 2, 2048))
    _fill(mm, rng)
    mm.flush()
    before = np.asarray(mm).copy()
    del mm
    host = _aligned((4, 2, 2048), np.uint16)
    with DiskTier(path, (6, 2, 2048), np.uint16) as d:
        assert not d.created and d.data_offset == 128 and not d.is_direct
        d.load_blocks(host, [5, 0], [1, 2])
        assert np.array_equal(host[1], before[5]) and np.array_equal(host[2], before[0])
        host[3] = 0xABCD
        d.save_blocks(host, [3], [4])
    after = np.load(path, mmap_mode="r")
    want = before.copy()
    want[4] = 0xABCD
    assert np.array_equal(after, want)


def test_format_2_headers_are_understood(tmp_path):
    path = str(tmp_path / "v2.npy")
    data = np.arange(3 * 2 * 8, dtype=np.uint16).reshape(3, 2, 8)
    with open(path, "wb") as f:
        np.lib.format.write_array(f, data, version=(2, 0))
    with DiskTier(path, (3, 2, 8), np.uint16) as d:
        assert not d.created
        host = np.zeros((2, 2, 8), dtype=np.uint16)
        d.load_blocks(host, [2], [0])
    assert np.array_equal(host[0], data[2])


@pytest.mark.parametrize("what", ["shape", "dtype", "garbage", "truncated", "fortran"])
def test_a_file_that_does_not_match_is_recreated(tmp_path, what):
    """kv_worker.py:55-73: a changed configuration or an unreadable file is removed
    and a new, empty one takes its place."""
    path = str(tmp_path / "stale.npy")
    if what == "garbage":
        open(path, "wb").write(b"not an array" * 100)
    elif what == "truncated":
        np.save(path, np.ones((4, 2, 64), dtype=np.uint16))
        os.truncate(path, 300)
    elif what == "fortran":
        np.save(path, np.asfortranarray(np.ones((4, 2, 64), dtype=np.uint16)))
    else:
        shape = (5, 2, 64) if what == "shape" else (4, 2, 64)
        np.save(path, np.ones(shape, dtype=np.uint16 if what == "shape" else np.int16))
    with DiskTier(path, (4, 2, 64), np.uint16) as d:
        assert d.created
    a = np.load(path, mmap_mode="r")
    assert a.shape == (4, 2, 64) and a.dtype == np.uint16 and not np.asarray(a).any()


def test_errors(tmp_path):
    path = str(tmp_path / "e.npy")
    host = np.zeros((4, 2, 64), dtype=np.uint16)
    with DiskTier(path, (3, 2, 64), np.uint16) as d:
        with pytest.raises(IndexError, match="disk block id 3"):
            d.save_blocks(host, [0], [3])
        with pytest.raises(IndexError, match="host block id 4"):
            d.load_blocks(host, [0], [4])
        with pytest.raises(IndexError):
            d.save_blocks(host, [-1], [0])
        assert not np.asarray(np.load(path, mmap_mode="r")).any()      # nothing was written
        with pytest.raises(ValueError, match="differ in length"):
            d.save_blocks(host, [0, 1], [0])
        with pytest.raises(ValueError, match="do not match"):
            d.save_blocks(np.zeros((4, 2, 32), dtype=np.uint16), [0], [0])
        with pytest.raises(ValueError, match="do not match"):
            d.save_blocks(host.view(np.int16), [0], [0])
        ro = host.copy()
        ro.flags.writeable = False
        with pytest.raises(ValueError, match="read-only"):
            d.load_blocks(ro, [0], [0])
    with pytest.raises(ValueError, match="closed"):
        d.save_blocks(host, [0], [0])
    with pytest.raises(OSError):
        DiskTier(str(tmp_path / "no-such-dir" / "x.npy"), (3, 2, 64), np.uint16)
    with pytest.raises(ValueError):
        DiskTier(path, (0, 2, 64), np.uint16)
    h = _lib.lib()
    assert h.kvc_disk_close(None) == _lib.KVC_OK
    assert h.kvc_disk_sync(None) == _lib.KVC_ERR_INVALID_ARG
    assert h.kvc_disk_info(None, 0) == -1

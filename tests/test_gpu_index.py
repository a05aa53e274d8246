"""GPU parity of the page-table index preparation against the CPU oracle."""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
from oracle import kvc_oracle as orc

pytestmark = pytest.mark.gpu


def _up(a, gpu):
    return torch.from_numpy(np.asarray(a, dtype=np.int32)).to(gpu)


@pytest.mark.parametrize("page_size", [16, 4, 3])
def test_get_seq_lens_matches_oracle(gpu, page_size):
    rng = np.random.default_rng(page_size)
    B = 300
    pages = rng.integers(0, 40, size=B)
    pages[::17] = 0                                    # requests without pages: clamp
    indptr = np.cumsum(np.concatenate([[0], pages])).astype(np.int32)
    last = rng.integers(1, page_size + 1, size=B).astype(np.int32)
    want = orc.c_get_seq_lens(indptr, last, page_size)
    assert np.array_equal(want, orc.get_seq_lens_np(indptr, last, page_size))
    got = kvc.get_seq_lens(_up(indptr, gpu), _up(last, gpu), page_size)
    assert got.dtype == torch.int32
    assert np.array_equal(got.cpu().numpy(), want)
    assert kvc.get_seq_lens(_up([0], gpu), _up([], gpu), page_size).numel() == 0


def test_get_batch_indices_positions_matches_oracle(gpu):
    rng = np.random.default_rng(1)
    B = 257
    n_new = rng.integers(0, 9, size=B)                 # includes requests with no new token
    n_new[5] = 2048                                    # one long prefill chunk
    filled = rng.integers(0, 5000, size=B)
    seq_lens = (filled + n_new).astype(np.int32)
    indptr = np.cumsum(np.concatenate([[0], n_new])).astype(np.int32)
    nnz = int(indptr[-1])
    want_b, want_p = orc.c_get_batch_indices_positions(indptr, seq_lens, nnz)
    np_b, np_p = orc.get_batch_indices_positions_np(indptr, seq_lens, nnz)
    assert np.array_equal(want_b, np_b) and np.array_equal(want_p, np_p)
    got_b, got_p = kvc.get_batch_indices_positions(_up(indptr, gpu), _up(seq_lens, gpu), nnz)
    assert np.array_equal(got_b.cpu().numpy(), want_b)
    assert np.array_equal(got_p.cpu().numpy(), want_p)
    # positions are exactly range(filled, filled + n_new) per request
    at = 0
    for b in range(B):
        assert got_p[at:at + n_new[b]].cpu().tolist() == list(range(filled[b], filled[b] + n_new[b]))
        at += n_new[b]


def test_index_prep_rejects_wrong_dtypes_and_lengths(gpu):
    with pytest.raises(TypeError):
        kvc.get_seq_lens(torch.zeros(3, dtype=torch.int64, device=gpu), _up([1, 1], gpu), 16)
    with pytest.raises(ValueError):
        kvc.get_seq_lens(_up([0, 1], gpu), _up([1, 1], gpu), 16)
    with pytest.raises(ValueError):
        kvc.get_batch_indices_positions(_up([0, 1], gpu), _up([1, 1], gpu), 1)


@pytest.mark.parametrize("kind", ["decode", "chunked_prefill", "mixed", "large_batch", "empty"])
def test_one_launch_index_build_matches_the_host_construction(gpu, kind):
    """Prefix sums, last-page lengths, request indices, positions and slots from
    one device launch equal what the host-side construction (the restatement of
    the reference's list building) produces."""
    import workloads as wl
    rng = np.random.default_rng(11)
    bs = 16
    if kind == "decode":
        reqs = wl.decode_step(wl.LLAMA_3_8B, num_blocks=4096, batch=256, max_context=200, seed=5).inputs
    elif kind == "chunked_prefill":
        reqs = wl.chunked_prefill(wl.QWEN_2_5_7B, num_blocks=16384, seed=6).inputs
    elif kind == "mixed":
        filled = [0, 37, 5, 64, 200, 16, 15, 0]
        new = [70, 1, 1, 33, 1, 16, 2, 1]
        reqs = wl._write_workload(wl.LLAMA_3_2_1B, 256, filled, new, rng).inputs
    elif kind == "large_batch":                       # more requests than one scan chunk
        filled = rng.integers(0, 40, size=2500).tolist()
        new = rng.integers(1, 4, size=2500).tolist()
        reqs = wl._write_workload(wl.LLAMA_3_2_1B, 16384, filled, new, rng).inputs
    else:
        reqs = []
    host = kvc.make_kv_index_inputs(reqs, bs)
    dev = kvc.to_device_one_launch(reqs, bs, gpu)
    torch.cuda.synchronize()
    # the oracle's statement of the same index, from the per-request scalars in batch order
    ordered = [reqs[i] for i in host.order]
    want = orc.build_write_index_np([r.input_len for r in ordered], [r.context_len for r in ordered],
                                    [len(r.block_ids) for r in ordered],
                                    [b for r in ordered for b in r.block_ids], bs)
    for got, exp in zip((dev.cu_seqlens_q, dev.kv_block_indptrs, dev.kv_last_block_lens,
                         dev.batch_indices, dev.positions, dev.slot_mapping), want):
        assert np.array_equal(got.cpu().numpy(), exp)
    assert np.array_equal(dev.cu_seqlens_q.cpu().numpy(), host.cu_seqlens_q)
    assert np.array_equal(dev.kv_block_indptrs.cpu().numpy(), host.kv_block_indptrs)
    assert np.array_equal(dev.kv_last_block_lens.cpu().numpy(), host.kv_last_block_lens)
    assert np.array_equal(dev.kv_block_indices.cpu().numpy(), host.kv_block_indices)
    assert np.array_equal(dev.batch_indices.cpu().numpy(), host.batch_indices)
    assert np.array_equal(dev.positions.cpu().numpy(), host.position_ids)
    assert np.array_equal(dev.slot_mapping.cpu().numpy(), host.slot_mapping)
    assert dev.prefill_input_len == host.prefill_input_len
    # and it agrees with the two-call device path
    two = kvc.to_device(host, bs, gpu)
    assert torch.equal(two.batch_indices, dev.batch_indices)
    assert torch.equal(two.positions, dev.positions)


def test_one_launch_index_build_marks_positions_outside_the_table(gpu):
    cu, indptr, last, bi, pos, slots = kvc.build_write_index(
        _up([2, 1], gpu), _up([40, 5], gpu), _up([1, 1], gpu), _up([7, 3], gpu), 16, 3)
    assert cu.tolist() == [0, 2, 3] and indptr.tolist() == [0, 1, 2] and last.tolist() == [8, 5]
    assert pos.tolist() == [38, 39, 4]
    # request 0 claims 40 tokens with a single block: positions 38, 39 index past its table
    assert slots.tolist()[2] == 3 * 16 + 4
    assert slots.tolist()[0] == -1 and slots.tolist()[1] == -1
    # a position past the request's OWN table must not borrow the next request's block
    _, _, _, _, pos, slots = kvc.build_write_index(
        _up([1, 1], gpu), _up([20, 5], gpu), _up([1, 1], gpu), _up([7, 3], gpu), 16, 2)
    assert pos.tolist() == [19, 4] and slots.tolist() == [-1, 3 * 16 + 4]

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

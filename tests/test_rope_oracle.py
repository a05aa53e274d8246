"""Pins the rotary-embedding oracles and the cos/sin table (CPU)."""
import math

import numpy as np
import pytest
import torch

from lmserve_amd.rotary import make_cos_sin_cache
from oracle import rope_oracle as ro

LLAMA3_SCALING = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                  "original_max_position_embeddings": 8192}


def _inputs(T=7, Hq=4, Hkv=2, D=16, rd=16, P=50, seed=0):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((T, Hq * D))
    k = rng.standard_normal((T, Hkv * D))
    pos = rng.integers(0, P, size=T)
    cs = ro.cos_sin_table_f64(rd, P)
    return q, k, pos, cs


def test_rotation_is_complex_multiplication():
    """(x + iy)(cos + i sin): an independent statement of the same rotation."""
    T, Hq, Hkv, D, rd = 7, 4, 2, 16, 16
    q, k, pos, cs = _inputs(T, Hq, Hkv, D, rd)
    q_out, k_out = ro.rotary_pos_emb_f64(q, k, pos, cs, D)
    half = rd // 2
    for x, out in ((q, q_out), (k, k_out)):
        xh = x.reshape(T, -1, D)
        z = xh[:, :, :half] + 1j * xh[:, :, half:rd]
        w = cs[pos, :half] + 1j * cs[pos, rd:rd + half]          # cos + i sin of the x lanes
        zz = z * w[:, None, :]
        oh = out.reshape(T, -1, D)
        assert np.allclose(oh[:, :, :half], zz.real, rtol=0, atol=1e-12)
        assert np.allclose(oh[:, :, half:rd], zz.imag, rtol=0, atol=1e-12)


def test_position_zero_is_the_identity_and_norms_are_preserved():
    q, k, pos, cs = _inputs()
    q0, k0 = ro.rotary_pos_emb_f64(q, k, np.zeros_like(pos), cs, 16)
    assert np.array_equal(q0, q) and np.array_equal(k0, k)
    q1, k1 = ro.rotary_pos_emb_f64(q, k, pos, cs, 16)
    assert not np.allclose(q1, q)
    for a, b in ((q, q1), (k, k1)):
        ah, bh = a.reshape(7, -1, 2, 8), b.reshape(7, -1, 2, 8)     # [T, H, (x|y), lane]
        assert np.allclose((ah ** 2).sum(axis=2), (bh ** 2).sum(axis=2), rtol=1e-12)


def test_angles_add():
    """Rotating to position a and then by position b equals position a + b."""
    q, k, _, cs = _inputs(P=64)
    a = np.full(7, 11)
    b = np.full(7, 30)
    q1, k1 = ro.rotary_pos_emb_f64(q, k, a, cs, 16)
    q2, k2 = ro.rotary_pos_emb_f64(q1, k1, b, cs, 16)
    q3, k3 = ro.rotary_pos_emb_f64(q, k, a + b, cs, 16)
    assert np.allclose(q2, q3, atol=1e-10) and np.allclose(k2, k3, atol=1e-10)


def test_partial_rotary_leaves_the_tail_lanes():
    T, D, rd = 5, 16, 8
    q, k, pos, _ = _inputs(T=T, D=D, rd=rd)
    cs = ro.cos_sin_table_f64(rd, 50)
    q1, _ = ro.rotary_pos_emb_f64(q, k, pos, cs, D)
    assert np.array_equal(q1.reshape(T, -1, D)[:, :, rd:], q.reshape(T, -1, D)[:, :, rd:])
    assert not np.allclose(q1.reshape(T, -1, D)[:, :, :rd], q.reshape(T, -1, D)[:, :, :rd])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_torch_references_stay_within_their_rounding_of_the_f64_formula(dtype):
    T, Hq, Hkv, D = 33, 4, 2, 32
    g = torch.Generator().manual_seed(1)
    q = torch.randn(T, Hq * D, generator=g).to(dtype)
    k = torch.randn(T, Hkv * D, generator=g).to(dtype)
    pos = torch.randint(0, 500, (T,), generator=g)
    cs = make_cos_sin_cache(D, 500, dtype=dtype)
    exact_q, exact_k = ro.rotary_pos_emb_f64(q.double().numpy(), k.double().numpy(), pos.numpy(),
                                             cs.double().numpy(), D)
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -24}[dtype]
    fq, fk = ro.rotary_pos_emb_fp32(q, k, pos, cs, D)
    pq, pk = ro.rotary_pos_emb_per_op(q, k, pos, cs, D)
    # magnitude of the two products feeding each output lane
    mag_q = np.abs(exact_q) + 2 * np.abs(q.double().numpy()).reshape(T, -1, D).max(axis=2).repeat(D, axis=1)
    for got, exact in ((fq, exact_q), (fk, exact_k)):
        err = np.abs(got.double().numpy() - exact)
        assert (err <= eps * np.abs(exact) * 1.01 + 1e-6 * eps + 3e-7).all()     # half an ulp
    err = np.abs(pq.double().numpy() - exact_q)
    assert (err <= 4 * eps * mag_q).all()                                          # per-op rounding


def test_cos_sin_table_matches_the_closed_form():
    for rd, P, base, scaling in ((64, 300, 10000.0, None), (128, 200, 500000.0, LLAMA3_SCALING),
                                 (8, 40, 10000.0, None)):
        want = ro.cos_sin_table_f64(rd, P, base, scaling)
        got32 = make_cos_sin_cache(rd, P, base, scaling, dtype=torch.float32).double().numpy()
        # fp32 angles p * inv_freq carry an absolute error that grows with p
        assert np.abs(got32 - want).max() < 2e-4
        got16 = make_cos_sin_cache(rd, P, base, scaling, dtype=torch.bfloat16).double().numpy()
        assert np.abs(got16 - want).max() < 2.0 ** -8 + 2e-4
        assert got32.shape == (P, 2 * rd)
        assert np.allclose(got32[:, :rd] ** 2 + got32[:, rd:] ** 2, 1.0, atol=1e-5)
        assert np.array_equal(got32[:, :rd // 2], got32[:, rd // 2:rd])            # cat(freqs, freqs)
        assert np.array_equal(got32[0, :rd], np.ones(rd)) and np.array_equal(got32[0, rd:], np.zeros(rd))


def test_llama3_scaling_bands():
    rd, base = 128, 500000.0
    plain = ro.cos_sin_table_f64(rd, 2, base)
    scaled = ro.cos_sin_table_f64(rd, 2, base, LLAMA3_SCALING)
    ang_plain = np.arctan2(plain[1, rd:rd + rd // 2], plain[1, :rd // 2])          # = inv_freq
    ang_scaled = np.arctan2(scaled[1, rd:rd + rd // 2], scaled[1, :rd // 2])
    wavelen = 2 * math.pi / ang_plain
    high = wavelen < 8192 / 4.0
    low = wavelen > 8192 / 1.0
    assert high.any() and low.any() and (~high & ~low).any()
    assert np.allclose(ang_scaled[high], ang_plain[high])                          # untouched
    assert np.allclose(ang_scaled[low], ang_plain[low] / 8.0)                      # divided by factor
    mid = ~high & ~low
    assert (ang_scaled[mid] < ang_plain[mid]).all() and (ang_scaled[mid] > ang_plain[mid] / 8.0).all()
    # factor 1 changes nothing
    same = ro.cos_sin_table_f64(rd, 2, base, dict(LLAMA3_SCALING, factor=1.0))
    assert np.allclose(same, plain)
    # and the product's table follows the same bands
    got = make_cos_sin_cache(rd, 2, base, LLAMA3_SCALING, dtype=torch.float32).double().numpy()
    assert np.abs(got - scaled).max() < 1e-6


def test_fma_variants_sit_between_one_and_three_roundings():
    """The two-rounding variants: within u*|rounded product| + u*|result| of the float64
    formula (u = 2^-8 for bf16: half an ulp of 8 significant bits), i.e. tighter than the three-rounding bound and
    looser than a single rounding; at position 0 (cos = 1, sin = 0) they are the
    identity like the others."""
    import torch
    from lmserve_amd import rotary
    g = torch.Generator().manual_seed(5)
    T, H, D = 64, 4, 64
    q = torch.randn(T, H * D, generator=g).to(torch.bfloat16)
    k = torch.randn(T, H * D, generator=g).to(torch.bfloat16)
    pos = torch.randint(0, 512, (T,), generator=g)
    cs = rotary.make_cos_sin_cache(D, 512, 10000.0, dtype=torch.bfloat16)
    exact_q, _ = ro.rotary_pos_emb_f64(q.double().numpy(), k.double().numpy(), pos.numpy(), cs.double().numpy(), D)
    u = 2.0 ** -8
    xh = q.double().numpy().reshape(T, H, D)
    c = cs[pos].double().numpy()
    cos, sin = c[:, None, :D], c[:, None, D:]
    half = D // 2
    a, b = xh[:, :, :half], xh[:, :, half:]
    prods = {"first": np.concatenate([np.abs(a * cos[:, :, :half]), np.abs(b * cos[:, :, half:])], axis=2),
             "second": np.concatenate([np.abs(b * sin[:, :, :half]), np.abs(a * sin[:, :, half:])], axis=2)}
    for which in ("first", "second"):
        got, _ = ro.rotary_pos_emb_fma(q, k, pos, cs, D, rounded=which)
        err = np.abs(got.double().numpy() - exact_q)
        bound = u * prods[which].reshape(T, -1) + u * np.abs(exact_q) * 1.001 + 1e-30
        assert (err <= bound).all(), which
        zero = torch.zeros(T, dtype=torch.long)
        same_q, same_k = ro.rotary_pos_emb_fma(q, k, zero, cs, D, rounded=which)
        assert torch.equal(same_q, q) and torch.equal(same_k, k)
    with pytest.raises(ValueError):
        ro.rotary_pos_emb_fma(q, k, pos, cs, D, rounded="both")

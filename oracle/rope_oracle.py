"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

CPU restatements of the reference's rotary position embedding
(runtime/worker/llm_worker/ops/triton/rotary_embedding.py:5-66 with the wrapper
ops/rotary_embedding_ops.py:8-35) and of its cos/sin table
(models/layers/rotary_embedding.py:27-70). Floating point, so three views:

  rotary_pos_emb_f64      the kernel's formula in float64 (no rounding): the
                          yardstick the tolerance is measured from
  rotary_pos_emb_fp32     torch reference: upcast to fp32, one rounding to the
                          storage dtype (what the HIP kernel implements)
  rotary_pos_emb_per_op   every product and sum rounded to the storage dtype,
                          the way a bf16-typed Triton expression evaluates
                          (three roundings per lane)
  rotary_pos_emb_fma      the same expression with one product contracted into
                          a fused multiply-add: two roundings per lane, either
                          product being the one that is rounded on its own

Pinned in tests/test_rope_oracle.py against complex multiplication
(x + iy)(cos + i sin), the identity at position 0, norm preservation and
additivity of angles. Which of the roundings the reference's Triton build
performs on NVIDIA hardware cannot be established here (no reference-held
vectors, kernel not runnable): bit-level parity with it is UNPINNED; the tests
hold the HIP kernel to half an ulp of the float64 formula, which bounds its
distance to either rounding order by one ulp of the larger product.
"""
from __future__ import annotations

import math

import numpy as np
import torch


def rotary_pos_emb_f64(query, key, positions, cos_sin_cache, head_dim):
    """query [T, Hq*D], key [T, Hkv*D], cos_sin_cache [P, 2*rd] as float arrays
    (any dtype convertible to float64). Returns float64 (q_out, k_out); lanes at
    or beyond rotary_dim are passed through."""
    q = np.asarray(query, dtype=np.float64)
    k = np.asarray(key, dtype=np.float64)
    cs = np.asarray(cos_sin_cache, dtype=np.float64)
    pos = np.asarray(positions, dtype=np.int64)
    rd = cs.shape[1] // 2
    half = rd // 2
    cos, sin = cs[pos, :rd], cs[pos, rd:]            # [T, rd] each

    def rotate(x):
        T = x.shape[0]
        xh = x.reshape(T, -1, head_dim).copy()
        a, b = xh[:, :, :half].copy(), xh[:, :, half:rd].copy()
        xh[:, :, :half] = a * cos[:, None, :half] - b * sin[:, None, :half]
        xh[:, :, half:rd] = b * cos[:, None, half:] + a * sin[:, None, half:]
        return xh.reshape(x.shape)

    return rotate(q), rotate(k)


def _rotate_torch(x, cos, sin, head_dim, rd, compute_dtype, out_dtype):
    T = x.shape[0]
    half = rd // 2
    xh = x.reshape(T, -1, head_dim).to(compute_dtype)
    c = cos.to(compute_dtype)[:, None, :]
    s = sin.to(compute_dtype)[:, None, :]
    a, b = xh[:, :, :half], xh[:, :, half:rd]
    out = xh.clone()
    out[:, :, :half] = a * c[:, :, :half] - b * s[:, :, :half]
    out[:, :, half:rd] = b * c[:, :, half:] + a * s[:, :, half:]
    return out.to(out_dtype).reshape(x.shape)


def rotary_pos_emb_fp32(query, key, positions, cos_sin_cache, head_dim):
    """torch tensors in their storage dtype -> rotated tensors of the same dtype,
    fp32 arithmetic, one rounding."""
    rd = cos_sin_cache.shape[1] // 2
    cs = cos_sin_cache[positions.long()]
    cos, sin = cs[:, :rd], cs[:, rd:]
    return (_rotate_torch(query, cos, sin, head_dim, rd, torch.float32, query.dtype),
            _rotate_torch(key, cos, sin, head_dim, rd, torch.float32, key.dtype))


def rotary_pos_emb_per_op(query, key, positions, cos_sin_cache, head_dim):
    """Same formula with every intermediate rounded to the storage dtype."""
    rd = cos_sin_cache.shape[1] // 2
    cs = cos_sin_cache[positions.long()]
    cos, sin = cs[:, :rd], cs[:, rd:]
    return (_rotate_torch(query, cos, sin, head_dim, rd, query.dtype, query.dtype),
            _rotate_torch(key, cos, sin, head_dim, rd, key.dtype, key.dtype))


def rotary_pos_emb_fma(query, key, positions, cos_sin_cache, head_dim, rounded="second"):
    """`a*b - c*d` evaluated as a fused multiply-add over ONE product rounded to the
    storage dtype: `rounded="second"` is fma(a, b, -rn(c*d)), `"first"` is
    fma(-c, d, rn(a*b)); the sum is rounded once. The exact products of two
    16-bit-or-narrower operands fit float64, so float64 stands in for the
    unrounded fma. Storage dtypes bf16 / fp16."""
    if rounded not in ("first", "second"):
        raise ValueError("rounded must be 'first' or 'second'")
    rd = cos_sin_cache.shape[1] // 2
    half = rd // 2
    cs = cos_sin_cache[positions.long()]
    cos, sin = cs[:, None, :rd].double(), cs[:, None, rd:].double()

    def rotate(x):
        dt = x.dtype
        T = x.shape[0]
        xh = x.reshape(T, -1, head_dim)
        a, b = xh[:, :, :half].double(), xh[:, :, half:rd].double()

        def rn(t):
            return t.to(dt).double()

        def fused(p1, p2):          # p1 - p2 (or p1 + p2 below) with one of them pre-rounded
            return (rn(p1) - p2) if rounded == "first" else (p1 - rn(p2))

        out = xh.clone()
        out[:, :, :half] = fused(a * cos[:, :, :half], b * sin[:, :, :half]).to(dt)
        # y*cos + x*sin = y*cos - (-(x*sin))
        out[:, :, half:rd] = fused(b * cos[:, :, half:], -(a * sin[:, :, half:])).to(dt)
        return out.reshape(x.shape)

    return rotate(query), rotate(key)


def cos_sin_table_f64(rotary_dim, max_position, base=10000.0, rope_scaling=None):
    """Closed form of the table in float64: angle[p, i] = p * inv_freq[i mod rd/2]."""
    i = np.arange(0, rotary_dim, 2, dtype=np.float64)
    inv_freq = 1.0 / (base ** (i / rotary_dim))
    if rope_scaling is not None:
        factor = rope_scaling["factor"]
        lo, hi = rope_scaling["low_freq_factor"], rope_scaling["high_freq_factor"]
        old = rope_scaling["original_max_position_embeddings"]
        wavelen = 2 * math.pi / inv_freq
        out = inv_freq.copy()
        for j, w in enumerate(wavelen):
            if w > old / lo:
                out[j] = inv_freq[j] / factor
            elif w >= old / hi:          # medium band: smooth interpolation
                smooth = (old / w - lo) / (hi - lo)
                out[j] = (1 - smooth) * inv_freq[j] / factor + smooth * inv_freq[j]
        inv_freq = out
    angle = np.arange(max_position, dtype=np.float64)[:, None] * inv_freq[None, :]
    emb = np.concatenate([angle, angle], axis=1)
    return np.concatenate([np.cos(emb), np.sin(emb)], axis=1)

"""Seeded synthetic inputs for the KV-cache data-movement configurations.

Host-only (NumPy): block tables, slot mappings, page-table index arrays, block
pair lists and swap id lists in the shapes the reference's scheduler produces
(runtime/src/llm_engine/scheduler.rs:453-541,
 runtime/src/llm_engine/block_manager.rs:62-140: the free list starts as
 0..nb and turns into an arbitrary order under churn, so tables are drawn from
 a seeded permutation of the pool). Used by the tests and by bench.py; not part of the lmserve_amd package.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Tuple

import numpy as np

from lmserve_amd.index_prep import InferInput, KVIndexInputs, make_kv_index_inputs


@dataclass(frozen=True)
class KVShape:
    name: str
    num_layers: int
    num_kv_heads: int
    head_dim: int
    block_size: int = 16
    elem_bytes: int = 2  # bf16

    @property
    def row_elems(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def row_bytes(self) -> int:
        return self.row_elems * self.elem_bytes

    @property
    def block_elems(self) -> int:
        """K and V of one block of one layer."""
        return 2 * self.block_size * self.row_elems

    @property
    def block_bytes(self) -> int:
        return self.block_elems * self.elem_bytes

    def shard(self, tp: int) -> "KVShape":
        """The head slice one rank holds under tensor parallelism of degree `tp`
        (runtime/worker/llm_worker/models/llama.py:105-106: num_kv_heads // tp_size;
        block tables and mappings are the same on every rank)."""
        if tp < 1 or self.num_kv_heads % tp:
            raise ValueError(f"{self.num_kv_heads} KV heads do not split over {tp} ranks")
        return KVShape(f"{self.name}/tp{tp}", self.num_layers, self.num_kv_heads // tp,
                       self.head_dim, self.block_size, self.elem_bytes)


LLAMA_3_2_1B = KVShape("llama-3.2-1b", 16, 8, 64)
LLAMA_3_8B = KVShape("llama-3-8b", 32, 8, 128)
QWEN_2_5_7B = KVShape("qwen2.5-7b", 28, 4, 128)
LLAMA_3_1_70B = KVShape("llama-3.1-70b", 80, 8, 128)


@dataclass
class WriteWorkload:
    shape: KVShape
    num_blocks: int
    inputs: List[InferInput]
    index: KVIndexInputs          # request-sorted index arrays + slot_mapping

    @property
    def num_tokens(self) -> int:
        return int(self.index.slot_mapping.shape[0])

    def algorithmic_bytes(self, layers: int) -> int:
        """read K,V + write K,V for `layers` layers, plus 8 bytes of slot index per token."""
        return 2 * self.num_tokens * 2 * self.shape.row_bytes * layers + 8 * self.num_tokens


def _tables(rng: np.random.Generator, num_blocks: int, blocks_needed: List[int]) -> List[np.ndarray]:
    """Disjoint block tables drawn without replacement from a permutation of the pool."""
    total = int(sum(blocks_needed))
    if total > num_blocks:
        raise ValueError(f"{total} blocks needed, pool holds {num_blocks}")
    perm = rng.permutation(num_blocks)
    out, at = [], 0
    for n in blocks_needed:
        out.append(perm[at:at + n].astype(np.int64))
        at += n
    return out


def _write_workload(shape: KVShape, num_blocks: int, filled: List[int], new_tokens: List[int],
                    rng: np.random.Generator) -> WriteWorkload:
    bs = shape.block_size
    ctx = [f + n for f, n in zip(filled, new_tokens)]
    tables = _tables(rng, num_blocks, [(c + bs - 1) // bs for c in ctx])
    inputs = [
        InferInput(seq_id=i, input_ids=[0] * n, input_len=n, filled_token_len=f, context_len=c,
                   block_ids=t.tolist())
        for i, (f, n, c, t) in enumerate(zip(filled, new_tokens, ctx, tables))
    ]
    return WriteWorkload(shape, num_blocks, inputs, make_kv_index_inputs(inputs, bs))


def random_free_slots(shape: KVShape = LLAMA_3_2_1B, num_blocks: int = 1024, num_tokens: int = 256,
                      seed: int = 0) -> np.ndarray:
    """Config 1: `num_tokens` distinct free slots of the pool, seeded (int64)."""
    rng = np.random.default_rng(seed)
    return rng.permutation(num_blocks * shape.block_size)[:num_tokens].astype(np.int64)


def decode_step(shape: KVShape = LLAMA_3_8B, num_blocks: int = 65536, batch: int = 256,
                max_context: int = 4096, seed: int = 0) -> WriteWorkload:
    """Config 2: `batch` sequences x 1 new token; sequence b already holds
    c_b in [1, max_context) tokens and its slot is the next one of its table."""
    rng = np.random.default_rng(seed)
    filled = rng.integers(1, max_context, size=batch).tolist()
    return _write_workload(shape, num_blocks, filled, [1] * batch, rng)


def chunked_prefill(shape: KVShape = QWEN_2_5_7B, num_blocks: int = 16384, num_seqs: int = 4,
                    chunk_tokens: int = 2048, min_context: int = 1024, max_context: int = 32768,
                    seed: int = 0) -> WriteWorkload:
    """Config 3: one `chunk_tokens` chunk split evenly over `num_seqs` sequences
    whose existing context lengths are uniform in [min_context, max_context]."""
    rng = np.random.default_rng(seed)
    filled = rng.integers(min_context, max_context + 1, size=num_seqs).tolist()
    per = chunk_tokens // num_seqs
    return _write_workload(shape, num_blocks, filled, [per] * num_seqs, rng)


def copy_on_write_pairs(num_blocks: int = 65536, num_pairs: int = 4096,
                        seed: int = 0) -> Tuple[np.ndarray, Dict[int, List[int]]]:
    """Config 4: `num_pairs` (src, dst) pairs, dsts distinct and disjoint from the srcs.
    Returns the flattened int64 `[src0, dst0, ...]` list and the reference's dict form."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(num_blocks)
    src = perm[:num_pairs]
    dst = perm[num_pairs:2 * num_pairs]
    flat = np.empty(2 * num_pairs, dtype=np.int64)
    flat[0::2] = src
    flat[1::2] = dst
    return flat, {int(s): [int(d)] for s, d in zip(src, dst)}


def swap_round_trip(num_gpu_blocks: int = 16384, n: int = 8192,
                    seed: int = 0) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Config 5: (gpu ids swapped out, host ids 0..n-1, fresh gpu ids swapped back in)."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(num_gpu_blocks)
    return (perm[:n].astype(np.int64), np.arange(n, dtype=np.int64),
            perm[n:2 * n].astype(np.int64))

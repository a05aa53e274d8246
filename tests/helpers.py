"""Shared input builders for the tests (CPU side)."""
from __future__ import annotations

import numpy as np
import torch

# bf16 bit patterns 0xFFC0..0xFFFF are NaNs with the sign bit set: values a
# float->bf16 conversion of N(0,1) samples never produces, so a pool pre-filled
# with them shows every written element and every stray write.
SENTINEL_BASE = 0xFFC0


def bf16_bits(shape, seed: int) -> np.ndarray:
    """K/V ~ N(0,1) in fp32, rounded to bf16 by torch, returned as uint16 bit patterns."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g, dtype=torch.float32).to(torch.bfloat16)
    return x.view(torch.int16).numpy().view(np.uint16).copy()


def sentinel_pool(shape, seed: int = 0) -> np.ndarray:
    """uint16 pool whose every element is a position-dependent sentinel."""
    n = int(np.prod(shape, dtype=np.int64))
    idx = np.arange(n, dtype=np.uint64)
    mixed = (idx * np.uint64(0x9E3779B97F4A7C15) + np.uint64(seed)) >> np.uint64(58)  # 6 bits
    return (np.uint16(SENTINEL_BASE) + mixed.astype(np.uint16)).reshape(shape)


def random_pool(shape, seed: int) -> np.ndarray:
    """uint16 pool of arbitrary bit patterns (for copy/swap, where all bits matter)."""
    rng = np.random.default_rng(seed)
    return rng.integers(0, 1 << 16, size=shape, dtype=np.uint16)


def to_bf16(a: np.ndarray, device=None) -> torch.Tensor:
    """uint16 bit patterns -> torch bf16 tensor (optionally on a device)."""
    t = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return t.to(device) if device is not None else t


def bits_of(t: torch.Tensor) -> np.ndarray:
    """torch tensor of a 16-bit dtype -> uint16 bit patterns on the host."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


class FifoBlockIds:
    """Block ids in the order the reference's allocator produces them under churn
    (runtime/src/llm_engine/block_manager.rs:62-140): ids are taken from the front
    of a queue that starts as 0..n-1 and go to its back when their last user
    lets go, so live block tables end up scattered over the pool. Test input
    generator only."""

    def __init__(self, n: int):
        from collections import deque
        self.queue = deque(range(n))
        self.users = [0] * n

    def take(self, count: int = 1):
        if count > len(self.queue):
            raise RuntimeError("no free block ids left")
        ids = [self.queue.popleft() for _ in range(count)]
        for i in ids:
            self.users[i] = 1
        return ids

    def share(self, block_id: int) -> int:
        """One more user of a block (prefix sharing); a free id is claimed."""
        if self.users[block_id] == 0:
            self.queue.remove(block_id)
        self.users[block_id] += 1
        return block_id

    def give_back(self, ids) -> None:
        for i in ids:
            assert self.users[i] > 0, f"block {i} given back twice"
            self.users[i] -= 1
            if self.users[i] == 0:
                self.queue.append(i)

"""One rank's head slice of the tensor-parallel shapes, against the oracle.

Under tensor parallelism every rank runs the same operators with the same
block tables on num_kv_heads / tp heads
(runtime/worker/llm_worker/models/llama.py:105-106), so a row and a block
shrink by tp: Llama-3.1-70B at tp=8 is one KV head, 256-byte rows and 8 KiB
blocks over 80 layers. These are the shapes a single GPU of such a job sees."""
import numpy as np
import pytest
import torch

import lmserve_amd as kvc
import workloads as wl
from oracle import kvc_oracle as orc

pytestmark = pytest.mark.gpu

SHARDS = [(wl.LLAMA_3_1_70B, 8), (wl.LLAMA_3_1_70B, 4), (wl.LLAMA_3_8B, 8), (wl.QWEN_2_5_7B, 4),
          (wl.LLAMA_3_2_1B, 8)]


def _dev(a, gpu):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(gpu)


def _host(t):
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("full,tp", SHARDS, ids=[f"{s.name}-tp{t}" for s, t in SHARDS])
def test_shard_write_copy_swap(gpu, full, tp):
    s = full.shard(tp)
    assert s.row_bytes * tp == full.row_bytes and s.block_bytes * tp == full.block_bytes
    rng = np.random.default_rng(tp * 131 + full.num_layers)
    L, nb, bs, H, D = s.num_layers, 192, s.block_size, s.num_kv_heads, s.head_dim
    pool = rng.integers(0, 1 << 16, size=(L, nb, 2, bs, H, D), dtype=np.uint16)

    # a decode step and a prefill chunk with the tables every rank receives
    for w in (wl.decode_step(s, nb, batch=48, max_context=60, seed=tp),
              wl.chunked_prefill(s, nb, num_seqs=3, chunk_tokens=96, min_context=5, max_context=300,
                                 seed=tp + 1)):
        T, idx = w.num_tokens, w.index
        key = rng.integers(0, 1 << 16, size=(L, T, H, D), dtype=np.uint16)
        value = rng.integers(0, 1 << 16, size=(L, T, H, D), dtype=np.uint16)
        want = pool.copy()
        for l in range(L):
            orc.c_append_paged_kv_cache(key[l], value[l], idx.batch_indices, idx.positions, want[l],
                                        idx.kv_block_indices, idx.kv_block_indptrs)
        dev = kvc.to_device(idx, bs, gpu)
        dk, dv = _dev(key, gpu), _dev(value, gpu)
        a, b, c = (_dev(pool, gpu) for _ in range(3))
        kvc.reshape_and_cache_layers(dk, dv, a, dev.slot_mapping)
        kvc.append_paged_kv_cache_layers(dk, dv, dev.batch_indices, dev.positions, b,
                                         dev.kv_block_indices, dev.kv_block_indptrs,
                                         dev.kv_last_block_lens)
        for l in range(L):
            kvc.append_paged_kv_cache(dk[l], dv[l], dev.batch_indices, dev.positions, c[l],
                                      dev.kv_block_indices, dev.kv_block_indptrs,
                                      dev.kv_last_block_lens)
        torch.cuda.synchronize()
        for name, got in (("slot one launch", a), ("paged one launch", b), ("paged per layer", c)):
            assert np.array_equal(_host(got), want), f"{s.name}: {name}"
        pool = want

    flat, pairs = wl.copy_on_write_pairs(nb, 40, seed=tp)
    orc.c_copy_blocks(pool, flat)
    kvc.copy_blocks(a, pairs, validate=True)
    torch.cuda.synchronize()
    assert np.array_equal(_host(a), pool), f"{s.name}: copy_blocks"

    old, host_ids, new = wl.swap_round_trip(nb, 24, seed=tp)
    for mode in ("direct", "staged"):
        worker = kvc.KVWorker(a, 24, swap_mode=mode)
        try:
            worker.host_kv_caches[...] = 0
            host = np.zeros_like(worker.host_kv_caches)
            gpu_np = pool.reshape(L, nb, -1)
            orc.c_save_blocks_to_host(gpu_np, host, old, host_ids)
            orc.c_load_blocks_from_host(gpu_np, host, host_ids, new)
            worker.copy_kv_sync([kvc.BlockMapping.from_pairs(zip(old.tolist(), host_ids.tolist()))],
                                kvc.Device.GPU, kvc.Device.Host)
            worker.copy_kv_sync([kvc.BlockMapping.from_pairs(zip(host_ids.tolist(), new.tolist()))],
                                kvc.Device.Host, kvc.Device.GPU)
            assert np.array_equal(worker.host_kv_caches, host), f"{s.name}: swap-out {mode}"
            assert np.array_equal(_host(a).reshape(L, nb, -1), gpu_np), f"{s.name}: swap-in {mode}"
        finally:
            worker.close()

"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py
from the element-by-element restatement): the fast oracles must reproduce them
on the CPU, and the HIP library must reproduce them on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import kvc_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLDEN, name), allow_pickle=False))


# --------------------------------------------------------------------------- CPU

@pytest.mark.parametrize("impl", ["np", "c"])
def test_oracles_reproduce_the_write_fixture(impl):
    g = load("write.npz")
    paged = orc.append_paged_kv_cache_np if impl == "np" else orc.c_append_paged_kv_cache
    slotted = orc.reshape_and_cache_np if impl == "np" else orc.c_reshape_and_cache
    fill = orc.fill_key_cache_np if impl == "np" else orc.c_fill_key_cache
    a, b = g["pool_before"].copy(), g["pool_before"].copy()
    for l in range(a.shape[0]):
        paged(g["key"][l], g["value"][l], g["batch_indices"], g["positions"], a[l],
              g["kv_indices"], g["kv_indptr"])
        slotted(g["key"][l], g["value"][l], b[l], g["slot_mapping"])
    assert np.array_equal(a, g["pool_after"]) and np.array_equal(b, g["pool_after"])
    kc, vc = g["kc_before"].copy(), g["vc_before"].copy()
    fill(g["key"][0], g["value"][0], kc, vc, g["slot_mapping"])
    assert np.array_equal(kc, g["kc_after"]) and np.array_equal(vc, g["vc_after"])
    page_size = g["pool_before"].shape[3]
    sl = (orc.get_seq_lens_np if impl == "np" else orc.c_get_seq_lens)(
        g["kv_indptr"], g["kv_last_page_len"], page_size)
    bi, pos = (orc.get_batch_indices_positions_np if impl == "np"
               else orc.c_get_batch_indices_positions)(g["cu_seqlens_q"], sl, len(g["positions"]))
    assert np.array_equal(bi, g["batch_indices"]) and np.array_equal(pos, g["positions"])


@pytest.mark.parametrize("impl", ["np", "c"])
def test_oracles_reproduce_the_copy_and_swap_fixtures(impl):
    g = load("copy_blocks.npz")
    pool = g["pool_before"].copy()
    (orc.copy_blocks_np if impl == "np" else orc.c_copy_blocks)(pool, g["block_maps"])
    assert np.array_equal(pool, g["pool_after"])
    g = load("swap.npz")
    host, gpu = g["host_before"].copy(), g["gpu_before"].copy()
    (orc.save_blocks_to_host_np if impl == "np" else orc.c_save_blocks_to_host)(
        gpu, host, g["out_src"], g["out_dst"])
    assert np.array_equal(host, g["host_after"]) and np.array_equal(gpu, g["gpu_before"])
    (orc.load_blocks_from_host_np if impl == "np" else orc.c_load_blocks_from_host)(
        gpu, host, g["in_src"], g["in_dst"])
    assert np.array_equal(gpu, g["gpu_after"])


# --------------------------------------------------------------------------- GPU

def _bf16(a, dev):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(dev)


def _bits(t):
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.gpu
def test_hip_write_reproduces_the_fixture(gpu):
    import lmserve_amd as kvc
    g = load("write.npz")
    L = g["pool_before"].shape[0]
    page_size = g["pool_before"].shape[3]
    key, value = _bf16(g["key"], gpu), _bf16(g["value"], gpu)

    def i32(name):
        return torch.from_numpy(g[name]).to(gpu)

    cu, indptr, last = i32("cu_seqlens_q"), i32("kv_indptr"), i32("kv_last_page_len")
    bi, pos = kvc.get_batch_indices_positions(cu, kvc.get_seq_lens(indptr, last, page_size),
                                              len(g["positions"]))
    assert np.array_equal(bi.cpu().numpy(), g["batch_indices"])
    assert np.array_equal(pos.cpu().numpy(), g["positions"])
    slots = torch.from_numpy(g["slot_mapping"]).to(gpu)

    per_layer, fused, slotted, slotted_fused = (_bf16(g["pool_before"], gpu) for _ in range(4))
    for l in range(L):
        kvc.append_paged_kv_cache(key[l], value[l], bi, pos, per_layer[l], i32("kv_indices"), indptr, last)
        kvc.reshape_and_cache(key[l], value[l], slotted[l], slots)
    kvc.append_paged_kv_cache_layers(key, value, bi, pos, fused, i32("kv_indices"), indptr, last)
    kvc.reshape_and_cache_layers(key, value, slotted_fused, slots)
    kc, vc = _bf16(g["kc_before"], gpu), _bf16(g["vc_before"], gpu)
    kvc.fill_key_cache(key[0], value[0], kc, vc, slots)
    torch.cuda.synchronize()
    for got in (per_layer, fused, slotted, slotted_fused):
        assert np.array_equal(_bits(got), g["pool_after"])
    assert np.array_equal(_bits(kc), g["kc_after"]) and np.array_equal(_bits(vc), g["vc_after"])


@pytest.mark.gpu
def test_hip_copy_blocks_reproduces_the_fixture(gpu):
    import lmserve_amd as kvc
    g = load("copy_blocks.npz")
    pool = _bf16(g["pool_before"], gpu)
    kvc.copy_blocks(pool, {7: [0, 3], 2: [9], 5: [5], 4: [1]})
    torch.cuda.synchronize()
    assert kvc.flatten_block_maps({7: [0, 3], 2: [9], 5: [5], 4: [1]}) == g["block_maps"].tolist()
    assert np.array_equal(_bits(pool), g["pool_after"])


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["staged", "direct"])
def test_hip_swap_reproduces_the_fixture(gpu, mode):
    import lmserve_amd as kvc
    g = load("swap.npz")
    pool = _bf16(g["gpu_before"], gpu)
    w = kvc.KVWorker(pool, g["host_before"].shape[0], swap_mode=mode)
    try:
        w.host_kv_caches[...] = g["host_before"]
        w.copy_kv_sync([kvc.BlockMapping.from_pairs(zip(g["out_src"].tolist(), g["out_dst"].tolist()))],
                       kvc.Device.GPU, kvc.Device.Host)
        assert np.array_equal(w.host_kv_caches, g["host_after"])
        w.copy_kv_sync([kvc.BlockMapping.from_pairs(zip(g["in_src"].tolist(), g["in_dst"].tolist()))],
                       kvc.Device.Host, kvc.Device.GPU)
        assert np.array_equal(_bits(pool), g["gpu_after"])
    finally:
        w.close()

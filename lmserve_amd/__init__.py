"""MI355X-native paged KV-cache data movement behind LMServe's operator surface.

    cache_ops   copy_blocks, fill_key_cache, reshape_and_cache(_layers), gather/scatter_blocks,
                swap_out / swap_in (functional form of the GPU <-> host swap)
    paged       append_paged_kv_cache(_layers), get_seq_lens, get_batch_indices_positions
    kv_worker   KVWorker (GPU <-> pinned host swap), Device, BlockMapping
    index_prep  host-side block-table / slot-mapping construction
    rotary      rotary position embedding, alone or fused with the K/V write
    disk_tier   DiskTier (host <-> block file, native positional I/O)
    kv_pool     pool sizing, layer-sync handle and model-side hooks, hand-over to a second process
    kv_service  the KV worker as a process of its own (pool mapped from an IPC handle)
    step_graph  KVWriteStep: fixed-capacity index buffers and plans, so that a step's index build
                and per-layer writes can be recorded once into a hipGraph and replayed for later steps

Every operator runs a hand-written HIP kernel from libkvcache.so through the
C ABI of include/kvcache.h; the disk tier is host-side file I/O in the same
library. Nothing here has a CPU fallback.
"""
from . import _lib
from .cache_ops import (check_block_maps, copy_blocks, fill_key_cache, flatten_block_maps,
                        gather_blocks, reshape_and_cache, reshape_and_cache_layers, scatter_blocks,
                        swap_in, swap_out)
from .disk_tier import DiskTier
from .index_prep import (InferInput, KVIndexInputs, make_kv_index_inputs, to_device,
                         to_device_one_launch)
from .kv_pool import (CachePlan, KVWorkerHandle, KVWorkerParams, LayerSyncHooks,
                      allocate_kv_caches, make_kv_worker_params, open_kv_worker_params, plan_cache)
from .kv_service import serve_kv_worker
from .kv_worker import (BlockMapping, BlockMappingEntry, Device, KVWorker, PinnedHostPool,
                        flatten_block_mappings)
from .rotary import (PagedRotaryWritePlan, RotaryEmbedding, make_cos_sin_cache, rotary_pos_emb,
                     rotary_pos_emb_and_append_paged, rotary_pos_emb_and_cache)
from .paged import (BlockRuns, PagedKVWritePlan, append_paged_kv_cache, append_paged_kv_cache_layers,
                    build_write_index, get_batch_indices_positions, get_seq_lens, max_block_runs,
                    slot_block_runs, write_block_runs_layers)
from .step_graph import KVWriteStep

__all__ = [
    "copy_blocks", "fill_key_cache", "reshape_and_cache", "reshape_and_cache_layers",
    "flatten_block_maps", "check_block_maps", "gather_blocks", "scatter_blocks",
    "swap_out", "swap_in",
    "append_paged_kv_cache", "append_paged_kv_cache_layers", "PagedKVWritePlan", "get_seq_lens",
    "get_batch_indices_positions",
    "KVWorker", "Device", "BlockMapping", "BlockMappingEntry", "PinnedHostPool",
    "flatten_block_mappings", "DiskTier",
    "RotaryEmbedding", "make_cos_sin_cache", "rotary_pos_emb", "rotary_pos_emb_and_cache",
    "rotary_pos_emb_and_append_paged", "PagedRotaryWritePlan",
    "CachePlan", "KVWorkerHandle", "KVWorkerParams", "LayerSyncHooks", "allocate_kv_caches",
    "make_kv_worker_params", "open_kv_worker_params", "serve_kv_worker",
    "plan_cache",
    "InferInput", "KVIndexInputs", "make_kv_index_inputs", "to_device", "to_device_one_launch",
    "build_write_index", "BlockRuns", "max_block_runs", "slot_block_runs", "write_block_runs_layers",
    "KVWriteStep",
]

/*
 * kvc_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded CPU restatement of the reference's paged KV-cache
 * data-movement operations, used only as the checker for the HIP library
 * (tests/, the smoke check, and the CPU-baseline leg of bench.py). Nothing in
 * lmserve_amd/ may call into this file.
 *
 * Every function moves opaque elements of `elem_bytes` bytes, so bf16/fp16/fp32
 * pools are all covered bit-exactly. Citations are paths under the reference
 * tree's runtime/worker/llm_worker/ unless a longer path is given.
 *
 * Pinning status (the reference ships no tests or golden vectors for these
 * operations, so each function is pinned by mathematics in
 * tests/test_oracle_pinning.py):
 *   oracle_fill_key_cache             pinned: identity / permutation special
 *                                     cases against memcpy and np.take, changed-
 *                                     row census, element-wise brute force
 *   oracle_copy_blocks                pinned: np.take equivalence on disjoint
 *                                     pairs, self-pair no-op, idempotence,
 *                                     brute force
 *   oracle_save/load_blocks_to/from_host
 *                                     pinned: contiguous-id case against
 *                                     np.swapaxes, round-trip identity, brute force
 *   oracle_append_paged_kv_cache,
 *   oracle_get_seq_lens,
 *   oracle_get_batch_indices_positions
 *                                     pinned against the reference's OWN index
 *                                     construction (positions == position_ids,
 *                                     seq_lens == context_len; model_worker.py:346,
 *                                     :399-433) and against the slot rule of
 *                                     scheduler.rs/block_manager.rs; parity with
 *                                     the third-party flashinfer binary itself
 *                                     (not in the tree, not installable here)
 *                                     is UNPINNED.
 */
#include <stdint.h>
#include <string.h>

/* ops/triton/cache_kernels.py:39-58 (fill_key_cache_kernel) with the wrapper's
 * argument derivation, ops/cache_ops.py:39-59: program i copies the H*D
 * elements of key[i] to key_cache + slot*H*D (flat, dense), same for value. */
void oracle_fill_key_cache(const void* key, const void* value, void* key_cache,
                           void* value_cache, const int64_t* slot_mapping,
                           int64_t num_tokens, int64_t num_kv_heads, int64_t head_size,
                           int64_t elem_bytes) {
  const int64_t row = num_kv_heads * head_size * elem_bytes;
  for (int64_t i = 0; i < num_tokens; ++i) {
    const int64_t slot = slot_mapping[i];
    memcpy((char*)key_cache + slot * row, (const char*)key + i * row, (size_t)row);
    memcpy((char*)value_cache + slot * row, (const char*)value + i * row, (size_t)row);
  }
}

/* The same write addressed into one layer of the interleaved pool
 * [nb, 2, bs, H, D] (model_worker.py:221-228): slot = blk*bs + e
 * (runtime/src/llm_engine/block_manager.rs:241-273 gives the block table,
 * scheduler.rs:489-511 the positions). */
void oracle_reshape_and_cache(const void* key, const void* value, void* kv_cache,
                              const int64_t* slot_mapping, int64_t num_tokens,
                              int64_t block_size, int64_t num_kv_heads, int64_t head_size,
                              int64_t elem_bytes) {
  const int64_t row = num_kv_heads * head_size * elem_bytes;
  for (int64_t i = 0; i < num_tokens; ++i) {
    const int64_t blk = slot_mapping[i] / block_size;
    const int64_t e = slot_mapping[i] % block_size;
    char* page = (char*)kv_cache + blk * 2 * block_size * row;
    memcpy(page + e * row, (const char*)key + i * row, (size_t)row);
    memcpy(page + (block_size + e) * row, (const char*)value + i * row, (size_t)row);
  }
}

/* flashinfer.append_paged_kv_cache as called at models/layers/attention.py:76-85,
 * NHD single-tensor cache [num_pages, 2, page_size, H, D]:
 *   page = kv_indices[kv_indptr[b] + p / page_size], e = p % page_size. */
void oracle_append_paged_kv_cache(const void* append_key, const void* append_value,
                                  const int32_t* batch_indices, const int32_t* positions,
                                  void* paged_kv_cache, const int32_t* kv_indices,
                                  const int32_t* kv_indptr, int64_t nnz, int64_t num_kv_heads,
                                  int64_t head_dim, int64_t page_size, int64_t elem_bytes) {
  const int64_t row = num_kv_heads * head_dim * elem_bytes;
  for (int64_t i = 0; i < nnz; ++i) {
    const int64_t b = batch_indices[i];
    const int64_t p = positions[i];
    const int64_t page = kv_indices[(int64_t)kv_indptr[b] + p / page_size];
    const int64_t e = p % page_size;
    char* base = (char*)paged_kv_cache + page * 2 * page_size * row;
    memcpy(base + e * row, (const char*)append_key + i * row, (size_t)row);
    memcpy(base + (page_size + e) * row, (const char*)append_value + i * row, (size_t)row);
  }
}

/* flashinfer.get_seq_lens as called at model_worker.py:427-431. */
void oracle_get_seq_lens(const int32_t* kv_indptr, const int32_t* kv_last_page_len,
                         int64_t batch_size, int32_t page_size, int32_t* seq_lens) {
  for (int64_t b = 0; b < batch_size; ++b) {
    int32_t full = kv_indptr[b + 1] - kv_indptr[b] - 1;
    if (full < 0) full = 0;
    seq_lens[b] = full * page_size + kv_last_page_len[b];
  }
}

/* flashinfer.get_batch_indices_positions as called at model_worker.py:425-433. */
void oracle_get_batch_indices_positions(const int32_t* append_indptr, const int32_t* seq_lens,
                                        int64_t batch_size, int32_t* batch_indices,
                                        int32_t* positions) {
  for (int64_t b = 0; b < batch_size; ++b) {
    const int32_t n_new = append_indptr[b + 1] - append_indptr[b];
    for (int32_t j = 0; j < n_new; ++j) {
      batch_indices[append_indptr[b] + j] = (int32_t)b;
      positions[append_indptr[b] + j] = seq_lens[b] - n_new + j;
    }
  }
}

/* ops/triton/cache_kernels.py:5-36 (copy_blocks_kernel) with the wrapper's
 * argument derivation, ops/cache_ops.py:8-36: program (layer, pair j) copies
 * numel_per_block elements from block maps[2j] to block maps[2j+1] of that
 * layer. The reference orders neither layers nor pairs; this restatement runs
 * them pair-major, which gives the reference's result whenever that result is
 * defined (distinct dsts, no dst that is also a src). */
void oracle_copy_blocks(void* kv_caches, const int64_t* block_maps, int64_t num_pairs,
                        int64_t num_layers, int64_t numel_per_layer, int64_t numel_per_block,
                        int64_t elem_bytes) {
  for (int64_t j = 0; j < num_pairs; ++j) {
    const int64_t src = block_maps[2 * j];
    const int64_t dst = block_maps[2 * j + 1];
    for (int64_t l = 0; l < num_layers; ++l) {
      char* layer = (char*)kv_caches + l * numel_per_layer * elem_bytes;
      memmove(layer + dst * numel_per_block * elem_bytes,
              layer + src * numel_per_block * elem_bytes,
              (size_t)(numel_per_block * elem_bytes));
    }
  }
}

/* kv_worker.py:213-227 (_save_layer_kv_blocks_to_host) inside the layer loop of
 * kv_worker.py:272-295: host[dst, l, :] = gpu[l, src, :]. gpu is
 * [L, num_gpu_blocks, block_bytes], host is [num_host_blocks, L, block_bytes]
 * (kv_worker.py:104-108, :123-127). */
void oracle_save_blocks_to_host(const void* gpu, void* host, const int64_t* src_ids,
                                const int64_t* dst_ids, int64_t n, int64_t num_layers,
                                int64_t num_gpu_blocks, int64_t block_bytes,
                                int64_t layer_begin, int64_t layer_end) {
  for (int64_t l = layer_begin; l < layer_end; ++l)
    for (int64_t i = 0; i < n; ++i)
      memcpy((char*)host + (dst_ids[i] * num_layers + l) * block_bytes,
             (const char*)gpu + (l * num_gpu_blocks + src_ids[i]) * block_bytes,
             (size_t)block_bytes);
}

/* kv_worker.py:197-211 (_load_layer_kv_blocks_from_host) inside the layer loop
 * of kv_worker.py:249-270: gpu[l, dst, :] = host[src, l, :]. */
void oracle_load_blocks_from_host(void* gpu, const void* host, const int64_t* src_ids,
                                  const int64_t* dst_ids, int64_t n, int64_t num_layers,
                                  int64_t num_gpu_blocks, int64_t block_bytes,
                                  int64_t layer_begin, int64_t layer_end) {
  for (int64_t l = layer_begin; l < layer_end; ++l)
    for (int64_t i = 0; i < n; ++i)
      memcpy((char*)gpu + (l * num_gpu_blocks + dst_ids[i]) * block_bytes,
             (const char*)host + (src_ids[i] * num_layers + l) * block_bytes,
             (size_t)block_bytes);
}

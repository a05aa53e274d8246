/*
 * kvcache.h -- C ABI of libkvcache, the MI355X (gfx950) paged KV-cache
 * data-movement library: slot-mapped and page-table K/V write (alone or fused
 * with the rotary embedding), block copy, block gather/scatter between the HBM
 * pool and a pinned host pool, the index preparation of a step, and the
 * host <-> disk tier of the block cache.
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes only; `stream` arguments are hipStream_t passed
 *     as void* (NULL = the null stream);
 *   - returns KVC_OK (0) or a negative kvc_status; never throws; the text of the
 *     last failure on the calling thread is kvc_last_error_string();
 *   - asynchronous on the given stream(s) unless the name ends in _sync;
 *   - never allocates or frees device memory; the caller owns every buffer
 *     (host-side helpers own small pinned bounce buffers, events and, in the
 *     disk tier, per-thread staging; kvc_thread_release returns the swap's);
 *   - every offset is computed in 64 bits (one layer of a 65536-block Llama-3-8B
 *     pool already holds 2^31 elements);
 *   - block ids / slots outside [0, capacity) are skipped by the kernels
 *     (the reference leaves them undefined), host-resident id lists are
 *     rejected with KVC_ERR_OUT_OF_RANGE before anything is launched.
 *
 * STABLE SURFACE. Everything declared in this file keeps its name, arguments and
 * meaning until KVC_ABI_VERSION changes; kvc_abi_version() lets a binding check
 * at load time. Launch-shape knobs, launch introspection, the host-side row
 * mover and the run-descriptor write are declared in kvcache_experimental.h and
 * may change without a version bump.
 *
 * Pool layout (runtime/worker/llm_worker/model_worker.py:221-228):
 *   kv_caches[L, num_blocks, 2, block_size, H, D], contiguous; kv_caches[l] is
 *   the per-layer "NHD" paged cache handed to attention.
 * Host pool layout (runtime/worker/llm_worker/kv_worker.py:123-127):
 *   host[num_host_blocks, L, 2*block_size*H*D], C order, pinned.
 */
#ifndef KVCACHE_H_
#define KVCACHE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVC_ABI_VERSION 6

typedef enum kvc_status {
  KVC_OK = 0,
  KVC_ERR_INVALID_ARG = -1,   /* null pointer, negative size, bad stride ...   */
  KVC_ERR_UNSUPPORTED = -2,   /* elem_bytes / index width not supported        */
  KVC_ERR_OUT_OF_RANGE = -3,  /* a host-resident block id is outside its pool  */
  KVC_ERR_STAGING = -4,       /* staging buffer too small for the request      */
  KVC_ERR_HIP = -5,           /* a HIP runtime call failed (see error string)  */
  KVC_ERR_IO = -6,            /* a file operation of the disk tier failed      */
  KVC_ERR_TIMEOUT = -7,       /* a host-side wait gave up at its deadline      */
  KVC_ERR_CANCELLED = -8      /* a host-side wait was cancelled by the caller  */
} kvc_status;

/* how kvc_swap_out / kvc_swap_in move the bytes over PCIe */
typedef enum kvc_swap_mode {
  KVC_SWAP_STAGED = 0, /* gather/scatter kernel <-> device staging ring, large
                          hipMemcpyAsync extents on the copy stream, overlapped */
  KVC_SWAP_DIRECT = 1, /* one kernel that loads/stores the pinned host pool
                          through its device mapping (no staging traffic)       */
  KVC_SWAP_AUTO = 2    /* per call: staged when the host ids of the call form
                          runs that make the PCIe copies 1 MiB or more in the
                          mean (knob auto_min_extent_bytes), direct otherwise,
                          and direct when `staging` holds no ring               */
} kvc_swap_mode;

int kvc_abi_version(void);
const char* kvc_last_error_string(void);

/* ---------------------------------------------------------------------------
 * K/V write, slot-mapped.
 * Replaces fill_key_cache / fill_key_cache_kernel
 *   (runtime/worker/llm_worker/ops/cache_ops.py:39-59,
 *    runtime/worker/llm_worker/ops/triton/cache_kernels.py:39-58).
 * For token i: s = slot_mapping[i]; the row of row_elems elements at
 *   key + i*key_token_stride is copied to
 *   key_cache + (s / block_size)*cache_block_stride + (s % block_size)*cache_slot_stride,
 * likewise value -> value_cache. All strides are in ELEMENTS of elem_bytes.
 * The reference's packed caches [num_slots, H, D] are
 *   cache_block_stride = block_size*H*D, cache_slot_stride = H*D;
 * one layer of the interleaved pool [nb, 2, bs, H, D] is
 *   value_cache = key_cache + bs*H*D, cache_block_stride = 2*bs*H*D.
 * slot_mapping lives on the device, slot_bytes is 4 (int32) or 8 (int64).
 * A slot < 0 or >= num_cache_blocks*block_size is skipped.
 * ------------------------------------------------------------------------- */
int kvc_reshape_and_cache(const void* key, const void* value,
                          void* key_cache, void* value_cache,
                          const void* slot_mapping, int slot_bytes,
                          int64_t num_tokens, int64_t row_elems,
                          int64_t key_token_stride, int64_t value_token_stride,
                          int64_t block_size, int64_t cache_block_stride,
                          int64_t cache_slot_stride, int64_t num_cache_blocks,
                          int elem_bytes, void* stream);

/* Same write for num_layers layers in ONE launch: layer l reads
 * key + l*key_layer_stride (value likewise) and writes the caches at
 * + l*cache_layer_stride; every layer uses the same slot_mapping, as the
 * reference's block tables are shared by all layers
 * (runtime/worker/llm_worker/model_worker.py:399-423 builds them once per step).
 * No counterpart launch exists in the reference, which writes one layer per
 * attention call (runtime/worker/llm_worker/models/layers/attention.py:76-85). */
int kvc_reshape_and_cache_layers(const void* key, const void* value,
                                 void* key_cache, void* value_cache,
                                 const void* slot_mapping, int slot_bytes,
                                 int64_t num_tokens, int64_t row_elems,
                                 int64_t key_token_stride, int64_t value_token_stride,
                                 int64_t block_size, int64_t cache_block_stride,
                                 int64_t cache_slot_stride, int64_t num_cache_blocks,
                                 int64_t num_layers, int64_t key_layer_stride,
                                 int64_t value_layer_stride, int64_t cache_layer_stride,
                                 int elem_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * K/V write, page-table addressed (the reference's live write).
 * Replaces the flashinfer.append_paged_kv_cache call at
 *   runtime/worker/llm_worker/models/layers/attention.py:76-85
 * (flashinfer-python 0.3.1.post1, "NHD" single-tensor cache
 *  [num_pages, 2, page_size, H, D], runtime/worker/llm_worker/model_worker.py:65-66).
 * For token i: b = batch_indices[i], p = positions[i],
 *   page = kv_indices[kv_indptr[b] + p / page_size], e = p % page_size,
 *   paged_kv_cache[page, 0, e] = append_key[i], paged_kv_cache[page, 1, e] = append_value[i].
 * Index arrays are int32 on the device. kv_last_page_len is accepted for
 * signature parity and not read (flashinfer does not read it either).
 * page_stride is the distance between pages in elements (2*page_size*H*D when
 * contiguous). b outside [0, batch_size), a page-table index outside the
 * request's own table [kv_indptr[b], kv_indptr[b+1]) or outside
 * [0, num_kv_indices), or a page outside [0, num_pages) skips the token.
 * The _layers form adds the layer loop exactly as kvc_reshape_and_cache_layers.
 * ------------------------------------------------------------------------- */
int kvc_append_paged_kv_cache(const void* append_key, const void* append_value,
                              const int32_t* batch_indices, const int32_t* positions,
                              void* paged_kv_cache,
                              const int32_t* kv_indices, const int32_t* kv_indptr,
                              const int32_t* kv_last_page_len,
                              int64_t nnz, int64_t batch_size, int64_t num_kv_indices,
                              int64_t num_kv_heads, int64_t head_dim, int64_t page_size,
                              int64_t key_token_stride, int64_t value_token_stride,
                              int64_t page_stride, int64_t num_pages,
                              int elem_bytes, void* stream);

int kvc_append_paged_kv_cache_layers(const void* append_key, const void* append_value,
                                     const int32_t* batch_indices, const int32_t* positions,
                                     void* paged_kv_cache,
                                     const int32_t* kv_indices, const int32_t* kv_indptr,
                                     const int32_t* kv_last_page_len,
                                     int64_t nnz, int64_t batch_size, int64_t num_kv_indices,
                                     int64_t num_kv_heads, int64_t head_dim, int64_t page_size,
                                     int64_t key_token_stride, int64_t value_token_stride,
                                     int64_t page_stride, int64_t num_pages,
                                     int64_t num_layers, int64_t key_layer_stride,
                                     int64_t value_layer_stride, int64_t cache_layer_stride,
                                     int elem_bytes, void* stream);

/* The page-table write with its per-step arguments held by the library, so a
 * layer-by-layer forward pass hands over three pointers per layer instead of
 * twenty arguments. The reference builds the same five index tensors once per
 * step (runtime/worker/llm_worker/model_worker.py:399-446) and passes them to
 * every layer's append call (runtime/worker/llm_worker/models/llama.py:236-242,
 * runtime/worker/llm_worker/models/layers/attention.py:76-85).
 * kvc_write_plan_create copies the ARGUMENTS (pointers and sizes), not the
 * arrays: the index arrays must stay valid on the device for as long as the
 * plan is used. kvc_write_plan_append is kvc_append_paged_kv_cache with the
 * plan's arguments and the layer's key, value (token strides in elements) and
 * cache; same checks, same errors. Host-side object: create/destroy touch
 * no device memory. */
typedef struct kvc_write_plan kvc_write_plan;

int kvc_write_plan_create(const int32_t* batch_indices, const int32_t* positions,
                          const int32_t* kv_indices, const int32_t* kv_indptr,
                          const int32_t* kv_last_page_len,
                          int64_t nnz, int64_t batch_size, int64_t num_kv_indices,
                          int64_t num_kv_heads, int64_t head_dim, int64_t page_size,
                          int elem_bytes, kvc_write_plan** out);
int kvc_write_plan_append(const kvc_write_plan* plan, const void* append_key,
                          const void* append_value, int64_t key_token_stride,
                          int64_t value_token_stride, void* paged_kv_cache,
                          int64_t page_stride, int64_t num_pages, void* stream);
int kvc_write_plan_destroy(kvc_write_plan* plan);

/* Optional: walk the page table ONCE per step instead of once per layer. One
 * small launch on `stream` writes every token's slot (page * page_size + entry,
 * or -1 for a token the page-table write would skip) into `slots`, nnz int64
 * entries of device memory that the caller owns and keeps valid while the plan
 * is used. From then on kvc_write_plan_append addresses the cache through these
 * slots, exactly as kvc_reshape_and_cache would: the per-layer launch loses its
 * chain of three dependent index loads. The results are identical. Appends must
 * be ordered after this call (same stream, or an event). */
int kvc_write_plan_resolve_slots(kvc_write_plan* plan, int64_t* slots, void* stream);

/* The same with slots the caller already has on the device (the slot_mapping
 * output of kvc_build_write_index): no launch, the plan only remembers the
 * pointer. A plan made once over fixed-capacity index buffers and given their
 * slot_mapping this way can be recorded into a hipGraph together with the index
 * build: every replay then writes the step whose scalars the buffers hold.
 * NULL returns the plan to page-table addressing. */
int kvc_write_plan_set_slots(kvc_write_plan* plan, const int64_t* slots);

/* ---------------------------------------------------------------------------
 * Index preparation for the paged write.
 * Replace the flashinfer.get_seq_lens / flashinfer.get_batch_indices_positions
 * calls at runtime/worker/llm_worker/model_worker.py:425-433.
 *   seq_lens[b] = max(kv_indptr[b+1]-kv_indptr[b]-1, 0)*page_size + kv_last_page_len[b]
 *   for j in [append_indptr[b], append_indptr[b+1]):
 *     batch_indices[j] = b
 *     positions[j]     = seq_lens[b] - (append_indptr[b+1]-append_indptr[b]) + (j - append_indptr[b])
 * Entries of the outputs at j >= append_indptr[batch_size] (up to nnz) are left
 * untouched. All arrays int32 on the device.
 * ------------------------------------------------------------------------- */
int kvc_get_seq_lens(const int32_t* kv_indptr, const int32_t* kv_last_page_len,
                     int64_t batch_size, int64_t page_size, int32_t* seq_lens,
                     void* stream);

int kvc_get_batch_indices_positions(const int32_t* append_indptr, const int32_t* seq_lens,
                                    int64_t batch_size, int64_t nnz,
                                    int32_t* batch_indices, int32_t* positions,
                                    void* stream);

/* The whole index preparation of a step in ONE launch, from the per-request
 * scalars the scheduler sends (proto/worker.proto:40-47: input_len, context_len,
 * block_ids). Replaces the host-side cumulative sums and list building of
 * ModelWorker._make_inputs (runtime/worker/llm_worker/model_worker.py:346,
 * :362-365, :399-423), the two flashinfer index calls (:425-433) and the slot
 * rule of the scheduler (runtime/src/llm_engine/scheduler.rs:489-511):
 *   cu_seqlens_q[b+1]  = sum_{i<=b} input_lens[i]           (cu_seqlens_q[0] = 0)
 *   kv_indptr[b+1]     = sum_{i<=b} num_blocks[i]           (kv_indptr[0] = 0)
 *   kv_last_page_len[b]= (context_lens[b]-1) % page_size + 1
 *   for the j-th new token of request b, at out = cu_seqlens_q[b] + j:
 *     batch_indices[out] = b, positions[out] = context_lens[b] - input_lens[b] + j,
 *     slot_mapping[out]  = kv_indices[kv_indptr[b] + pos/page_size]*page_size + pos%page_size
 * kv_indices is the concatenation of the requests' block tables. slot_mapping
 * may be NULL; a position outside its request's table yields slot -1.
 * Outputs: cu_seqlens_q, kv_indptr [batch_size+1], kv_last_page_len [batch_size],
 * batch_indices, positions (int32) and slot_mapping (int64) [nnz].
 *
 * Every size argument is a CAPACITY, so one recorded launch (a hipGraph node)
 * serves every later step that fits: the step's own sizes are read from device
 * memory. Requests with input_lens[b] = 0 (and num_blocks[b] = 0) pad the batch;
 * per-token outputs from the step's token count up to nnz are set to -1, which
 * every write entry point skips; num_kv_indices bounds the block-table array.
 *
 * Optional block runs (runs != NULL): a run is a maximal range of one request's
 * new tokens that falls into one block -- consecutive tokens on the source side,
 * consecutive entries of one block on the cache side, which is how a prefill
 * chunk fills whole blocks (runtime/src/llm_engine/scheduler.rs:466-512).
 *   run_indptr[b+1] = runs of requests 0..b                 (run_indptr[0] = 0)
 *   runs[r] = {first token, block id (-1: outside the table), first entry, token count}
 *   *num_runs = run_indptr[batch_size]
 * runs is int32 [max_runs][4], 16-byte aligned; max_runs must be at least
 * min(nnz, nnz / page_size + 2 * batch_size) (checked). Descriptors from
 * *num_runs up to max_runs are set empty. */
int kvc_build_write_index(const int32_t* input_lens, const int32_t* context_lens,
                          const int32_t* num_blocks, const int32_t* kv_indices,
                          int64_t batch_size, int64_t num_kv_indices, int64_t page_size,
                          int64_t nnz, int32_t* cu_seqlens_q, int32_t* kv_indptr,
                          int32_t* kv_last_page_len, int32_t* batch_indices,
                          int32_t* positions, int64_t* slot_mapping,
                          int32_t* run_indptr, int32_t* runs, int32_t* num_runs,
                          int64_t max_runs, void* stream);

/* ---------------------------------------------------------------------------
 * Block copy inside the pool (prefix-sharing copy-on-write).
 * Replaces copy_blocks / copy_blocks_kernel
 *   (runtime/worker/llm_worker/ops/cache_ops.py:8-36,
 *    runtime/worker/llm_worker/ops/triton/cache_kernels.py:5-36).
 * block_maps is the device array [src0, dst0, src1, dst1, ...] of int64 that the
 * reference wrapper builds; for every layer l and pair j
 *   kv_caches[l, dst_j, :] = kv_caches[l, src_j, :]   (block_bytes bytes each).
 * layer_stride_bytes = num_blocks*block_bytes for the contiguous pool.
 * Defined when the dsts are distinct and no dst is also a src (the reference
 * gives no ordering between pairs); src == dst is a no-op.
 * ------------------------------------------------------------------------- */
int kvc_copy_blocks(void* kv_caches, const int64_t* block_maps, int64_t num_pairs,
                    int64_t num_layers, int64_t layer_stride_bytes,
                    int64_t block_bytes, int64_t num_blocks, void* stream);

/* ---------------------------------------------------------------------------
 * Swap between the HBM pool and the pinned host pool.
 * Replace the per-(layer, block) memcpy loops
 *   _save_layer_kv_blocks_to_host  (runtime/worker/llm_worker/kv_worker.py:213-227)
 *   _load_layer_kv_blocks_from_host (runtime/worker/llm_worker/kv_worker.py:197-211)
 * and their layer loops (kv_worker.py:249-295).
 *   swap_out: host[dst_ids[i], l, :] = pool[l, src_ids[i], :]
 *   swap_in : pool[l, dst_ids[i], :] = host[src_ids[i], l, :]
 * for i in [0, n) and l in [layer_begin, layer_end) -- the layer range keeps the
 * reference's layer-pipelined protocol expressible (one call per finished layer
 * or one call for all).
 * src_ids / dst_ids are HOST arrays of int64 (they arrive as BlockMapping
 * entries over gRPC, proto/worker.proto:78-85) and are range-checked here.
 * host_pool must be pinned memory that the device can address (kvc_host_alloc_pinned).
 * staging is a device buffer of staging_bytes >= kvc_swap_staging_bytes(...):
 * its head holds the device copy of the id lists, the rest is the two-slot
 * ring used by KVC_SWAP_STAGED (chunk_blocks blocks per slot; 0 = about 64 MiB
 * per slot, more when the call would otherwise take over 128 chunks).
 * KVC_SWAP_AUTO wants the staged size and falls back to the direct kernel when
 * the buffer holds the id lists only. The staged PCIe copies follow the runs of
 * consecutive host ids; these two entry points order the pairs of the call by
 * host id first (on a copy), so its host blocks form the longest runs they can.
 * Kernels run on kernel_stream, PCIe
 * copies on copy_stream. Pass the same stream for both unless measured
 * otherwise: the gather or scatter of a chunk takes a hundredth of its PCIe
 * time, so two streams gain 1 % at best, and late in a busy process (graphs
 * captured, many streams) the event-ordered pipeline fell to a quarter of the
 * link rate where one stream kept all of it (a staged call of one chunk uses
 * kernel_stream for both in any case). On return all
 * work is enqueued and kernel_stream has been made to wait for copy_stream's
 * part, so synchronising kernel_stream alone completes the swap.
 * ------------------------------------------------------------------------- */
int64_t kvc_swap_staging_bytes(int64_t n, int64_t num_layers_in_range,
                               int64_t block_bytes, int mode, int64_t chunk_blocks);

int kvc_swap_out(const void* pool, void* host_pool,
                 const int64_t* src_ids, const int64_t* dst_ids, int64_t n,
                 int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                 int64_t num_gpu_blocks, int64_t num_host_blocks,
                 int64_t layer_begin, int64_t layer_end,
                 void* staging, int64_t staging_bytes, int mode,
                 void* kernel_stream, void* copy_stream);

int kvc_swap_in(void* pool, const void* host_pool,
                const int64_t* src_ids, const int64_t* dst_ids, int64_t n,
                int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                int64_t num_gpu_blocks, int64_t num_host_blocks,
                int64_t layer_begin, int64_t layer_end,
                void* staging, int64_t staging_bytes, int mode,
                void* kernel_stream, void* copy_stream);

/* Which way a KVC_SWAP_AUTO call goes, without making it: KVC_SWAP_STAGED or
 * KVC_SWAP_DIRECT for n pairs with these HOST host ids (in the order the call
 * would use: ascending for kvc_swap_out / kvc_swap_in, as given for the prepared
 * calls), a layer range of num_layers_in_range layers and a staging buffer of
 * staging_bytes. The direct kernel holds the PCIe rate whatever the ids are, but
 * holds back the kernels of other streams while it runs (a forward pass beside a
 * direct write-through of 1 GiB took 2.3 times as long on MI355X); a caller that
 * runs a model on the same GPU should give AUTO a staging buffer of
 * kvc_swap_staging_bytes(..., KVC_SWAP_STAGED, ...) and host blocks that form
 * runs, or move the rows through a dense pinned buffer (kvcache_experimental.h).
 * kvc_swap_last_mode: the mode the calling thread's most recent swap call ran in
 * (-1 before the first). */
int kvc_swap_resolve_mode(const int64_t* host_ids, int64_t n, int64_t num_layers_in_range,
                          int64_t block_bytes, int64_t staging_bytes);
int kvc_swap_last_mode(void);

/* Orders the (gpu id, host id) pairs of one swap call by ascending host block id,
 * stably and in place (HOST arrays of n entries; no GPU work). The result of a
 * swap does not depend on the order of its pairs (the reference copies them one
 * after the other, runtime/worker/llm_worker/kv_worker.py:197-227, and they
 * touch distinct blocks), but the staged PCIe leg moves one extent per run of
 * consecutive host ids in the order given. kvc_swap_out / kvc_swap_in do this
 * themselves on a copy of their lists (staged and auto mode); call it before
 * kvc_swap_prepare, whose order the prepared calls keep. */
int kvc_order_pairs_by_host_id(int64_t* gpu_ids, int64_t* host_ids, int64_t n);

/* The id lists of a swap checked and uploaded ONCE, for callers that move the
 * same blocks in several calls -- the reference's layer loops issue one call per
 * layer with the same mappings (runtime/worker/llm_worker/kv_worker.py:249-295).
 *   kvc_swap_prepare: range-checks gpu_ids against num_gpu_blocks and host_ids
 *     against num_host_blocks (HOST int64 arrays of n entries) and uploads
 *     [gpu_ids | host_ids] to the head of `staging` on `stream`.
 *   kvc_swap_out_prepared / kvc_swap_in_prepared: kvc_swap_out / kvc_swap_in for a
 *     layer range with the id lists read from the head of `staging` as
 *     kvc_swap_prepare left them (gpu ids are the sources of a swap-out and the
 *     destinations of a swap-in). Neither checks nor uploads anything; in
 *     KVC_SWAP_DIRECT mode the call is one kernel launch and host_ids may be
 *     NULL; KVC_SWAP_STAGED still needs the HOST array host_ids for its PCIe
 *     extents, and KVC_SWAP_AUTO reads it to choose (NULL: direct). The caller
 *     orders these calls after the prepare call (same stream, or an event) and
 *     keeps `staging` untouched in between.
 * kvc_thread_release frees what the swap entry points keep per calling thread
 * (events, pinned id bounce buffers); it waits for that thread's pending id
 * uploads. Optional: a thread that never calls it keeps a few KiB of pinned
 * memory until the process ends. */
int kvc_swap_prepare(const int64_t* gpu_ids, const int64_t* host_ids, int64_t n,
                     int64_t num_gpu_blocks, int64_t num_host_blocks,
                     void* staging, int64_t staging_bytes, void* stream);

int kvc_swap_out_prepared(const void* pool, void* host_pool, const int64_t* host_ids, int64_t n,
                          int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                          int64_t num_gpu_blocks, int64_t num_host_blocks,
                          int64_t layer_begin, int64_t layer_end,
                          void* staging, int64_t staging_bytes, int mode,
                          void* kernel_stream, void* copy_stream);

int kvc_swap_in_prepared(void* pool, const void* host_pool, const int64_t* host_ids, int64_t n,
                         int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                         int64_t num_gpu_blocks, int64_t num_host_blocks,
                         int64_t layer_begin, int64_t layer_end,
                         void* staging, int64_t staging_bytes, int mode,
                         void* kernel_stream, void* copy_stream);

int kvc_thread_release(void);

/* A direct swap that allocates nothing and needs no workspace. It has no
 * counterpart in the reference; it is for callers that cannot allocate: tight
 * serving loops and harnesses that forbid hipMalloc, and code that records its
 * stream into a hipGraph (after one call outside the capture, see below).
 * kvc_swap_out / kvc_swap_in in KVC_SWAP_DIRECT mode with `staging` replaced by
 * a static device array inside the library (KVC_NOALLOC_MAX_BLOCKS id pairs,
 * 128 KiB per device, held until the process ends):
 *   to_host != 0: host[host_ids[i], l, :] = pool[l, gpu_ids[i], :]
 *   to_host == 0: pool[l, gpu_ids[i], :] = host[host_ids[i], l, :]
 * for l in [layer_begin, layer_end). gpu_ids / host_ids are HOST int64 arrays,
 * range-checked before anything is launched; they travel to the device as
 * kernel arguments, so the call consists of kernel launches on `stream` only:
 * no hipMalloc, no hipFree, no pinned bounce buffer, no memcpy, no events.
 * n > KVC_NOALLOC_MAX_BLOCKS: KVC_ERR_UNSUPPORTED, nothing launched. The first
 * call on a device looks up the array's address there (hipGetSymbolAddress, which
 * may load the code object and is not a stream operation): make one call, n = 1
 * is enough, at start-up and outside any stream capture. A call moves its ids in
 * packets of 448 pairs, one small launch each ahead of the copy kernel: up to
 * 19 + 1 launches at the maximum size. A recorded call replays the ids it was
 * recorded with.
 * Every call on one device shares that device's array: calls on one stream are
 * ordered by the stream; calls that overlap on different streams of one device
 * race on the id lists and must be ordered by the caller. */
#define KVC_NOALLOC_MAX_BLOCKS 8192

int kvc_swap_noalloc(int to_host, void* pool, void* host_pool,
                     const int64_t* gpu_ids, const int64_t* host_ids, int64_t n,
                     int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                     int64_t num_gpu_blocks, int64_t num_host_blocks,
                     int64_t layer_begin, int64_t layer_end, void* stream);

/* ---------------------------------------------------------------------------
 * Rotary position embedding, alone or fused with the K/V write.
 * (Widening beyond the copy path: the rotation runs immediately before the
 * write on the same K tensor, runtime/worker/llm_worker/models/llama.py:156-167.)
 * Replaces rotary_pos_emb / apply_rotary_pos_emb_kernel
 *   (runtime/worker/llm_worker/ops/rotary_embedding_ops.py:8-35,
 *    runtime/worker/llm_worker/ops/triton/rotary_embedding.py:5-66):
 * for token t with p = positions[t], every head, and lane i in [0, rotary_dim/2):
 *   x = in[i], y = in[rotary_dim/2 + i]
 *   out[i]                = x*cos[p, i]                - y*sin[p, i]
 *   out[rotary_dim/2 + i] = y*cos[p, rotary_dim/2 + i] + x*sin[p, rotary_dim/2 + i]
 * with cos_sin_cache[max_position, 2*rotary_dim] = cos | sin in the tensors'
 * dtype (runtime/worker/llm_worker/models/layers/rotary_embedding.py:62-70).
 * Arithmetic is fp32 with one rounding to the storage dtype. Lanes in
 * [rotary_dim, head_dim) are copied through (the reference leaves them
 * unwritten). query_out may alias query, key_out may alias key. A position
 * outside [0, max_position) leaves the token untouched. Strides in elements.
 *
 * _and_cache / _and_append_paged additionally store the ROTATED key row and
 * the value row into the token's cache slot, addressed exactly as
 * kvc_reshape_and_cache / kvc_append_paged_kv_cache address it (one layer);
 * key_out may then be NULL. In the page-table form `positions` serves both
 * the rotation and the page lookup, as the reference passes the same values
 * for both (runtime/worker/llm_worker/model_worker.py:346, :425-433).
 * ------------------------------------------------------------------------- */
typedef enum kvc_dtype { KVC_DTYPE_BF16 = 0, KVC_DTYPE_F16 = 1, KVC_DTYPE_F32 = 2 } kvc_dtype;

int kvc_rotary_pos_emb(const void* query, const void* key, const void* positions, int pos_bytes,
                       const void* cos_sin_cache, int64_t max_position, int64_t num_tokens,
                       int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                       int64_t rotary_dim, int64_t q_token_stride, int64_t k_token_stride,
                       void* query_out, void* key_out, int64_t qo_token_stride,
                       int64_t ko_token_stride, int dtype, void* stream);

int kvc_rotary_pos_emb_and_cache(const void* query, const void* key, const void* value,
                                 const void* positions, int pos_bytes, const void* cos_sin_cache,
                                 int64_t max_position, int64_t num_tokens, int64_t num_heads,
                                 int64_t num_kv_heads, int64_t head_dim, int64_t rotary_dim,
                                 int64_t q_token_stride, int64_t k_token_stride,
                                 int64_t v_token_stride, void* query_out, void* key_out,
                                 int64_t qo_token_stride, int64_t ko_token_stride,
                                 void* key_cache, void* value_cache, const void* slot_mapping,
                                 int slot_bytes, int64_t block_size, int64_t cache_block_stride,
                                 int64_t cache_slot_stride, int64_t num_cache_blocks, int dtype,
                                 void* stream);

int kvc_rotary_pos_emb_and_append_paged(const void* query, const void* key, const void* value,
                                        const int32_t* batch_indices, const int32_t* positions,
                                        const void* cos_sin_cache, int64_t max_position,
                                        int64_t nnz, int64_t num_heads, int64_t num_kv_heads,
                                        int64_t head_dim, int64_t rotary_dim,
                                        int64_t q_token_stride, int64_t k_token_stride,
                                        int64_t v_token_stride, void* query_out, void* key_out,
                                        int64_t qo_token_stride, int64_t ko_token_stride,
                                        void* paged_kv_cache, const int32_t* kv_indices,
                                        const int32_t* kv_indptr, int64_t batch_size,
                                        int64_t num_kv_indices, int64_t page_size,
                                        int64_t page_stride, int64_t num_pages, int dtype,
                                        void* stream);

/* kvc_rotary_pos_emb_and_append_paged with its per-step arguments held by the
 * library (see kvc_write_plan): per layer the caller hands over the layer's
 * query/key/value with their token strides in elements (slices of a fused QKV
 * projection are read in place), the output buffers (dense rows: query_out
 * stride = num_heads*head_dim, key_out stride = num_kv_heads*head_dim; key_out
 * may be NULL) and the layer's cache. The reference calls the rotation
 * and the append once per layer with the same positions and index tensors
 * (runtime/worker/llm_worker/models/llama.py:156-167, :236-242). */
typedef struct kvc_rotary_plan kvc_rotary_plan;

int kvc_rotary_plan_create(const int32_t* batch_indices, const int32_t* positions,
                           const void* cos_sin_cache, int64_t max_position, int64_t nnz,
                           int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                           int64_t rotary_dim, const int32_t* kv_indices,
                           const int32_t* kv_indptr, int64_t batch_size,
                           int64_t num_kv_indices, int64_t page_size, int dtype,
                           kvc_rotary_plan** out);
int kvc_rotary_plan_run(const kvc_rotary_plan* plan, const void* query, const void* key,
                        const void* value, int64_t q_token_stride, int64_t k_token_stride,
                        int64_t v_token_stride, void* query_out, void* key_out,
                        void* paged_kv_cache, int64_t page_stride, int64_t num_pages,
                        void* stream);
int kvc_rotary_plan_destroy(kvc_rotary_plan* plan);
/* As kvc_write_plan_resolve_slots: the page table is walked once per step and
 * kvc_rotary_plan_run addresses the cache through `slots` (nnz int64 entries of
 * caller-owned device memory), as kvc_rotary_pos_emb_and_cache would. */
int kvc_rotary_plan_resolve_slots(kvc_rotary_plan* plan, int64_t* slots, void* stream);
/* As kvc_write_plan_set_slots. */
int kvc_rotary_plan_set_slots(kvc_rotary_plan* plan, const int64_t* slots);

/* The on-device half of a swap on its own: gather scattered pool blocks into a
 * dense device buffer laid out like the host pool, [n, layer_end-layer_begin,
 * block_bytes], or scatter such a buffer back:
 *   gather : buffer[i, l-layer_begin, :] = pool[l, block_ids[i], :]
 *   scatter: pool[l, block_ids[i], :]    = buffer[i, l-layer_begin, :]
 * The same row semantics as kv_worker.py:213-227 / :197-211 of the reference
 * with the host pool replaced by device memory and host ids 0..n-1; what a
 * prefill-to-decode hand-off over a device-to-device link would send. block_ids
 * is an int64 array on the DEVICE; ids outside [0, num_blocks) are skipped. */
int kvc_gather_blocks(const void* pool, void* buffer, const int64_t* block_ids, int64_t n,
                      int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                      int64_t num_blocks, int64_t layer_begin, int64_t layer_end, void* stream);

int kvc_scatter_blocks(void* pool, const void* buffer, const int64_t* block_ids, int64_t n,
                       int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                       int64_t num_blocks, int64_t layer_begin, int64_t layer_end, void* stream);

/*
 * Host <-> disk tier: whole blocks between the host pool and a block file.
 * Replaces
 *   memmap_disk_kv_cache              (runtime/worker/llm_worker/kv_worker.py:48-85)
 *   _load_layer_kv_blocks_from_disk   (kv_worker.py:229-237)
 *   _save_layer_kv_blocks_to_disk     (kv_worker.py:239-247)
 *   load/save_kv_blocks_from/to_disk  (kv_worker.py:297-322, one task per layer on 4 threads)
 * The file is a NumPy `.npy` array of shape (num_blocks, num_layers, block_elems)
 * and dtype string `descr` ("<u2" for bf16 lanes carried as uint16, kv_worker.py:17-22).
 * kvc_disk_open reuses a file whose stored shape and dtype match and removes and
 * recreates any other, as the reference does; a new file is sparse (unless
 * KVC_DISK_PREALLOCATE asks for its blocks to be reserved) and starts its data
 * at byte 4096. With KVC_DISK_DIRECT the transfers bypass the page
 * cache (O_DIRECT) whenever the data offset and one block's bytes over all
 * layers are multiples of 4096 and the file system allows it; otherwise they are
 * ordinary buffered reads and writes. The host side of an O_DIRECT transfer is
 * handed to the kernel in place when the pool is 4096-aligned ordinary memory;
 * a pool the kernel cannot pin (EFAULT: memory mapped by the GPU driver, i.e.
 * kvc_host_alloc_pinned) or an unaligned one goes through a 4 MiB aligned
 * staging buffer per thread.
 *   save: disk[dst_disk_ids[i]] = host[src_host_ids[i]]   (all layers of the block)
 *   load: host[dst_host_ids[i]] = disk[src_disk_ids[i]]
 * Pairs whose ids are consecutive on both sides travel as one extent; extents
 * are spread over `threads` threads (<= 0: 8). Synchronous: returns when the
 * data has been handed to the kernel (kvc_disk_sync forces it to the device).
 * Ids are HOST int64 arrays, range-checked before any I/O. Destinations must be
 * distinct. No GPU work; safe to call from any thread, one call per handle at a
 * time for overlapping blocks.
 */
typedef struct kvc_disk kvc_disk;

enum {
  KVC_DISK_DIRECT = 1,      /* bypass the page cache where alignment allows            */
  KVC_DISK_PREALLOCATE = 2 /* a new file reserves all its blocks at once (posix_fallocate) */
};
enum {
  KVC_DISK_INFO_DATA_OFFSET = 0, /* byte offset of block 0 in the file            */
  KVC_DISK_INFO_DIRECT = 1,      /* 1 if an O_DIRECT descriptor is in use         */
  KVC_DISK_INFO_CREATED = 2,     /* 1 if kvc_disk_open made a new file            */
  KVC_DISK_INFO_ROW_BYTES = 3,   /* bytes of one block over all layers            */
  KVC_DISK_INFO_NUM_BLOCKS = 4,
  KVC_DISK_INFO_BOUNCED = 5      /* 1 if the last transfer staged the host side   */
};

int kvc_disk_open(const char* path, const char* descr, int64_t num_blocks, int64_t num_layers,
                  int64_t block_elems, int elem_bytes, int flags, kvc_disk** out);
int kvc_disk_close(kvc_disk* disk);
int kvc_disk_sync(kvc_disk* disk);
int64_t kvc_disk_info(const kvc_disk* disk, int what);
int kvc_disk_save_blocks(kvc_disk* disk, const void* host_pool, int64_t num_host_blocks,
                         const int64_t* src_host_ids, const int64_t* dst_disk_ids, int64_t n,
                         int threads);
int kvc_disk_load_blocks(kvc_disk* disk, void* host_pool, int64_t num_host_blocks,
                         const int64_t* src_disk_ids, const int64_t* dst_host_ids, int64_t n,
                         int threads);

/* Pinned, device-addressable host memory for the host pool; replaces
 * pycuda.driver.pagelocked_empty (runtime/worker/llm_worker/kv_worker.py:123-127).
 * Returns NULL on failure. */
void* kvc_host_alloc_pinned(size_t bytes);
int kvc_host_free_pinned(void* ptr);

#ifdef __cplusplus
}
#endif
#endif /* KVCACHE_H_ */

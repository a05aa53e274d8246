/*
 * kvcache_experimental.h -- entry points of libkvcache that are NOT part of the
 * stable surface (kvcache.h): they exist for measurement sweeps, for tests that
 * must know which kernel instantiation ran, and for the KV worker's own host
 * threads. Names, arguments and meaning may change without a change of
 * KVC_ABI_VERSION. None of them has a counterpart in the reference.
 */
#ifndef KVCACHE_EXPERIMENTAL_H_
#define KVCACHE_EXPERIMENTAL_H_

#include "kvcache.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launch-shape knobs for measurement sweeps; process-wide, not thread-safe
 * against concurrent launches. No counterpart in the reference. Keys:
 *   "copy_unroll", "gather_unroll"   16-byte vectors per lane in the tile kernel (1, 2, 4, 8, 16;
 *                                     0 = by launch size)
 *   "copy_nt"                         non-temporal loads and stores in the tile kernel (0/1)
 *   "copy_order"                      1 = walk all blocks of a layer before the next layer
 *   "copy_max_wgs"                    grid cap of the tile kernel (0 = one workgroup per chunk)
 *   "direct_max_wgs"                  grid cap of the direct swap kernel
 *   "direct_max_wgs_in"               the same for Host->GPU (0 = direct_max_wgs)
 *   "write_vpt"                       vectors per lane in the write kernel (0 = by size, 1, 2, 4, 8)
 *   "write_threads"                   lanes per workgroup in the write kernel (0 = by size, 64, 128, 256)
 *   "write_nt"                        bit 0: non-temporal stores, bit 1: non-temporal loads (applied to rows
 *                                     of 1 KiB or more); default 3
 *   "write_order"                     1 = a token's workgroups are neighbours in the grid
 *   "write_planes"                    the plane kernel (lanes of a workgroup run over consecutive
 *                                     tokens of one (layer, K|V) plane): 0 = never, 1 = by row
 *                                     width and launch size, 2 = whenever the row shape allows
 *   "write_planes_vpt"                planes per lane in that kernel (0 = by size, 1, 2, 4, 8)
 *   "write_planes_threads"            lanes per workgroup in that kernel (0 = by rule, 256, 512, 1024)
 *   "write_planes_min_bytes"          rows under 1 KiB: source bytes per launch from which it runs
 *   "write_planes_max_vpr"            widest row it takes, in 16-byte vectors (at most 256)
 *   "write_pipe"                      1 = a lane waits for each of its loads before issuing the
 *                                     next, 0 = loads back to back, -1 = by rule
 *   "runs_unroll", "runs_order", "runs_nt"   the run-descriptor write below
 *   "auto_min_extent_bytes"           KVC_SWAP_AUTO: mean bytes per PCIe copy from which a call is staged
 *   "rope_threads"                    lanes per workgroup in the rotation kernel (0 = default, 64, 128, 256)
 *   "rope_nt"                         non-temporal loads in that kernel: bit 0 the K and V rows, bit 1 the Q rows
 *   "disk_bounce_mib"                 MiB of aligned staging per thread in the disk tier
 *   "host_rows_nt"                    row copies on host threads: 1 = stores that go past the cache (default)
 * Unknown key: KVC_ERR_INVALID_ARG. kvc_reset_tuning puts every knob back to its
 * default; kvc_tuning_modified counts the knobs that are not at their default. */
int kvc_set_tuning(const char* key, int value);
int kvc_get_tuning(const char* key, int* value);
int kvc_reset_tuning(void);
int kvc_tuning_modified(void);

/* Shape of the most recent kernel launch made by the calling thread (for tests
 * and sweeps that must know which instantiation ran). No counterpart in the
 * reference. Unknown `what`: KVC_ERR_INVALID_ARG. */
enum {
  KVC_KERNEL_NONE = 0,
  KVC_KERNEL_WRITE_ROWS = 1,        /* token per workgroup                          */
  KVC_KERNEL_COPY_TILES = 2,        /* block copy, gather, scatter, direct swap     */
  KVC_KERNEL_WRITE_PLANES = 3,      /* lanes over consecutive tokens of one plane   */
  KVC_KERNEL_WRITE_RUNS = 4         /* workgroup per chunk of a (block run, plane)  */
};
enum {
  KVC_LAUNCH_KERNEL = 0,       /* one of KVC_KERNEL_*                               */
  KVC_LAUNCH_VEC_BYTES = 1,    /* bytes per load/store instruction per lane         */
  KVC_LAUNCH_PER_LANE = 2,     /* vectors (or planes) in flight per lane            */
  KVC_LAUNCH_THREADS = 3,      /* lanes per workgroup                               */
  KVC_LAUNCH_GRID = 4,         /* workgroups                                        */
  KVC_LAUNCH_NON_TEMPORAL = 5, /* bit 0 stores, bit 1 loads (tile kernel: both = 1) */
  KVC_LAUNCH_PIPE = 6,         /* write kernels: 1 = a lane waits for each of its loads */
  KVC_LAUNCH_SWAP_MODE = 7     /* the kvc_swap_mode this thread's last swap call ran in  */
};
int64_t kvc_last_launch_info(int what);

/* ---------------------------------------------------------------------------
 * The K/V write as tile copies over block runs (see kvc_build_write_index for
 * the descriptors). For run r = {first token t0, block b, first entry e, count c}
 * and every layer l:
 *   key_cache  [l][b][e .. e+c) = key  [l][t0 .. t0+c)
 *   value_cache[l][b][e .. e+c) = value[l][t0 .. t0+c)
 * with the geometry arguments of kvc_reshape_and_cache_layers (strides in
 * ELEMENTS). The launch is sized for max_runs runs and reads the number of runs
 * from *num_runs on the device, so a recorded launch serves any step that fits.
 * A run with a block id outside [0, num_cache_blocks), a count < 1, entries
 * beyond the block or tokens beyond num_tokens is skipped. Same result as
 * kvc_reshape_and_cache_layers on the slot mapping the runs describe.
 * kvc_slot_runs derives the descriptors from any slot mapping on the device
 * (one small launch): token t opens a run when slot[t] >= 0 and slot[t] is not
 * slot[t-1] + 1 inside the same block; max_runs >= num_tokens (checked).
 * Tuning keys: "runs_unroll" (vectors per lane: 1, 2, 4; 0 = by launch size),
 * "runs_order" (1 = all runs of a plane are neighbours in the grid, the default;
 * 0 = all planes of a run), "runs_nt".
 * ------------------------------------------------------------------------- */
int kvc_slot_runs(const void* slot_mapping, int slot_bytes, int64_t num_tokens,
                  int64_t block_size, int32_t* runs, int32_t* num_runs, int64_t max_runs,
                  void* stream);

int kvc_write_runs_layers(const void* key, const void* value,
                          void* key_cache, void* value_cache,
                          const int32_t* runs, const int32_t* num_runs, int64_t max_runs,
                          int64_t num_tokens, int64_t row_elems,
                          int64_t key_token_stride, int64_t value_token_stride,
                          int64_t block_size, int64_t cache_block_stride,
                          int64_t cache_slot_stride, int64_t num_cache_blocks,
                          int64_t num_layers, int64_t key_layer_stride,
                          int64_t value_layer_stride, int64_t cache_layer_stride,
                          int elem_bytes, void* stream);

/*
 * Do two streams feed the same hardware queue? The runtime maps every stream of
 * a process onto a few hardware queues (4 unless GPU_MAX_HW_QUEUES says
 * otherwise). Kernels of streams that share one run one after the other, and a
 * wait that one of them queues (a kernel behind a copy-engine transfer, an
 * event of another stream) holds back the other as well: swap-out and swap-in
 * issued together then take turns instead of overlapping (55 against 94 GB/s
 * in sum), and a forward pass beside a write-through takes twice its time.
 * The call finds out by doing it: stream_x is kept busy for 200 us by a kernel
 * that watches the clock, an empty kernel is launched on stream_y, and the host
 * sees which finishes first (up to three rounds; both streams are synchronised
 * before it returns; about 0.3 ms). *shared = 1 when y's kernel never finished
 * before x's, 0 otherwise; the same handle twice gives 1 without a launch.
 * Ask while both streams are idle: work already queued on stream_y delays its
 * empty kernel as a shared queue would (the answer then errs towards 1).
 * Not under stream capture (KVC_ERR_INVALID_ARG). No counterpart in the
 * reference, whose two streams (kv_worker.py:159-160) live in a process of
 * their own; KVWorker uses it to choose its streams.
 */
int kvc_streams_share_hw_queue(void* stream_x, void* stream_y, int* shared);

/*
 * Host side of a one-layer swap to or from scattered host blocks, on host threads.
 * Serves
 *   _save_layer_kv_blocks_to_host     (runtime/worker/llm_worker/kv_worker.py:213-227)
 *   _load_layer_kv_blocks_from_host   (kv_worker.py:197-211)
 * when the layer's rows do not neighbour each other in the host pool
 * [num_host_blocks, L, block] (kv_worker.py:123-127): the PCIe leg of the layer
 * is then one copy between the GPU and a dense pinned buffer
 * (kvc_swap_out_prepared / kvc_swap_in_prepared with that buffer as a one-layer
 * host pool and host ids 0..n-1), and this call moves the rows between the
 * buffer and their places in the pool:
 *   to_pool != 0: pool[host_ids[i]] [pool_offset .. pool_offset + row_bytes) = dense[i]
 *   to_pool == 0: dense[i] = pool[host_ids[i]] [pool_offset .. pool_offset + row_bytes)
 * with pool_block_bytes the bytes of one host block over all layers,
 * pool_offset = layer * block bytes and dense rows row_bytes apart. Ids are
 * range-checked first. Synchronous, `threads` host threads (<= 0: 4; fewer for
 * small calls); no GPU work, callable from any thread. Rows of one call must be
 * distinct when to_pool != 0.
 */
int kvc_host_copy_rows(void* host_pool, int64_t num_host_blocks, int64_t pool_block_bytes,
                       int64_t pool_offset, void* dense, const int64_t* host_ids, int64_t n,
                       int64_t row_bytes, int to_pool, int threads);

/*
 * The same row copies as a queue with a thread of its own, so that the caller's
 * loop over the layers (kv_worker.py:249-295) never waits for the host side:
 * kvc_row_mover_submit checks the ids, copies them and returns a ticket
 * (0, 1, 2, ... in the order of the calls; a negative kvc_status on error);
 * the mover's thread takes the jobs in that order, waits for `after_event` first
 * when one is given (a hipEvent_t of the device that is current at the submit:
 * "the layer has landed in the dense buffer" for a save, "the GPU has read the
 * region" for a load), and moves the rows on `threads` host threads.
 * kvc_row_mover_submit_after_flag is the same with a host word in place of the
 * event: the job starts once *flag is non-zero (another host thread, or another
 * process through shared memory, sets it).
 * kvc_row_mover_done tells without blocking whether a ticket's job has finished
 * (1) or not (0); kvc_row_mover_wait blocks until it has, together with every
 * job submitted before it, and returns the status of the first job that failed
 * since the last wait. The event or flag, the pool and the dense buffer must stay
 * valid until the job is done.
 *
 * No wait is unbounded. A job whose event or flag is not reached within the
 * mover's timeout (kvc_row_mover_set_timeout_ms; 30 000 ms unless set; negative =
 * no limit) fails with KVC_ERR_TIMEOUT: its rows are not copied, and neither are
 * those of the jobs already queued behind it, which complete at once with
 * KVC_ERR_CANCELLED (they wait for work of the same stream). kvc_row_mover_cancel
 * does the same on request to every job submitted so far, the one that is waiting
 * included. Jobs submitted afterwards run as usual. kvc_row_mover_destroy lets the
 * queued jobs finish first, each bounded as above, so it returns within one
 * timeout of the call.
 * One thread submits to a mover at a time; done, wait, cancel and set_timeout may
 * be called from any thread.
 */
typedef struct kvc_row_mover kvc_row_mover;
int kvc_row_mover_create(int threads, kvc_row_mover** out);
int64_t kvc_row_mover_submit(kvc_row_mover* mover, void* after_event, void* host_pool,
                             int64_t num_host_blocks, int64_t pool_block_bytes, int64_t pool_offset,
                             void* dense, const int64_t* host_ids, int64_t n, int64_t row_bytes,
                             int to_pool);
int64_t kvc_row_mover_submit_after_flag(kvc_row_mover* mover, const int32_t* flag, void* host_pool,
                                        int64_t num_host_blocks, int64_t pool_block_bytes,
                                        int64_t pool_offset, void* dense, const int64_t* host_ids,
                                        int64_t n, int64_t row_bytes, int to_pool);
int kvc_row_mover_set_timeout_ms(kvc_row_mover* mover, int64_t timeout_ms);
int kvc_row_mover_cancel(kvc_row_mover* mover);
int kvc_row_mover_done(kvc_row_mover* mover, int64_t ticket);
int kvc_row_mover_wait(kvc_row_mover* mover, int64_t ticket);
int kvc_row_mover_destroy(kvc_row_mover* mover);

#ifdef __cplusplus
}
#endif
#endif /* KVCACHE_EXPERIMENTAL_H_ */

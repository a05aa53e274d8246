// libkvcache: paged KV-cache data movement for MI355X (gfx950, CDNA4).
//
// Four kernels carry the whole path; all are HBM-bound byte movers, so the
// design is about coalescing and bytes in flight, not arithmetic:
//
//   write_rows_kernel   a workgroup owns ONE token and a run of 16-byte vectors
//                       out of that token's rows (K and V of every layer in
//                       the launch). The slot lookup is workgroup-uniform, so
//                       the index chain is resolved once on the scalar unit and
//                       each lane only streams: VPT loads, then VPT stores;
//                       lanes of a wavefront cover consecutive vectors of a row
//                       on both sides. Small launches and launches of many
//                       resident sets.
//   write_planes_kernel the lanes of a workgroup run over consecutive tokens of
//                       one (layer, K|V) plane, 1-8 planes per lane: rows under
//                       1 KiB, and launches that fit one resident set of lanes
//                       that way (the decode step of all layers at once).
//   copy_tiles_kernel   a "tile" is one block of one layer (block_bytes
//                       contiguous on both sides). A workgroup owns a chunk of
//                       256 lanes x UNROLL x 16 bytes, issues all its loads
//                       before its first store, and walks chunks grid-stride.
//                       The same kernel serves copy_blocks (pool -> pool), the
//                       swap gather/scatter (pool <-> staging ring in host
//                       layout) and the direct swap (pool <-> mapped host pool).
//   index kernels       seq_lens and (batch_indices, positions) for the paged
//                       write; a few KiB of int32.
//
// The C ABI is declared in include/kvcache.h.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <numeric>
#include <vector>

#include "common.h"
#include "kvcache.h"
#include "kvcache_experimental.h"

// ---------------------------------------------------------------------------
// error plumbing (shared with the other translation units through common.h)
// ---------------------------------------------------------------------------
namespace kvc {
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace kvc

namespace {
using kvc::fail;

// ---------------------------------------------------------------------------
// tuning knobs (kvc_set_tuning); defaults are the measured best on MI355X
// ---------------------------------------------------------------------------
struct Tuning {
  int copy_unroll = 0;      // 16-byte vectors in flight per lane in copy_tiles, 0 = by size
  int gather_unroll = 0;    // the same for pool -> dense buffer; by size, 1 for large launches (dense
                            // writes measured best with 4 KiB per workgroup: 6.27 vs 5.68 TB/s at 4)
  int copy_nt = 1;          // non-temporal loads/stores in copy_tiles
  int copy_max_wgs = 0;     // 0 = one workgroup per chunk, else grid cap
  int copy_order = 0;       // copy_tiles: 1 = walk all blocks of a layer before the next layer
  int write_vpt = 0;        // vectors per lane in write_rows, 0 = by size
  int write_nt = 3;         // write kernels: bit 0 non-temporal stores, bit 1 non-temporal loads (rows of
                            // 1 KiB or more only: narrower rows measured 4 % slower with them). Loads:
                            // -3 % at the 64 MiB decode step, -2 to -3 % at 224-256 MiB, -10 to -15 %
                            // for one layer per launch when the K/V rows come from HBM, neutral when
                            // they are still in cache (one source set, or a producer kernel in front)
  int write_order = 0;      // write_rows: 1 = a token's workgroups are neighbours in the grid
  int write_threads = 0;    // write_rows: lanes per workgroup (64, 128, 256), 0 = by size
  int write_planes = 1;     // the plane kernel (lanes of a workgroup run over consecutive tokens of
                            // one (layer, K|V) plane): 0 = never, 1 = by row width and launch size,
                            // 2 = whenever the row shape allows
  int write_planes_min_bytes = 256 << 10;  // rows under 1 KiB: source bytes of a launch from which it runs
  int write_planes_max_vpr = 256;        // widest row (in 16-byte vectors) that kernel takes
  int write_planes_threads = 0;          // lanes per workgroup of that kernel (256, 512, 1024), 0 = by rule
  int write_pipe = -1;                   // 1 = a lane waits for each load before issuing its next,
                                         // 0 = loads back to back, -1 = by rule
  int write_planes_vpt = 0; // planes per lane in that kernel (1, 2, 4, 8), 0 = by size
  int direct_max_wgs = 96;  // grid cap of the direct swap kernel: one direction of PCIe saturates
                            // with 48-64 workgroups (more cost a 16 MiB one-layer launch 2-4 %),
                            // both directions at once want 96 or more each (91-92 against 87 GB/s
                            // in sum); the rest of the GPU stays free for the model
  int direct_max_wgs_in = 16;  // the same cap for Host->GPU (0 = direct_max_wgs). Reads over PCIe hold back
                               // the kernels of other streams in proportion to what is in flight: 16
                               // workgroups keep the link rate (57.1 against 57.3 GB/s) and let a forward
                               // pass that waits for each fetched layer through after 22.8 ms instead of
                               // 31.5 (13.8 alone, fetch alone 19.5); 8-12 are through after 22.1-22.3 but
                               // lose the rate on large calls (36-52 GB/s). The price: beside a direct
                               // swap-out the fetch gets less of the link (54 against 91 GB/s in sum).
                               // Stores over PCIe hold others back whatever the cap (4 workgroups: +110 %)
  int runs_unroll = 0;       // write_runs: 16-byte vectors per lane (1, 2, 4), 0 = by size
  int runs_order = 1;        // write_runs: 1 = all runs of a plane are neighbours in the grid, 0 = all planes of a run
  int runs_nt = 1;           // write_runs: non-temporal loads and stores
  int auto_min_extent_bytes = 1 << 20;  // KVC_SWAP_AUTO: mean bytes per PCIe copy from which a call
                                        // goes through the copy engines. A copy costs about 10 us
                                        // beyond its transfer time (65 % of the link rate at 1 MiB,
                                        // 88 % at 4 MiB, 11 % at 64 KiB), but what the choice is for
                                        // is the forward pass beside it: one-layer calls of 1, 2, 4
                                        // and 8 MiB behind a 13 ms forward pass lengthen it by 5, 10,
                                        // 18 and 34 % through the direct kernel and by 1-6 % (8 MiB:
                                        // 20 %) through the engines
};
Tuning g_tune;

// name -> knob, for kvc_set_tuning / kvc_get_tuning / kvc_reset_tuning
struct Knob {
  const char* name;
  int* value;
  int initial;
};
Knob* knobs(int* count) {
  static Knob table[] = {
      {"copy_unroll", &g_tune.copy_unroll, 0},
      {"gather_unroll", &g_tune.gather_unroll, 0},
      {"copy_nt", &g_tune.copy_nt, 1},
      {"copy_max_wgs", &g_tune.copy_max_wgs, 0},
      {"copy_order", &g_tune.copy_order, 0},
      {"write_vpt", &g_tune.write_vpt, 0},
      {"write_nt", &g_tune.write_nt, 3},
      {"write_order", &g_tune.write_order, 0},
      {"write_threads", &g_tune.write_threads, 0},
      {"write_planes", &g_tune.write_planes, 1},
      {"write_planes_vpt", &g_tune.write_planes_vpt, 0},
      {"write_planes_min_bytes", &g_tune.write_planes_min_bytes, 256 << 10},
      {"write_planes_max_vpr", &g_tune.write_planes_max_vpr, 256},
      {"write_planes_threads", &g_tune.write_planes_threads, 0},
      {"write_pipe", &g_tune.write_pipe, -1},
      {"direct_max_wgs", &g_tune.direct_max_wgs, 96},
      {"direct_max_wgs_in", &g_tune.direct_max_wgs_in, 16},
      {"auto_min_extent_bytes", &g_tune.auto_min_extent_bytes, 1 << 20},
      {"runs_unroll", &g_tune.runs_unroll, 0},
      {"runs_order", &g_tune.runs_order, 1},
      {"runs_nt", &g_tune.runs_nt, 1},
      {"rope_threads", &kvc::g_rope_tune.threads, 0},
      {"rope_nt", &kvc::g_rope_tune.nt, 0},
      {"disk_bounce_mib", &kvc::g_disk_bounce_mib, 4},
      {"host_rows_nt", &kvc::g_host_rows_nt, 1},
  };
  *count = (int)(sizeof(table) / sizeof(table[0]));
  return table;
}
// grid cap of the direct swap kernel for one direction
inline int direct_wgs(bool to_host) {
  return (!to_host && g_tune.direct_max_wgs_in > 0) ? g_tune.direct_max_wgs_in : g_tune.direct_max_wgs;
}

Knob* find_knob(const char* key) {
  int n = 0;
  Knob* t = knobs(&n);
  for (int i = 0; i < n; ++i)
    if (!strcmp(key, t[i].name)) return &t[i];
  return nullptr;
}

// What the most recent kernel launch of this thread looked like (kvc_last_launch_info).
struct LastLaunch {
  int64_t kernel = KVC_KERNEL_NONE, vec = 0, per_lane = 0, threads = 0, grid = 0, nt = 0, pipe = 0;
};
thread_local LastLaunch g_last;
thread_local int g_last_swap_mode = -1;  // the mode this thread's most recent swap call ran in

constexpr int kThreads = 256;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int BYTES> struct VecOf;
template <> struct VecOf<16> { using type = u32x4; };
template <> struct VecOf<8> { using type = u32x2; };
template <> struct VecOf<4> { using type = uint32_t; };
template <> struct VecOf<2> { using type = uint16_t; };
template <> struct VecOf<1> { using type = uint8_t; };

template <bool NT, typename V>
__device__ __forceinline__ V ld(const V* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, typename V>
__device__ __forceinline__ void st(V* p, V v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// ---------------------------------------------------------------------------
// write_rows_kernel
// ---------------------------------------------------------------------------
struct WriteArgs {
  const char* key;
  const char* value;
  char* key_cache;
  char* value_cache;
  // slot-mapped addressing
  const void* slot_mapping;
  int slot_bytes;
  // page-table addressing (used when batch_indices != nullptr)
  const int32_t* batch_indices;
  const int32_t* positions;
  const int32_t* kv_indices;
  const int32_t* kv_indptr;
  int64_t batch_size;
  int64_t num_kv_indices;
  // geometry; every stride in BYTES
  uint32_t num_tokens;       // tokens of this launch (host splits huge T)
  uint32_t vecs_per_row;
  int vpr_shift;             // log2(vecs_per_row) or -1
  uint32_t items_per_token;  // 2 * num_layers * vecs_per_row; item = (layer, K|V, vec)
  uint32_t num_groups;       // workgroups per token
  int groups_fastest;        // blockIdx.x = token * num_groups + group (else group * T + token)
  int pipe;                  // 1 = a lane waits for each of its loads before issuing the next one,
                             // so that the lanes of a launch that is resident all at once drift
                             // apart and reads overlap writes
  int64_t key_token_stride, value_token_stride;
  int64_t key_layer_stride, value_layer_stride;
  int64_t block_size;
  int bs_shift;              // log2(block_size) or -1
  int64_t cache_block_stride, cache_slot_stride, cache_layer_stride;
  int64_t num_cache_blocks;
  // plane kernel only
  uint32_t num_planes;        // 2 * num_layers; plane = (layer, K|V)
  uint32_t tokens_per_wg;     // blockDim.x / vecs_per_row
  uint32_t num_token_groups;  // ceil(num_tokens / tokens_per_wg)
};

// One workgroup = one token x a run of VPT*blockDim.x vectors out of the
// token's 2*L rows (K and V of every layer). The token, hence its slot and
// every base address, is uniform across the workgroup.
// Order of work: the source addresses need only the token, so every lane first
// issues its VPT independent 16-byte loads; the index chain (slot_mapping, or
// batch_indices -> kv_indptr -> kv_indices) is resolved on the scalar unit
// while those loads are in flight; the stores follow. A token whose slot is
// invalid simply returns with its loads unused.
template <int VEC, int VPT, bool PAGED, bool NT, bool NTL>
__global__ __launch_bounds__(kThreads) void write_rows_kernel(WriteArgs a) {
  using V = typename VecOf<VEC>::type;
  // blockIdx.x = group * num_tokens + token by default: neighbouring workgroups
  // read neighbouring token rows of the same layers
  uint32_t group, t;
  if (a.groups_fastest) {
    t = blockIdx.x / a.num_groups;
    group = blockIdx.x - t * a.num_groups;
  } else {
    group = blockIdx.x / a.num_tokens;
    t = blockIdx.x - group * a.num_tokens;
  }
  const char* key_row = a.key + (int64_t)t * a.key_token_stride;
  const char* value_row = a.value + (int64_t)t * a.value_token_stride;
  const uint32_t first = group * (VPT * blockDim.x) + threadIdx.x;
  // item -> (row r = 2*layer + K|V, vector inside the row)
  const auto split = [&](uint32_t item, uint32_t& r, uint32_t& vec) {
    if (a.vpr_shift >= 0) {
      r = item >> a.vpr_shift;
      vec = item & (a.vecs_per_row - 1u);
    } else {
      r = item / a.vecs_per_row;
      vec = item - r * a.vecs_per_row;
    }
  };
  // Loads are unconditional (an item index past the token's last vector is
  // clamped to it and its store skipped): straight-line code keeps the register
  // count at the data registers plus a few addresses, whatever VPT.
  V data[VPT];
  const uint32_t last_item = a.items_per_token - 1u;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    uint32_t r, vec;
    split(min(first + j * blockDim.x, last_item), r, vec);
    const int64_t layer = r >> 1;
    const char* src = ((r & 1u) ? value_row + layer * a.value_layer_stride
                                : key_row + layer * a.key_layer_stride) + (int64_t)vec * VEC;
    data[j] = ld<NTL>(reinterpret_cast<const V*>(src));
    if (VPT > 1 && a.pipe == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }

  int64_t blk, off;
  if constexpr (PAGED) {
    const int64_t b = a.batch_indices[t];
    const int64_t p = a.positions[t];
    if (b < 0 || b >= a.batch_size || p < 0) return;
    int64_t pg;
    if (a.bs_shift >= 0) {
      pg = p >> a.bs_shift;
      off = p & (a.block_size - 1);
    } else {
      pg = p / a.block_size;
      off = p - pg * a.block_size;
    }
    // the page must lie inside this request's own table (and inside the array)
    const int64_t it = (int64_t)a.kv_indptr[b] + pg;
    if (it < 0 || it >= (int64_t)a.kv_indptr[b + 1] || it >= a.num_kv_indices) return;
    blk = a.kv_indices[it];
  } else {
    const int64_t s = (a.slot_bytes == 8)
                          ? reinterpret_cast<const int64_t*>(a.slot_mapping)[t]
                          : (int64_t) reinterpret_cast<const int32_t*>(a.slot_mapping)[t];
    if (s < 0) return;
    if (a.bs_shift >= 0) {
      blk = s >> a.bs_shift;
      off = s & (a.block_size - 1);
    } else {
      blk = s / a.block_size;
      off = s - blk * a.block_size;
    }
  }
  if (blk < 0 || blk >= a.num_cache_blocks) return;
  const int64_t slot_off = blk * a.cache_block_stride + off * a.cache_slot_stride;
  char* kc_row = a.key_cache + slot_off;
  char* vc_row = a.value_cache + slot_off;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const uint32_t item = first + j * blockDim.x;
    if (item <= last_item) {
      uint32_t r, vec;
      split(item, r, vec);
      char* dst = ((r & 1u) ? vc_row : kc_row) + (int64_t)(r >> 1) * a.cache_layer_stride + (int64_t)vec * VEC;
      st<NT>(reinterpret_cast<V*>(dst), data[j]);
    }
  }
}

// The lanes of a workgroup run over consecutive TOKENS of one (layer, K|V)
// plane: the source side is one contiguous run of blockDim.x * 16 bytes, the
// cache side one row per token. Each lane looks up its own token's slot (lanes
// of one row read the same index words) and reuses it for its VPT planes, whose
// loads are issued before the lookup. Two regimes use it:
//   - rows shorter than the 1 KiB a wavefront moves per instruction (one KV head
//     of a tensor-parallel shard: 256-byte rows), where a token per workgroup
//     leaves a wavefront spanning several rows of several layers and neither
//     side is one run;
//   - launches that a few planes per lane bring down to one resident set of
//     lanes (a decode step of every layer at once): no second round of workgroups,
//     several loads in flight per lane.
// 16-byte vectors and a power-of-two number of them per row (up to 256) only;
// blockIdx.x = plane_group * num_token_groups + token_group.
template <int VPT, bool PAGED, bool NT, bool NTL>
__global__ __launch_bounds__(1024) void write_planes_kernel(WriteArgs a) {
  using V = u32x4;
  const uint32_t pg = blockIdx.x / a.num_token_groups;
  const uint32_t tg = blockIdx.x - pg * a.num_token_groups;
  const uint32_t t = tg * a.tokens_per_wg + (threadIdx.x >> a.vpr_shift);
  if (t >= a.num_tokens) return;
  const int64_t vec_off = (int64_t)(threadIdx.x & (a.vecs_per_row - 1u)) * 16;
  const char* key_row = a.key + (int64_t)t * a.key_token_stride + vec_off;
  const char* value_row = a.value + (int64_t)t * a.value_token_stride + vec_off;
  // Loads are unconditional (a plane index past the end is clamped to the last
  // plane and its store skipped): straight-line code keeps the register count
  // at the data registers plus a few addresses.
  V data[VPT];
  const uint32_t last_plane = a.num_planes - 1u;
  const auto load_plane = [&](int j) {
    const uint32_t plane = min(pg * VPT + j, last_plane);
    const int64_t layer = plane >> 1;
    const char* src = (plane & 1u) ? value_row + layer * a.value_layer_stride
                                   : key_row + layer * a.key_layer_stride;
    return ld<NTL>(reinterpret_cast<const V*>(src));
  };
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    data[j] = load_plane(j);
    if (VPT > 1 && a.pipe == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  int64_t blk, off;
  if constexpr (PAGED) {
    const int64_t b = a.batch_indices[t];
    const int64_t p = a.positions[t];
    if (b < 0 || b >= a.batch_size || p < 0) return;
    int64_t pgi;
    if (a.bs_shift >= 0) {
      pgi = p >> a.bs_shift;
      off = p & (a.block_size - 1);
    } else {
      pgi = p / a.block_size;
      off = p - pgi * a.block_size;
    }
    const int64_t it = (int64_t)a.kv_indptr[b] + pgi;
    if (it < 0 || it >= (int64_t)a.kv_indptr[b + 1] || it >= a.num_kv_indices) return;
    blk = a.kv_indices[it];
  } else {
    const int64_t s = (a.slot_bytes == 8)
                          ? reinterpret_cast<const int64_t*>(a.slot_mapping)[t]
                          : (int64_t) reinterpret_cast<const int32_t*>(a.slot_mapping)[t];
    if (s < 0) return;
    if (a.bs_shift >= 0) {
      blk = s >> a.bs_shift;
      off = s & (a.block_size - 1);
    } else {
      blk = s / a.block_size;
      off = s - blk * a.block_size;
    }
  }
  if (blk < 0 || blk >= a.num_cache_blocks) return;
  const int64_t slot_off = blk * a.cache_block_stride + off * a.cache_slot_stride + vec_off;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const uint32_t plane = pg * VPT + j;
    if (plane < a.num_planes) {
      char* dst = ((plane & 1u) ? a.value_cache : a.key_cache) + slot_off +
                  (int64_t)(plane >> 1) * a.cache_layer_stride;
      st<NT>(reinterpret_cast<V*>(dst), data[j]);
    }
  }
}

// ---------------------------------------------------------------------------
// copy_tiles_kernel
// ---------------------------------------------------------------------------
struct TileArgs {
  const char* src_base;
  char* dst_base;
  const int64_t* src_ids;  // device; nullptr = identity (i)
  const int64_t* dst_ids;  // device; nullptr = identity (i)
  int id_stride;           // 1, or 2 for the interleaved [src,dst,...] pair list
  int64_t src_layer_stride, src_block_stride;
  int64_t dst_layer_stride, dst_block_stride;
  int64_t num_src_blocks, num_dst_blocks;  // bounds for the id lists
  int64_t tile_bytes;
  uint32_t chunks_per_tile;
  uint32_t num_layers;
  uint32_t num_items;      // n: blocks (or pairs) of the launch
  int layer_slowest;       // tile order: 0 = layers of one block are neighbours, 1 = blocks of one layer
  uint64_t total_chunks;   // n * num_layers * chunks_per_tile
};

template <int VEC, int UNROLL, bool NT>
__global__ __launch_bounds__(kThreads) void copy_tiles_kernel(TileArgs a) {
  using V = typename VecOf<VEC>::type;
  constexpr int64_t kChunk = (int64_t)kThreads * UNROLL * VEC;
  for (uint64_t w = blockIdx.x; w < a.total_chunks; w += gridDim.x) {
    // chunk fastest, then layer, then block: neighbouring workgroups stream
    // neighbouring addresses of one tile
    uint32_t chunk, layer;
    int64_t i;
    if (a.total_chunks <= 0xffffffffull) {  // 32-bit divisions when they suffice
      const uint32_t w32 = (uint32_t)w;
      const uint32_t tile = w32 / a.chunks_per_tile;
      chunk = w32 - tile * a.chunks_per_tile;
      if (a.layer_slowest) {
        layer = tile / a.num_items;
        i = tile - layer * a.num_items;
      } else {
        const uint32_t blk = tile / a.num_layers;
        layer = tile - blk * a.num_layers;
        i = blk;
      }
    } else {
      chunk = (uint32_t)(w % a.chunks_per_tile);
      const uint64_t tile = w / a.chunks_per_tile;
      if (a.layer_slowest) {
        layer = (uint32_t)(tile / a.num_items);
        i = (int64_t)(tile % a.num_items);
      } else {
        layer = (uint32_t)(tile % a.num_layers);
        i = (int64_t)(tile / a.num_layers);
      }
    }
    const int64_t sid = a.src_ids ? a.src_ids[i * a.id_stride] : i;
    const int64_t did = a.dst_ids ? a.dst_ids[i * a.id_stride] : i;
    if (sid < 0 || sid >= a.num_src_blocks || did < 0 || did >= a.num_dst_blocks) continue;
    const char* src = a.src_base + layer * a.src_layer_stride + sid * a.src_block_stride;
    char* dst = a.dst_base + layer * a.dst_layer_stride + did * a.dst_block_stride;
    if (src == dst) continue;
    const int64_t base = chunk * kChunk + (int64_t)threadIdx.x * VEC;
    V data[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int64_t off = base + (int64_t)j * kThreads * VEC;
      if (off < a.tile_bytes) data[j] = ld<NT>(reinterpret_cast<const V*>(src + off));
    }
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
      const int64_t off = base + (int64_t)j * kThreads * VEC;
      if (off < a.tile_bytes) st<NT>(reinterpret_cast<V*>(dst + off), data[j]);
    }
  }
}

// ---------------------------------------------------------------------------
// write_runs_kernel
// ---------------------------------------------------------------------------
// The K/V write as a tile copy. A block run (see build_write_index_kernel) of
// one (layer, K|V) plane is contiguous on both sides when rows are dense: up to
// block_size rows of the source plane go to consecutive entries of one cache
// block. A workgroup owns a chunk of 256 lanes x UNROLL x VEC bytes of one
// (run, plane), reads the run's descriptor on the scalar unit, issues all its
// loads before its first store. The grid is sized for `max_runs` runs; the
// number of runs of this step is read from device memory, so a recorded launch
// serves steps of any size up to that capacity.
struct RunArgs {
  const char* key;
  const char* value;
  char* key_cache;
  char* value_cache;
  const int32_t* runs;      // [max_runs][4]: first token, block id, first entry, token count
  const int32_t* num_runs;  // device scalar
  uint32_t max_runs, num_planes, chunks_per_run;
  uint32_t vecs_per_row;
  int vpr_shift;            // log2(vecs_per_row) or -1
  int plane_major;          // 1: blockIdx = (plane, run, chunk); 0: (run, plane, chunk)
  int64_t key_token_stride, value_token_stride;  // bytes
  int64_t key_layer_stride, value_layer_stride;
  int64_t cache_block_stride, cache_slot_stride, cache_layer_stride;
  int64_t num_cache_blocks, block_size, num_tokens;
};

template <int VEC, int UNROLL, bool NT>
__global__ __launch_bounds__(kThreads) void write_runs_kernel(RunArgs a) {
  using V = typename VecOf<VEC>::type;
  const uint32_t chunk = blockIdx.x % a.chunks_per_run;
  const uint32_t rest = blockIdx.x / a.chunks_per_run;
  uint32_t run, plane;
  if (a.plane_major) {
    plane = rest / a.max_runs;
    run = rest - plane * a.max_runs;
  } else {
    run = rest / a.num_planes;
    plane = rest - run * a.num_planes;
  }
  if (run >= (uint32_t)*a.num_runs) return;
  const int4 d = reinterpret_cast<const int4*>(a.runs)[run];
  const int64_t first_token = d.x, block = d.y, entry = d.z, count = d.w;
  if (block < 0 || block >= a.num_cache_blocks || count <= 0 || entry < 0 ||
      entry + count > a.block_size || first_token < 0 || first_token + count > a.num_tokens)
    return;
  const uint32_t nvec = (uint32_t)count * a.vecs_per_row;
  const uint32_t v_first = chunk * (kThreads * UNROLL);
  if (v_first >= nvec) return;  // a short run needs fewer chunks than a full one
  const int64_t layer = plane >> 1;
  const bool is_v = plane & 1u;
  const char* src = (is_v ? a.value + layer * a.value_layer_stride : a.key + layer * a.key_layer_stride);
  const int64_t src_token_stride = is_v ? a.value_token_stride : a.key_token_stride;
  src += first_token * src_token_stride;
  char* dst = (is_v ? a.value_cache : a.key_cache) + layer * a.cache_layer_stride +
              block * a.cache_block_stride + entry * a.cache_slot_stride;
  const auto split = [&](uint32_t v, uint32_t& tok, uint32_t& vec) {
    if (a.vpr_shift >= 0) {
      tok = v >> a.vpr_shift;
      vec = v & (a.vecs_per_row - 1u);
    } else {
      tok = v / a.vecs_per_row;
      vec = v - tok * a.vecs_per_row;
    }
  };
  V data[UNROLL];
#pragma unroll
  for (int j = 0; j < UNROLL; ++j) {
    uint32_t tok, vec;
    split(min(v_first + j * kThreads + threadIdx.x, nvec - 1u), tok, vec);
    data[j] = ld<NT>(reinterpret_cast<const V*>(src + (int64_t)tok * src_token_stride + (int64_t)vec * VEC));
  }
#pragma unroll
  for (int j = 0; j < UNROLL; ++j) {
    const uint32_t v = v_first + j * kThreads + threadIdx.x;
    if (v < nvec) {
      uint32_t tok, vec;
      split(v, tok, vec);
      st<NT>(reinterpret_cast<V*>(dst + (int64_t)tok * a.cache_slot_stride + (int64_t)vec * VEC), data[j]);
    }
  }
}

// ---------------------------------------------------------------------------
// index kernels
// ---------------------------------------------------------------------------
__global__ void seq_lens_kernel(const int32_t* kv_indptr, const int32_t* last_page_len,
                                int64_t batch_size, int32_t page_size, int32_t* seq_lens) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch_size) return;
  int32_t pages = kv_indptr[b + 1] - kv_indptr[b] - 1;
  if (pages < 0) pages = 0;
  seq_lens[b] = pages * page_size + last_page_len[b];
}

// slot of every token of a page-table write: page * page_size + entry, or -1
// where the write would skip the token (the rules of the write kernels)
__global__ void resolve_slots_kernel(const int32_t* batch_indices, const int32_t* positions,
                                     const int32_t* kv_indices, const int32_t* kv_indptr,
                                     int64_t batch_size, int64_t num_kv_indices, int64_t page_size,
                                     int64_t nnz, int64_t* slots) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= nnz) return;
  int64_t slot = -1;
  const int64_t b = batch_indices[t];
  const int64_t p = positions[t];
  if (b >= 0 && b < batch_size && p >= 0) {
    const int64_t pg = p / page_size;
    const int64_t it = (int64_t)kv_indptr[b] + pg;
    if (it >= 0 && it < (int64_t)kv_indptr[b + 1] && it < num_kv_indices) {
      const int64_t blk = kv_indices[it];
      if (blk >= 0) slot = blk * page_size + (p - pg * page_size);
    }
  }
  slots[t] = slot;
}

__global__ void batch_indices_positions_kernel(const int32_t* append_indptr,
                                               const int32_t* seq_lens, int64_t nnz,
                                               int32_t* batch_indices, int32_t* positions) {
  const int32_t b = blockIdx.x;
  const int32_t begin = append_indptr[b];
  const int32_t end = append_indptr[b + 1];
  const int32_t first_pos = seq_lens[b] - (end - begin);
  for (int32_t j = begin + (int32_t)threadIdx.x; j < end; j += blockDim.x) {
    if (j < 0 || j >= nnz) continue;
    batch_indices[j] = b;
    positions[j] = first_pos + (j - begin);
  }
}

// Whole index preparation of a step in one launch (one workgroup): prefix sums
// of the per-request new-token counts, block counts and block-run counts, the
// last-page fill, and for every new token its request, absolute position and
// slot. The per-token outputs are CAPACITY-bound: entries from the step's token
// count up to `nnz` are filled with -1 (a request index, position and slot every
// write kernel skips), so a launch recorded once for `nnz` tokens serves steps
// of any smaller size.
// A block run is a maximal range of a request's new tokens that falls into one
// block: consecutive tokens on the source side, consecutive cache entries on
// the other. Its descriptor is four int32: first token, block id, first entry,
// token count. The first token of every run writes it.
constexpr int kPrepThreads = 1024;

// Inclusive scan of three values over the workgroup's 1024 lanes: shuffles inside
// each wavefront, then the 16 wavefront totals through LDS (two barriers).
__device__ __forceinline__ void scan3(int32_t& q, int32_t& n, int32_t& r, int32_t (*wave_sums)[3]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int32_t uq = __shfl_up(q, off, 64), un = __shfl_up(n, off, 64), ur = __shfl_up(r, off, 64);
    if (lane >= off) {
      q += uq;
      n += un;
      r += ur;
    }
  }
  __syncthreads();  // the previous round's readers are done with wave_sums
  if (lane == 63) {
    wave_sums[wave][0] = q;
    wave_sums[wave][1] = n;
    wave_sums[wave][2] = r;
  }
  __syncthreads();
  for (int w = 0; w < wave; ++w) {
    q += wave_sums[w][0];
    n += wave_sums[w][1];
    r += wave_sums[w][2];
  }
}

__global__ __launch_bounds__(kPrepThreads) void build_write_index_kernel(
    const int32_t* input_lens, const int32_t* context_lens, const int32_t* num_blocks,
    const int32_t* kv_indices, int32_t batch_size, int64_t num_kv_indices, int32_t page_size,
    int64_t nnz, int32_t* cu_seqlens_q, int32_t* kv_indptr, int32_t* kv_last_page_len,
    int32_t* batch_indices, int32_t* positions, int64_t* slot_mapping, int32_t* run_indptr,
    int32_t* runs, int32_t* num_runs, int64_t max_runs) {
  __shared__ int32_t carry[3];
  __shared__ int32_t wave_sums[kPrepThreads / 64][3];
  // prefix sums of a batch that fits one chunk stay in LDS for the per-token part
  __shared__ int32_t lds_cu[kPrepThreads + 1], lds_indptr[kPrepThreads + 1], lds_runptr[kPrepThreads + 1];
  const int tid = threadIdx.x;
  const bool in_lds = batch_size <= kPrepThreads;
  if (tid == 0) {
    carry[0] = carry[1] = carry[2] = 0;
    cu_seqlens_q[0] = 0;
    kv_indptr[0] = 0;
    if (run_indptr) run_indptr[0] = 0;
    lds_cu[0] = lds_indptr[0] = lds_runptr[0] = 0;
  }
  // every descriptor starts out empty: a run whose first token lies beyond `nnz` is never written
  if (runs)
    for (int64_t r = tid; r < max_runs; r += kPrepThreads)
      reinterpret_cast<int4*>(runs)[r] = make_int4(0, -1, 0, 0);
  __syncthreads();
  for (int32_t base = 0; base < batch_size; base += kPrepThreads) {
    const int32_t b = base + tid;
    int32_t q = b < batch_size ? input_lens[b] : 0;
    int32_t n = b < batch_size ? num_blocks[b] : 0;
    const int32_t ctx = b < batch_size ? context_lens[b] : 0;
    // runs of the request: the blocks its new positions [ctx - q, ctx) touch
    int32_t nr = (q > 0 && ctx >= q) ? (ctx - 1) / page_size - (ctx - q) / page_size + 1 : 0;
    scan3(q, n, nr, wave_sums);
    q += carry[0];
    n += carry[1];
    nr += carry[2];
    if (b < batch_size) {
      cu_seqlens_q[b + 1] = q;
      kv_indptr[b + 1] = n;
      if (run_indptr) run_indptr[b + 1] = nr;
      kv_last_page_len[b] = ctx > 0 ? (ctx - 1) % page_size + 1 : 0;
      if (in_lds) {
        lds_cu[b + 1] = q;
        lds_indptr[b + 1] = n;
        lds_runptr[b + 1] = nr;
      }
    }
    __syncthreads();  // everyone has read the carry
    if (tid == kPrepThreads - 1) {
      carry[0] = q;
      carry[1] = n;
      carry[2] = nr;
    }
    __syncthreads();
  }
  if (tid == 0 && num_runs) *num_runs = (int32_t)(carry[2] < max_runs ? carry[2] : max_runs);
  // per token: find its request by bisection over the prefix sums just written
  // (visible to the whole workgroup after the barrier above); the request's new
  // tokens occupy positions [context - input, context)
  const int32_t* cu = in_lds ? lds_cu : cu_seqlens_q;
  const int32_t* indptr = in_lds ? lds_indptr : kv_indptr;
  const int32_t* runptr = in_lds ? lds_runptr : run_indptr;
  const int64_t total = carry[0];
  const int64_t limit = total < nnz ? total : nnz;
  for (int64_t out = tid; out < nnz; out += kPrepThreads) {
    if (out >= limit) {  // beyond this step's tokens: entries every write kernel skips
      batch_indices[out] = -1;
      positions[out] = -1;
      if (slot_mapping) slot_mapping[out] = -1;
      continue;
    }
    int32_t lo = 0, hi = batch_size;  // invariant: cu[lo] <= out < cu[hi]
    while (hi - lo > 1) {
      const int32_t mid = (lo + hi) >> 1;
      if (cu[mid] <= out) lo = mid;
      else hi = mid;
    }
    const int32_t b = lo;
    const int32_t begin = cu[b];
    const int32_t n_new = cu[b + 1] - begin;
    const int32_t j = (int32_t)(out - begin);
    const int32_t ctx = context_lens[b];
    const int32_t pos = ctx - n_new + j;
    batch_indices[out] = b;
    positions[out] = pos;
    const int64_t it = (int64_t)indptr[b] + pos / page_size;
    const int64_t table_end = indptr[b + 1] < num_kv_indices ? indptr[b + 1] : num_kv_indices;
    const bool in_table = pos >= 0 && it >= 0 && it < table_end;
    const int32_t block = in_table ? kv_indices[it] : -1;
    if (slot_mapping) slot_mapping[out] = in_table ? (int64_t)block * page_size + pos % page_size : -1;
    if (runs && pos >= 0 && ctx >= n_new && (j == 0 || pos % page_size == 0)) {
      const int32_t first_pos = ctx - n_new;
      const int64_t r = (int64_t)runptr[b] + (pos / page_size - first_pos / page_size);
      if (r >= 0 && r < max_runs) {
        int64_t count = page_size - pos % page_size;
        if (count > n_new - j) count = n_new - j;
        if (count > nnz - out) count = nnz - out;
        reinterpret_cast<int4*>(runs)[r] = make_int4((int32_t)out, block, pos % page_size, (int32_t)count);
      }
    }
  }
}

// Block runs of an arbitrary slot mapping (one workgroup): token t opens a run
// when its slot is valid and is not the successor of token t-1's slot inside
// the same block. Same descriptors as the index build writes.
__global__ __launch_bounds__(kPrepThreads) void slot_runs_kernel(const void* slot_mapping, int slot_bytes,
                                                                 int64_t num_tokens, int64_t block_size,
                                                                 int32_t* runs, int32_t* num_runs,
                                                                 int64_t max_runs) {
  __shared__ int32_t part[kPrepThreads];
  __shared__ int32_t carry;
  const int tid = threadIdx.x;
  const auto slot_of = [&](int64_t t) -> int64_t {
    return slot_bytes == 8 ? reinterpret_cast<const int64_t*>(slot_mapping)[t]
                           : (int64_t) reinterpret_cast<const int32_t*>(slot_mapping)[t];
  };
  const auto opens = [&](int64_t t, int64_t s) {
    if (s < 0) return false;
    if (t == 0 || s % block_size == 0) return true;
    return slot_of(t - 1) != s - 1;
  };
  if (tid == 0) carry = 0;
  for (int64_t r = tid; r < max_runs; r += kPrepThreads)
    reinterpret_cast<int4*>(runs)[r] = make_int4(0, -1, 0, 0);
  __syncthreads();
  // pass 1: the first token of a run writes its descriptor with a count of 0
  for (int64_t base = 0; base < num_tokens; base += kPrepThreads) {
    const int64_t t = base + tid;
    const int64_t s = t < num_tokens ? slot_of(t) : -1;
    const bool head = t < num_tokens && opens(t, s);
    part[tid] = head ? 1 : 0;
    __syncthreads();
    for (int off = 1; off < kPrepThreads; off <<= 1) {
      const int32_t add = tid >= off ? part[tid - off] : 0;
      __syncthreads();
      part[tid] += add;
      __syncthreads();
    }
    if (head) {
      const int64_t r = (int64_t)carry + part[tid] - 1;
      if (r < max_runs)
        reinterpret_cast<int4*>(runs)[r] =
            make_int4((int32_t)t, (int32_t)(s / block_size), (int32_t)(s % block_size), 0);
    }
    __syncthreads();
    if (tid == kPrepThreads - 1) carry += part[tid];
    __syncthreads();
  }
  if (tid == 0) {
    *num_runs = (int32_t)(carry < max_runs ? carry : max_runs);
    carry = 0;
  }
  __syncthreads();
  // pass 2: the last token of a run writes the count (descriptors of pass 1 are
  // visible to the workgroup after the barriers above)
  for (int64_t base = 0; base < num_tokens; base += kPrepThreads) {
    const int64_t t = base + tid;
    const int64_t s = t < num_tokens ? slot_of(t) : -1;
    const bool head = t < num_tokens && opens(t, s);
    part[tid] = head ? 1 : 0;
    __syncthreads();
    for (int off = 1; off < kPrepThreads; off <<= 1) {
      const int32_t add = tid >= off ? part[tid - off] : 0;
      __syncthreads();
      part[tid] += add;
      __syncthreads();
    }
    if (t < num_tokens && s >= 0) {
      const bool last = t + 1 == num_tokens || opens(t + 1, slot_of(t + 1)) || slot_of(t + 1) < 0;
      const int64_t r = (int64_t)carry + part[tid] - 1;
      if (last && r >= 0 && r < max_runs) runs[4 * r + 3] = (int32_t)(t - runs[4 * r] + 1);
    }
    __syncthreads();
    if (tid == kPrepThreads - 1) carry += part[tid];
    __syncthreads();
  }
}

// Two kernels for kvc_streams_share_hw_queue: one keeps its hardware queue busy
// for `ticks` of the 100 MHz wall clock (one wavefront that sleeps between
// looks at the clock; `max_iters` bounds the loop whatever the clock reads),
// the other does nothing.
__global__ void hold_queue_kernel(uint64_t ticks, uint32_t max_iters) {
  const uint64_t begin = wall_clock64();
  for (uint32_t i = 0; i < max_iters; ++i) {
    if (wall_clock64() - begin >= ticks) break;
    __builtin_amdgcn_s_sleep(32);
  }
}
__global__ void touch_queue_kernel() {}

// ---------------------------------------------------------------------------
// host helpers
// ---------------------------------------------------------------------------
using kvc::log2_exact;

// widest vector (bytes) that divides every value given (addresses and strides)
inline int common_vec(std::initializer_list<uint64_t> vals) {
  uint64_t acc = 16;
  for (uint64_t v : vals) {
    while (acc > 1 && (v % acc)) acc >>= 1;
  }
  return (int)acc;
}

// Workgroups of kThreads lanes the current device holds at once (2048 lanes per CU).
int resident_workgroups() {
  static thread_local int cached_dev = -1, cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 2048;
  if (dev != cached_dev) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached = cus * (2048 / kThreads);
    cached_dev = dev;
  }
  return cached;
}

struct WriteLaunch {
  unsigned grid;     // workgroups
  unsigned threads;  // lanes per workgroup
  int vpt;
  bool nt;   // non-temporal stores
  bool ntl;  // non-temporal loads
};

template <int VEC, int VPT, bool PAGED>
void launch_write_nt(const WriteArgs& a, const WriteLaunch& l, hipStream_t s) {
  const dim3 grid(l.grid), block(l.threads);
  if (l.nt && l.ntl) hipLaunchKernelGGL((write_rows_kernel<VEC, VPT, PAGED, true, true>), grid, block, 0, s, a);
  else if (l.nt) hipLaunchKernelGGL((write_rows_kernel<VEC, VPT, PAGED, true, false>), grid, block, 0, s, a);
  else if (l.ntl) hipLaunchKernelGGL((write_rows_kernel<VEC, VPT, PAGED, false, true>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((write_rows_kernel<VEC, VPT, PAGED, false, false>), grid, block, 0, s, a);
}

template <int VEC, bool PAGED>
void launch_write_vpt(const WriteArgs& a, const WriteLaunch& l, hipStream_t s) {
  switch (l.vpt) {
    case 1: launch_write_nt<VEC, 1, PAGED>(a, l, s); break;
    case 2: launch_write_nt<VEC, 2, PAGED>(a, l, s); break;
    case 4: launch_write_nt<VEC, 4, PAGED>(a, l, s); break;
    default: launch_write_nt<VEC, 8, PAGED>(a, l, s); break;
  }
}

template <bool PAGED>
void launch_write(const WriteArgs& a, int vec, const WriteLaunch& l, hipStream_t s) {
  switch (vec) {
    case 16: launch_write_vpt<16, PAGED>(a, l, s); break;
    case 8: launch_write_vpt<8, PAGED>(a, l, s); break;
    case 4: launch_write_vpt<4, PAGED>(a, l, s); break;
    case 2: launch_write_vpt<2, PAGED>(a, l, s); break;
    default: launch_write_vpt<1, PAGED>(a, l, s); break;
  }
}

template <int VPT, bool PAGED>
void launch_planes_nt(const WriteArgs& a, const WriteLaunch& l, hipStream_t s) {
  const dim3 grid(l.grid), block(l.threads);
  if (l.nt && l.ntl) hipLaunchKernelGGL((write_planes_kernel<VPT, PAGED, true, true>), grid, block, 0, s, a);
  else if (l.nt) hipLaunchKernelGGL((write_planes_kernel<VPT, PAGED, true, false>), grid, block, 0, s, a);
  else if (l.ntl) hipLaunchKernelGGL((write_planes_kernel<VPT, PAGED, false, true>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((write_planes_kernel<VPT, PAGED, false, false>), grid, block, 0, s, a);
}

template <bool PAGED>
void launch_planes(const WriteArgs& a, const WriteLaunch& l, hipStream_t s) {
  switch (l.vpt) {
    case 1: launch_planes_nt<1, PAGED>(a, l, s); break;
    case 2: launch_planes_nt<2, PAGED>(a, l, s); break;
    case 4: launch_planes_nt<4, PAGED>(a, l, s); break;
    default: launch_planes_nt<8, PAGED>(a, l, s); break;
  }
}

struct WriteGeom {
  int64_t num_tokens, row_elems;
  int64_t key_token_stride, value_token_stride;       // elements
  int64_t block_size, cache_block_stride, cache_slot_stride, num_cache_blocks;
  int64_t num_layers, key_layer_stride, value_layer_stride, cache_layer_stride;
  int elem_bytes;
};

int check_write_geom(const char* fn, const void* key, const void* value, const void* kc,
                     const void* vc, const WriteGeom& g) {
  if (g.elem_bytes != 1 && g.elem_bytes != 2 && g.elem_bytes != 4 && g.elem_bytes != 8)
    return fail(KVC_ERR_UNSUPPORTED, "%s: elem_bytes=%d (need 1, 2, 4 or 8)", fn, g.elem_bytes);
  if (g.num_tokens < 0 || g.row_elems < 0 || g.num_layers < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: negative size (tokens=%lld row_elems=%lld layers=%lld)", fn,
                (long long)g.num_tokens, (long long)g.row_elems, (long long)g.num_layers);
  if (g.block_size <= 0 || g.num_cache_blocks < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: block_size=%lld num_cache_blocks=%lld", fn,
                (long long)g.block_size, (long long)g.num_cache_blocks);
  if (g.num_tokens == 0 || g.row_elems == 0 || g.num_layers == 0) return KVC_OK;
  if (!key || !value || !kc || !vc)
    return fail(KVC_ERR_INVALID_ARG, "%s: null key/value/cache pointer", fn);
  if (g.key_token_stride < g.row_elems || g.value_token_stride < g.row_elems)
    return fail(KVC_ERR_INVALID_ARG, "%s: token stride smaller than the row (%lld/%lld < %lld)", fn,
                (long long)g.key_token_stride, (long long)g.value_token_stride, (long long)g.row_elems);
  if (g.cache_slot_stride < g.row_elems || g.cache_block_stride < 0 || g.cache_layer_stride < 0 ||
      g.key_layer_stride < 0 || g.value_layer_stride < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: bad cache/layer stride", fn);
  if (g.num_layers > 32767)
    return fail(KVC_ERR_UNSUPPORTED, "%s: num_layers=%lld exceeds 32767", fn, (long long)g.num_layers);
  if (g.row_elems * g.elem_bytes > (int64_t(1) << 30))
    return fail(KVC_ERR_UNSUPPORTED, "%s: row of %lld bytes is beyond 1 GiB", fn,
                (long long)(g.row_elems * g.elem_bytes));
  return KVC_OK;
}

// shared driver of the four write entry points
int run_write(const char* fn, const void* key, const void* value, void* kc, void* vc,
              const void* slot_mapping, int slot_bytes, const int32_t* batch_indices,
              const int32_t* positions, const int32_t* kv_indices, const int32_t* kv_indptr,
              int64_t batch_size, int64_t num_kv_indices, const WriteGeom& g, void* stream) {
  int rc = check_write_geom(fn, key, value, kc, vc, g);
  if (rc != KVC_OK) return rc;
  if (g.num_tokens == 0 || g.row_elems == 0 || g.num_layers == 0) return KVC_OK;
  const bool paged = batch_indices != nullptr;
  if (paged) {
    if (!positions || !kv_indices || !kv_indptr)
      return fail(KVC_ERR_INVALID_ARG, "%s: null index array", fn);
    if (batch_size < 0 || num_kv_indices < 0)
      return fail(KVC_ERR_INVALID_ARG, "%s: negative batch_size/num_kv_indices", fn);
  } else {
    if (!slot_mapping) return fail(KVC_ERR_INVALID_ARG, "%s: null slot_mapping", fn);
    if (slot_bytes != 4 && slot_bytes != 8)
      return fail(KVC_ERR_UNSUPPORTED, "%s: slot_bytes=%d (need 4 or 8)", fn, slot_bytes);
  }
  const int64_t E = g.elem_bytes;
  const int vec = common_vec({(uint64_t)(uintptr_t)key, (uint64_t)(uintptr_t)value,
                              (uint64_t)(uintptr_t)kc, (uint64_t)(uintptr_t)vc,
                              (uint64_t)(g.row_elems * E), (uint64_t)(g.key_token_stride * E),
                              (uint64_t)(g.value_token_stride * E),
                              (uint64_t)(g.key_layer_stride * E), (uint64_t)(g.value_layer_stride * E),
                              (uint64_t)(g.cache_block_stride * E), (uint64_t)(g.cache_slot_stride * E),
                              (uint64_t)(g.cache_layer_stride * E)});
  WriteArgs a{};
  a.key_cache = (char*)kc;
  a.value_cache = (char*)vc;
  a.slot_bytes = slot_bytes;
  a.batch_indices = batch_indices;
  a.positions = positions;
  a.kv_indices = kv_indices;
  a.kv_indptr = kv_indptr;
  a.batch_size = batch_size;
  a.num_kv_indices = num_kv_indices;
  a.vecs_per_row = (uint32_t)(g.row_elems * E / vec);
  a.vpr_shift = log2_exact(a.vecs_per_row);
  a.key_token_stride = g.key_token_stride * E;
  a.value_token_stride = g.value_token_stride * E;
  a.key_layer_stride = g.key_layer_stride * E;
  a.value_layer_stride = g.value_layer_stride * E;
  a.block_size = g.block_size;
  a.bs_shift = log2_exact(g.block_size);
  a.cache_block_stride = g.cache_block_stride * E;
  a.cache_slot_stride = g.cache_slot_stride * E;
  a.cache_layer_stride = g.cache_layer_stride * E;
  a.num_cache_blocks = g.num_cache_blocks;
  const int64_t items64 = 2 * g.num_layers * (int64_t)a.vecs_per_row;
  if (items64 > 0x7fffffffll)
    return fail(KVC_ERR_UNSUPPORTED, "%s: %lld vectors per token exceed 2^31", fn, (long long)items64);
  a.items_per_token = (uint32_t)items64;

  // The plane kernel (lanes over consecutive tokens of one (layer, K|V) plane)
  // takes rows of a power-of-two number of 16-byte vectors up to 4 KiB. The rule
  // below comes from sweeps on MI355X over rows of 256 B to 2 KiB, one layer and
  // all layers per launch, 1 MiB to 256 MiB moved, sources rotating through
  // 512 MiB (nothing cached) and through two sets (everything cached). It is
  // written in terms of fill(v): the lanes of the launch at v planes per lane
  // over the lanes the GPU holds at once (2048 per CU).
  //   - Small launches are latency-bound and go to the token kernel (many small
  //     workgroups, scalar slot lookup): wide rows below half a resident set at
  //     one plane per lane (a quarter for page-table launches, whose lookup the
  //     plane kernel amortises over two planes), rows under 1 KiB below 256 KiB
  //     of source rows (a token per workgroup leaves their wavefronts spanning
  //     several rows of several layers, which costs 10-30 % from 1 MiB on).
  //   - The fewest planes per lane (at most 4; 2 for rows under 1 KiB) that leave
  //     the GPU at most half full run as they are: 256-lane workgroups, loads
  //     back to back.
  //   - Otherwise the fewest planes per lane that fit one resident set: no second
  //     round of workgroups. There every lane of the GPU is resident at once; if
  //     all of them issue all their loads and then all their stores, the launch
  //     splits into a read phase and a write phase and loses 15-20 % (64 MiB
  //     decode step: 14.4 against 12.2 us; 32 MiB: 8.5 against 7.1). A lane that
  //     waits for each load before issuing the next drifts apart from its
  //     neighbours and the two directions overlap: slot-mapped launches do that
  //     (from 4 planes per lane in 512-lane workgroups; at 2 planes per lane only
  //     when the GPU is more than three quarters full). The page-table lookup, a
  //     chain of dependent loads per lane, has the same effect by itself.
  //   - Launches beyond one resident set at 8 planes per lane stream best through
  //     the token kernel, with two exceptions: rows under 1 KiB (see above), and
  //     page-table launches of so few planes that every token-kernel workgroup
  //     would walk a cold index chain for 4 KiB of work (one layer of a long
  //     prefill chunk: 15.5 against 17.9 us at 64 MiB).
  const int64_t resident_lanes = (int64_t)resident_workgroups() * kThreads;
  const bool plane_rows = vec == 16 && a.vpr_shift >= 0 &&
                          (int64_t)a.vecs_per_row <= std::min(g_tune.write_planes_max_vpr, 256);
  const int64_t num_planes = 2 * g.num_layers;
  const auto plane_lanes = [&](int v) {  // lanes of the launch at v planes per lane, 256-lane workgroups
    const int64_t tpw = kThreads / (int64_t)a.vecs_per_row;
    return (g.num_tokens + tpw - 1) / tpw * ((num_planes + v - 1) / v) * kThreads;
  };
  const bool narrow = a.vecs_per_row < 64;
  int rule_vpt = 0, rule_pipe = 0, rule_lanes = kThreads;  // rule_vpt 0 = token kernel
  if (plane_rows) {
    bool pays;
    if (narrow) pays = g.num_tokens * num_planes * g.row_elems * E >= g_tune.write_planes_min_bytes;
    else pays = plane_lanes(1) * (paged ? 4 : 2) >= resident_lanes;
    if (pays) {
      const int v_first = paged ? 2 : 1;  // a lookup per lane wants two planes to pay for itself
      const int v_last = (int)std::min<int64_t>(8, num_planes);
      for (int v = v_first; v <= std::min(v_last, narrow ? 2 : 4) && !rule_vpt; v *= 2)
        if (2 * plane_lanes(v) <= resident_lanes) rule_vpt = v;
      for (int v = v_first; v <= v_last && !rule_vpt; v *= 2)
        if (plane_lanes(v) <= resident_lanes) {
          rule_vpt = v;
          if (!paged && v >= 4) { rule_pipe = 1; rule_lanes = 512; }
          else if (!paged && v == 2 && 4 * plane_lanes(v) > 3 * resident_lanes) rule_pipe = 1;
        }
      if (!rule_vpt) {  // beyond one resident set
        if (narrow) rule_vpt = v_first;
        else if (paged && num_planes * (int64_t)a.vecs_per_row <= 2 * kThreads) rule_vpt = 2;
      }
    }
    if (g_tune.write_planes >= 2 && !rule_vpt) rule_vpt = paged ? 2 : 1;  // forced
  }
  if (g_tune.write_planes && rule_vpt) {
    WriteLaunch l{};
    l.vpt = g_tune.write_planes_vpt;
    if (l.vpt != 1 && l.vpt != 2 && l.vpt != 4 && l.vpt != 8) l.vpt = rule_vpt;
    else if (l.vpt != rule_vpt) { rule_pipe = (!paged && l.vpt >= 4) ? 1 : 0; rule_lanes = rule_pipe ? 512 : kThreads; }
    while (l.vpt > 1 && (int64_t)(l.vpt / 2) >= num_planes) l.vpt /= 2;
    int wg_lanes = g_tune.write_planes_threads;
    if (wg_lanes != 256 && wg_lanes != 512 && wg_lanes != 1024) wg_lanes = rule_lanes;
    a.pipe = g_tune.write_pipe >= 0 ? g_tune.write_pipe : rule_pipe;
    const int64_t lanes_all = g.num_tokens * (int64_t)a.vecs_per_row;
    l.threads = (unsigned)std::min<int64_t>(wg_lanes, (lanes_all + 63) / 64 * 64);
    if (l.threads < a.vecs_per_row) l.threads = a.vecs_per_row;  // a row never splits over workgroups
    a.tokens_per_wg = l.threads / a.vecs_per_row;
    a.num_planes = (uint32_t)num_planes;
    l.nt = (g_tune.write_nt & 1) != 0;
    l.ntl = (g_tune.write_nt & 2) != 0 && !narrow;
    const int64_t plane_groups = (a.num_planes + l.vpt - 1) / l.vpt;
    const int64_t max_groups = std::max<int64_t>(1, 0x7fffffffll / plane_groups);
    const int64_t max_tokens = max_groups * a.tokens_per_wg;
    for (int64_t t0 = 0; t0 < g.num_tokens; t0 += max_tokens) {
      const int64_t n_tok = std::min(max_tokens, g.num_tokens - t0);
      a.num_tokens = (uint32_t)n_tok;
      a.num_token_groups = (uint32_t)((n_tok + a.tokens_per_wg - 1) / a.tokens_per_wg);
      l.grid = (unsigned)(a.num_token_groups * plane_groups);
      a.key = (const char*)key + t0 * a.key_token_stride;
      a.value = (const char*)value + t0 * a.value_token_stride;
      if (paged) {
        a.batch_indices = batch_indices + t0;
        a.positions = positions + t0;
        launch_planes<true>(a, l, (hipStream_t)stream);
      } else {
        a.slot_mapping = (const char*)slot_mapping + t0 * slot_bytes;
        launch_planes<false>(a, l, (hipStream_t)stream);
      }
      KVC_HIP(hipGetLastError());
    }
    g_last = LastLaunch{KVC_KERNEL_WRITE_PLANES, 16, l.vpt, l.threads, l.grid, (l.nt ? 1 : 0) | (l.ntl ? 2 : 0), a.pipe};
    return KVC_OK;
  }

  // Launch shape, from sweeps on MI355X. 256-lane workgroups with one vector per
  // lane (the leanest lane, the most workgroups) are best whenever the launch is
  // either smaller than one resident set of workgroups (2048 lanes per CU) or
  // many times larger. In between, a launch that 2 or 4 vectors per lane shrink
  // to exactly one resident set runs 3-5 % faster that way (no second round of
  // workgroup dispatch, several loads in flight per lane), and another 3 % faster
  // with that set made of 128-lane workgroups: the 64 MiB decode step of an
  // 8-head model is that case. Rows under 1 KiB never gain: a lane's vectors
  // then fall in different layers' rows.
  WriteLaunch l{};
  const auto wgs = [&](int64_t lanes_per_wg, int v) {
    return g.num_tokens * ((items64 + (int64_t)v * lanes_per_wg - 1) / ((int64_t)v * lanes_per_wg));
  };
  const bool fixed_wg = g_tune.write_threads == 64 || g_tune.write_threads == 128 || g_tune.write_threads == 256;
  int64_t wg = fixed_wg ? g_tune.write_threads : kThreads;
  l.vpt = g_tune.write_vpt;
  if (l.vpt != 1 && l.vpt != 2 && l.vpt != 4 && l.vpt != 8) {
    l.vpt = 1;
    const int64_t resident256 = (int64_t)resident_workgroups();
    if (g.row_elems * E >= 1024 && wgs(kThreads, 1) > resident256) {
      const int64_t shaped = fixed_wg ? wg : 128;
      const int64_t resident = resident256 * (kThreads / shaped);
      if (wgs(shaped, 2) <= resident) {
        l.vpt = 2;
        wg = shaped;
      } else if (wgs(shaped, 4) <= resident) {
        l.vpt = 4;
        wg = shaped;
      }
    }
  }
  while (l.vpt > 1 && (int64_t)(l.vpt / 2) * wg >= items64) l.vpt /= 2;
  const int64_t lanes = (items64 + l.vpt - 1) / l.vpt;
  l.threads = (unsigned)std::min<int64_t>(wg, (lanes + 63) / 64 * 64);
  l.nt = (g_tune.write_nt & 1) != 0;
  l.ntl = (g_tune.write_nt & 2) != 0 && g.row_elems * E >= 1024;
  a.pipe = g_tune.write_pipe >= 0 ? g_tune.write_pipe : (l.vpt > 1 ? 1 : 0);
  const int64_t groups = (items64 + (int64_t)l.vpt * l.threads - 1) / ((int64_t)l.vpt * l.threads);

  a.num_groups = (uint32_t)groups;
  a.groups_fastest = g_tune.write_order;

  // keep groups * tokens inside 31 bits per launch
  const int64_t max_tokens = std::max<int64_t>(1, 0x7fffffffll / groups);
  for (int64_t t0 = 0; t0 < g.num_tokens; t0 += max_tokens) {
    const int64_t n_tok = std::min(max_tokens, g.num_tokens - t0);
    a.num_tokens = (uint32_t)n_tok;
    l.grid = (unsigned)(n_tok * groups);
    a.key = (const char*)key + t0 * a.key_token_stride;
    a.value = (const char*)value + t0 * a.value_token_stride;
    if (paged) {
      a.batch_indices = batch_indices + t0;
      a.positions = positions + t0;
      launch_write<true>(a, vec, l, (hipStream_t)stream);
    } else {
      a.slot_mapping = (const char*)slot_mapping + t0 * slot_bytes;
      launch_write<false>(a, vec, l, (hipStream_t)stream);
    }
    KVC_HIP(hipGetLastError());
  }
  g_last = LastLaunch{KVC_KERNEL_WRITE_ROWS, vec, l.vpt, l.threads, l.grid, (l.nt ? 1 : 0) | (l.ntl ? 2 : 0), a.pipe};
  return KVC_OK;
}

// --------------------------- run write launch -------------------------------
template <int VEC, int UNROLL>
void launch_runs_nt(const RunArgs& a, unsigned grid, hipStream_t s, bool nt) {
  if (nt) hipLaunchKernelGGL((write_runs_kernel<VEC, UNROLL, true>), dim3(grid), dim3(kThreads), 0, s, a);
  else hipLaunchKernelGGL((write_runs_kernel<VEC, UNROLL, false>), dim3(grid), dim3(kThreads), 0, s, a);
}

template <int VEC>
void launch_runs_unroll(const RunArgs& a, int unroll, unsigned grid, hipStream_t s, bool nt) {
  switch (unroll) {
    case 1: launch_runs_nt<VEC, 1>(a, grid, s, nt); break;
    case 2: launch_runs_nt<VEC, 2>(a, grid, s, nt); break;
    default: launch_runs_nt<VEC, 4>(a, grid, s, nt); break;
  }
}

// The K/V write of `max_runs` block runs x 2 * num_layers planes as tile copies.
int run_write_runs(const char* fn, const void* key, const void* value, void* kc, void* vc,
                   const int32_t* runs, const int32_t* num_runs, int64_t max_runs, const WriteGeom& g,
                   void* stream) {
  int rc = check_write_geom(fn, key, value, kc, vc, g);
  if (rc != KVC_OK) return rc;
  if (max_runs < 0) return fail(KVC_ERR_INVALID_ARG, "%s: negative max_runs", fn);
  if (g.num_tokens == 0 || g.row_elems == 0 || g.num_layers == 0 || max_runs == 0) return KVC_OK;
  if (!runs || !num_runs) return fail(KVC_ERR_INVALID_ARG, "%s: null run list", fn);
  if ((uintptr_t)runs % 16) return fail(KVC_ERR_INVALID_ARG, "%s: the run list must be 16-byte aligned", fn);
  if (g.num_tokens > 0x7fffffffll) return fail(KVC_ERR_UNSUPPORTED, "%s: %lld tokens", fn, (long long)g.num_tokens);
  const int64_t E = g.elem_bytes;
  const int vec = common_vec({(uint64_t)(uintptr_t)key, (uint64_t)(uintptr_t)value,
                              (uint64_t)(uintptr_t)kc, (uint64_t)(uintptr_t)vc,
                              (uint64_t)(g.row_elems * E), (uint64_t)(g.key_token_stride * E),
                              (uint64_t)(g.value_token_stride * E),
                              (uint64_t)(g.key_layer_stride * E), (uint64_t)(g.value_layer_stride * E),
                              (uint64_t)(g.cache_block_stride * E), (uint64_t)(g.cache_slot_stride * E),
                              (uint64_t)(g.cache_layer_stride * E)});
  RunArgs a{};
  a.key = (const char*)key;
  a.value = (const char*)value;
  a.key_cache = (char*)kc;
  a.value_cache = (char*)vc;
  a.runs = runs;
  a.num_runs = num_runs;
  a.max_runs = (uint32_t)max_runs;
  a.num_planes = (uint32_t)(2 * g.num_layers);
  a.vecs_per_row = (uint32_t)(g.row_elems * E / vec);
  a.vpr_shift = log2_exact(a.vecs_per_row);
  a.plane_major = g_tune.runs_order != 0;
  a.key_token_stride = g.key_token_stride * E;
  a.value_token_stride = g.value_token_stride * E;
  a.key_layer_stride = g.key_layer_stride * E;
  a.value_layer_stride = g.value_layer_stride * E;
  a.cache_block_stride = g.cache_block_stride * E;
  a.cache_slot_stride = g.cache_slot_stride * E;
  a.cache_layer_stride = g.cache_layer_stride * E;
  a.num_cache_blocks = g.num_cache_blocks;
  a.block_size = g.block_size;
  a.num_tokens = g.num_tokens;
  const int64_t vecs_per_run = g.block_size * (int64_t)a.vecs_per_row;  // of a full run
  if (vecs_per_run > 0x7fffffffll)
    return fail(KVC_ERR_UNSUPPORTED, "%s: %lld vectors per run exceed 2^31", fn, (long long)vecs_per_run);
  // One vector per lane (4 KiB per workgroup at 16-byte vectors) and all runs of a
  // plane next to each other in the grid measured best at the 2048-token chunk of
  // 28 layers (43.1 us; 2 and 4 vectors per lane 45.5-46.9, run-major order 43.3,
  // an XCD-aware order 44.2-45.2; the token kernel 44.1-44.4). One layer per
  // launch prefers 2 (4.05 against 4.49 us), where the grid is a quarter of a
  // resident set.
  int unroll = g_tune.runs_unroll;
  if (unroll != 1 && unroll != 2 && unroll != 4)
    unroll = max_runs * (int64_t)a.num_planes * ((vecs_per_run + kThreads - 1) / kThreads) <= resident_workgroups() ? 2 : 1;
  while (unroll > 1 && (int64_t)kThreads * (unroll / 2) >= vecs_per_run) unroll /= 2;
  const int64_t per_wg = (int64_t)kThreads * unroll;
  a.chunks_per_run = (uint32_t)((vecs_per_run + per_wg - 1) / per_wg);
  const int64_t grid = max_runs * (int64_t)a.num_planes * a.chunks_per_run;
  if (grid > 0x7fffffffll || max_runs > 0x7fffffffll)
    return fail(KVC_ERR_UNSUPPORTED, "%s: %lld workgroups exceed 2^31", fn, (long long)grid);
  const bool nt = g_tune.runs_nt != 0;
  hipStream_t s = (hipStream_t)stream;
  switch (vec) {
    case 16: launch_runs_unroll<16>(a, unroll, (unsigned)grid, s, nt); break;
    case 8: launch_runs_unroll<8>(a, unroll, (unsigned)grid, s, nt); break;
    case 4: launch_runs_unroll<4>(a, unroll, (unsigned)grid, s, nt); break;
    case 2: launch_runs_unroll<2>(a, unroll, (unsigned)grid, s, nt); break;
    default: launch_runs_unroll<1>(a, unroll, (unsigned)grid, s, nt); break;
  }
  KVC_HIP(hipGetLastError());
  g_last = LastLaunch{KVC_KERNEL_WRITE_RUNS, vec, unroll, kThreads, grid, nt ? 3 : 0, 0};
  return KVC_OK;
}

// --------------------------- tile copy launch -------------------------------
template <int VEC, int UNROLL>
void launch_tiles_nt(const TileArgs& a, unsigned grid, hipStream_t s, bool nt) {
  if (nt) hipLaunchKernelGGL((copy_tiles_kernel<VEC, UNROLL, true>), dim3(grid), dim3(kThreads), 0, s, a);
  else hipLaunchKernelGGL((copy_tiles_kernel<VEC, UNROLL, false>), dim3(grid), dim3(kThreads), 0, s, a);
}

template <int VEC>
int launch_tiles_vec(TileArgs a, int unroll, int max_wgs, hipStream_t s, bool nt, int64_t n, int large) {
  if (unroll <= 0) {
    // By size, from sweeps of copy_blocks (1 to 4096 pairs x 32 layers x 64 KiB):
    // a launch that fits a quarter of the resident workgroups runs best as few,
    // deep workgroups (the smallest depth that gets it there; up to a whole tile
    // per workgroup while that stays within half the resident set): 6-8 % faster
    // than 4 vectors per lane from 32 to 128 MiB (a gather: 12-15 % faster than
    // with 1). Larger launches stream best with `large` vectors per lane: 2, or 1
    // when the scattered side is the one being read (gather).
    const int64_t resident = resident_workgroups();
    const auto chunks = [&](int u) {
      const int64_t c = (int64_t)kThreads * VEC * u;
      return n * (int64_t)a.num_layers * ((a.tile_bytes + c - 1) / c);
    };
    unroll = 0;
    for (int u = 1; u <= 16 && !unroll; u *= 2)
      if (chunks(u) <= resident / 4) unroll = u;
    if (!unroll) unroll = chunks(16) <= resident / 2 ? 16 : large;
  }
  // do not carry more vectors per lane than the tile can fill
  while (unroll > 1 && (int64_t)kThreads * VEC * (unroll / 2) >= a.tile_bytes) unroll /= 2;
  const int64_t chunk = (int64_t)kThreads * VEC * unroll;
  a.chunks_per_tile = (uint32_t)((a.tile_bytes + chunk - 1) / chunk);
  a.total_chunks = (uint64_t)n * a.num_layers * a.chunks_per_tile;
  a.num_items = (uint32_t)n;
  a.layer_slowest = g_tune.copy_order;
  uint64_t grid = a.total_chunks;
  if (max_wgs > 0) grid = std::min<uint64_t>(grid, (uint64_t)max_wgs);
  grid = std::min<uint64_t>(grid, 0x7fffffffull);
  switch (unroll) {
    case 1: launch_tiles_nt<VEC, 1>(a, (unsigned)grid, s, nt); break;
    case 2: launch_tiles_nt<VEC, 2>(a, (unsigned)grid, s, nt); break;
    case 4: launch_tiles_nt<VEC, 4>(a, (unsigned)grid, s, nt); break;
    case 8: launch_tiles_nt<VEC, 8>(a, (unsigned)grid, s, nt); break;
    default: launch_tiles_nt<VEC, 16>(a, (unsigned)grid, s, nt); break;
  }
  g_last = LastLaunch{KVC_KERNEL_COPY_TILES, VEC, unroll, kThreads, (int64_t)grid, nt ? 1 : 0};
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}

// unroll > 0: fixed; 0: the copy_unroll knob (by size unless set); gather: the gather_unroll knob
int launch_tiles(const TileArgs& a, int64_t n, int max_wgs, hipStream_t s, bool gather = false) {
  if (n == 0 || a.num_layers == 0 || a.tile_bytes == 0) return KVC_OK;
  const int vec = common_vec({(uint64_t)(uintptr_t)a.src_base, (uint64_t)(uintptr_t)a.dst_base,
                              (uint64_t)a.src_layer_stride, (uint64_t)a.src_block_stride,
                              (uint64_t)a.dst_layer_stride, (uint64_t)a.dst_block_stride,
                              (uint64_t)a.tile_bytes});
  int unroll = gather ? g_tune.gather_unroll : g_tune.copy_unroll;
  if (unroll != 1 && unroll != 2 && unroll != 4 && unroll != 8 && unroll != 16) unroll = 0;  // by size
  const bool nt = g_tune.copy_nt != 0;
  switch (vec) {
    case 16: return launch_tiles_vec<16>(a, unroll, max_wgs, s, nt, n, gather ? 1 : 2);
    case 8: return launch_tiles_vec<8>(a, unroll, max_wgs, s, nt, n, gather ? 1 : 2);
    case 4: return launch_tiles_vec<4>(a, unroll, max_wgs, s, nt, n, gather ? 1 : 2);
    case 2: return launch_tiles_vec<2>(a, unroll, max_wgs, s, nt, n, gather ? 1 : 2);
    default: return launch_tiles_vec<1>(a, unroll, max_wgs, s, nt, n, gather ? 1 : 2);
  }
}

// --------------------------- swap plumbing ----------------------------------
constexpr int64_t kIdAlign = 256;
inline int64_t round_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }
inline int64_t ids_region_bytes(int64_t n) { return round_up(2 * n * (int64_t)sizeof(int64_t), kIdAlign); }

// Per-thread resources of the swap entry points: events that order the two
// streams of a staged swap, and a small ring of pinned bounce buffers from
// which id lists are uploaded (the caller's lists may be pageable and may be
// freed as soon as the call returns). A bounce slot is reused only after its
// upload has run, so a call waits on the host only when kBounceSlots uploads of
// this thread are still queued. A slot that is too small is replaced by a
// larger one (at least twice its size); the outgrown buffer is kept until
// kvc_thread_release, because freeing pinned memory synchronises the device.
constexpr int kBounceSlots = 4;

struct Bounce {
  int64_t* buf = nullptr;
  int64_t cap = 0;  // int64 entries
  hipEvent_t done = nullptr;
  bool pending = false;
};

struct SwapCtx {
  hipEvent_t start = nullptr, tail = nullptr;
  hipEvent_t filled[2] = {nullptr, nullptr};   // staging slot holds fresh data
  hipEvent_t drained[2] = {nullptr, nullptr};  // staging slot may be overwritten
  Bounce bounce[kBounceSlots];
  int next_bounce = 0;
  int64_t** retired = nullptr;  // outgrown bounce buffers
  int num_retired = 0, cap_retired = 0;
  int device = -1;

  void all_events(hipEvent_t** out) {
    int k = 0;
    out[k++] = &start; out[k++] = &tail;
    out[k++] = &filled[0]; out[k++] = &filled[1];
    out[k++] = &drained[0]; out[k++] = &drained[1];
    for (int i = 0; i < kBounceSlots; ++i) out[k++] = &bounce[i].done;
  }
};
constexpr int kSwapEvents = 6 + kBounceSlots;
thread_local SwapCtx g_swap;

void swap_ctx_drop_events(SwapCtx& c) {
  for (int i = 0; i < kBounceSlots; ++i) {
    if (c.bounce[i].pending) (void)hipEventSynchronize(c.bounce[i].done);
    c.bounce[i].pending = false;
  }
  hipEvent_t* evs[kSwapEvents];
  c.all_events(evs);
  for (hipEvent_t* e : evs) {
    if (*e) (void)hipEventDestroy(*e);
    *e = nullptr;
  }
}

// events of this thread on the current device (they belong to the device they
// were created on: a thread that moves to another device starts over)
int swap_ctx_prepare() {
  int dev = 0;
  KVC_HIP(hipGetDevice(&dev));
  SwapCtx& c = g_swap;
  if (c.device != dev) {
    swap_ctx_drop_events(c);  // also what an earlier, failed attempt left behind
    c.device = -1;
    hipEvent_t* evs[kSwapEvents];
    c.all_events(evs);
    for (hipEvent_t* e : evs) KVC_HIP(hipEventCreateWithFlags(e, hipEventDisableTiming));
    c.device = dev;
  }
  return KVC_OK;
}

int swap_ctx_release() {
  SwapCtx& c = g_swap;
  if (c.device >= 0) swap_ctx_drop_events(c);
  c.device = -1;
  int rc = KVC_OK;
  for (int i = 0; i < kBounceSlots; ++i) {
    if (c.bounce[i].buf && hipHostFree(c.bounce[i].buf) != hipSuccess) rc = KVC_ERR_HIP;
    c.bounce[i] = Bounce{};
  }
  for (int i = 0; i < c.num_retired; ++i)
    if (hipHostFree(c.retired[i]) != hipSuccess) rc = KVC_ERR_HIP;
  std::free(c.retired);
  c.retired = nullptr;
  c.num_retired = c.cap_retired = 0;
  c.next_bounce = 0;
  if (rc != KVC_OK) return fail(rc, "kvc_thread_release: hipHostFree failed");
  return KVC_OK;
}

struct SwapGeom {
  int64_t n, num_layers, layer_stride_bytes, block_bytes;
  int64_t num_gpu_blocks, num_host_blocks, layer_begin, layer_end;
};

int check_ids(const char* fn, const int64_t* gpu_ids, const int64_t* host_ids, int64_t n,
              int64_t num_gpu_blocks, int64_t num_host_blocks) {
  for (int64_t i = 0; i < n; ++i) {
    if (gpu_ids[i] < 0 || gpu_ids[i] >= num_gpu_blocks)
      return fail(KVC_ERR_OUT_OF_RANGE, "%s: gpu block id %lld (entry %lld) outside [0, %lld)", fn,
                  (long long)gpu_ids[i], (long long)i, (long long)num_gpu_blocks);
    if (host_ids[i] < 0 || host_ids[i] >= num_host_blocks)
      return fail(KVC_ERR_OUT_OF_RANGE, "%s: host block id %lld (entry %lld) outside [0, %lld)", fn,
                  (long long)host_ids[i], (long long)i, (long long)num_host_blocks);
  }
  return KVC_OK;
}

// prepared: the id lists already sit at the head of the staging buffer
// (kvc_swap_prepare checked and uploaded them); gpu_ids is then unused and
// host_ids is needed only by the staged mode's PCIe extents.
int check_swap(const char* fn, const void* pool, const void* host, const int64_t* gpu_ids,
               const int64_t* host_ids, const SwapGeom& g, const void* staging,
               int64_t staging_bytes, int mode, bool prepared, int64_t* chunk_blocks) {
  if (g.n < 0 || g.num_layers < 0 || g.block_bytes < 0 || g.layer_stride_bytes < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: negative size", fn);
  if (g.layer_begin < 0 || g.layer_end < g.layer_begin || g.layer_end > g.num_layers)
    return fail(KVC_ERR_INVALID_ARG, "%s: layer range [%lld, %lld) outside [0, %lld)", fn,
                (long long)g.layer_begin, (long long)g.layer_end, (long long)g.num_layers);
  if (mode != KVC_SWAP_STAGED && mode != KVC_SWAP_DIRECT)
    return fail(KVC_ERR_INVALID_ARG, "%s: unknown swap mode %d", fn, mode);
  const int64_t nl = g.layer_end - g.layer_begin;
  *chunk_blocks = 0;
  if (g.n == 0 || nl == 0 || g.block_bytes == 0) return KVC_OK;
  if (!pool || !host) return fail(KVC_ERR_INVALID_ARG, "%s: null pool/host pointer", fn);
  if (prepared ? (mode == KVC_SWAP_STAGED && !host_ids) : (!gpu_ids || !host_ids))
    return fail(KVC_ERR_INVALID_ARG, "%s: null id list", fn);
  if (g.layer_stride_bytes < g.block_bytes)
    return fail(KVC_ERR_INVALID_ARG, "%s: layer stride smaller than a block", fn);
  if (nl > 0xffffffffll) return fail(KVC_ERR_UNSUPPORTED, "%s: too many layers", fn);
  if (!prepared) {
    const int rc = check_ids(fn, gpu_ids, host_ids, g.n, g.num_gpu_blocks, g.num_host_blocks);
    if (rc != KVC_OK) return rc;
  }
  if (!staging) return fail(KVC_ERR_STAGING, "%s: null staging buffer", fn);
  if ((uintptr_t)staging % kIdAlign)
    return fail(KVC_ERR_STAGING, "%s: staging buffer must be %lld-byte aligned", fn, (long long)kIdAlign);
  const int64_t ids_bytes = ids_region_bytes(g.n);
  if (staging_bytes < ids_bytes)
    return fail(KVC_ERR_STAGING, "%s: staging of %lld bytes cannot hold the id lists (%lld)", fn,
                (long long)staging_bytes, (long long)ids_bytes);
  if (mode == KVC_SWAP_STAGED) {
    const int64_t per_block = round_up(nl * g.block_bytes, kIdAlign);
    const int64_t cb = (staging_bytes - ids_bytes) / 2 / per_block;
    if (cb < 1)
      return fail(KVC_ERR_STAGING, "%s: staging of %lld bytes holds no ring slot (need >= %lld)", fn,
                  (long long)staging_bytes, (long long)(ids_bytes + 2 * per_block));
    *chunk_blocks = std::min(cb, g.n);
  }
  return KVC_OK;
}

// upload [gpu_ids | host_ids] to the head of the staging buffer on `s`
int upload_ids(const int64_t* gpu_ids, const int64_t* host_ids, int64_t n, void* staging,
               hipStream_t s) {
  SwapCtx& c = g_swap;
  Bounce& b = c.bounce[c.next_bounce];
  c.next_bounce = (c.next_bounce + 1) % kBounceSlots;
  if (b.pending) {
    KVC_HIP(hipEventSynchronize(b.done));
    b.pending = false;
  }
  if (2 * n > b.cap) {
    if (b.buf) {
      if (c.num_retired == c.cap_retired) {
        const int cap = c.cap_retired ? 2 * c.cap_retired : 8;
        int64_t** grown = (int64_t**)std::realloc(c.retired, cap * sizeof(int64_t*));
        if (!grown) return fail(KVC_ERR_HIP, "out of host memory");
        c.retired = grown;
        c.cap_retired = cap;
      }
      c.retired[c.num_retired++] = b.buf;
      b.buf = nullptr;
    }
    const int64_t cap = std::max<int64_t>(std::max<int64_t>(2 * n, 2 * b.cap), 4096);
    b.cap = 0;
    KVC_HIP(hipHostMalloc((void**)&b.buf, cap * sizeof(int64_t), hipHostMallocDefault));
    b.cap = cap;
  }
  std::memcpy(b.buf, gpu_ids, n * sizeof(int64_t));
  std::memcpy(b.buf + n, host_ids, n * sizeof(int64_t));
  KVC_HIP(hipMemcpyAsync(staging, b.buf, 2 * n * sizeof(int64_t), hipMemcpyHostToDevice, s));
  KVC_HIP(hipEventRecord(b.done, s));
  b.pending = true;
  return KVC_OK;
}

// PCIe leg of one staged chunk: rows of `width` bytes, one per block of the
// chunk, between the ring slot (dense) and the host pool (row pitch = a whole
// host block). Runs of consecutive host ids go out as one extent.
int copy_chunk_rows(char* slot, char* host_pool, const int64_t* host_ids, int64_t count,
                    int64_t width, int64_t host_block_bytes, int64_t host_row_offset,
                    bool to_host, hipStream_t s) {
  int64_t i = 0;
  while (i < count) {
    int64_t j = i + 1;
    while (j < count && host_ids[j] == host_ids[j - 1] + 1) ++j;
    const int64_t run = j - i;
    char* h = host_pool + host_ids[i] * host_block_bytes + host_row_offset;
    char* d = slot + i * width;
    if (width == host_block_bytes || run == 1) {
      if (to_host) KVC_HIP(hipMemcpyAsync(h, d, run * width, hipMemcpyDeviceToHost, s));
      else KVC_HIP(hipMemcpyAsync(d, h, run * width, hipMemcpyHostToDevice, s));
    } else {
      if (to_host)
        KVC_HIP(hipMemcpy2DAsync(h, host_block_bytes, d, width, width, run, hipMemcpyDeviceToHost, s));
      else
        KVC_HIP(hipMemcpy2DAsync(d, width, h, host_block_bytes, width, run, hipMemcpyHostToDevice, s));
    }
    i = j;
  }
  return KVC_OK;
}

// the tile-kernel arguments of a direct swap: pool <-> mapped host pool
TileArgs direct_swap_tiles(bool out, char* pool, char* host_pool, const int64_t* d_gpu_ids,
                           const int64_t* d_host_ids, const SwapGeom& g) {
  const int64_t host_block_bytes = g.num_layers * g.block_bytes;
  char* pool_l0 = pool + g.layer_begin * g.layer_stride_bytes;
  char* host_l0 = host_pool + g.layer_begin * g.block_bytes;
  TileArgs t{};
  t.id_stride = 1;
  t.tile_bytes = g.block_bytes;
  t.num_layers = (uint32_t)(g.layer_end - g.layer_begin);
  if (out) {
    t.src_base = pool_l0; t.src_ids = d_gpu_ids;
    t.src_layer_stride = g.layer_stride_bytes; t.src_block_stride = g.block_bytes;
    t.num_src_blocks = g.num_gpu_blocks;
    t.dst_base = host_l0; t.dst_ids = d_host_ids;
    t.dst_layer_stride = g.block_bytes; t.dst_block_stride = host_block_bytes;
    t.num_dst_blocks = g.num_host_blocks;
  } else {
    t.src_base = host_l0; t.src_ids = d_host_ids;
    t.src_layer_stride = g.block_bytes; t.src_block_stride = host_block_bytes;
    t.num_src_blocks = g.num_host_blocks;
    t.dst_base = pool_l0; t.dst_ids = d_gpu_ids;
    t.dst_layer_stride = g.layer_stride_bytes; t.dst_block_stride = g.block_bytes;
    t.num_dst_blocks = g.num_gpu_blocks;
  }
  return t;
}

// The pairs of one call in ascending order of their host block id (stable), in
// place. Blocks that lie next to each other in the host pool are then next to
// each other in the call and leave as one PCIe extent.
int order_pairs_by_host_id(int64_t* gpu_ids, int64_t* host_ids, int64_t n) {
  bool ascending = true;
  for (int64_t i = 1; i < n && ascending; ++i) ascending = host_ids[i] >= host_ids[i - 1];
  if (ascending) return KVC_OK;
  try {
    std::vector<int64_t> order((size_t)n);
    std::iota(order.begin(), order.end(), int64_t(0));
    std::stable_sort(order.begin(), order.end(),
                     [&](int64_t a, int64_t b) { return host_ids[a] < host_ids[b]; });
    std::vector<int64_t> tmp((size_t)n);
    for (int64_t i = 0; i < n; ++i) tmp[(size_t)i] = gpu_ids[order[(size_t)i]];
    std::memcpy(gpu_ids, tmp.data(), (size_t)n * sizeof(int64_t));
    for (int64_t i = 0; i < n; ++i) tmp[(size_t)i] = host_ids[order[(size_t)i]];
    std::memcpy(host_ids, tmp.data(), (size_t)n * sizeof(int64_t));
  } catch (const std::bad_alloc&) {
    return fail(KVC_ERR_HIP, "out of host memory while ordering %lld pairs", (long long)n);
  }
  return KVC_OK;
}

// this thread's ordered copy of the id lists of an unprepared call: [gpu ids | host ids]
thread_local std::vector<int64_t> g_ordered_ids;

// KVC_SWAP_AUTO: the copy engines when the PCIe leg of this call is made of large
// extents, the direct kernel when it would fall apart into small copies. The
// engines leave the kernels of other streams alone, but every copy costs about
// 10 us beyond its transfer time, so scattered host blocks of one layer (64 KiB
// each) move at a ninth of the link rate; the direct kernel holds the link rate
// whatever the ids are, but holds back the kernels of other streams while it runs.
int resolve_auto_mode(const int64_t* host_ids, const SwapGeom& g, const void* staging,
                      int64_t staging_bytes) {
  const int64_t nl = g.layer_end - g.layer_begin;
  if (!host_ids || !staging || g.n <= 0 || nl <= 0 || g.block_bytes <= 0) return KVC_SWAP_DIRECT;
  const int64_t width = nl * g.block_bytes;
  if (staging_bytes < ids_region_bytes(g.n) + 2 * round_up(width, kIdAlign)) return KVC_SWAP_DIRECT;
  int64_t runs = 1;
  for (int64_t i = 1; i < g.n; ++i) runs += host_ids[i] != host_ids[i - 1] + 1;
  // mean extent = n * width / runs, compared without the division
  return (g.n * width >= runs * (int64_t)g_tune.auto_min_extent_bytes) ? KVC_SWAP_STAGED
                                                                        : KVC_SWAP_DIRECT;
}

int run_swap(const char* fn, bool out, char* pool, char* host_pool, const int64_t* gpu_ids,
             const int64_t* host_ids, const SwapGeom& g, void* staging, int64_t staging_bytes,
             int mode, bool prepared, void* kernel_stream, void* copy_stream) {
  // An unprepared call that may go through the copy engines orders its pairs by
  // host block id first (the result of a swap does not depend on their order):
  // the staged PCIe leg follows the runs of consecutive host ids. A prepared
  // call keeps the order in which kvc_swap_prepare uploaded the lists.
  if (!prepared && mode != KVC_SWAP_DIRECT && gpu_ids && host_ids && g.n > 1) {
    try {
      g_ordered_ids.resize((size_t)(2 * g.n));
    } catch (const std::bad_alloc&) {
      return fail(KVC_ERR_HIP, "%s: out of host memory", fn);
    }
    int64_t* og = g_ordered_ids.data();
    int64_t* oh = og + g.n;
    std::memcpy(og, gpu_ids, (size_t)g.n * sizeof(int64_t));
    std::memcpy(oh, host_ids, (size_t)g.n * sizeof(int64_t));
    const int rc_order = order_pairs_by_host_id(og, oh, g.n);
    if (rc_order != KVC_OK) return rc_order;
    gpu_ids = og;
    host_ids = oh;
  }
  if (mode == KVC_SWAP_AUTO) mode = resolve_auto_mode(host_ids, g, staging, staging_bytes);
  g_last_swap_mode = mode;
  int64_t chunk_blocks = 0;
  int rc = check_swap(fn, pool, host_pool, gpu_ids, host_ids, g, staging, staging_bytes, mode,
                      prepared, &chunk_blocks);
  if (rc != KVC_OK) return rc;
  const int64_t nl = g.layer_end - g.layer_begin;
  if (g.n == 0 || nl == 0 || g.block_bytes == 0) return KVC_OK;
  hipStream_t ks = (hipStream_t)kernel_stream;
  hipStream_t cs = (hipStream_t)copy_stream;
  // A staged call of a single chunk has nothing to overlap inside itself: it
  // runs kernel and copy on kernel_stream alone and saves the two cross-stream
  // waits (about 0.15 ms each here), which a one-layer call of a few dozen MiB
  // would otherwise pay per layer.
  if (mode == KVC_SWAP_STAGED && g.n <= chunk_blocks) cs = ks;
  const bool two_streams = ks != cs;
  const int64_t* d_gpu_ids = (const int64_t*)staging;
  const int64_t* d_host_ids = d_gpu_ids + g.n;

  if (mode == KVC_SWAP_DIRECT && prepared) {
    // nothing but the launch: no events, no upload
    const TileArgs t = direct_swap_tiles(out, pool, host_pool, d_gpu_ids, d_host_ids, g);
    return launch_tiles(t, g.n, direct_wgs(out), ks);
  }
  rc = swap_ctx_prepare();
  if (rc != KVC_OK) return rc;
  SwapCtx& c = g_swap;
  if (!prepared) {
    rc = upload_ids(gpu_ids, host_ids, g.n, staging, ks);
    if (rc != KVC_OK) return rc;
  }
  const int64_t host_block_bytes = g.num_layers * g.block_bytes;
  char* pool_l0 = pool + g.layer_begin * g.layer_stride_bytes;
  const int64_t host_row_offset = g.layer_begin * g.block_bytes;

  if (mode == KVC_SWAP_DIRECT) {
    // pool <-> mapped host pool in a single kernel
    const TileArgs t = direct_swap_tiles(out, pool, host_pool, d_gpu_ids, d_host_ids, g);
    return launch_tiles(t, g.n, direct_wgs(out), ks);
  }

  TileArgs t{};
  t.id_stride = 1;
  t.tile_bytes = g.block_bytes;
  t.num_layers = (uint32_t)nl;

  // staged: two ring slots, kernel on ks, PCIe extents on cs
  const int64_t width = nl * g.block_bytes;  // bytes of one block's layer range
  const int64_t slot_bytes = round_up(width, kIdAlign) * chunk_blocks;
  char* ring = (char*)staging + ids_region_bytes(g.n);
  if (two_streams) {
    KVC_HIP(hipEventRecord(c.start, ks));
    KVC_HIP(hipStreamWaitEvent(cs, c.start, 0));
  }
  int64_t done = 0;
  for (int64_t k = 0; done < g.n; ++k, done += chunk_blocks) {
    const int64_t count = std::min(chunk_blocks, g.n - done);
    const int sl = (int)(k & 1);
    char* slot = ring + sl * slot_bytes;
    if (out) {
      // gather pool blocks -> slot (host layout [count, nl, block]) -> host
      if (two_streams && k >= 2) KVC_HIP(hipStreamWaitEvent(ks, c.drained[sl], 0));
      t.src_base = pool_l0; t.src_ids = d_gpu_ids + done;
      t.src_layer_stride = g.layer_stride_bytes; t.src_block_stride = g.block_bytes;
      t.num_src_blocks = g.num_gpu_blocks;
      t.dst_base = slot; t.dst_ids = nullptr;
      t.dst_layer_stride = g.block_bytes; t.dst_block_stride = width;
      t.num_dst_blocks = count;
      rc = launch_tiles(t, count, g_tune.copy_max_wgs, ks, true);
      if (rc != KVC_OK) return rc;
      if (two_streams) {
        KVC_HIP(hipEventRecord(c.filled[sl], ks));
        KVC_HIP(hipStreamWaitEvent(cs, c.filled[sl], 0));
      }
      rc = copy_chunk_rows(slot, host_pool, host_ids + done, count, width, host_block_bytes,
                           host_row_offset, true, cs);
      if (rc != KVC_OK) return rc;
      if (two_streams) KVC_HIP(hipEventRecord(c.drained[sl], cs));
    } else {
      // host -> slot -> scatter into pool blocks
      if (two_streams && k >= 2) KVC_HIP(hipStreamWaitEvent(cs, c.drained[sl], 0));
      rc = copy_chunk_rows(slot, host_pool, host_ids + done, count, width, host_block_bytes,
                           host_row_offset, false, cs);
      if (rc != KVC_OK) return rc;
      if (two_streams) {
        KVC_HIP(hipEventRecord(c.filled[sl], cs));
        KVC_HIP(hipStreamWaitEvent(ks, c.filled[sl], 0));
      }
      t.src_base = slot; t.src_ids = nullptr;
      t.src_layer_stride = g.block_bytes; t.src_block_stride = width;
      t.num_src_blocks = count;
      t.dst_base = pool_l0; t.dst_ids = d_gpu_ids + done;
      t.dst_layer_stride = g.layer_stride_bytes; t.dst_block_stride = g.block_bytes;
      t.num_dst_blocks = g.num_gpu_blocks;
      rc = launch_tiles(t, count, g_tune.copy_max_wgs, ks);
      if (rc != KVC_OK) return rc;
      if (two_streams) KVC_HIP(hipEventRecord(c.drained[sl], ks));
    }
  }
  if (two_streams && out) {
    // the last PCIe extents sit on the copy stream: fold them into kernel_stream
    KVC_HIP(hipEventRecord(c.tail, cs));
    KVC_HIP(hipStreamWaitEvent(ks, c.tail, 0));
  }
  return KVC_OK;
}

// --------------------------- swap that allocates nothing ---------------------
// The id lists of a direct swap live in a static device array instead of a
// caller-provided workspace, and reach it as kernel arguments instead of through
// a pinned bounce buffer and a copy: the call is kernel launches only.
static __device__ __align__(256) int64_t scratch[2 * KVC_NOALLOC_MAX_BLOCKS];  // [gpu ids | host ids]

constexpr int kMaxDevices = 64;
constexpr int kIdsPerPacket = 448;  // id pairs per staging launch: 3584 bytes of kernel arguments

struct IdPacket {
  int32_t gpu[kIdsPerPacket];
  int32_t host[kIdsPerPacket];
};

// scratch_ptr[first + i] = gpu id, scratch_ptr[n + first + i] = host id, for i in [0, count)
__global__ __launch_bounds__(kIdsPerPacket) void stage_ids_kernel(IdPacket p, int64_t* scratch_ptr,
                                                                  int64_t first, int count, int64_t n) {
  const int i = threadIdx.x;
  if (i < count) {
    scratch_ptr[first + i] = p.gpu[i];
    scratch_ptr[n + first + i] = p.host[i];
  }
}

// Device address of `scratch` on the current device. In host code the array's
// name is only a handle for the runtime; every device holds its own copy at its
// own address, looked up once per device.
int scratch_of_current_device(int64_t** out) {
  static std::mutex mu;
  static int64_t* ptrs[kMaxDevices] = {};
  int dev = 0;
  KVC_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(KVC_ERR_UNSUPPORTED, "device ordinal %d is beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    KVC_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(KVC_ERR_HIP, "hipGetSymbolAddress returned a null address for the id scratch");
    ptrs[dev] = (int64_t*)p;
  }
  *out = ptrs[dev];
  return KVC_OK;
}

}  // namespace

namespace kvc {
int launch_resolve_slots(const char* fn, const int32_t* batch_indices, const int32_t* positions,
                         const int32_t* kv_indices, const int32_t* kv_indptr, int64_t batch_size,
                         int64_t num_kv_indices, int64_t page_size, int64_t nnz, int64_t* slots,
                         hipStream_t stream) {
  if (nnz == 0) return KVC_OK;
  if (!slots) return fail(KVC_ERR_INVALID_ARG, "%s: null slot array", fn);
  if (nnz > (int64_t(1) << 40)) return fail(KVC_ERR_UNSUPPORTED, "%s: %lld tokens", fn, (long long)nnz);
  const unsigned grid = (unsigned)((nnz + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(resolve_slots_kernel, dim3(grid), dim3(kThreads), 0, stream, batch_indices,
                     positions, kv_indices, kv_indptr, batch_size, num_kv_indices, page_size, nnz, slots);
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}
}  // namespace kvc

// ===========================================================================
// C ABI
// ===========================================================================
extern "C" {

int kvc_abi_version(void) { return KVC_ABI_VERSION; }

const char* kvc_last_error_string(void) { return kvc::g_err; }

// Tuning hook for sweeps (not part of the reference surface): returns 0, or
// KVC_ERR_INVALID_ARG for an unknown key.
int kvc_set_tuning(const char* key, int value) {
  if (!key) return fail(KVC_ERR_INVALID_ARG, "kvc_set_tuning: null key");
  Knob* k = find_knob(key);
  if (!k) return fail(KVC_ERR_INVALID_ARG, "kvc_set_tuning: unknown key '%s'", key);
  *k->value = value;
  return KVC_OK;
}

int kvc_get_tuning(const char* key, int* value) {
  if (!key || !value) return fail(KVC_ERR_INVALID_ARG, "kvc_get_tuning: null argument");
  Knob* k = find_knob(key);
  if (!k) return fail(KVC_ERR_INVALID_ARG, "kvc_get_tuning: unknown key '%s'", key);
  *value = *k->value;
  return KVC_OK;
}

int kvc_reset_tuning(void) {
  int n = 0;
  Knob* t = knobs(&n);
  for (int i = 0; i < n; ++i) *t[i].value = t[i].initial;
  return KVC_OK;
}

int kvc_tuning_modified(void) {
  int n = 0, changed = 0;
  Knob* t = knobs(&n);
  for (int i = 0; i < n; ++i) changed += *t[i].value != t[i].initial;
  return changed;
}

int64_t kvc_last_launch_info(int what) {
  switch (what) {
    case KVC_LAUNCH_KERNEL: return g_last.kernel;
    case KVC_LAUNCH_VEC_BYTES: return g_last.vec;
    case KVC_LAUNCH_PER_LANE: return g_last.per_lane;
    case KVC_LAUNCH_THREADS: return g_last.threads;
    case KVC_LAUNCH_GRID: return g_last.grid;
    case KVC_LAUNCH_NON_TEMPORAL: return g_last.nt;
    case KVC_LAUNCH_PIPE: return g_last.pipe;
    case KVC_LAUNCH_SWAP_MODE: return g_last_swap_mode;
    default: return KVC_ERR_INVALID_ARG;
  }
}

int kvc_reshape_and_cache_layers(const void* key, const void* value, void* key_cache,
                                 void* value_cache, const void* slot_mapping, int slot_bytes,
                                 int64_t num_tokens, int64_t row_elems, int64_t key_token_stride,
                                 int64_t value_token_stride, int64_t block_size,
                                 int64_t cache_block_stride, int64_t cache_slot_stride,
                                 int64_t num_cache_blocks, int64_t num_layers,
                                 int64_t key_layer_stride, int64_t value_layer_stride,
                                 int64_t cache_layer_stride, int elem_bytes, void* stream) {
  WriteGeom g{num_tokens, row_elems, key_token_stride, value_token_stride, block_size,
              cache_block_stride, cache_slot_stride, num_cache_blocks, num_layers,
              key_layer_stride, value_layer_stride, cache_layer_stride, elem_bytes};
  return run_write("kvc_reshape_and_cache", key, value, key_cache, value_cache, slot_mapping,
                   slot_bytes, nullptr, nullptr, nullptr, nullptr, 0, 0, g, stream);
}

int kvc_reshape_and_cache(const void* key, const void* value, void* key_cache, void* value_cache,
                          const void* slot_mapping, int slot_bytes, int64_t num_tokens,
                          int64_t row_elems, int64_t key_token_stride, int64_t value_token_stride,
                          int64_t block_size, int64_t cache_block_stride, int64_t cache_slot_stride,
                          int64_t num_cache_blocks, int elem_bytes, void* stream) {
  return kvc_reshape_and_cache_layers(key, value, key_cache, value_cache, slot_mapping, slot_bytes,
                                      num_tokens, row_elems, key_token_stride, value_token_stride,
                                      block_size, cache_block_stride, cache_slot_stride,
                                      num_cache_blocks, 1, 0, 0, 0, elem_bytes, stream);
}

int kvc_append_paged_kv_cache_layers(const void* append_key, const void* append_value,
                                     const int32_t* batch_indices, const int32_t* positions,
                                     void* paged_kv_cache, const int32_t* kv_indices,
                                     const int32_t* kv_indptr, const int32_t* kv_last_page_len,
                                     int64_t nnz, int64_t batch_size, int64_t num_kv_indices,
                                     int64_t num_kv_heads, int64_t head_dim, int64_t page_size,
                                     int64_t key_token_stride, int64_t value_token_stride,
                                     int64_t page_stride, int64_t num_pages, int64_t num_layers,
                                     int64_t key_layer_stride, int64_t value_layer_stride,
                                     int64_t cache_layer_stride, int elem_bytes, void* stream) {
  (void)kv_last_page_len;
  if (num_kv_heads < 0 || head_dim < 0 || page_size <= 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_append_paged_kv_cache: bad H/D/page_size");
  const int64_t row = num_kv_heads * head_dim;
  if (nnz > 0 && !batch_indices)
    return fail(KVC_ERR_INVALID_ARG, "kvc_append_paged_kv_cache: null batch_indices");
  if (page_stride < 2 * page_size * row)
    return fail(KVC_ERR_INVALID_ARG, "kvc_append_paged_kv_cache: page_stride %lld < 2*page_size*H*D",
                (long long)page_stride);
  WriteGeom g{nnz, row, key_token_stride, value_token_stride, page_size, page_stride, row,
              num_pages, num_layers, key_layer_stride, value_layer_stride, cache_layer_stride,
              elem_bytes};
  char* vc = paged_kv_cache ? (char*)paged_kv_cache + page_size * row * (int64_t)elem_bytes : nullptr;
  return run_write("kvc_append_paged_kv_cache", append_key, append_value, paged_kv_cache, vc,
                   nullptr, 0, batch_indices, positions, kv_indices, kv_indptr, batch_size,
                   num_kv_indices, g, stream);
}

int kvc_append_paged_kv_cache(const void* append_key, const void* append_value,
                              const int32_t* batch_indices, const int32_t* positions,
                              void* paged_kv_cache, const int32_t* kv_indices,
                              const int32_t* kv_indptr, const int32_t* kv_last_page_len,
                              int64_t nnz, int64_t batch_size, int64_t num_kv_indices,
                              int64_t num_kv_heads, int64_t head_dim, int64_t page_size,
                              int64_t key_token_stride, int64_t value_token_stride,
                              int64_t page_stride, int64_t num_pages, int elem_bytes,
                              void* stream) {
  return kvc_append_paged_kv_cache_layers(append_key, append_value, batch_indices, positions,
                                          paged_kv_cache, kv_indices, kv_indptr, kv_last_page_len,
                                          nnz, batch_size, num_kv_indices, num_kv_heads, head_dim,
                                          page_size, key_token_stride, value_token_stride,
                                          page_stride, num_pages, 1, 0, 0, 0, elem_bytes, stream);
}

// ---- per-step plan of the page-table write ----------------------------------
struct kvc_write_plan {
  const int32_t* batch_indices;
  const int32_t* positions;
  const int32_t* kv_indices;
  const int32_t* kv_indptr;
  const int32_t* kv_last_page_len;
  int64_t nnz, batch_size, num_kv_indices, num_kv_heads, head_dim, page_size;
  int elem_bytes;
  const int64_t* slots;  // resolved by kvc_write_plan_resolve_slots, else null
};

int kvc_write_plan_create(const int32_t* batch_indices, const int32_t* positions,
                          const int32_t* kv_indices, const int32_t* kv_indptr,
                          const int32_t* kv_last_page_len, int64_t nnz, int64_t batch_size,
                          int64_t num_kv_indices, int64_t num_kv_heads, int64_t head_dim,
                          int64_t page_size, int elem_bytes, kvc_write_plan** out) {
  if (!out) return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_create: null out");
  *out = nullptr;
  if (num_kv_heads < 0 || head_dim < 0 || page_size <= 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_create: bad H/D/page_size");
  if (nnz < 0 || batch_size < 0 || num_kv_indices < 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_create: negative size");
  if (nnz > 0 && (!batch_indices || !positions || !kv_indices || !kv_indptr))
    return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_create: null index array");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return fail(KVC_ERR_UNSUPPORTED, "kvc_write_plan_create: elem_bytes=%d (need 1, 2, 4 or 8)", elem_bytes);
  kvc_write_plan* p = new (std::nothrow) kvc_write_plan{
      batch_indices, positions, kv_indices, kv_indptr, kv_last_page_len, nnz, batch_size,
      num_kv_indices, num_kv_heads, head_dim, page_size, elem_bytes, nullptr};
  if (!p) return fail(KVC_ERR_HIP, "kvc_write_plan_create: out of host memory");
  *out = p;
  return KVC_OK;
}

int kvc_write_plan_append(const kvc_write_plan* plan, const void* append_key,
                          const void* append_value, int64_t key_token_stride,
                          int64_t value_token_stride, void* paged_kv_cache, int64_t page_stride,
                          int64_t num_pages, void* stream) {
  if (!plan) return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_append: null plan");
  if (plan->slots) {
    const int64_t row = plan->num_kv_heads * plan->head_dim;
    if (page_stride < 2 * plan->page_size * row)
      return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_append: page_stride %lld < 2*page_size*H*D",
                  (long long)page_stride);
    WriteGeom g{plan->nnz, row, key_token_stride, value_token_stride, plan->page_size, page_stride,
                row, num_pages, 1, 0, 0, 0, plan->elem_bytes};
    char* vc = paged_kv_cache ? (char*)paged_kv_cache + plan->page_size * row * (int64_t)plan->elem_bytes
                              : nullptr;
    return run_write("kvc_write_plan_append", append_key, append_value, paged_kv_cache, vc,
                     plan->slots, 8, nullptr, nullptr, nullptr, nullptr, 0, 0, g, stream);
  }
  return kvc_append_paged_kv_cache(append_key, append_value, plan->batch_indices, plan->positions,
                                   paged_kv_cache, plan->kv_indices, plan->kv_indptr,
                                   plan->kv_last_page_len, plan->nnz, plan->batch_size,
                                   plan->num_kv_indices, plan->num_kv_heads, plan->head_dim,
                                   plan->page_size, key_token_stride, value_token_stride,
                                   page_stride, num_pages, plan->elem_bytes, stream);
}

int kvc_write_plan_resolve_slots(kvc_write_plan* plan, int64_t* slots, void* stream) {
  if (!plan) return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_resolve_slots: null plan");
  const int rc = kvc::launch_resolve_slots("kvc_write_plan_resolve_slots", plan->batch_indices,
                                           plan->positions, plan->kv_indices, plan->kv_indptr,
                                           plan->batch_size, plan->num_kv_indices, plan->page_size,
                                           plan->nnz, slots, (hipStream_t)stream);
  if (rc == KVC_OK && plan->nnz > 0) plan->slots = slots;
  return rc;
}

int kvc_write_plan_set_slots(kvc_write_plan* plan, const int64_t* slots) {
  if (!plan) return fail(KVC_ERR_INVALID_ARG, "kvc_write_plan_set_slots: null plan");
  plan->slots = slots;
  return KVC_OK;
}

int kvc_write_plan_destroy(kvc_write_plan* plan) {
  delete plan;
  return KVC_OK;
}

int kvc_get_seq_lens(const int32_t* kv_indptr, const int32_t* kv_last_page_len, int64_t batch_size,
                     int64_t page_size, int32_t* seq_lens, void* stream) {
  if (batch_size < 0 || page_size <= 0 || page_size > INT32_MAX)
    return fail(KVC_ERR_INVALID_ARG, "kvc_get_seq_lens: batch_size=%lld page_size=%lld",
                (long long)batch_size, (long long)page_size);
  if (batch_size == 0) return KVC_OK;
  if (!kv_indptr || !kv_last_page_len || !seq_lens)
    return fail(KVC_ERR_INVALID_ARG, "kvc_get_seq_lens: null pointer");
  const unsigned grid = (unsigned)((batch_size + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(seq_lens_kernel, dim3(grid), dim3(kThreads), 0, (hipStream_t)stream, kv_indptr,
                     kv_last_page_len, batch_size, (int32_t)page_size, seq_lens);
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}

int kvc_get_batch_indices_positions(const int32_t* append_indptr, const int32_t* seq_lens,
                                    int64_t batch_size, int64_t nnz, int32_t* batch_indices,
                                    int32_t* positions, void* stream) {
  if (batch_size < 0 || nnz < 0 || batch_size > 0x7fffffffll)
    return fail(KVC_ERR_INVALID_ARG, "kvc_get_batch_indices_positions: batch_size=%lld nnz=%lld",
                (long long)batch_size, (long long)nnz);
  if (batch_size == 0 || nnz == 0) return KVC_OK;
  if (!append_indptr || !seq_lens || !batch_indices || !positions)
    return fail(KVC_ERR_INVALID_ARG, "kvc_get_batch_indices_positions: null pointer");
  hipLaunchKernelGGL(batch_indices_positions_kernel, dim3((unsigned)batch_size), dim3(kThreads), 0,
                     (hipStream_t)stream, append_indptr, seq_lens, nnz, batch_indices, positions);
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}

int kvc_build_write_index(const int32_t* input_lens, const int32_t* context_lens,
                          const int32_t* num_blocks, const int32_t* kv_indices, int64_t batch_size,
                          int64_t num_kv_indices, int64_t page_size, int64_t nnz,
                          int32_t* cu_seqlens_q, int32_t* kv_indptr, int32_t* kv_last_page_len,
                          int32_t* batch_indices, int32_t* positions, int64_t* slot_mapping,
                          int32_t* run_indptr, int32_t* runs, int32_t* num_runs, int64_t max_runs,
                          void* stream) {
  if (batch_size < 0 || nnz < 0 || num_kv_indices < 0 || page_size <= 0 ||
      batch_size > 0x7fffffffll || page_size > 0x7fffffffll || nnz > 0x7fffffffll)
    return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: batch_size=%lld nnz=%lld page_size=%lld",
                (long long)batch_size, (long long)nnz, (long long)page_size);
  if (!cu_seqlens_q || !kv_indptr)
    return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: null prefix-sum output");
  if (batch_size > 0 && (!input_lens || !context_lens || !num_blocks || !kv_last_page_len))
    return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: null per-request array");
  if (nnz > 0 && (!batch_indices || !positions))
    return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: null per-token output");
  if (slot_mapping && num_kv_indices > 0 && !kv_indices)
    return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: null kv_indices");
  if (runs) {
    if (!run_indptr || !num_runs)
      return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: runs need run_indptr and num_runs");
    if ((uintptr_t)runs % 16)
      return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: the run list must be 16-byte aligned");
    // nnz tokens over batch_size requests form at most nnz / page_size + 2 * batch_size runs
    const int64_t bound = nnz / page_size + 2 * batch_size;
    if (max_runs < std::min(bound, nnz))
      return fail(KVC_ERR_INVALID_ARG, "kvc_build_write_index: max_runs=%lld cannot hold the %lld runs "
                  "%lld tokens of %lld requests may form", (long long)max_runs,
                  (long long)std::min(bound, nnz), (long long)nnz, (long long)batch_size);
  } else {
    run_indptr = nullptr;
    num_runs = nullptr;
    max_runs = 0;
  }
  hipLaunchKernelGGL(build_write_index_kernel, dim3(1), dim3(kPrepThreads), 0, (hipStream_t)stream,
                     input_lens, context_lens, num_blocks, kv_indices, (int32_t)batch_size,
                     num_kv_indices, (int32_t)page_size, nnz, cu_seqlens_q, kv_indptr,
                     kv_last_page_len, batch_indices, positions, slot_mapping, run_indptr, runs,
                     num_runs, max_runs);
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}

int kvc_streams_share_hw_queue(void* stream_x, void* stream_y, int* shared) {
  const char* fn = "kvc_streams_share_hw_queue";
  if (!shared) return fail(KVC_ERR_INVALID_ARG, "%s: null result pointer", fn);
  *shared = 1;
  hipStream_t x = (hipStream_t)stream_x, y = (hipStream_t)stream_y;
  if (x == y) return KVC_OK;
  for (hipStream_t s : {x, y}) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    KVC_HIP(hipStreamIsCapturing(s, &capturing));
    if (capturing != hipStreamCaptureStatusNone)
      return fail(KVC_ERR_INVALID_ARG, "%s: a stream is being captured", fn);
  }
  // first use of a stream creates or attaches its hardware queue: keep that out of the timing
  hipLaunchKernelGGL(touch_queue_kernel, dim3(1), dim3(64), 0, x);
  hipLaunchKernelGGL(touch_queue_kernel, dim3(1), dim3(64), 0, y);
  KVC_HIP(hipGetLastError());
  KVC_HIP(hipStreamSynchronize(x));
  KVC_HIP(hipStreamSynchronize(y));
  hipEvent_t ex = nullptr, ey = nullptr;
  KVC_HIP(hipEventCreateWithFlags(&ex, hipEventDisableTiming));
  if (hipEventCreateWithFlags(&ey, hipEventDisableTiming) != hipSuccess) {
    (void)hipEventDestroy(ex);
    return fail(KVC_ERR_HIP, "%s: hipEventCreateWithFlags failed", fn);
  }
  // x is held for 200 us; y's empty kernel takes about 10 us from launch to done unless
  // it sits behind x's in the same hardware queue. A host thread that loses the
  // processor for the whole hold would see both done at once: three rounds, and the
  // streams count as sharing only if every round says so.
  int rc = KVC_OK;
  int blocked_rounds = 0;
  constexpr int kRounds = 3;
  for (int round = 0; round < kRounds && rc == KVC_OK; ++round) {
    hipLaunchKernelGGL(hold_queue_kernel, dim3(1), dim3(64), 0, x, (uint64_t)20000, (uint32_t)4000);
    hipError_t e = hipEventRecord(ex, x);
    if (e == hipSuccess) {
      hipLaunchKernelGGL(touch_queue_kernel, dim3(1), dim3(64), 0, y);
      e = hipEventRecord(ey, y);
    }
    bool blocked = false;
    if (e == hipSuccess) {
      for (;;) {
        const hipError_t qx = hipEventQuery(ex);   // x first: "y done, x not" proves y was not held up
        const hipError_t qy = hipEventQuery(ey);
        if ((qx != hipSuccess && qx != hipErrorNotReady) || (qy != hipSuccess && qy != hipErrorNotReady)) {
          e = qx != hipSuccess && qx != hipErrorNotReady ? qx : qy;
          break;
        }
        if (qy == hipSuccess) {
          blocked = qx == hipSuccess;
          break;
        }
      }
    }
    const hipError_t sx = hipStreamSynchronize(x), sy = hipStreamSynchronize(y);
    if (e == hipSuccess) e = sx != hipSuccess ? sx : sy;
    if (e != hipSuccess) rc = fail(KVC_ERR_HIP, "%s: %s", fn, hipGetErrorString(e));
    if (!blocked) break;
    ++blocked_rounds;
  }
  (void)hipEventDestroy(ex);
  (void)hipEventDestroy(ey);
  if (rc != KVC_OK) return rc;
  *shared = blocked_rounds == kRounds ? 1 : 0;
  return KVC_OK;
}

int kvc_slot_runs(const void* slot_mapping, int slot_bytes, int64_t num_tokens, int64_t block_size,
                  int32_t* runs, int32_t* num_runs, int64_t max_runs, void* stream) {
  if (num_tokens < 0 || block_size <= 0 || max_runs < 0 || num_tokens > 0x7fffffffll)
    return fail(KVC_ERR_INVALID_ARG, "kvc_slot_runs: num_tokens=%lld block_size=%lld max_runs=%lld",
                (long long)num_tokens, (long long)block_size, (long long)max_runs);
  if (slot_bytes != 4 && slot_bytes != 8)
    return fail(KVC_ERR_UNSUPPORTED, "kvc_slot_runs: slot_bytes=%d (need 4 or 8)", slot_bytes);
  if (!num_runs || (max_runs > 0 && !runs) || (num_tokens > 0 && !slot_mapping))
    return fail(KVC_ERR_INVALID_ARG, "kvc_slot_runs: null pointer");
  if ((uintptr_t)runs % 16)
    return fail(KVC_ERR_INVALID_ARG, "kvc_slot_runs: the run list must be 16-byte aligned");
  if (max_runs < num_tokens)
    return fail(KVC_ERR_INVALID_ARG, "kvc_slot_runs: max_runs=%lld cannot hold the %lld runs that many "
                "tokens may form", (long long)max_runs, (long long)num_tokens);
  hipLaunchKernelGGL(slot_runs_kernel, dim3(1), dim3(kPrepThreads), 0, (hipStream_t)stream,
                     slot_mapping, slot_bytes, num_tokens, block_size, runs, num_runs, max_runs);
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}

int kvc_write_runs_layers(const void* key, const void* value, void* key_cache, void* value_cache,
                          const int32_t* runs, const int32_t* num_runs, int64_t max_runs,
                          int64_t num_tokens, int64_t row_elems, int64_t key_token_stride,
                          int64_t value_token_stride, int64_t block_size, int64_t cache_block_stride,
                          int64_t cache_slot_stride, int64_t num_cache_blocks, int64_t num_layers,
                          int64_t key_layer_stride, int64_t value_layer_stride,
                          int64_t cache_layer_stride, int elem_bytes, void* stream) {
  WriteGeom g{num_tokens, row_elems, key_token_stride, value_token_stride, block_size,
              cache_block_stride, cache_slot_stride, num_cache_blocks, num_layers,
              key_layer_stride, value_layer_stride, cache_layer_stride, elem_bytes};
  return run_write_runs("kvc_write_runs_layers", key, value, key_cache, value_cache, runs, num_runs,
                        max_runs, g, stream);
}

int kvc_copy_blocks(void* kv_caches, const int64_t* block_maps, int64_t num_pairs,
                    int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                    int64_t num_blocks, void* stream) {
  if (num_pairs < 0 || num_layers < 0 || block_bytes < 0 || num_blocks < 0 || layer_stride_bytes < 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_copy_blocks: negative size");
  if (num_pairs == 0 || num_layers == 0 || block_bytes == 0) return KVC_OK;
  if (!kv_caches || !block_maps) return fail(KVC_ERR_INVALID_ARG, "kvc_copy_blocks: null pointer");
  if (layer_stride_bytes < block_bytes)
    return fail(KVC_ERR_INVALID_ARG, "kvc_copy_blocks: layer stride %lld < block bytes %lld",
                (long long)layer_stride_bytes, (long long)block_bytes);
  if (num_layers > 0xffffffffll) return fail(KVC_ERR_UNSUPPORTED, "kvc_copy_blocks: too many layers");
  TileArgs t{};
  t.src_base = (const char*)kv_caches;
  t.dst_base = (char*)kv_caches;
  t.src_ids = block_maps;
  t.dst_ids = block_maps + 1;
  t.id_stride = 2;
  t.src_layer_stride = t.dst_layer_stride = layer_stride_bytes;
  t.src_block_stride = t.dst_block_stride = block_bytes;
  t.num_src_blocks = t.num_dst_blocks = num_blocks;
  t.tile_bytes = block_bytes;
  t.num_layers = (uint32_t)num_layers;
  return launch_tiles(t, num_pairs, g_tune.copy_max_wgs, (hipStream_t)stream);
}

// device-to-device gather / scatter between pool blocks and a dense buffer in
// host-pool layout [n, layer_end-layer_begin, block]
static int run_gather_scatter(const char* fn, bool gather, char* pool, char* buffer,
                              const int64_t* block_ids, int64_t n, int64_t num_layers,
                              int64_t layer_stride_bytes, int64_t block_bytes,
                              int64_t num_blocks, int64_t layer_begin, int64_t layer_end,
                              void* stream) {
  if (n < 0 || num_layers < 0 || block_bytes < 0 || layer_stride_bytes < 0 || num_blocks < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: negative size", fn);
  if (layer_begin < 0 || layer_end < layer_begin || layer_end > num_layers)
    return fail(KVC_ERR_INVALID_ARG, "%s: layer range [%lld, %lld) outside [0, %lld)", fn,
                (long long)layer_begin, (long long)layer_end, (long long)num_layers);
  const int64_t nl = layer_end - layer_begin;
  if (n == 0 || nl == 0 || block_bytes == 0) return KVC_OK;
  if (!pool || !buffer || !block_ids) return fail(KVC_ERR_INVALID_ARG, "%s: null pointer", fn);
  if (layer_stride_bytes < block_bytes)
    return fail(KVC_ERR_INVALID_ARG, "%s: layer stride smaller than a block", fn);
  if (nl > 0xffffffffll) return fail(KVC_ERR_UNSUPPORTED, "%s: too many layers", fn);
  TileArgs t{};
  t.id_stride = 1;
  t.tile_bytes = block_bytes;
  t.num_layers = (uint32_t)nl;
  char* pool_l0 = pool + layer_begin * layer_stride_bytes;
  if (gather) {
    t.src_base = pool_l0; t.src_ids = block_ids;
    t.src_layer_stride = layer_stride_bytes; t.src_block_stride = block_bytes;
    t.num_src_blocks = num_blocks;
    t.dst_base = buffer; t.dst_ids = nullptr;
    t.dst_layer_stride = block_bytes; t.dst_block_stride = nl * block_bytes;
    t.num_dst_blocks = n;
  } else {
    t.src_base = buffer; t.src_ids = nullptr;
    t.src_layer_stride = block_bytes; t.src_block_stride = nl * block_bytes;
    t.num_src_blocks = n;
    t.dst_base = pool_l0; t.dst_ids = block_ids;
    t.dst_layer_stride = layer_stride_bytes; t.dst_block_stride = block_bytes;
    t.num_dst_blocks = num_blocks;
  }
  return launch_tiles(t, n, g_tune.copy_max_wgs, (hipStream_t)stream, gather);
}

int kvc_gather_blocks(const void* pool, void* buffer, const int64_t* block_ids, int64_t n,
                      int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                      int64_t num_blocks, int64_t layer_begin, int64_t layer_end, void* stream) {
  return run_gather_scatter("kvc_gather_blocks", true, (char*)pool, (char*)buffer, block_ids, n,
                            num_layers, layer_stride_bytes, block_bytes, num_blocks, layer_begin,
                            layer_end, stream);
}

int kvc_scatter_blocks(void* pool, const void* buffer, const int64_t* block_ids, int64_t n,
                       int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                       int64_t num_blocks, int64_t layer_begin, int64_t layer_end, void* stream) {
  return run_gather_scatter("kvc_scatter_blocks", false, (char*)pool, (char*)buffer, block_ids, n,
                            num_layers, layer_stride_bytes, block_bytes, num_blocks, layer_begin,
                            layer_end, stream);
}

int64_t kvc_swap_staging_bytes(int64_t n, int64_t num_layers_in_range, int64_t block_bytes,
                               int mode, int64_t chunk_blocks) {
  if (n < 0 || num_layers_in_range < 0 || block_bytes < 0) return KVC_ERR_INVALID_ARG;
  const int64_t ids = std::max<int64_t>(ids_region_bytes(n), kIdAlign);
  if (mode != KVC_SWAP_STAGED && mode != KVC_SWAP_AUTO && mode != KVC_SWAP_DIRECT)
    return KVC_ERR_INVALID_ARG;
  if (mode == KVC_SWAP_DIRECT || n == 0) return ids;
  const int64_t per_block = round_up(num_layers_in_range * block_bytes, kIdAlign);
  if (per_block == 0) return ids;
  if (chunk_blocks <= 0) {
    // default ring slot: about 64 MiB, large enough for the DMA engines to run
    // at link rate and small next to HBM; larger when the call would otherwise
    // take more than 128 chunks (a call of several hundred chunks, each a
    // kernel, a copy and four event operations across two streams, falls to
    // half the link rate at 340 chunks and a quarter at 680)
    chunk_blocks = std::max<int64_t>(1, (int64_t(64) << 20) / per_block);
    chunk_blocks = std::max<int64_t>(chunk_blocks, (n + 127) / 128);
  }
  chunk_blocks = std::min(chunk_blocks, n);
  return ids + 2 * per_block * chunk_blocks;
}

int kvc_swap_out(const void* pool, void* host_pool, const int64_t* src_ids, const int64_t* dst_ids,
                 int64_t n, int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                 int64_t num_gpu_blocks, int64_t num_host_blocks, int64_t layer_begin,
                 int64_t layer_end, void* staging, int64_t staging_bytes, int mode,
                 void* kernel_stream, void* copy_stream) {
  SwapGeom g{n, num_layers, layer_stride_bytes, block_bytes, num_gpu_blocks, num_host_blocks,
             layer_begin, layer_end};
  return run_swap("kvc_swap_out", true, (char*)pool, (char*)host_pool, src_ids, dst_ids, g,
                  staging, staging_bytes, mode, false, kernel_stream, copy_stream);
}

int kvc_swap_in(void* pool, const void* host_pool, const int64_t* src_ids, const int64_t* dst_ids,
                int64_t n, int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                int64_t num_gpu_blocks, int64_t num_host_blocks, int64_t layer_begin,
                int64_t layer_end, void* staging, int64_t staging_bytes, int mode,
                void* kernel_stream, void* copy_stream) {
  SwapGeom g{n, num_layers, layer_stride_bytes, block_bytes, num_gpu_blocks, num_host_blocks,
             layer_begin, layer_end};
  return run_swap("kvc_swap_in", false, (char*)pool, (char*)host_pool, dst_ids, src_ids, g, staging,
                  staging_bytes, mode, false, kernel_stream, copy_stream);
}

int kvc_swap_resolve_mode(const int64_t* host_ids, int64_t n, int64_t num_layers_in_range,
                          int64_t block_bytes, int64_t staging_bytes) {
  if (n < 0 || num_layers_in_range < 0 || block_bytes < 0 || staging_bytes < 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_swap_resolve_mode: negative size");
  const SwapGeom g{n, num_layers_in_range, 0, block_bytes, 0, 0, 0, num_layers_in_range};
  static const char some_staging = 0;   // only its presence is looked at
  return resolve_auto_mode(host_ids, g, staging_bytes > 0 ? &some_staging : nullptr, staging_bytes);
}

int kvc_swap_last_mode(void) { return g_last_swap_mode; }

int kvc_order_pairs_by_host_id(int64_t* gpu_ids, int64_t* host_ids, int64_t n) {
  if (n < 0) return fail(KVC_ERR_INVALID_ARG, "kvc_order_pairs_by_host_id: negative size");
  if (n > 0 && (!gpu_ids || !host_ids))
    return fail(KVC_ERR_INVALID_ARG, "kvc_order_pairs_by_host_id: null id list");
  return order_pairs_by_host_id(gpu_ids, host_ids, n);
}

int kvc_swap_prepare(const int64_t* gpu_ids, const int64_t* host_ids, int64_t n,
                     int64_t num_gpu_blocks, int64_t num_host_blocks, void* staging,
                     int64_t staging_bytes, void* stream) {
  if (n < 0 || num_gpu_blocks < 0 || num_host_blocks < 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_swap_prepare: negative size");
  if (n == 0) return KVC_OK;
  if (!gpu_ids || !host_ids) return fail(KVC_ERR_INVALID_ARG, "kvc_swap_prepare: null id list");
  int rc = check_ids("kvc_swap_prepare", gpu_ids, host_ids, n, num_gpu_blocks, num_host_blocks);
  if (rc != KVC_OK) return rc;
  if (!staging) return fail(KVC_ERR_STAGING, "kvc_swap_prepare: null staging buffer");
  if ((uintptr_t)staging % kIdAlign)
    return fail(KVC_ERR_STAGING, "kvc_swap_prepare: staging buffer must be %lld-byte aligned",
                (long long)kIdAlign);
  if (staging_bytes < ids_region_bytes(n))
    return fail(KVC_ERR_STAGING, "kvc_swap_prepare: staging of %lld bytes cannot hold the id lists (%lld)",
                (long long)staging_bytes, (long long)ids_region_bytes(n));
  rc = swap_ctx_prepare();
  if (rc != KVC_OK) return rc;
  return upload_ids(gpu_ids, host_ids, n, staging, (hipStream_t)stream);
}

int kvc_swap_out_prepared(const void* pool, void* host_pool, const int64_t* host_ids, int64_t n,
                          int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                          int64_t num_gpu_blocks, int64_t num_host_blocks, int64_t layer_begin,
                          int64_t layer_end, void* staging, int64_t staging_bytes, int mode,
                          void* kernel_stream, void* copy_stream) {
  SwapGeom g{n, num_layers, layer_stride_bytes, block_bytes, num_gpu_blocks, num_host_blocks,
             layer_begin, layer_end};
  return run_swap("kvc_swap_out_prepared", true, (char*)pool, (char*)host_pool, nullptr, host_ids, g,
                  staging, staging_bytes, mode, true, kernel_stream, copy_stream);
}

int kvc_swap_in_prepared(void* pool, const void* host_pool, const int64_t* host_ids, int64_t n,
                         int64_t num_layers, int64_t layer_stride_bytes, int64_t block_bytes,
                         int64_t num_gpu_blocks, int64_t num_host_blocks, int64_t layer_begin,
                         int64_t layer_end, void* staging, int64_t staging_bytes, int mode,
                         void* kernel_stream, void* copy_stream) {
  SwapGeom g{n, num_layers, layer_stride_bytes, block_bytes, num_gpu_blocks, num_host_blocks,
             layer_begin, layer_end};
  return run_swap("kvc_swap_in_prepared", false, (char*)pool, (char*)host_pool, nullptr, host_ids, g,
                  staging, staging_bytes, mode, true, kernel_stream, copy_stream);
}

int kvc_thread_release(void) { return swap_ctx_release(); }

int kvc_swap_noalloc(int to_host, void* pool, void* host_pool, const int64_t* gpu_ids,
                     const int64_t* host_ids, int64_t n, int64_t num_layers,
                     int64_t layer_stride_bytes, int64_t block_bytes, int64_t num_gpu_blocks,
                     int64_t num_host_blocks, int64_t layer_begin, int64_t layer_end, void* stream) {
  const char* fn = "kvc_swap_noalloc";
  if (n < 0 || num_layers < 0 || block_bytes < 0 || layer_stride_bytes < 0 || num_gpu_blocks < 0 ||
      num_host_blocks < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: negative size", fn);
  if (layer_begin < 0 || layer_end < layer_begin || layer_end > num_layers)
    return fail(KVC_ERR_INVALID_ARG, "%s: layer range [%lld, %lld) outside [0, %lld)", fn,
                (long long)layer_begin, (long long)layer_end, (long long)num_layers);
  if (n > KVC_NOALLOC_MAX_BLOCKS)
    return fail(KVC_ERR_UNSUPPORTED, "%s: %lld blocks exceed the %d this entry point holds ids for "
                "(use kvc_swap_out / kvc_swap_in with a workspace)", fn, (long long)n,
                KVC_NOALLOC_MAX_BLOCKS);
  const int64_t nl = layer_end - layer_begin;
  if (n == 0 || nl == 0 || block_bytes == 0) return KVC_OK;
  if (!pool || !host_pool || !gpu_ids || !host_ids)
    return fail(KVC_ERR_INVALID_ARG, "%s: null pool/host/id pointer", fn);
  if (layer_stride_bytes < block_bytes)
    return fail(KVC_ERR_INVALID_ARG, "%s: layer stride smaller than a block", fn);
  if (nl > 0xffffffffll) return fail(KVC_ERR_UNSUPPORTED, "%s: too many layers", fn);
  if (num_gpu_blocks > INT32_MAX || num_host_blocks > INT32_MAX)
    return fail(KVC_ERR_UNSUPPORTED, "%s: block ids beyond 31 bits", fn);
  int rc = check_ids(fn, gpu_ids, host_ids, n, num_gpu_blocks, num_host_blocks);
  if (rc != KVC_OK) return rc;
  int64_t* ids = nullptr;  // device address of the static id array on this device
  rc = scratch_of_current_device(&ids);
  if (rc != KVC_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  IdPacket packet;
  for (int64_t first = 0; first < n; first += kIdsPerPacket) {
    const int count = (int)std::min<int64_t>(kIdsPerPacket, n - first);
    for (int i = 0; i < count; ++i) {
      packet.gpu[i] = (int32_t)gpu_ids[first + i];
      packet.host[i] = (int32_t)host_ids[first + i];
    }
    hipLaunchKernelGGL(stage_ids_kernel, dim3(1), dim3((count + 63) / 64 * 64), 0, s, packet, ids, first,
                       count, n);
    KVC_HIP(hipGetLastError());
  }
  const SwapGeom g{n, num_layers, layer_stride_bytes, block_bytes, num_gpu_blocks, num_host_blocks,
                   layer_begin, layer_end};
  const TileArgs t = direct_swap_tiles(to_host != 0, (char*)pool, (char*)host_pool, ids, ids + n, g);
  return launch_tiles(t, n, direct_wgs(to_host != 0), s);
}

void* kvc_host_alloc_pinned(size_t bytes) {
  void* p = nullptr;
  if (bytes == 0) bytes = 1;
  hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocDefault);
  if (e != hipSuccess) {
    fail(KVC_ERR_HIP, "hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    return nullptr;
  }
  return p;
}

int kvc_host_free_pinned(void* ptr) {
  if (!ptr) return KVC_OK;
  KVC_HIP(hipHostFree(ptr));
  return KVC_OK;
}

}  // extern "C"

// Rotary position embedding fused with the K/V write (gfx950).
//
// In the reference's attention layer the rotation of Q and K runs as its own
// launch immediately before the cache write, on the same K tensor. Here a
// workgroup owns a run of 16-byte work items of ONE token (so position, cos/sin
// row and cache slot are workgroup-uniform): it stages the token's cos/sin row
// in LDS as fp32, rotates Q and K in fp32 with a single rounding to the storage
// type, and, when a cache is given, stores the rotated K and the V row straight
// into the token's slot. K is read once and V never takes a separate launch.
// Without a cache the kernel is the plain rotation.
//
// Vectors are 16 bytes (8 bf16/fp16 or 4 fp32 elements); a "pair-vector" is the
// x half and the y half of the same rotation lanes of one head.

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <new>

#include "common.h"
#include "kvcache.h"

namespace kvc {
RopeTuning g_rope_tune;
}

namespace {

using kvc::fail;
using kvc::log2_exact;

constexpr int kThreads = 256;
constexpr int kMaxRotaryDim = 512;  // cos + sin of one position in LDS as fp32: 4 KiB

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---- storage types ---------------------------------------------------------
struct BF16 {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float load(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
  // Round to nearest, ties to even, through the native conversion: gfx950 has a
  // packed f32 -> bf16 convert instruction, which the compiler selects for this.
  static __device__ __forceinline__ uint16_t store(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
  }
  static __device__ __forceinline__ uint32_t store2(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
};
struct F16 {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float load(uint16_t b) { return __half2float(__ushort_as_half(b)); }
  static __device__ __forceinline__ uint16_t store(float f) { return __half_as_ushort(__float2half_rn(f)); }
  static __device__ __forceinline__ uint32_t store2(float lo, float hi) {
    return (uint32_t)store(lo) | ((uint32_t)store(hi) << 16);
  }
};
struct F32 {
  static constexpr int kBytes = 4;
};

// unpack / pack one 16-byte vector to fp32 lanes
template <typename T>
struct Vec {
  static constexpr int kElems = 16 / T::kBytes;
  static __device__ __forceinline__ void unpack(u32x4 v, float* out) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = T::load((uint16_t)(v[i] & 0xffffu));
      out[2 * i + 1] = T::load((uint16_t)(v[i] >> 16));
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float* in) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      v[i] = T::store2(in[2 * i], in[2 * i + 1]);
    return v;
  }
  static __device__ __forceinline__ float load1(const char* p) { return T::load(*(const uint16_t*)p); }
  static __device__ __forceinline__ void store1(char* p, float f) { *(uint16_t*)p = T::store(f); }
};
template <>
struct Vec<F32> {
  static constexpr int kElems = 4;
  static __device__ __forceinline__ void unpack(u32x4 v, float* out) {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = __uint_as_float(v[i]);
  }
  static __device__ __forceinline__ u32x4 pack(const float* in) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(in[i]);
    return v;
  }
  static __device__ __forceinline__ float load1(const char* p) { return *(const float*)p; }
  static __device__ __forceinline__ void store1(char* p, float f) { *(float*)p = f; }
};

struct RopeArgs {
  const char* query;
  const char* key;
  const char* value;       // null without a cache
  char* query_out;
  char* key_out;           // may be null when a cache takes the rotated K
  const void* positions;   // rotation positions; with page-table addressing also the KV positions
  int pos_bytes;
  const char* cos_sin_cache;  // [max_position, 2*rotary_dim]: cos | sin
  int64_t max_position;
  uint32_t num_heads, num_kv_heads, head_dim, rotary_dim;
  int64_t q_token_stride, k_token_stride, v_token_stride;     // bytes
  int64_t qo_token_stride, ko_token_stride;                   // bytes
  // cache side (key_cache == null: plain rotation)
  char* key_cache;
  char* value_cache;
  const void* slot_mapping;
  int slot_bytes;
  const int32_t* batch_indices;  // non-null: page-table addressing
  const int32_t* kv_indices;
  const int32_t* kv_indptr;
  int64_t batch_size, num_kv_indices;
  int64_t block_size;
  int bs_shift;
  int64_t cache_block_stride, cache_slot_stride;  // bytes
  int64_t num_cache_blocks;
  uint32_t groups_per_token;  // workgroups per token
  int pv_shift;               // log2(pair-vectors per head) or -1
  int cs_vector;              // cos/sin rows are 16-byte aligned runs of whole vectors
};

// Work items of one token, in this order: rotation pair-vectors of the Q heads
// then the K heads, pass-through vectors beyond rotary_dim, V vectors. A
// workgroup takes IPL * blockDim.x consecutive items of one token, IPL per lane
// (item = first + j * blockDim.x, so the lanes of a wavefront stay on
// consecutive vectors): all of the lane's global loads are issued first, the
// cos/sin row is staged in LDS while they are in flight, then the lane computes
// and stores.
template <bool NT>
__device__ __forceinline__ u32x4 ld16(const char* p) {
  if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  else return *reinterpret_cast<const u32x4*>(p);
}

// NTL: non-temporal loads, bit 0 for the K and V rows, bit 1 for the Q rows.
template <typename T, bool VECTOR, int IPL, int NTL>
__global__ __launch_bounds__(kThreads) void rope_cache_kernel(RopeArgs a) {
  using VT = Vec<T>;
  constexpr int EV = VECTOR ? VT::kElems : 1;
  constexpr int E = T::kBytes;
  __shared__ float cs[2 * kMaxRotaryDim];  // cos[0, rd) | sin[0, rd)

  const uint32_t t = blockIdx.x / a.groups_per_token;
  const uint32_t group = blockIdx.x - t * a.groups_per_token;
  const int64_t pos = a.pos_bytes == 8 ? reinterpret_cast<const int64_t*>(a.positions)[t]
                                       : (int64_t) reinterpret_cast<const int32_t*>(a.positions)[t];
  if (pos < 0 || pos >= a.max_position) return;  // no cos/sin row: the token is left alone
  const uint32_t rd = a.rotary_dim;
  const uint32_t half = rd >> 1;
  const uint32_t D = a.head_dim;
  const uint32_t heads = a.num_heads + a.num_kv_heads;
  const uint32_t pv_per_head = half / EV;
  const uint32_t rot_items = heads * pv_per_head;
  const uint32_t tail_per_head = (D - rd) / EV;
  const uint32_t tail_items = heads * tail_per_head;
  const uint32_t v_items = a.key_cache ? a.num_kv_heads * D / EV : 0;

  // ---- this lane's items and their loads ----
  enum : int { kNone, kRotate, kTail, kValue };
  int kind[IPL];
  bool is_k[IPL];
  uint32_t e0[IPL];     // first lane inside the head (rotation / tail)
  int64_t in_off[IPL];  // byte offset of the item inside its source row == inside its out row
  u32x4 rx[IPL], ry[IPL];  // 16-byte path: x half and y half (or the one pass-through vector)
  float sx[IPL], sy[IPL];  // element path
  const uint32_t first = group * (IPL * blockDim.x) + threadIdx.x;
#pragma unroll
  for (int j = 0; j < IPL; ++j) {
    const uint32_t item = first + j * blockDim.x;
    kind[j] = kNone;
    is_k[j] = false;
    e0[j] = 0;
    in_off[j] = 0;
    sx[j] = sy[j] = 0.f;
    if (item < rot_items) {
      kind[j] = kRotate;
      const uint32_t h = a.pv_shift >= 0 ? item >> a.pv_shift : item / pv_per_head;
      e0[j] = (item - h * pv_per_head) * EV;
      is_k[j] = h >= a.num_heads;
      const uint32_t hh = is_k[j] ? h - a.num_heads : h;
      in_off[j] = (int64_t)hh * D * E;
      const char* in = (is_k[j] ? a.key + (int64_t)t * a.k_token_stride
                                : a.query + (int64_t)t * a.q_token_stride) + in_off[j];
      if constexpr (VECTOR) {
        if (is_k[j]) {
          rx[j] = ld16<(NTL & 1) != 0>(in + (int64_t)e0[j] * E);
          ry[j] = ld16<(NTL & 1) != 0>(in + (int64_t)(half + e0[j]) * E);
        } else {
          rx[j] = ld16<(NTL & 2) != 0>(in + (int64_t)e0[j] * E);
          ry[j] = ld16<(NTL & 2) != 0>(in + (int64_t)(half + e0[j]) * E);
        }
      } else {
        sx[j] = VT::load1(in + (int64_t)e0[j] * E);
        sy[j] = VT::load1(in + (int64_t)(half + e0[j]) * E);
      }
    } else if (item < rot_items + tail_items) {
      kind[j] = kTail;
      const uint32_t it = item - rot_items;
      const uint32_t h = it / tail_per_head;
      e0[j] = rd + (it - h * tail_per_head) * EV;
      is_k[j] = h >= a.num_heads;
      const uint32_t hh = is_k[j] ? h - a.num_heads : h;
      in_off[j] = ((int64_t)hh * D + e0[j]) * E;
      const char* in = (is_k[j] ? a.key + (int64_t)t * a.k_token_stride
                                : a.query + (int64_t)t * a.q_token_stride) + in_off[j];
      if constexpr (VECTOR) rx[j] = is_k[j] ? ld16<(NTL & 1) != 0>(in) : ld16<(NTL & 2) != 0>(in);
      else sx[j] = VT::load1(in);
    } else if (item < rot_items + tail_items + v_items) {
      kind[j] = kValue;
      in_off[j] = (int64_t)(item - rot_items - tail_items) * EV * E;
      const char* in = a.value + (int64_t)t * a.v_token_stride + in_off[j];
      if constexpr (VECTOR) rx[j] = ld16<(NTL & 1) != 0>(in);
      else sx[j] = VT::load1(in);
    }
  }

  // ---- cos/sin row of this position: issue the loads (first vector of each lane) ----
  const char* cs_row = a.cos_sin_cache + pos * (int64_t)(2 * rd) * E;
  constexpr int CV = VT::kElems;  // whole 16-byte vectors when the row is aligned and a multiple of them
  const uint32_t cs_vecs = 2 * rd / CV;
  u32x4 cs_first = {0, 0, 0, 0};
  if (a.cs_vector && threadIdx.x < cs_vecs)
    cs_first = *reinterpret_cast<const u32x4*>(cs_row + (int64_t)threadIdx.x * 16);

  // ---- slot of this token (workgroup-uniform) ----
  // Placed after every vector load has been issued and before the first wait on
  // them: the chain of dependent scalar loads runs while they are in flight.
  char* kc_row = nullptr;
  char* vc_row = nullptr;
  if (a.key_cache) {
    int64_t blk = -1, off = 0;
    if (a.batch_indices) {
      const int64_t b = a.batch_indices[t];
      if (b >= 0 && b < a.batch_size) {
        const int64_t pg = a.bs_shift >= 0 ? (pos >> a.bs_shift) : pos / a.block_size;
        off = pos - pg * a.block_size;
        const int64_t it = (int64_t)a.kv_indptr[b] + pg;
        if (it >= 0 && it < (int64_t)a.kv_indptr[b + 1] && it < a.num_kv_indices) blk = a.kv_indices[it];
      }
    } else {
      const int64_t s = a.slot_bytes == 8 ? reinterpret_cast<const int64_t*>(a.slot_mapping)[t]
                                          : (int64_t) reinterpret_cast<const int32_t*>(a.slot_mapping)[t];
      if (s >= 0) {
        blk = a.bs_shift >= 0 ? (s >> a.bs_shift) : s / a.block_size;
        off = s - blk * a.block_size;
      }
    }
    if (blk >= 0 && blk < a.num_cache_blocks) {
      const int64_t slot_off = blk * a.cache_block_stride + off * a.cache_slot_stride;
      kc_row = a.key_cache + slot_off;
      vc_row = a.value_cache + slot_off;
    }
  }
  // ---- cos/sin row into LDS as fp32, shared by all heads ----
  if (a.cs_vector) {
    for (uint32_t i = threadIdx.x; i < cs_vecs; i += blockDim.x) {
      float f[CV];
      VT::unpack(i == threadIdx.x ? cs_first : *reinterpret_cast<const u32x4*>(cs_row + (int64_t)i * 16), f);
#pragma unroll
      for (int e = 0; e < CV; ++e) cs[i * CV + e] = f[e];
    }
  } else {
    for (uint32_t i = threadIdx.x; i < 2 * rd; i += blockDim.x) cs[i] = VT::load1(cs_row + (int64_t)i * E);
  }
  __syncthreads();

  // ---- compute and store ----
  char* qo_row = a.query_out + (int64_t)t * a.qo_token_stride;
  char* ko_row = a.key_out ? a.key_out + (int64_t)t * a.ko_token_stride : nullptr;
#pragma unroll
  for (int j = 0; j < IPL; ++j) {
    // outs[0]: the rotated tensor handed back (read again by attention right away);
    // outs[1]: the cache row of a K item (not read again by this step: non-temporal)
    char* outs[2] = {is_k[j] ? ko_row : qo_row, is_k[j] ? kc_row : nullptr};
    if (kind[j] == kRotate) {
      float x[EV], y[EV], ox[EV], oy[EV];
      if constexpr (VECTOR) {
        VT::unpack(rx[j], x);
        VT::unpack(ry[j], y);
      } else {
        x[0] = sx[j];
        y[0] = sy[j];
      }
#pragma unroll
      for (int i = 0; i < EV; ++i) {
        const float cos_x = cs[e0[j] + i], cos_y = cs[half + e0[j] + i];
        const float sin_x = cs[rd + e0[j] + i], sin_y = cs[rd + half + e0[j] + i];
        ox[i] = x[i] * cos_x - y[i] * sin_x;
        oy[i] = y[i] * cos_y + x[i] * sin_y;
      }
#pragma unroll
      for (int o = 0; o < 2; ++o) {
        if (!outs[o]) continue;
        char* out = outs[o] + in_off[j];
        if constexpr (VECTOR) {
          u32x4* px = reinterpret_cast<u32x4*>(out + (int64_t)e0[j] * E);
          u32x4* py = reinterpret_cast<u32x4*>(out + (int64_t)(half + e0[j]) * E);
          if (o == 1) {
            __builtin_nontemporal_store(VT::pack(ox), px);
            __builtin_nontemporal_store(VT::pack(oy), py);
          } else {
            *px = VT::pack(ox);
            *py = VT::pack(oy);
          }
        } else {
          VT::store1(out + (int64_t)e0[j] * E, ox[0]);
          VT::store1(out + (int64_t)(half + e0[j]) * E, oy[0]);
        }
      }
    } else if (kind[j] == kTail) {
      // lanes beyond rotary_dim pass through unchanged (partial rotary)
#pragma unroll
      for (int o = 0; o < 2; ++o) {
        if (!outs[o]) continue;
        if constexpr (VECTOR) *reinterpret_cast<u32x4*>(outs[o] + in_off[j]) = rx[j];
        else VT::store1(outs[o] + in_off[j], sx[j]);
      }
    } else if (kind[j] == kValue && vc_row) {
      // the V row goes to the cache as it is
      if constexpr (VECTOR) __builtin_nontemporal_store(rx[j], reinterpret_cast<u32x4*>(vc_row + in_off[j]));
      else VT::store1(vc_row + in_off[j], sx[j]);
    }
  }
}

// One item per lane is what runs: 2 and 4 items per lane were measured from
// 6 MiB to 324 MiB per launch and never gained (the launch is either latency-bound
// or already has enough workgroups in flight).
template <typename T, bool VECTOR>
void launch_rope_ipl(const RopeArgs& a, dim3 grid, dim3 block, hipStream_t s) {
  if constexpr (VECTOR) {
    switch (kvc::g_rope_tune.nt & 3) {
      case 1: hipLaunchKernelGGL((rope_cache_kernel<T, true, 1, 1>), grid, block, 0, s, a); break;
      case 2: hipLaunchKernelGGL((rope_cache_kernel<T, true, 1, 2>), grid, block, 0, s, a); break;
      case 3: hipLaunchKernelGGL((rope_cache_kernel<T, true, 1, 3>), grid, block, 0, s, a); break;
      default: hipLaunchKernelGGL((rope_cache_kernel<T, true, 1, 0>), grid, block, 0, s, a); break;
    }
  } else {
    hipLaunchKernelGGL((rope_cache_kernel<T, false, 1, 0>), grid, block, 0, s, a);
  }
}

template <typename T>
void launch_rope(const RopeArgs& a, int64_t num_tokens, bool vector, unsigned threads,
                 hipStream_t s) {
  const dim3 grid((unsigned)(num_tokens * a.groups_per_token)), block(threads);
  if (vector) launch_rope_ipl<T, true>(a, grid, block, s);
  else launch_rope_ipl<T, false>(a, grid, block, s);
}

struct RopeGeom {
  int64_t num_tokens, num_heads, num_kv_heads, head_dim, rotary_dim, max_position;
  int64_t q_token_stride, k_token_stride, v_token_stride, qo_token_stride, ko_token_stride;  // elements
  int dtype;
};

struct CacheGeom {
  void* key_cache;
  void* value_cache;
  const void* slot_mapping;
  int slot_bytes;
  const int32_t* batch_indices;
  const int32_t* kv_indices;
  const int32_t* kv_indptr;
  int64_t batch_size, num_kv_indices;
  int64_t block_size, cache_block_stride, cache_slot_stride, num_cache_blocks;  // strides in elements
};

int run_rope(const char* fn, const void* query, const void* key, const void* value,
             void* query_out, void* key_out, const void* positions, int pos_bytes,
             const void* cos_sin_cache, const RopeGeom& g, const CacheGeom* c, void* stream) {
  int E;
  switch (g.dtype) {
    case KVC_DTYPE_BF16: case KVC_DTYPE_F16: E = 2; break;
    case KVC_DTYPE_F32: E = 4; break;
    default: return fail(KVC_ERR_UNSUPPORTED, "%s: dtype %d (need bf16, f16 or f32)", fn, g.dtype);
  }
  if (g.num_tokens < 0 || g.num_heads < 0 || g.num_kv_heads < 0 || g.head_dim <= 0 ||
      g.rotary_dim < 0 || g.max_position < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: negative size", fn);
  if (g.rotary_dim > g.head_dim || (g.rotary_dim & 1))
    return fail(KVC_ERR_INVALID_ARG, "%s: rotary_dim %lld must be even and <= head_dim %lld", fn,
                (long long)g.rotary_dim, (long long)g.head_dim);
  if (g.rotary_dim > kMaxRotaryDim)
    return fail(KVC_ERR_UNSUPPORTED, "%s: rotary_dim %lld exceeds %d", fn, (long long)g.rotary_dim,
                kMaxRotaryDim);
  if (pos_bytes != 4 && pos_bytes != 8)
    return fail(KVC_ERR_UNSUPPORTED, "%s: pos_bytes=%d (need 4 or 8)", fn, pos_bytes);
  if (g.num_tokens > 0x7fffffffll || g.num_heads + g.num_kv_heads > 0xffffll)
    return fail(KVC_ERR_UNSUPPORTED, "%s: too many tokens or heads", fn);
  if (g.num_tokens == 0 || g.num_heads + g.num_kv_heads == 0) return KVC_OK;
  if (!query || !key || !query_out || !positions || !cos_sin_cache)
    return fail(KVC_ERR_INVALID_ARG, "%s: null pointer", fn);
  if (!c && !key_out) return fail(KVC_ERR_INVALID_ARG, "%s: no destination for the rotated key", fn);
  if (g.q_token_stride < g.num_heads * g.head_dim || g.qo_token_stride < g.num_heads * g.head_dim ||
      g.k_token_stride < g.num_kv_heads * g.head_dim ||
      (key_out && g.ko_token_stride < g.num_kv_heads * g.head_dim))
    return fail(KVC_ERR_INVALID_ARG, "%s: token stride smaller than a row", fn);

  RopeArgs a{};
  a.query = (const char*)query;
  a.key = (const char*)key;
  a.value = (const char*)value;
  a.query_out = (char*)query_out;
  a.key_out = (char*)key_out;
  a.positions = positions;
  a.pos_bytes = pos_bytes;
  a.cos_sin_cache = (const char*)cos_sin_cache;
  a.max_position = g.max_position;
  a.num_heads = (uint32_t)g.num_heads;
  a.num_kv_heads = (uint32_t)g.num_kv_heads;
  a.head_dim = (uint32_t)g.head_dim;
  a.rotary_dim = (uint32_t)g.rotary_dim;
  a.q_token_stride = g.q_token_stride * E;
  a.k_token_stride = g.k_token_stride * E;
  a.v_token_stride = g.v_token_stride * E;
  a.qo_token_stride = g.qo_token_stride * E;
  a.ko_token_stride = g.ko_token_stride * E;

  uint64_t align = (uintptr_t)query | (uintptr_t)key | (uintptr_t)query_out | (uintptr_t)key_out |
                   (uint64_t)a.q_token_stride | (uint64_t)a.k_token_stride |
                   (uint64_t)a.qo_token_stride | (uint64_t)a.ko_token_stride;
  if (c) {
    if (!value || !c->key_cache || !c->value_cache)
      return fail(KVC_ERR_INVALID_ARG, "%s: null value/cache pointer", fn);
    if (g.v_token_stride < g.num_kv_heads * g.head_dim)
      return fail(KVC_ERR_INVALID_ARG, "%s: value token stride smaller than a row", fn);
    if (c->block_size <= 0 || c->num_cache_blocks < 0 || c->cache_block_stride < 0 ||
        c->cache_slot_stride < g.num_kv_heads * g.head_dim)
      return fail(KVC_ERR_INVALID_ARG, "%s: bad cache geometry", fn);
    if (c->batch_indices) {
      if (!c->kv_indices || !c->kv_indptr || c->batch_size < 0 || c->num_kv_indices < 0)
        return fail(KVC_ERR_INVALID_ARG, "%s: bad page-table arguments", fn);
      if (pos_bytes != 4)
        return fail(KVC_ERR_UNSUPPORTED, "%s: page-table addressing takes int32 positions", fn);
    } else {
      if (!c->slot_mapping) return fail(KVC_ERR_INVALID_ARG, "%s: null slot_mapping", fn);
      if (c->slot_bytes != 4 && c->slot_bytes != 8)
        return fail(KVC_ERR_UNSUPPORTED, "%s: slot_bytes=%d (need 4 or 8)", fn, c->slot_bytes);
    }
    a.key_cache = (char*)c->key_cache;
    a.value_cache = (char*)c->value_cache;
    a.slot_mapping = c->slot_mapping;
    a.slot_bytes = c->slot_bytes;
    a.batch_indices = c->batch_indices;
    a.kv_indices = c->kv_indices;
    a.kv_indptr = c->kv_indptr;
    a.batch_size = c->batch_size;
    a.num_kv_indices = c->num_kv_indices;
    a.block_size = c->block_size;
    a.bs_shift = log2_exact(c->block_size);
    a.cache_block_stride = c->cache_block_stride * E;
    a.cache_slot_stride = c->cache_slot_stride * E;
    a.num_cache_blocks = c->num_cache_blocks;
    align |= (uintptr_t)value | (uintptr_t)c->key_cache | (uintptr_t)c->value_cache |
             (uint64_t)a.v_token_stride | (uint64_t)a.cache_block_stride |
             (uint64_t)a.cache_slot_stride;
  }
  // 16-byte vectors need aligned rows and halves that hold whole vectors
  const int ev = 16 / E;
  const bool vector = (align % 16 == 0) && ((g.rotary_dim / 2) % ev == 0) &&
                      ((g.head_dim - g.rotary_dim) % ev == 0) && (g.head_dim % ev == 0);
  const int64_t ev_used = vector ? ev : 1;
  const int64_t heads = g.num_heads + g.num_kv_heads;
  const int64_t items = heads * ((g.rotary_dim / 2) / ev_used) +
                        heads * ((g.head_dim - g.rotary_dim) / ev_used) +
                        (c ? g.num_kv_heads * g.head_dim / ev_used : 0);
  a.pv_shift = log2_exact((g.rotary_dim / 2) / ev_used);
  a.cs_vector = ((uintptr_t)a.cos_sin_cache % 16 == 0) && ((2 * g.rotary_dim * E) % 16 == 0) ? 1 : 0;
  // Lanes per workgroup, from graph-timed sweeps (64 to 8192 tokens): the plain
  // rotation runs the same with 64 or 128 lanes and slower with 256; with the
  // cache write fused in, one wavefront per workgroup is 3-9 % faster than two
  // (the barrier then costs nothing, and a workgroup whose slot chain is late
  // holds back fewer lanes).
  unsigned threads = (unsigned)kvc::g_rope_tune.threads;
  if (threads != 64 && threads != 128 && threads != 256) threads = c ? 64 : 128;
  a.groups_per_token = (uint32_t)std::max<int64_t>(1, (items + threads - 1) / threads);
  if (g.num_tokens * (int64_t)a.groups_per_token > 0x7fffffffll)
    return fail(KVC_ERR_UNSUPPORTED, "%s: launch of %lld workgroups is too large", fn,
                (long long)(g.num_tokens * (int64_t)a.groups_per_token));
  hipStream_t s = (hipStream_t)stream;
  switch (g.dtype) {
    case KVC_DTYPE_BF16: launch_rope<BF16>(a, g.num_tokens, vector, threads, s); break;
    case KVC_DTYPE_F16: launch_rope<F16>(a, g.num_tokens, vector, threads, s); break;
    default: launch_rope<F32>(a, g.num_tokens, vector, threads, s); break;
  }
  KVC_HIP(hipGetLastError());
  return KVC_OK;
}

}  // namespace

extern "C" {

int kvc_rotary_pos_emb(const void* query, const void* key, const void* positions, int pos_bytes,
                       const void* cos_sin_cache, int64_t max_position, int64_t num_tokens,
                       int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                       int64_t rotary_dim, int64_t q_token_stride, int64_t k_token_stride,
                       void* query_out, void* key_out, int64_t qo_token_stride,
                       int64_t ko_token_stride, int dtype, void* stream) {
  RopeGeom g{num_tokens, num_heads, num_kv_heads, head_dim, rotary_dim, max_position,
             q_token_stride, k_token_stride, 0, qo_token_stride, ko_token_stride, dtype};
  return run_rope("kvc_rotary_pos_emb", query, key, nullptr, query_out, key_out, positions,
                  pos_bytes, cos_sin_cache, g, nullptr, stream);
}

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
                                 void* stream) {
  RopeGeom g{num_tokens, num_heads, num_kv_heads, head_dim, rotary_dim, max_position,
             q_token_stride, k_token_stride, v_token_stride, qo_token_stride, ko_token_stride, dtype};
  CacheGeom c{key_cache, value_cache, slot_mapping, slot_bytes, nullptr, nullptr, nullptr, 0, 0,
              block_size, cache_block_stride, cache_slot_stride, num_cache_blocks};
  return run_rope("kvc_rotary_pos_emb_and_cache", query, key, value, query_out, key_out, positions,
                  pos_bytes, cos_sin_cache, g, &c, stream);
}

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
                                        void* stream) {
  if (nnz > 0 && !batch_indices)
    return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_pos_emb_and_append_paged: null batch_indices");
  if (num_kv_heads < 0 || head_dim <= 0 || page_size <= 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_pos_emb_and_append_paged: bad H/D/page_size");
  const int64_t row = num_kv_heads * head_dim;
  if (page_stride < 2 * page_size * row)
    return fail(KVC_ERR_INVALID_ARG,
                "kvc_rotary_pos_emb_and_append_paged: page_stride %lld < 2*page_size*H*D",
                (long long)page_stride);
  const int E = dtype == KVC_DTYPE_F32 ? 4 : 2;
  RopeGeom g{nnz, num_heads, num_kv_heads, head_dim, rotary_dim, max_position,
             q_token_stride, k_token_stride, v_token_stride, qo_token_stride, ko_token_stride, dtype};
  char* vc = paged_kv_cache ? (char*)paged_kv_cache + page_size * row * E : nullptr;
  CacheGeom c{paged_kv_cache, vc, nullptr, 0, batch_indices, kv_indices, kv_indptr, batch_size,
              num_kv_indices, page_size, page_stride, row, num_pages};
  return run_rope("kvc_rotary_pos_emb_and_append_paged", query, key, value, query_out, key_out,
                  positions, 4, cos_sin_cache, g, &c, stream);
}

// ---- per-step plan of the fused rotation + page-table write ------------------
struct kvc_rotary_plan {
  const int32_t* batch_indices;
  const int32_t* positions;
  const void* cos_sin_cache;
  const int32_t* kv_indices;
  const int32_t* kv_indptr;
  int64_t max_position, nnz, num_heads, num_kv_heads, head_dim, rotary_dim;
  int64_t batch_size, num_kv_indices, page_size;
  int dtype;
  const int64_t* slots;  // resolved by kvc_rotary_plan_resolve_slots, else null
};

int kvc_rotary_plan_create(const int32_t* batch_indices, const int32_t* positions,
                           const void* cos_sin_cache, int64_t max_position, int64_t nnz,
                           int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                           int64_t rotary_dim, const int32_t* kv_indices,
                           const int32_t* kv_indptr, int64_t batch_size, int64_t num_kv_indices,
                           int64_t page_size, int dtype, kvc_rotary_plan** out) {
  if (!out) return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_create: null out");
  *out = nullptr;
  if (dtype != KVC_DTYPE_BF16 && dtype != KVC_DTYPE_F16 && dtype != KVC_DTYPE_F32)
    return fail(KVC_ERR_UNSUPPORTED, "kvc_rotary_plan_create: dtype %d (need bf16, f16 or f32)", dtype);
  if (nnz < 0 || num_heads < 0 || num_kv_heads < 0 || head_dim <= 0 || rotary_dim < 0 ||
      max_position < 0 || batch_size < 0 || num_kv_indices < 0 || page_size <= 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_create: bad size");
  if (rotary_dim > head_dim || (rotary_dim & 1))
    return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_create: rotary_dim %lld must be even and <= head_dim %lld",
                (long long)rotary_dim, (long long)head_dim);
  if (rotary_dim > kMaxRotaryDim)
    return fail(KVC_ERR_UNSUPPORTED, "kvc_rotary_plan_create: rotary_dim %lld exceeds %d",
                (long long)rotary_dim, kMaxRotaryDim);
  if (nnz > 0 && (!batch_indices || !positions || !cos_sin_cache || !kv_indices || !kv_indptr))
    return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_create: null pointer");
  kvc_rotary_plan* p = new (std::nothrow) kvc_rotary_plan{
      batch_indices, positions, cos_sin_cache, kv_indices, kv_indptr, max_position, nnz, num_heads,
      num_kv_heads, head_dim, rotary_dim, batch_size, num_kv_indices, page_size, dtype, nullptr};
  if (!p) return fail(KVC_ERR_HIP, "kvc_rotary_plan_create: out of host memory");
  *out = p;
  return KVC_OK;
}

int kvc_rotary_plan_run(const kvc_rotary_plan* plan, const void* query, const void* key,
                        const void* value, int64_t q_token_stride, int64_t k_token_stride,
                        int64_t v_token_stride, void* query_out, void* key_out,
                        void* paged_kv_cache, int64_t page_stride, int64_t num_pages,
                        void* stream) {
  if (!plan) return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_run: null plan");
  const int64_t q_row = plan->num_heads * plan->head_dim;
  const int64_t k_row = plan->num_kv_heads * plan->head_dim;
  if (plan->slots) {
    if (page_stride < 2 * plan->page_size * k_row)
      return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_run: page_stride %lld < 2*page_size*H*D",
                  (long long)page_stride);
    const int E = plan->dtype == KVC_DTYPE_F32 ? 4 : 2;
    char* vc = paged_kv_cache ? (char*)paged_kv_cache + plan->page_size * k_row * E : nullptr;
    return kvc_rotary_pos_emb_and_cache(
        query, key, value, plan->positions, 4, plan->cos_sin_cache, plan->max_position, plan->nnz,
        plan->num_heads, plan->num_kv_heads, plan->head_dim, plan->rotary_dim, q_token_stride,
        k_token_stride, v_token_stride, query_out, key_out, q_row, k_row, paged_kv_cache, vc,
        plan->slots, 8, plan->page_size, page_stride, k_row, num_pages, plan->dtype, stream);
  }
  return kvc_rotary_pos_emb_and_append_paged(
      query, key, value, plan->batch_indices, plan->positions, plan->cos_sin_cache,
      plan->max_position, plan->nnz, plan->num_heads, plan->num_kv_heads, plan->head_dim,
      plan->rotary_dim, q_token_stride, k_token_stride, v_token_stride, query_out, key_out, q_row,
      k_row, paged_kv_cache, plan->kv_indices, plan->kv_indptr, plan->batch_size,
      plan->num_kv_indices, plan->page_size, page_stride, num_pages, plan->dtype, stream);
}

int kvc_rotary_plan_resolve_slots(kvc_rotary_plan* plan, int64_t* slots, void* stream) {
  if (!plan) return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_resolve_slots: null plan");
  const int rc = kvc::launch_resolve_slots("kvc_rotary_plan_resolve_slots", plan->batch_indices,
                                           plan->positions, plan->kv_indices, plan->kv_indptr,
                                           plan->batch_size, plan->num_kv_indices, plan->page_size,
                                           plan->nnz, slots, (hipStream_t)stream);
  if (rc == KVC_OK && plan->nnz > 0) plan->slots = slots;
  return rc;
}

int kvc_rotary_plan_set_slots(kvc_rotary_plan* plan, const int64_t* slots) {
  if (!plan) return fail(KVC_ERR_INVALID_ARG, "kvc_rotary_plan_set_slots: null plan");
  plan->slots = slots;
  return KVC_OK;
}

int kvc_rotary_plan_destroy(kvc_rotary_plan* plan) {
  delete plan;
  return KVC_OK;
}

}  // extern "C"

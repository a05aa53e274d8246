// Calls libkvcache through its C ABI from a plain HIP program (no Python, no
// torch): every operator of the copy path, the one-launch index build and the
// disk tier on small seeded inputs, compared byte for byte with the C oracle
// (oracle/kvc_oracle.c, linked in) or with arrays written out by hand.
// Exit status 0 and a final "ABI CHECK PASSED" line on success.
#include <hip/hip_runtime.h>
#include <time.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <random>
#include <string>
#include <vector>

#include "kvcache.h"
#include "kvcache_experimental.h"

extern "C" {
void oracle_reshape_and_cache(const void*, const void*, void*, const int64_t*, int64_t, int64_t,
                              int64_t, int64_t, int64_t);
void oracle_append_paged_kv_cache(const void*, const void*, const int32_t*, const int32_t*, void*,
                                  const int32_t*, const int32_t*, int64_t, int64_t, int64_t, int64_t,
                                  int64_t);
void oracle_copy_blocks(void*, const int64_t*, int64_t, int64_t, int64_t, int64_t, int64_t);
void oracle_save_blocks_to_host(const void*, void*, const int64_t*, const int64_t*, int64_t, int64_t,
                                int64_t, int64_t, int64_t, int64_t);
void oracle_load_blocks_from_host(void*, const void*, const int64_t*, const int64_t*, int64_t,
                                  int64_t, int64_t, int64_t, int64_t, int64_t);
}

#define HIP_OK(x)                                                                     \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                    \
      return 2;                                                                       \
    }                                                                                 \
  } while (0)
#define KVC_OK_OR_DIE(x)                                                              \
  do {                                                                                \
    int rc_ = (x);                                                                    \
    if (rc_ != KVC_OK) {                                                              \
      std::fprintf(stderr, "%s -> %d: %s\n", #x, rc_, kvc_last_error_string());       \
      return 3;                                                                       \
    }                                                                                 \
  } while (0)

static int fails = 0;
static void expect_equal(const char* what, const void* a, const void* b, size_t n) {
  if (std::memcmp(a, b, n) != 0) {
    std::fprintf(stderr, "MISMATCH: %s\n", what);
    ++fails;
  } else {
    std::printf("ok: %s\n", what);
  }
  std::fflush(stdout);
}

int main() {
  const int64_t L = 3, nb = 48, bs = 16, H = 2, D = 64, E = 2;
  const int64_t row = H * D, blk_elems = 2 * bs * row, blk_bytes = blk_elems * E;
  const int64_t layer_elems = nb * blk_elems;
  const size_t pool_bytes = (size_t)(L * layer_elems * E);
  std::mt19937_64 rng(7);
  std::vector<uint16_t> pool(L * layer_elems);
  for (auto& x : pool) x = (uint16_t)rng();

  // --- a mixed step: request 0 appends 20 tokens after 5, request 1 one token after 33
  std::vector<int32_t> kv_indices = {7, 19, 3, 40, 11, 25};  // tables: [7,19] and [3,40,11]; 25 unused
  std::vector<int32_t> kv_indptr = {0, 2, 5};
  std::vector<int32_t> last = {(25 - 1) % 16 + 1, (34 - 1) % 16 + 1};
  std::vector<int32_t> bi, pos;
  std::vector<int64_t> slots;
  for (int p = 5; p < 25; ++p) { bi.push_back(0); pos.push_back(p); slots.push_back((int64_t)kv_indices[p / 16] * 16 + p % 16); }
  bi.push_back(1); pos.push_back(33); slots.push_back((int64_t)kv_indices[2 + 33 / 16] * 16 + 33 % 16);
  const int64_t T = (int64_t)bi.size();
  std::vector<uint16_t> key(L * T * row), value(L * T * row);
  for (auto& x : key) x = (uint16_t)rng();
  for (auto& x : value) x = (uint16_t)rng();

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  void *d_pool, *d_key, *d_value, *d_slots, *d_bi, *d_pos, *d_ind, *d_ptr, *d_last, *d_maps;
  HIP_OK(hipMalloc(&d_pool, pool_bytes));
  HIP_OK(hipMalloc(&d_key, key.size() * E));
  HIP_OK(hipMalloc(&d_value, value.size() * E));
  HIP_OK(hipMalloc(&d_slots, T * 8));
  HIP_OK(hipMalloc(&d_bi, T * 4));
  HIP_OK(hipMalloc(&d_pos, T * 4));
  HIP_OK(hipMalloc(&d_ind, kv_indices.size() * 4));
  HIP_OK(hipMalloc(&d_ptr, kv_indptr.size() * 4));
  HIP_OK(hipMalloc(&d_last, last.size() * 4));
  HIP_OK(hipMemcpy(d_key, key.data(), key.size() * E, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_value, value.data(), value.size() * E, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_slots, slots.data(), T * 8, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_bi, bi.data(), T * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_pos, pos.data(), T * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_ind, kv_indices.data(), kv_indices.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_ptr, kv_indptr.data(), kv_indptr.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_last, last.data(), last.size() * 4, hipMemcpyHostToDevice));

  std::vector<uint16_t> got(pool.size()), want(pool);
  std::printf("abi version %d\n", kvc_abi_version());

  // 1. slot-mapped write, one launch per layer
  HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
  for (int64_t l = 0; l < L; ++l) {
    char* layer = (char*)d_pool + l * layer_elems * E;
    KVC_OK_OR_DIE(kvc_reshape_and_cache((char*)d_key + l * T * row * E, (char*)d_value + l * T * row * E,
                                        layer, layer + bs * row * E, d_slots, 8, T, row, row, row, bs,
                                        blk_elems, row, nb, (int)E, stream));
    oracle_reshape_and_cache(key.data() + l * T * row, value.data() + l * T * row,
                             want.data() + l * layer_elems, slots.data(), T, bs, H, D, E);
  }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
  expect_equal("kvc_reshape_and_cache (per layer) == oracle", got.data(), want.data(), pool_bytes);

  // 2. the same write for all layers in one launch
  HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
  KVC_OK_OR_DIE(kvc_reshape_and_cache_layers(d_key, d_value, d_pool, (char*)d_pool + bs * row * E,
                                             d_slots, 8, T, row, row, row, bs, blk_elems, row, nb, L,
                                             T * row, T * row, layer_elems, (int)E, stream));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
  expect_equal("kvc_reshape_and_cache_layers == oracle", got.data(), want.data(), pool_bytes);

  // 3. page-table addressed write (must land on the same slots)
  std::vector<uint16_t> want_paged(pool);
  HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
  for (int64_t l = 0; l < L; ++l) {
    KVC_OK_OR_DIE(kvc_append_paged_kv_cache(
        (char*)d_key + l * T * row * E, (char*)d_value + l * T * row * E, (const int32_t*)d_bi,
        (const int32_t*)d_pos, (char*)d_pool + l * layer_elems * E, (const int32_t*)d_ind,
        (const int32_t*)d_ptr, (const int32_t*)d_last, T, 2, (int64_t)kv_indices.size(), H, D, bs,
        row, row, blk_elems, nb, (int)E, stream));
    oracle_append_paged_kv_cache(key.data() + l * T * row, value.data() + l * T * row, bi.data(),
                                 pos.data(), want_paged.data() + l * layer_elems, kv_indices.data(),
                                 kv_indptr.data(), T, H, D, bs, E);
  }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
  expect_equal("kvc_append_paged_kv_cache == oracle", got.data(), want_paged.data(), pool_bytes);
  expect_equal("page-table write == slot-mapped write", want_paged.data(), want.data(), pool_bytes);
  // all layers in one launch
  HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
  KVC_OK_OR_DIE(kvc_append_paged_kv_cache_layers(
      d_key, d_value, (const int32_t*)d_bi, (const int32_t*)d_pos, d_pool, (const int32_t*)d_ind,
      (const int32_t*)d_ptr, (const int32_t*)d_last, T, 2, (int64_t)kv_indices.size(), H, D, bs, row, row,
      blk_elems, nb, L, T * row, T * row, layer_elems, (int)E, stream));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
  expect_equal("kvc_append_paged_kv_cache_layers == oracle", got.data(), want_paged.data(), pool_bytes);
  // the two index functions of the step: seq_lens = (pages - 1) * bs + last, then (request, position) per token
  {
    const std::vector<int32_t> cu = {0, 20, 21}, want_seq = {25, 34};
    void *d_cu, *d_seq, *d_bi2, *d_pos2;
    HIP_OK(hipMalloc(&d_cu, 3 * 4)); HIP_OK(hipMalloc(&d_seq, 2 * 4));
    HIP_OK(hipMalloc(&d_bi2, T * 4)); HIP_OK(hipMalloc(&d_pos2, T * 4));
    HIP_OK(hipMemcpy(d_cu, cu.data(), 3 * 4, hipMemcpyHostToDevice));
    KVC_OK_OR_DIE(kvc_get_seq_lens((const int32_t*)d_ptr, (const int32_t*)d_last, 2, bs, (int32_t*)d_seq, stream));
    KVC_OK_OR_DIE(kvc_get_batch_indices_positions((const int32_t*)d_cu, (const int32_t*)d_seq, 2, T,
                                                  (int32_t*)d_bi2, (int32_t*)d_pos2, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int32_t> g_seq(2), g_bi(T), g_pos(T);
    HIP_OK(hipMemcpy(g_seq.data(), d_seq, 2 * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_bi.data(), d_bi2, T * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_pos.data(), d_pos2, T * 4, hipMemcpyDeviceToHost));
    expect_equal("kvc_get_seq_lens == context lengths", g_seq.data(), want_seq.data(), 2 * 4);
    expect_equal("kvc_get_batch_indices_positions: requests", g_bi.data(), bi.data(), T * 4);
    expect_equal("kvc_get_batch_indices_positions: positions", g_pos.data(), pos.data(), T * 4);
    HIP_OK(hipFree(d_cu)); HIP_OK(hipFree(d_seq)); HIP_OK(hipFree(d_bi2)); HIP_OK(hipFree(d_pos2));
  }

  // 3b. the same page-table write through a per-step plan: three pointers per layer
  {
    HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
    kvc_write_plan* plan = nullptr;
    KVC_OK_OR_DIE(kvc_write_plan_create((const int32_t*)d_bi, (const int32_t*)d_pos, (const int32_t*)d_ind,
                                        (const int32_t*)d_ptr, (const int32_t*)d_last, T, 2,
                                        (int64_t)kv_indices.size(), H, D, bs, (int)E, &plan));
    for (int64_t l = 0; l < L; ++l)
      KVC_OK_OR_DIE(kvc_write_plan_append(plan, (char*)d_key + l * T * row * E,
                                          (char*)d_value + l * T * row * E, row, row,
                                          (char*)d_pool + l * layer_elems * E, blk_elems, nb, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
    expect_equal("kvc_write_plan_append == oracle", got.data(), want_paged.data(), pool_bytes);
    if (kvc_last_launch_info(KVC_LAUNCH_KERNEL) != KVC_KERNEL_WRITE_ROWS ||
        kvc_last_launch_info(KVC_LAUNCH_VEC_BYTES) != 16) {
      std::fprintf(stderr, "a small launch of 256-byte rows did not take the token-per-workgroup kernel\n");
      ++fails;
    }
    // the same plan with the page table walked once: slots == the scheduler's rule, same pool
    int64_t* d_resolved = nullptr;  // the plan uses it until it is destroyed
    {
      HIP_OK(hipMalloc(&d_resolved, T * sizeof(int64_t)));
      HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
      KVC_OK_OR_DIE(kvc_write_plan_resolve_slots(plan, d_resolved, stream));
      for (int64_t l = 0; l < L; ++l)
        KVC_OK_OR_DIE(kvc_write_plan_append(plan, (char*)d_key + l * T * row * E,
                                            (char*)d_value + l * T * row * E, row, row,
                                            (char*)d_pool + l * layer_elems * E, blk_elems, nb, stream));
      HIP_OK(hipStreamSynchronize(stream));
      std::vector<int64_t> resolved(T);
      HIP_OK(hipMemcpy(resolved.data(), d_resolved, T * sizeof(int64_t), hipMemcpyDeviceToHost));
      expect_equal("kvc_write_plan_resolve_slots == slot rule", resolved.data(), slots.data(),
                   T * sizeof(int64_t));
      HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
      expect_equal("kvc_write_plan_append through resolved slots == oracle", got.data(), want_paged.data(),
                   pool_bytes);
    }
    // host cost of one planned launch (informational)
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    const int reps = 2000;
    timespec t0, t1;
    HIP_OK(hipEventRecord(e0, stream));
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int i = 0; i < reps; ++i)
      KVC_OK_OR_DIE(kvc_write_plan_append(plan, d_key, d_value, row, row, d_pool, blk_elems, nb, stream));
    clock_gettime(CLOCK_MONOTONIC, &t1);
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipStreamSynchronize(stream));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    std::printf("kvc_write_plan_append: %.2f us of host time per call, %.2f us per call on the stream\n",
                ((t1.tv_sec - t0.tv_sec) * 1e9 + (t1.tv_nsec - t0.tv_nsec)) / 1e3 / reps, ms * 1e3 / reps);
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    KVC_OK_OR_DIE(kvc_write_plan_destroy(plan));
    HIP_OK(hipFree(d_resolved));
    if (kvc_write_plan_append(nullptr, d_key, d_value, row, row, d_pool, blk_elems, nb, stream) !=
        KVC_ERR_INVALID_ARG) {
      std::fprintf(stderr, "expected KVC_ERR_INVALID_ARG for a null plan\n");
      ++fails;
    }
    // tuning knobs: set, read back, reset
    int v = -1;
    KVC_OK_OR_DIE(kvc_set_tuning("write_planes", 2));
    KVC_OK_OR_DIE(kvc_get_tuning("write_planes", &v));
    if (v != 2 || kvc_tuning_modified() != 1) { std::fprintf(stderr, "tuning read-back failed\n"); ++fails; }
    HIP_OK(hipMemcpy(d_pool, pool.data(), pool_bytes, hipMemcpyHostToDevice));
    for (int64_t l = 0; l < L; ++l)
      KVC_OK_OR_DIE(kvc_reshape_and_cache((char*)d_key + l * T * row * E, (char*)d_value + l * T * row * E,
                                          (char*)d_pool + l * layer_elems * E,
                                          (char*)d_pool + l * layer_elems * E + bs * row * E, d_slots, 8, T,
                                          row, row, row, bs, blk_elems, row, nb, (int)E, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
    expect_equal("plane kernel on 256-byte rows == oracle", got.data(), want.data(), pool_bytes);
    if (kvc_last_launch_info(KVC_LAUNCH_KERNEL) != KVC_KERNEL_WRITE_PLANES) {
      std::fprintf(stderr, "write_planes = 2 did not select the plane kernel\n");
      ++fails;
    }
    KVC_OK_OR_DIE(kvc_reset_tuning());
    KVC_OK_OR_DIE(kvc_get_tuning("write_planes", &v));
    if (v != 1 || kvc_tuning_modified() != 0) { std::fprintf(stderr, "tuning reset failed\n"); ++fails; }
  }

  // 4. copy_blocks
  std::vector<int64_t> maps = {7, 0, 7, 1, 19, 30, 5, 5, 40, 47};
  HIP_OK(hipMalloc(&d_maps, maps.size() * 8));
  HIP_OK(hipMemcpy(d_maps, maps.data(), maps.size() * 8, hipMemcpyHostToDevice));
  KVC_OK_OR_DIE(kvc_copy_blocks(d_pool, (const int64_t*)d_maps, (int64_t)maps.size() / 2, L,
                                layer_elems * E, blk_bytes, nb, stream));
  oracle_copy_blocks(want.data(), maps.data(), (int64_t)maps.size() / 2, L, layer_elems, blk_elems, E);
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
  expect_equal("kvc_copy_blocks == oracle", got.data(), want.data(), pool_bytes);

  // 5. swap out / in, every mode, through library-pinned host memory
  const int64_t nhb = 10, n = 6;
  std::vector<int64_t> out_src = {30, 0, 47, 19, 5, 11}, out_dst = {2, 3, 4, 9, 0, 6};
  std::vector<int64_t> in_src = {9, 0, 3}, in_dst = {44, 45, 13};
  const size_t host_bytes = (size_t)(nhb * L * blk_bytes);
  for (int mode = 0; mode < 3; ++mode) {
    const std::string tag = mode == KVC_SWAP_STAGED ? " (staged)" : mode == KVC_SWAP_DIRECT ? " (direct)" : " (auto)";
    uint16_t* host = (uint16_t*)kvc_host_alloc_pinned(host_bytes);
    if (!host) { std::fprintf(stderr, "pinned alloc failed: %s\n", kvc_last_error_string()); return 4; }
    std::vector<uint16_t> want_host(host_bytes / 2);
    for (size_t i = 0; i < want_host.size(); ++i) host[i] = want_host[i] = (uint16_t)(0xFFC0 + i % 61);
    const int64_t staging_bytes = kvc_swap_staging_bytes(n, L, blk_bytes, mode, 2);
    void* staging;
    HIP_OK(hipMalloc(&staging, staging_bytes));
    hipStream_t copy_stream;
    HIP_OK(hipStreamCreate(&copy_stream));
    KVC_OK_OR_DIE(kvc_swap_out(d_pool, host, out_src.data(), out_dst.data(), n, L, layer_elems * E,
                               blk_bytes, nb, nhb, 0, L, staging, staging_bytes, mode, stream, copy_stream));
    HIP_OK(hipStreamSynchronize(stream));
    oracle_save_blocks_to_host(want.data(), want_host.data(), out_src.data(), out_dst.data(), n, L, nb,
                               blk_bytes, 0, L);
    expect_equal(("kvc_swap_out" + tag + " == oracle").c_str(), host, want_host.data(), host_bytes);
    if (mode == KVC_SWAP_AUTO) {
      // six scattered blocks of a few KiB: far under the extent size that pays for the copy engines
      if (kvc_last_launch_info(KVC_LAUNCH_SWAP_MODE) != KVC_SWAP_DIRECT) {
        std::fprintf(stderr, "KVC_SWAP_AUTO took mode %lld for small scattered extents\n",
                     (long long)kvc_last_launch_info(KVC_LAUNCH_SWAP_MODE));
        ++fails;
      }
      KVC_OK_OR_DIE(kvc_set_tuning("auto_min_extent_bytes", 1));  // from here on every call is staged
    }
    KVC_OK_OR_DIE(kvc_swap_in(d_pool, host, in_src.data(), in_dst.data(), 3, L, layer_elems * E,
                              blk_bytes, nb, nhb, 0, L, staging, staging_bytes, mode, stream, copy_stream));
    HIP_OK(hipStreamSynchronize(stream));
    oracle_load_blocks_from_host(want.data(), want_host.data(), in_src.data(), in_dst.data(), 3, L, nb,
                                 blk_bytes, 0, L);
    HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
    expect_equal(("kvc_swap_in" + tag + " == oracle").c_str(), got.data(), want.data(), pool_bytes);
    if (mode == KVC_SWAP_AUTO && kvc_last_launch_info(KVC_LAUNCH_SWAP_MODE) != KVC_SWAP_STAGED) {
      std::fprintf(stderr, "KVC_SWAP_AUTO did not take the staged path with the threshold at one byte\n");
      ++fails;
    }
    // the same ids checked and uploaded once, then one call per layer
    {
      std::vector<int64_t> p_gpu = {1, 46, 22, 9}, p_host = {1, 5, 7, 8};
      KVC_OK_OR_DIE(kvc_swap_prepare(p_gpu.data(), p_host.data(), 4, nb, nhb, staging, staging_bytes, stream));
      for (int64_t l = 0; l < L; ++l)
        KVC_OK_OR_DIE(kvc_swap_out_prepared(d_pool, host, p_host.data(), 4, L, layer_elems * E, blk_bytes,
                                            nb, nhb, l, l + 1, staging, staging_bytes, mode, stream,
                                            copy_stream));
      HIP_OK(hipStreamSynchronize(stream));
      oracle_save_blocks_to_host(want.data(), want_host.data(), p_gpu.data(), p_host.data(), 4, L, nb,
                                 blk_bytes, 0, L);
      expect_equal(("kvc_swap_out_prepared per layer" + tag + " == oracle").c_str(), host, want_host.data(),
                   host_bytes);
      std::vector<int64_t> q_gpu = {33, 34, 35, 2};
      KVC_OK_OR_DIE(kvc_swap_prepare(q_gpu.data(), p_host.data(), 4, nb, nhb, staging, staging_bytes, stream));
      for (int64_t l = L; l-- > 0;)
        KVC_OK_OR_DIE(kvc_swap_in_prepared(d_pool, host, p_host.data(), 4, L, layer_elems * E, blk_bytes,
                                           nb, nhb, l, l + 1, staging, staging_bytes, mode, stream,
                                           copy_stream));
      HIP_OK(hipStreamSynchronize(stream));
      oracle_load_blocks_from_host(want.data(), want_host.data(), p_host.data(), q_gpu.data(), 4, L, nb,
                                   blk_bytes, 0, L);
      HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
      expect_equal(("kvc_swap_in_prepared per layer" + tag + " == oracle").c_str(), got.data(), want.data(),
                   pool_bytes);
      std::vector<int64_t> bad_gpu = {nb};
      if (kvc_swap_prepare(bad_gpu.data(), p_host.data(), 1, nb, nhb, staging, staging_bytes, stream) !=
          KVC_ERR_OUT_OF_RANGE) {
        std::fprintf(stderr, "expected KVC_ERR_OUT_OF_RANGE from kvc_swap_prepare\n");
        ++fails;
      }
    }
    // an id outside the host pool is rejected before anything runs
    std::vector<int64_t> bad = {nhb};
    const int rc = kvc_swap_out(d_pool, host, out_src.data(), bad.data(), 1, L, layer_elems * E,
                                blk_bytes, nb, nhb, 0, L, staging, staging_bytes, mode, stream, copy_stream);
    if (rc != KVC_ERR_OUT_OF_RANGE) { std::fprintf(stderr, "expected KVC_ERR_OUT_OF_RANGE, got %d\n", rc); ++fails; }
    HIP_OK(hipStreamSynchronize(copy_stream));
    HIP_OK(hipStreamDestroy(copy_stream));
    HIP_OK(hipFree(staging));
    KVC_OK_OR_DIE(kvc_host_free_pinned(host));
    KVC_OK_OR_DIE(kvc_reset_tuning());
  }

  // 5b. the swap that allocates nothing: same result as the direct swap, no workspace argument
  {
    uint16_t* host = (uint16_t*)kvc_host_alloc_pinned(host_bytes);
    if (!host) { std::fprintf(stderr, "pinned alloc failed: %s\n", kvc_last_error_string()); return 4; }
    std::vector<uint16_t> want_host(host_bytes / 2);
    for (size_t i = 0; i < want_host.size(); ++i) host[i] = want_host[i] = (uint16_t)(0x1234 + i % 97);
    KVC_OK_OR_DIE(kvc_swap_noalloc(1, d_pool, host, out_src.data(), out_dst.data(), n, L, layer_elems * E,
                                   blk_bytes, nb, nhb, 0, L, stream));
    HIP_OK(hipStreamSynchronize(stream));
    oracle_save_blocks_to_host(want.data(), want_host.data(), out_src.data(), out_dst.data(), n, L, nb,
                               blk_bytes, 0, L);
    expect_equal("kvc_swap_noalloc to the host == oracle", host, want_host.data(), host_bytes);
    std::vector<int64_t> back_host = {2, 9}, back_gpu = {36, 37};   // a second, smaller call: layer 1 only
    KVC_OK_OR_DIE(kvc_swap_noalloc(0, d_pool, host, back_gpu.data(), back_host.data(), 2, L, layer_elems * E,
                                   blk_bytes, nb, nhb, 1, 2, stream));
    HIP_OK(hipStreamSynchronize(stream));
    oracle_load_blocks_from_host(want.data(), want_host.data(), back_host.data(), back_gpu.data(), 2, L, nb,
                                 blk_bytes, 1, 2);
    HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
    expect_equal("kvc_swap_noalloc from the host, one layer == oracle", got.data(), want.data(), pool_bytes);
    if (kvc_swap_noalloc(1, d_pool, host, out_src.data(), out_dst.data(), KVC_NOALLOC_MAX_BLOCKS + 1, L,
                         layer_elems * E, blk_bytes, nb, nhb, 0, L, stream) != KVC_ERR_UNSUPPORTED) {
      std::fprintf(stderr, "expected KVC_ERR_UNSUPPORTED beyond KVC_NOALLOC_MAX_BLOCKS\n");
      ++fails;
    }
    KVC_OK_OR_DIE(kvc_host_free_pinned(host));
  }

  // 6. device gather and scatter: the pool's blocks <-> a dense [n, L, blk] buffer.
  //    The dense buffer has the host pool's row layout, so the swap oracle applies.
  {
    std::vector<int64_t> ids = {41, 2, 17, 8}, dense_rows = {0, 1, 2, 3}, back = {20, 21, 22, 23};
    const int64_t m = (int64_t)ids.size();
    const size_t dense_bytes = (size_t)(m * L * blk_bytes);
    void *d_ids, *d_back, *d_dense;
    HIP_OK(hipMalloc(&d_ids, m * 8));
    HIP_OK(hipMalloc(&d_back, m * 8));
    HIP_OK(hipMalloc(&d_dense, dense_bytes));
    HIP_OK(hipMemcpy(d_ids, ids.data(), m * 8, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_back, back.data(), m * 8, hipMemcpyHostToDevice));
    HIP_OK(hipMemset(d_dense, 0, dense_bytes));
    KVC_OK_OR_DIE(kvc_gather_blocks(d_pool, d_dense, (const int64_t*)d_ids, m, L, layer_elems * E, blk_bytes,
                                    nb, 0, L, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> dense(dense_bytes / 2), want_dense(dense_bytes / 2, 0);
    HIP_OK(hipMemcpy(dense.data(), d_dense, dense_bytes, hipMemcpyDeviceToHost));
    oracle_save_blocks_to_host(want.data(), want_dense.data(), ids.data(), dense_rows.data(), m, L, nb,
                               blk_bytes, 0, L);
    expect_equal("kvc_gather_blocks == oracle", dense.data(), want_dense.data(), dense_bytes);
    KVC_OK_OR_DIE(kvc_scatter_blocks(d_pool, d_dense, (const int64_t*)d_back, m, L, layer_elems * E,
                                     blk_bytes, nb, 0, L, stream));
    HIP_OK(hipStreamSynchronize(stream));
    oracle_load_blocks_from_host(want.data(), want_dense.data(), dense_rows.data(), back.data(), m, L, nb,
                                 blk_bytes, 0, L);
    HIP_OK(hipMemcpy(got.data(), d_pool, pool_bytes, hipMemcpyDeviceToHost));
    expect_equal("kvc_scatter_blocks == oracle", got.data(), want.data(), pool_bytes);
    HIP_OK(hipFree(d_ids));
    HIP_OK(hipFree(d_back));
    HIP_OK(hipFree(d_dense));
  }

  // 7. the whole index of the step in one launch, against the arrays built by hand above
  {
    std::vector<int32_t> input_lens = {20, 1}, context_lens = {25, 34}, nblocks = {2, 3};
    void *d_il, *d_cl, *d_nb, *d_cu, *d_ptr2, *d_last2, *d_bi2, *d_pos2, *d_slots2;
    HIP_OK(hipMalloc(&d_il, 8)); HIP_OK(hipMalloc(&d_cl, 8)); HIP_OK(hipMalloc(&d_nb, 8));
    HIP_OK(hipMalloc(&d_cu, 12)); HIP_OK(hipMalloc(&d_ptr2, 12)); HIP_OK(hipMalloc(&d_last2, 8));
    HIP_OK(hipMalloc(&d_bi2, T * 4)); HIP_OK(hipMalloc(&d_pos2, T * 4)); HIP_OK(hipMalloc(&d_slots2, T * 8));
    HIP_OK(hipMemcpy(d_il, input_lens.data(), 8, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_cl, context_lens.data(), 8, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_nb, nblocks.data(), 8, hipMemcpyHostToDevice));
    KVC_OK_OR_DIE(kvc_build_write_index((const int32_t*)d_il, (const int32_t*)d_cl, (const int32_t*)d_nb,
                                        (const int32_t*)d_ind, 2, 5, bs, T, (int32_t*)d_cu, (int32_t*)d_ptr2,
                                        (int32_t*)d_last2, (int32_t*)d_bi2, (int32_t*)d_pos2,
                                        (int64_t*)d_slots2, nullptr, nullptr, nullptr, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int32_t> g_ptr(3), g_last(2), g_bi(T), g_pos(T), g_cu(3);
    std::vector<int64_t> g_slots(T);
    HIP_OK(hipMemcpy(g_cu.data(), d_cu, 12, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_ptr.data(), d_ptr2, 12, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_last.data(), d_last2, 8, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_bi.data(), d_bi2, T * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_pos.data(), d_pos2, T * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(g_slots.data(), d_slots2, T * 8, hipMemcpyDeviceToHost));
    const std::vector<int32_t> want_cu = {0, 20, 21};
    expect_equal("kvc_build_write_index cu_seqlens_q", g_cu.data(), want_cu.data(), 12);
    expect_equal("kvc_build_write_index kv_indptr", g_ptr.data(), kv_indptr.data(), 12);
    expect_equal("kvc_build_write_index kv_last_page_len", g_last.data(), last.data(), 8);
    expect_equal("kvc_build_write_index batch_indices", g_bi.data(), bi.data(), T * 4);
    expect_equal("kvc_build_write_index positions", g_pos.data(), pos.data(), T * 4);
    expect_equal("kvc_build_write_index slot_mapping", g_slots.data(), slots.data(), T * 8);
    for (void* p : {d_il, d_cl, d_nb, d_cu, d_ptr2, d_last2, d_bi2, d_pos2, d_slots2}) HIP_OK(hipFree(p));
  }

  // 8. host <-> disk tier behind the pinned pool: disk[dst] = host[src] and back
  {
    const int64_t ndb = 5;
    const size_t row_elems = (size_t)(L * blk_elems);
    uint16_t* host = (uint16_t*)kvc_host_alloc_pinned(host_bytes);
    if (!host) { std::fprintf(stderr, "pinned alloc failed: %s\n", kvc_last_error_string()); return 4; }
    for (size_t i = 0; i < host_bytes / 2; ++i) host[i] = (uint16_t)rng();
    std::vector<uint16_t> host0(host, host + host_bytes / 2);
    char path[64];
    std::snprintf(path, sizeof path, "/tmp/kvc-abi-check-%d.npy", (int)getpid());
    kvc_disk* disk = nullptr;
    KVC_OK_OR_DIE(kvc_disk_open(path, "<u2", ndb, L, blk_elems, 2, KVC_DISK_DIRECT, &disk));
    std::vector<int64_t> s_host = {7, 1, 2}, s_disk = {4, 0, 1}, l_disk = {1, 4}, l_host = {9, 8};
    KVC_OK_OR_DIE(kvc_disk_save_blocks(disk, host, nhb, s_host.data(), s_disk.data(), 3, 4));
    KVC_OK_OR_DIE(kvc_disk_sync(disk));
    KVC_OK_OR_DIE(kvc_disk_load_blocks(disk, host, nhb, l_disk.data(), l_host.data(), 2, 4));
    std::vector<uint16_t> want_h(host0);
    std::memcpy(&want_h[9 * row_elems], &host0[2 * row_elems], row_elems * 2);   // disk 1 holds host 2
    std::memcpy(&want_h[8 * row_elems], &host0[7 * row_elems], row_elems * 2);   // disk 4 holds host 7
    expect_equal("kvc_disk_save_blocks + kvc_disk_load_blocks round trip", host, want_h.data(), host_bytes);
    std::printf("disk tier: O_DIRECT %s, host side %s\n",
                kvc_disk_info(disk, KVC_DISK_INFO_DIRECT) ? "on" : "off",
                kvc_disk_info(disk, KVC_DISK_INFO_BOUNCED) ? "staged" : "in place");
    std::vector<int64_t> bad = {ndb};
    if (kvc_disk_save_blocks(disk, host, nhb, s_host.data(), bad.data(), 1, 1) != KVC_ERR_OUT_OF_RANGE) {
      std::fprintf(stderr, "expected KVC_ERR_OUT_OF_RANGE from the disk tier\n");
      ++fails;
    }
    KVC_OK_OR_DIE(kvc_disk_close(disk));
    std::remove(path);
    KVC_OK_OR_DIE(kvc_host_free_pinned(host));
  }

  // 9. one layer of scattered host blocks through a dense buffer (host threads only)
  {
    const int64_t n = 5, layer = 1;
    std::vector<uint16_t> host_pool((size_t)(nhb * L * blk_elems)), dense((size_t)(n * blk_elems));
    for (auto& x : host_pool) x = (uint16_t)rng();
    for (auto& x : dense) x = (uint16_t)rng();
    std::vector<int64_t> ids = {9, 0, 4, 2, 7};
    std::vector<uint16_t> want_p(host_pool);
    for (int64_t i = 0; i < n; ++i)
      std::memcpy(&want_p[(size_t)((ids[i] * L + layer) * blk_elems)], &dense[(size_t)(i * blk_elems)], blk_bytes);
    KVC_OK_OR_DIE(kvc_host_copy_rows(host_pool.data(), nhb, L * blk_bytes, layer * blk_bytes, dense.data(),
                                     ids.data(), n, blk_bytes, 1, 3));
    expect_equal("kvc_host_copy_rows into the pool", host_pool.data(), want_p.data(), host_pool.size() * 2);
    std::vector<uint16_t> back(dense.size());
    KVC_OK_OR_DIE(kvc_host_copy_rows(host_pool.data(), nhb, L * blk_bytes, layer * blk_bytes, back.data(),
                                     ids.data(), n, blk_bytes, 0, 3));
    expect_equal("kvc_host_copy_rows out of the pool", back.data(), dense.data(), dense.size() * 2);

    // the queue form: a job that waits for "the rows have landed in the pinned buffer"
    uint16_t* landing = (uint16_t*)kvc_host_alloc_pinned(dense.size() * 2);
    if (!landing) { std::fprintf(stderr, "pinned alloc failed: %s\n", kvc_last_error_string()); return 4; }
    void* d_rows;
    HIP_OK(hipMalloc(&d_rows, dense.size() * 2));
    std::vector<uint16_t> fresh(dense.size());
    for (auto& x : fresh) x = (uint16_t)rng();
    HIP_OK(hipMemcpy(d_rows, fresh.data(), fresh.size() * 2, hipMemcpyHostToDevice));
    hipEvent_t landed;
    HIP_OK(hipEventCreateWithFlags(&landed, hipEventDisableTiming));
    kvc_row_mover* mover = nullptr;
    KVC_OK_OR_DIE(kvc_row_mover_create(2, &mover));
    HIP_OK(hipMemcpyAsync(landing, d_rows, fresh.size() * 2, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipEventRecord(landed, stream));
    const int64_t ticket = kvc_row_mover_submit(mover, landed, host_pool.data(), nhb, L * blk_bytes, 2 * blk_bytes,
                                                landing, ids.data(), n, blk_bytes, 1);
    if (ticket != 0) { std::fprintf(stderr, "kvc_row_mover_submit: %s\n", kvc_last_error_string()); return 5; }
    KVC_OK_OR_DIE(kvc_row_mover_wait(mover, ticket));
    for (int64_t i = 0; i < n; ++i)
      std::memcpy(&want_p[(size_t)((ids[i] * L + 2) * blk_elems)], &fresh[(size_t)(i * blk_elems)], blk_bytes);
    expect_equal("kvc_row_mover job after an event", host_pool.data(), want_p.data(), host_pool.size() * 2);
    KVC_OK_OR_DIE(kvc_row_mover_destroy(mover));
    HIP_OK(hipEventDestroy(landed));
    HIP_OK(hipFree(d_rows));
    KVC_OK_OR_DIE(kvc_host_free_pinned(landing));
  }

  KVC_OK_OR_DIE(kvc_thread_release());
  HIP_OK(hipDeviceSynchronize());
  if (fails) {
    std::printf("ABI CHECK FAILED (%d mismatches)\n", fails);
    return 1;
  }
  std::printf("ABI CHECK PASSED\n");
  return 0;
}

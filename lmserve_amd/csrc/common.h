// Helpers shared by the translation units of libkvcache.
#ifndef KVC_COMMON_H_
#define KVC_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kvcache.h"

namespace kvc {

// Records the message for kvc_last_error_string() on this thread and returns `code`.
int fail(int code, const char* fmt, ...);

inline int log2_exact(int64_t x) {
  if (x <= 0 || (x & (x - 1))) return -1;
  int s = 0;
  while ((int64_t(1) << s) < x) ++s;
  return s;
}

// Launch shape of the rotation kernel, set through kvc_set_tuning
// ("rope_threads": 64/128/256 lanes per workgroup, 0 = by size; "rope_nt":
// non-temporal loads, bit 0 the K and V rows, bit 1 the Q rows). Off by default:
// with both bits a launch whose Q/K/V come from HBM gains 7-9 % (9.25 against
// 9.94 us per layer at a 2048-token chunk over 28 distinct source sets), but
// a forward pass hands the kernel rows its projection has just written, and
// with sources that are still in cache the same launch is 10 % slower (8.77
// against 7.95 us) and a 256-token decode launch is unchanged.
struct RopeTuning {
  int threads = 0;
  int nt = 0;
};
extern RopeTuning g_rope_tune;

// One launch on `stream`: slots[t] = page * page_size + entry of token t of a
// page-table write, or -1 where that write would skip the token.
int launch_resolve_slots(const char* fn, const int32_t* batch_indices, const int32_t* positions,
                         const int32_t* kv_indices, const int32_t* kv_indptr, int64_t batch_size,
                         int64_t num_kv_indices, int64_t page_size, int64_t nnz, int64_t* slots,
                         hipStream_t stream);

// MiB of aligned staging per thread in the disk tier ("disk_bounce_mib").
extern int g_disk_bounce_mib;

// Row copies on host threads ("host_rows_nt"): 1 = stores that go past the cache.
extern int g_host_rows_nt;

}  // namespace kvc

#define KVC_HIP(call)                                                          \
  do {                                                                         \
    hipError_t e_ = (call);                                                    \
    if (e_ != hipSuccess)                                                      \
      return kvc::fail(KVC_ERR_HIP, "%s failed: %s (%s:%d)", #call,            \
                       hipGetErrorString(e_), __FILE__, __LINE__);             \
  } while (0)

#endif  // KVC_COMMON_H_

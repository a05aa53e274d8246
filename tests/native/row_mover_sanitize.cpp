// Host-only driver for sanitizer builds of the row mover (csrc/host_rows.cpp):
// jobs triggered by host flags from several threads, a wait that times out, a
// cancel from another thread, and a destroy with waiting jobs queued. No GPU.
// Built and run by tests/test_host_sanitizers.py with -fsanitize=thread and
// -fsanitize=address,undefined; exits with the number of wrong results.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>
#include <chrono>
#include "kvcache.h"
#include "kvcache_experimental.h"
namespace kvc {
// the library's error recorder lives in the GPU source file; this build has only the host file
int fail(int code, const char* fmt, ...) { (void)fmt; return code; }
}
int main() {
  const int64_t nhb = 64, L = 4, row = 4096, blk = L * row;
  std::vector<char> pool(nhb * blk, 0), dense(16 * row);
  for (size_t i = 0; i < dense.size(); ++i) dense[i] = (char)(i * 7);
  kvc_row_mover* m = nullptr;
  if (kvc_row_mover_create(4, &m) != 0) return 1;
  int bad = 0;
  // 1) many jobs from two submitting threads, flags set by a third
  std::vector<int32_t> flags(64, 0);
  std::vector<int64_t> tickets(64, -1);
  auto submitter = [&](int lo, int hi) {
    for (int j = lo; j < hi; ++j) {
      int64_t ids[16];
      for (int i = 0; i < 16; ++i) ids[i] = (i * 4 + j) % nhb;   // distinct inside a job
      tickets[j] = kvc_row_mover_submit_after_flag(m, &flags[j], pool.data(), nhb, blk, (j % L) * row, dense.data(), ids, 16, row, 1);
    }
  };
  std::thread a(submitter, 0, 32), b(submitter, 32, 64);
  std::thread setter([&] {
    for (int j = 0; j < 64; ++j) {
      std::this_thread::sleep_for(std::chrono::microseconds(200));
      __atomic_store_n(&flags[j], 1, __ATOMIC_RELEASE);
    }
  });
  a.join(); b.join(); setter.join();
  for (int j = 0; j < 64; ++j) if (tickets[j] < 0 || kvc_row_mover_wait(m, tickets[j]) != 0) ++bad;
  // 2) a job whose flag never comes: timeout, then the queued ones are skipped
  kvc_row_mover_set_timeout_ms(m, 50);
  int32_t never = 0, yes = 1;
  int64_t ids[2] = {1, 2};
  int64_t t1 = kvc_row_mover_submit_after_flag(m, &never, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  int64_t t2 = kvc_row_mover_submit_after_flag(m, &yes, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  int r1 = kvc_row_mover_wait(m, t1);
  int r2 = kvc_row_mover_wait(m, t2);
  if (r1 != KVC_ERR_TIMEOUT) ++bad;
  (void)r2;
  int64_t t3 = kvc_row_mover_submit_after_flag(m, &yes, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  if (kvc_row_mover_wait(m, t3) != 0) { /* status of t2 (cancelled) may surface here */ }
  int64_t t3b = kvc_row_mover_submit_after_flag(m, &yes, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  if (kvc_row_mover_wait(m, t3b) != 0) ++bad;
  // 3) cancel from another thread while a job waits
  kvc_row_mover_set_timeout_ms(m, 5000);
  int64_t t4 = kvc_row_mover_submit_after_flag(m, &never, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  std::thread c([&] { std::this_thread::sleep_for(std::chrono::milliseconds(20)); kvc_row_mover_cancel(m); });
  int r4 = kvc_row_mover_wait(m, t4);
  c.join();
  if (r4 != KVC_ERR_CANCELLED) ++bad;
  // 4) destroy with a waiting job queued
  kvc_row_mover_set_timeout_ms(m, 100);
  kvc_row_mover_submit_after_flag(m, &never, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  kvc_row_mover_submit_after_flag(m, &never, pool.data(), nhb, blk, 0, dense.data(), ids, 2, row, 1);
  kvc_row_mover_destroy(m);
  std::printf("bad=%d\n", bad);
  return bad;
}

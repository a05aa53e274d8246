// libkvcache, host rows: one layer of many blocks between a dense pinned buffer
// and the host pool, moved by host threads.
//
// The host pool is [num_host_blocks, L, block] (kv_worker.py:123-127 of the
// reference): one layer of one block is a row of `block` bytes, and the rows of
// one layer of scattered blocks lie a whole host block or more apart. The copy
// engines pay about 10 us per such row; a kernel that stores them over PCIe
// holds back the kernels of every other stream while it runs. Here the PCIe leg
// of a layer is ONE copy between the GPU and a dense pinned buffer, and the rows
// go between that buffer and their places in the pool on a few host threads
// (one thread moves about 23 GB/s of 64 KiB rows, four match the link).
//
// No GPU work in this file.

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <deque>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "kvcache.h"
#include "kvcache_experimental.h"

namespace kvc {
int fail(int code, const char* fmt, ...);
}

namespace {
using kvc::fail;

struct RowCopy {
  char* pool;   // host pool + offset of the layer inside a block
  int64_t num_host_blocks, pool_block_bytes;
  char* dense;
  const int64_t* host_ids;
  int64_t n, row_bytes;
  int to_pool;
};

int check_rows(const char* fn, const void* host_pool, int64_t num_host_blocks, int64_t pool_block_bytes,
               int64_t pool_offset, const void* dense, const int64_t* host_ids, int64_t n,
               int64_t row_bytes) {
  if (n < 0 || row_bytes < 0 || num_host_blocks < 0 || pool_block_bytes < 0 || pool_offset < 0)
    return fail(KVC_ERR_INVALID_ARG, "%s: negative size", fn);
  if (n == 0 || row_bytes == 0) return KVC_OK;
  if (!host_pool || !dense || !host_ids) return fail(KVC_ERR_INVALID_ARG, "%s: null pointer", fn);
  if (pool_offset + row_bytes > pool_block_bytes)
    return fail(KVC_ERR_INVALID_ARG, "%s: row [%lld, %lld) outside a host block of %lld bytes", fn,
                (long long)pool_offset, (long long)(pool_offset + row_bytes), (long long)pool_block_bytes);
  for (int64_t i = 0; i < n; ++i)
    if (host_ids[i] < 0 || host_ids[i] >= num_host_blocks)
      return fail(KVC_ERR_OUT_OF_RANGE, "%s: host block id %lld (entry %lld) outside [0, %lld)", fn,
                  (long long)host_ids[i], (long long)i, (long long)num_host_blocks);
  return KVC_OK;
}

// the rows of one call on `threads` host threads (this thread is one of them); false = out of memory
bool copy_rows(const RowCopy& c, int threads) {
  // rows are handed out in runs of 8 so that a thread stays on neighbouring dense rows
  constexpr int64_t kRun = 8;
  std::atomic<int64_t> next{0};
  const auto work = [&]() {
    for (;;) {
      const int64_t first = next.fetch_add(kRun, std::memory_order_relaxed);
      if (first >= c.n) return;
      const int64_t last = std::min(c.n, first + kRun);
      for (int64_t i = first; i < last; ++i) {
        char* p = c.pool + c.host_ids[i] * c.pool_block_bytes;
        char* d = c.dense + i * c.row_bytes;
        if (c.to_pool) std::memcpy(p, d, (size_t)c.row_bytes);
        else std::memcpy(d, p, (size_t)c.row_bytes);
      }
    }
  };
  // a thread per MiB at most: small calls are not worth starting threads for
  int64_t nthreads = threads > 0 ? threads : 4;
  nthreads = std::min<int64_t>(nthreads, std::max<int64_t>(1, c.n * c.row_bytes >> 20));
  nthreads = std::min<int64_t>(nthreads, (c.n + kRun - 1) / kRun);
  if (nthreads <= 1) {
    work();
    return true;
  }
  std::vector<std::thread> helpers;
  try {
    helpers.reserve((size_t)nthreads - 1);
  } catch (...) {
    return false;
  }
  try {
    for (int64_t t = 1; t < nthreads; ++t) helpers.emplace_back(work);
  } catch (...) {
    // fewer threads than asked for: the ones that started and this one finish the rows
  }
  work();
  for (auto& t : helpers) t.join();
  return true;
}

}  // namespace

// ---- a queue of row copies, each after an event --------------------------------
struct kvc_row_mover {
  struct Job {
    RowCopy copy;
    std::vector<int64_t> ids;
    hipEvent_t after = nullptr;               // wait for this event of `device` first, or
    const volatile int32_t* flag = nullptr;   // for this host word to become non-zero
    int device = 0;
    int64_t ticket = 0;
  };
  std::mutex mu;
  std::condition_variable has_jobs, progressed;
  std::deque<Job> jobs;
  int64_t next_ticket = 0, done_ticket = -1;
  int status = KVC_OK;   // of the first job that failed since the last kvc_row_mover_wait
  char error[256] = "";
  bool stopping = false;
  int threads = 4;
  // A job's wait gives up after this long (KVC_ERR_TIMEOUT) or when kvc_row_mover_cancel
  // is called (KVC_ERR_CANCELLED). Either way the rows of that job stay where they are,
  // and so do those of every job that was already queued behind it (they wait for work
  // of the same stream): tickets below `skip_below` complete at once, without copying.
  // Jobs submitted after that run as usual.
  std::atomic<int64_t> timeout_ms{30000};
  std::atomic<bool> cancel{false};
  int64_t skip_below = 0;
  std::thread dispatcher;

  // KVC_OK once the job's condition holds; the caller's thread sleeps in 20 us steps
  // (hipEventSynchronize would spin on a core for an event made without the
  // blocking-sync flag, and the caller's events are torch's)
  int wait_for(const Job& job, char* text, size_t text_len) {
    if (!job.after && !job.flag) return KVC_OK;
    if (job.after) {
      const hipError_t e = hipSetDevice(job.device);
      if (e != hipSuccess) {
        std::snprintf(text, text_len, "kvc_row_mover: hipSetDevice failed: %s", hipGetErrorString(e));
        return KVC_ERR_HIP;
      }
    }
    const auto begin = std::chrono::steady_clock::now();
    for (;;) {
      if (job.after) {
        const hipError_t e = hipEventQuery(job.after);
        if (e == hipSuccess) return KVC_OK;
        if (e != hipErrorNotReady) {
          std::snprintf(text, text_len, "kvc_row_mover: waiting for the event failed: %s", hipGetErrorString(e));
          return KVC_ERR_HIP;
        }
      } else if (__atomic_load_n(job.flag, __ATOMIC_ACQUIRE) != 0) {
        return KVC_OK;
      }
      if (cancel.load(std::memory_order_acquire)) {
        std::snprintf(text, text_len, "kvc_row_mover: cancelled while job %lld waited", (long long)job.ticket);
        return KVC_ERR_CANCELLED;
      }
      const int64_t limit = timeout_ms.load(std::memory_order_relaxed);
      const auto waited = std::chrono::duration_cast<std::chrono::milliseconds>(
                              std::chrono::steady_clock::now() - begin).count();
      if (limit >= 0 && waited >= limit) {
        std::snprintf(text, text_len, "kvc_row_mover: job %lld: %s not reached after %lld ms", (long long)job.ticket,
                      job.after ? "event" : "host flag", (long long)waited);
        return KVC_ERR_TIMEOUT;
      }
      std::this_thread::sleep_for(std::chrono::microseconds(20));
    }
  }

  void run() {
    for (;;) {
      Job job;
      {
        std::unique_lock<std::mutex> lock(mu);
        has_jobs.wait(lock, [&] { return stopping || !jobs.empty(); });
        if (jobs.empty()) return;   // stopping, and nothing left to do
        job = std::move(jobs.front());
        jobs.pop_front();
      }
      int rc = KVC_OK;
      char text[256] = "";
      bool skip;
      {
        std::lock_guard<std::mutex> lock(mu);
        skip = job.ticket < skip_below;
        if (!skip) cancel.store(false, std::memory_order_release);   // a job newer than the last cancel
      }
      if (skip) {
        rc = KVC_ERR_CANCELLED;
        std::snprintf(text, sizeof text, "kvc_row_mover: job %lld skipped after an earlier job gave up",
                      (long long)job.ticket);
      } else {
        rc = wait_for(job, text, sizeof text);
      }
      if (rc == KVC_OK) {
        job.copy.host_ids = job.ids.data();
        if (!copy_rows(job.copy, threads)) {
          rc = KVC_ERR_HIP;
          std::snprintf(text, sizeof text, "kvc_row_mover: out of host memory");
        }
      }
      {
        std::lock_guard<std::mutex> lock(mu);
        if (rc != KVC_OK && status == KVC_OK) {
          status = rc;
          std::memcpy(error, text, sizeof error);
        }
        if (rc == KVC_ERR_TIMEOUT) skip_below = next_ticket;   // everything queued so far stays where it is
        done_ticket = job.ticket;
      }
      progressed.notify_all();
    }
  }
};

extern "C" {

int kvc_row_mover_create(int threads, kvc_row_mover** out) {
  if (!out) return fail(KVC_ERR_INVALID_ARG, "kvc_row_mover_create: null out");
  *out = nullptr;
  kvc_row_mover* m = new (std::nothrow) kvc_row_mover;
  if (!m) return fail(KVC_ERR_HIP, "kvc_row_mover_create: out of host memory");
  m->threads = threads > 0 ? threads : 4;
  try {
    m->dispatcher = std::thread([m] { m->run(); });
  } catch (...) {
    delete m;
    return fail(KVC_ERR_HIP, "kvc_row_mover_create: cannot start a thread");
  }
  *out = m;
  return KVC_OK;
}

static int64_t submit_job(const char* fn, kvc_row_mover* mover, void* after_event, const int32_t* flag,
                          void* host_pool, int64_t num_host_blocks, int64_t pool_block_bytes,
                          int64_t pool_offset, void* dense, const int64_t* host_ids, int64_t n,
                          int64_t row_bytes, int to_pool) {
  if (!mover) return fail(KVC_ERR_INVALID_ARG, "%s: null mover", fn);
  const int rc = check_rows(fn, host_pool, num_host_blocks, pool_block_bytes, pool_offset, dense, host_ids,
                            n, row_bytes);
  if (rc != KVC_OK) return rc;
  kvc_row_mover::Job job;
  job.after = (hipEvent_t)after_event;
  job.flag = flag;
  job.device = 0;
  if (after_event && hipGetDevice(&job.device) != hipSuccess)
    return fail(KVC_ERR_HIP, "%s: hipGetDevice failed", fn);
  try {
    if (n > 0 && row_bytes > 0) job.ids.assign(host_ids, host_ids + n);
  } catch (...) {
    return fail(KVC_ERR_HIP, "%s: out of host memory", fn);
  }
  const int64_t rows = (n > 0 && row_bytes > 0) ? n : 0;
  job.copy = RowCopy{host_pool ? (char*)host_pool + pool_offset : nullptr, num_host_blocks, pool_block_bytes,
                     (char*)dense, nullptr, rows, row_bytes, to_pool};
  int64_t ticket;
  {
    std::lock_guard<std::mutex> lock(mover->mu);
    if (mover->stopping) return fail(KVC_ERR_INVALID_ARG, "%s: the mover is being destroyed", fn);
    ticket = job.ticket = mover->next_ticket++;
    try {
      mover->jobs.push_back(std::move(job));
    } catch (...) {
      --mover->next_ticket;
      return fail(KVC_ERR_HIP, "%s: out of host memory", fn);
    }
  }
  mover->has_jobs.notify_one();
  return ticket;
}

int64_t kvc_row_mover_submit(kvc_row_mover* mover, void* after_event, void* host_pool,
                             int64_t num_host_blocks, int64_t pool_block_bytes, int64_t pool_offset,
                             void* dense, const int64_t* host_ids, int64_t n, int64_t row_bytes,
                             int to_pool) {
  return submit_job("kvc_row_mover_submit", mover, after_event, nullptr, host_pool, num_host_blocks,
                    pool_block_bytes, pool_offset, dense, host_ids, n, row_bytes, to_pool);
}

int64_t kvc_row_mover_submit_after_flag(kvc_row_mover* mover, const int32_t* flag, void* host_pool,
                                        int64_t num_host_blocks, int64_t pool_block_bytes,
                                        int64_t pool_offset, void* dense, const int64_t* host_ids,
                                        int64_t n, int64_t row_bytes, int to_pool) {
  return submit_job("kvc_row_mover_submit_after_flag", mover, nullptr, flag, host_pool, num_host_blocks,
                    pool_block_bytes, pool_offset, dense, host_ids, n, row_bytes, to_pool);
}

int kvc_row_mover_set_timeout_ms(kvc_row_mover* mover, int64_t timeout_ms) {
  if (!mover) return fail(KVC_ERR_INVALID_ARG, "kvc_row_mover_set_timeout_ms: null mover");
  mover->timeout_ms.store(timeout_ms, std::memory_order_relaxed);
  return KVC_OK;
}

int kvc_row_mover_cancel(kvc_row_mover* mover) {
  if (!mover) return fail(KVC_ERR_INVALID_ARG, "kvc_row_mover_cancel: null mover");
  std::lock_guard<std::mutex> lock(mover->mu);
  mover->skip_below = mover->next_ticket;                  // every job submitted so far
  mover->cancel.store(true, std::memory_order_release);    // the one that is waiting right now
  return KVC_OK;
}

int kvc_row_mover_done(kvc_row_mover* mover, int64_t ticket) {
  if (!mover) return fail(KVC_ERR_INVALID_ARG, "kvc_row_mover_done: null mover");
  std::lock_guard<std::mutex> lock(mover->mu);
  return mover->done_ticket >= ticket ? 1 : 0;
}

int kvc_row_mover_wait(kvc_row_mover* mover, int64_t ticket) {
  if (!mover) return fail(KVC_ERR_INVALID_ARG, "kvc_row_mover_wait: null mover");
  std::unique_lock<std::mutex> lock(mover->mu);
  if (ticket >= mover->next_ticket)
    return fail(KVC_ERR_INVALID_ARG, "kvc_row_mover_wait: ticket %lld was never handed out", (long long)ticket);
  mover->progressed.wait(lock, [&] { return mover->done_ticket >= ticket; });
  const int rc = mover->status;
  if (rc != KVC_OK) {
    mover->status = KVC_OK;
    return fail(rc, "%s", mover->error);
  }
  return KVC_OK;
}

int kvc_row_mover_destroy(kvc_row_mover* mover) {
  if (!mover) return KVC_OK;
  {
    std::lock_guard<std::mutex> lock(mover->mu);
    mover->stopping = true;
  }
  mover->has_jobs.notify_all();
  if (mover->dispatcher.joinable()) mover->dispatcher.join();   // after the jobs still queued
  delete mover;
  return KVC_OK;
}

int kvc_host_copy_rows(void* host_pool, int64_t num_host_blocks, int64_t pool_block_bytes,
                       int64_t pool_offset, void* dense, const int64_t* host_ids, int64_t n,
                       int64_t row_bytes, int to_pool, int threads) {
  const char* fn = "kvc_host_copy_rows";
  const int rc = check_rows(fn, host_pool, num_host_blocks, pool_block_bytes, pool_offset, dense, host_ids,
                            n, row_bytes);
  if (rc != KVC_OK) return rc;
  if (n == 0 || row_bytes == 0) return KVC_OK;
  const RowCopy c{(char*)host_pool + pool_offset, num_host_blocks, pool_block_bytes, (char*)dense, host_ids, n,
                  row_bytes, to_pool};
  if (!copy_rows(c, threads)) return fail(KVC_ERR_HIP, "%s: out of host memory", fn);
  return KVC_OK;
}

}  // extern "C"


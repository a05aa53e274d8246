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
// (into the pool one thread moves about 50 GB/s of 64 KiB rows and four 130-150,
// into the dense buffer 26 and 77; the link carries 55).
//
// No GPU work in this file.

#include <emmintrin.h>
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
int g_host_rows_nt = 1;
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

// One row. A row is written once and read next by a copy engine, a disk write
// or another process, never by this thread: when both ends are 64-byte aligned the
// stores go past the cache (16-byte non-temporal stores, a cache line at a time),
// which saves the read of the destination line a cached store starts with.
inline void copy_row(char* dst, const char* src, int64_t bytes, bool stream) {
  if (!stream || (((uintptr_t)dst | (uintptr_t)src | (uint64_t)bytes) & 63u) != 0) {
    std::memcpy(dst, src, (size_t)bytes);
    return;
  }
  const __m128i* s = reinterpret_cast<const __m128i*>(src);
  __m128i* d = reinterpret_cast<__m128i*>(dst);
  for (int64_t i = 0; i < bytes / 16; i += 4) {
    const __m128i a = _mm_load_si128(s + i), b = _mm_load_si128(s + i + 1);
    const __m128i c = _mm_load_si128(s + i + 2), e = _mm_load_si128(s + i + 3);
    _mm_stream_si128(d + i, a);
    _mm_stream_si128(d + i + 1, b);
    _mm_stream_si128(d + i + 2, c);
    _mm_stream_si128(d + i + 3, e);
  }
}

// Rows are handed out in runs of 8 so that a thread stays on neighbouring dense rows.
constexpr int64_t kRun = 8;
inline void copy_rows_share(const RowCopy& c, std::atomic<int64_t>& next, bool stream) {
  for (;;) {
    const int64_t first = next.fetch_add(kRun, std::memory_order_relaxed);
    if (first >= c.n) break;
    const int64_t last = std::min(c.n, first + kRun);
    for (int64_t i = first; i < last; ++i) {
      char* p = c.pool + c.host_ids[i] * c.pool_block_bytes;
      char* d = c.dense + i * c.row_bytes;
      if (c.to_pool) copy_row(p, d, c.row_bytes, stream);
      else copy_row(d, p, c.row_bytes, stream);
    }
  }
  // non-temporal stores are ordered by nothing else before the rows are handed on
  if (stream) _mm_sfence();
}

// threads worth starting for a call: one per MiB at most, one per run of rows at most
inline int64_t useful_threads(const RowCopy& c, int threads) {
  int64_t nthreads = threads > 0 ? threads : 4;
  nthreads = std::min<int64_t>(nthreads, std::max<int64_t>(1, c.n * c.row_bytes >> 20));
  return std::min<int64_t>(nthreads, std::max<int64_t>(1, (c.n + kRun - 1) / kRun));
}

// the rows of one call on `threads` host threads (this thread is one of them); false = out of memory
bool copy_rows(const RowCopy& c, int threads) {
  std::atomic<int64_t> next{0};
  const bool stream = kvc::g_host_rows_nt != 0;
  const auto work = [&]() { copy_rows_share(c, next, stream); };
  const int64_t nthreads = useful_threads(c, threads);
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

  // Helper threads that live as long as the mover (a job of one layer lasts a few
  // hundred microseconds: starting threads for each would cost a fifth of that).
  // The dispatcher publishes a job under `team_mu`, takes a share of the rows
  // itself and waits until the helpers it asked for have finished theirs.
  std::mutex team_mu;
  std::condition_variable team_start, team_finished;
  std::vector<std::thread> helpers;
  const RowCopy* team_job = nullptr;
  std::atomic<int64_t> team_next{0};
  bool team_stream = false;
  uint64_t team_generation = 0;
  int team_wanted = 0, team_running = 0;
  bool team_stop = false;

  void helper_main(int index) {
    uint64_t seen = 0;
    for (;;) {
      const RowCopy* job;
      bool stream;
      {
        std::unique_lock<std::mutex> lock(team_mu);
        team_start.wait(lock, [&] { return team_stop || team_generation != seen; });
        if (team_stop) return;
        seen = team_generation;
        if (index >= team_wanted) continue;   // a small job: not every helper is asked
        job = team_job;
        stream = team_stream;
      }
      copy_rows_share(*job, team_next, stream);
      {
        std::lock_guard<std::mutex> lock(team_mu);
        --team_running;
      }
      team_finished.notify_one();
    }
  }

  void start_helpers() {
    try {
      for (int i = 0; i + 1 < threads; ++i) helpers.emplace_back([this, i] { helper_main(i); });
    } catch (...) {
      // fewer helpers than asked for: the jobs run on those that started
    }
  }

  void stop_helpers() {
    {
      std::lock_guard<std::mutex> lock(team_mu);
      team_stop = true;
    }
    team_start.notify_all();
    for (auto& t : helpers) t.join();
    helpers.clear();
  }

  // the rows of one job on the dispatcher and as many helpers as the job is worth
  void team_copy(const RowCopy& c) {
    const bool stream = kvc::g_host_rows_nt != 0;
    const int wanted = (int)std::min<int64_t>(useful_threads(c, threads) - 1, (int64_t)helpers.size());
    team_next.store(0, std::memory_order_relaxed);
    if (wanted > 0) {
      {
        std::lock_guard<std::mutex> lock(team_mu);
        team_job = &c;
        team_stream = stream;
        team_wanted = team_running = wanted;
        ++team_generation;
      }
      team_start.notify_all();
    }
    copy_rows_share(c, team_next, stream);
    if (wanted > 0) {
      std::unique_lock<std::mutex> lock(team_mu);
      team_finished.wait(lock, [&] { return team_running == 0; });
    }
  }

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
        team_copy(job.copy);
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
  m->start_helpers();
  try {
    m->dispatcher = std::thread([m] { m->run(); });
  } catch (...) {
    m->stop_helpers();
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
  mover->stop_helpers();
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


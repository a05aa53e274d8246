// Host <-> disk tier of the KV cache: whole blocks between the pinned host
// pool and a block file, as large positional reads/writes on a few threads.
//
// Follows runtime/worker/llm_worker/kv_worker.py:
//   :48-85   memmap_disk_kv_cache   -- a NumPy `.npy` file of shape
//            (num_disk_blocks, L, block_elems); reused when its stored shape and
//            dtype match, recreated otherwise
//   :229-247 _load/_save_layer_kv_blocks_*_disk -- host[dst][l] = disk[src][l]
//            and disk[dst][l] = host[src][l], one (block, layer) row at a time
//   :297-322 one task per layer on a 4-thread pool
//
// A block's L layers are contiguous in both pools ([block][layer][elems]), so a
// block is ONE extent of L * block_bytes here (5 MiB for Llama-3.1-70B) instead
// of L row copies through a memory map, and neighbouring (src, dst) pairs merge
// into longer extents. The file stays a valid `.npy` (any NumPy reader can map
// it); files this code creates pad the header to 4096 bytes so that every block
// extent is aligned for O_DIRECT, which keeps tens of GiB of KV blocks out of
// the page cache. No GPU work in this file.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <utility>
#include <vector>

#include "kvcache.h"

namespace kvc {
int fail(int code, const char* fmt, ...);
int g_disk_bounce_mib = 4;  // per-thread staging of an O_DIRECT transfer (kvc_set_tuning "disk_bounce_mib")
}
using kvc::fail;

struct kvc_disk {
  int fd = -1;          // buffered descriptor
  int fd_direct = -1;   // O_DIRECT descriptor, -1 when the file system refuses it
  int64_t data_offset = 0;
  int64_t num_blocks = 0;
  int64_t row_bytes = 0;  // one block, all layers
  bool created = false;
  bool aligned = false;   // data_offset and row_bytes are multiples of kAlign
  // Host pool whose pages O_DIRECT could not take in place (EFAULT): memory the
  // GPU driver maps for pinning is such memory. Its transfers go through an
  // aligned bounce buffer per thread from then on.
  // Atomics: save and load calls may run on one handle from two threads.
  std::atomic<const void*> bounce_pool{nullptr};
  std::atomic<bool> last_bounced{false};
  std::string path;

  // Staging buffers of O_DIRECT transfers, kept with the handle so a call does
  // not fault fresh pages in every time: 2 MiB-aligned and advised as huge pages
  // (large physically contiguous segments make large block requests), touched
  // once when made.
  std::mutex stage_lock;
  std::vector<std::pair<char*, int64_t>> stages;

  char* take_stage(int64_t bytes) {
    {
      std::lock_guard<std::mutex> g(stage_lock);
      for (size_t i = 0; i < stages.size(); ++i) {
        if (stages[i].second == bytes) {
          char* p = stages[i].first;
          stages.erase(stages.begin() + (long)i);
          return p;
        }
      }
    }
    void* mem = nullptr;
    const size_t huge = size_t(2) << 20;
    const size_t size = ((size_t)bytes + huge - 1) / huge * huge;
    if (posix_memalign(&mem, huge, size) != 0) return nullptr;
    (void)madvise(mem, size, MADV_HUGEPAGE);
    memset(mem, 0, size);
    return static_cast<char*>(mem);
  }
  void give_stage(char* p, int64_t bytes) {
    std::lock_guard<std::mutex> g(stage_lock);
    if (stages.size() < 64) stages.emplace_back(p, bytes);
    else free(p);
  }
  ~kvc_disk() {
    for (auto& st : stages) free(st.first);
  }
};

namespace {

constexpr int64_t kAlign = 4096;
constexpr int64_t kMaxExtent = int64_t(64) << 20;  // split longer runs so threads share them

// "{'descr': '<u2', 'fortran_order': False, 'shape': (8192, 80, 32768), }" padded
// with spaces and a final newline to `total` bytes including the 10-byte preamble
// (format 1.0: magic, version, little-endian uint16 header length).
std::string npy_header(const char* descr, int64_t nb, int64_t nl, int64_t be, size_t total) {
  char dict[256];
  snprintf(dict, sizeof dict, "{'descr': '%s', 'fortran_order': False, 'shape': (%lld, %lld, %lld), }",
           descr, (long long)nb, (long long)nl, (long long)be);
  std::string h("\x93NUMPY\x01\x00", 8);
  const size_t hlen = total - 10;
  h.push_back((char)(hlen & 0xff));
  h.push_back((char)(hlen >> 8));
  h += dict;
  h.resize(total - 1, ' ');
  h.push_back('\n');
  return h;
}

// Value text after `'key':` in a header dict, trimmed of leading blanks; empty if absent.
std::string dict_value(const std::string& dict, const char* key) {
  const std::string k = std::string("'") + key + "'";
  size_t at = dict.find(k);
  if (at == std::string::npos) return "";
  at = dict.find(':', at + k.size());
  if (at == std::string::npos) return "";
  ++at;
  while (at < dict.size() && dict[at] == ' ') ++at;
  return dict.substr(at);
}

// Reads an existing file's `.npy` header. Returns true and fills the outputs when
// it is a C-order array; versions 1.0, 2.0 and 3.0 are understood.
bool parse_npy(int fd, std::string* descr, std::vector<int64_t>* shape, int64_t* data_offset) {
  unsigned char pre[12];
  if (pread(fd, pre, 10, 0) != 10 || memcmp(pre, "\x93NUMPY", 6) != 0) return false;
  size_t hlen, hoff;
  if (pre[6] == 1) {
    hlen = pre[8] | (size_t(pre[9]) << 8);
    hoff = 10;
  } else if (pre[6] == 2 || pre[6] == 3) {
    if (pread(fd, pre, 12, 0) != 12) return false;
    hlen = pre[8] | (size_t(pre[9]) << 8) | (size_t(pre[10]) << 16) | (size_t(pre[11]) << 24);
    hoff = 12;
  } else {
    return false;
  }
  if (hlen == 0 || hlen > (1u << 20)) return false;
  std::string dict(hlen, '\0');
  if (pread(fd, &dict[0], hlen, (off_t)hoff) != (ssize_t)hlen) return false;
  std::string d = dict_value(dict, "descr");
  if (d.size() < 3 || (d[0] != '\'' && d[0] != '"')) return false;
  const size_t q = d.find(d[0], 1);
  if (q == std::string::npos) return false;
  *descr = d.substr(1, q - 1);
  if (dict_value(dict, "fortran_order").compare(0, 5, "False") != 0) return false;
  std::string s = dict_value(dict, "shape");
  if (s.empty() || s[0] != '(') return false;
  const size_t close = s.find(')');
  if (close == std::string::npos) return false;
  shape->clear();
  const char* p = s.c_str() + 1;
  const char* end = s.c_str() + close;
  while (p < end) {
    while (p < end && (*p == ' ' || *p == ',')) ++p;
    if (p >= end) break;
    char* stop = nullptr;
    const long long v = strtoll(p, &stop, 10);
    if (stop == p || v < 0) return false;
    shape->push_back(v);
    p = stop;
  }
  *data_offset = (int64_t)(hoff + hlen);
  return true;
}

int write_all(int fd, const char* p, int64_t n, int64_t off) {
  while (n > 0) {
    const ssize_t w = pwrite(fd, p, (size_t)n, (off_t)off);
    if (w < 0) {
      if (errno == EINTR) continue;
      return errno ? errno : EIO;
    }
    p += w; off += w; n -= w;
  }
  return 0;
}

int read_all(int fd, char* p, int64_t n, int64_t off) {
  while (n > 0) {
    const ssize_t r = pread(fd, p, (size_t)n, (off_t)off);
    if (r < 0) {
      if (errno == EINTR) continue;
      return errno ? errno : EIO;
    }
    if (r == 0) return ENODATA;  // file shorter than its header promises
    p += r; off += r; n -= r;
  }
  return 0;
}

// One extent through an aligned staging buffer: the file side stays O_DIRECT, the
// host side is an ordinary memcpy.
int bounce_io(int fd, bool to_disk, char* host, int64_t len, int64_t off, char* stage,
              int64_t stage_bytes) {
  while (len > 0) {
    const int64_t n = std::min(len, stage_bytes);
    int err;
    if (to_disk) {
      memcpy(stage, host, (size_t)n);
      err = write_all(fd, stage, n, off);
    } else {
      err = read_all(fd, stage, n, off);
      if (!err) memcpy(host, stage, (size_t)n);
    }
    if (err) return err;
    host += n; off += n; len -= n;
  }
  return 0;
}

struct Extent {
  int64_t host_row, disk_row, rows;
};

// (host id, disk id) pairs -> extents of consecutive rows on both sides.
std::vector<Extent> merge_extents(const int64_t* host_ids, const int64_t* disk_ids, int64_t n,
                                  int64_t row_bytes) {
  const int64_t max_rows = std::max<int64_t>(1, kMaxExtent / std::max<int64_t>(1, row_bytes));
  std::vector<Extent> out;
  for (int64_t i = 0; i < n;) {
    int64_t j = i + 1;
    while (j < n && j - i < max_rows && host_ids[j] == host_ids[j - 1] + 1 &&
           disk_ids[j] == disk_ids[j - 1] + 1)
      ++j;
    out.push_back({host_ids[i], disk_ids[i], j - i});
    i = j;
  }
  return out;
}

int run_io(const char* fn, kvc_disk* d, bool to_disk, char* host_pool, int64_t num_host_blocks,
           const int64_t* host_ids, const int64_t* disk_ids, int64_t n, int threads) {
  if (!d || d->fd < 0) return fail(KVC_ERR_INVALID_ARG, "%s: disk tier is not open", fn);
  if (n < 0 || num_host_blocks < 0) return fail(KVC_ERR_INVALID_ARG, "%s: negative count", fn);
  if (n == 0) return KVC_OK;
  if (!host_pool || !host_ids || !disk_ids) return fail(KVC_ERR_INVALID_ARG, "%s: null pointer", fn);
  for (int64_t i = 0; i < n; ++i) {
    if (host_ids[i] < 0 || host_ids[i] >= num_host_blocks)
      return fail(KVC_ERR_OUT_OF_RANGE, "%s: host block id %lld at %lld outside [0, %lld)", fn,
                  (long long)host_ids[i], (long long)i, (long long)num_host_blocks);
    if (disk_ids[i] < 0 || disk_ids[i] >= d->num_blocks)
      return fail(KVC_ERR_OUT_OF_RANGE, "%s: disk block id %lld at %lld outside [0, %lld)", fn,
                  (long long)disk_ids[i], (long long)i, (long long)d->num_blocks);
  }
  const std::vector<Extent> ext = merge_extents(host_ids, disk_ids, n, d->row_bytes);
  // O_DIRECT whenever the file geometry allows it; the host side is handed over
  // in place when it is aligned and the kernel can pin its pages, else staged.
  const bool direct = d->fd_direct >= 0 && d->aligned;
  const bool in_place = direct && (reinterpret_cast<uintptr_t>(host_pool) % kAlign) == 0 &&
                        d->bounce_pool.load(std::memory_order_relaxed) != host_pool;
  const int fd = direct ? d->fd_direct : d->fd;
  const int nthreads = (int)std::max<int64_t>(1, std::min<int64_t>({(int64_t)(threads > 0 ? threads : 8),
                                                                   (int64_t)ext.size(), 64}));
  const int64_t stage_bytes = (int64_t)std::max(1, std::min(kvc::g_disk_bounce_mib, 256)) << 20;
  std::atomic<size_t> next{0};
  std::atomic<int> first_errno{0};
  std::atomic<bool> faulted{false};
  auto work = [&]() {
    char* stage = nullptr;
    for (;;) {
      const size_t k = next.fetch_add(1, std::memory_order_relaxed);
      if (k >= ext.size() || first_errno.load(std::memory_order_relaxed)) break;
      const Extent& e = ext[k];
      char* h = host_pool + e.host_row * d->row_bytes;
      const int64_t off = d->data_offset + e.disk_row * d->row_bytes;
      const int64_t len = e.rows * d->row_bytes;
      int err = EFAULT;
      if (!direct || (in_place && !faulted.load(std::memory_order_relaxed)))
        err = to_disk ? write_all(fd, h, len, off) : read_all(fd, h, len, off);
      if (direct && err == EFAULT) {
        if (in_place) faulted.store(true, std::memory_order_relaxed);
        if (!stage) stage = d->take_stage(stage_bytes);
        err = stage ? bounce_io(fd, to_disk, h, len, off, stage, stage_bytes) : ENOMEM;
      }
      if (err) {
        int expected = 0;
        first_errno.compare_exchange_strong(expected, err);
        break;
      }
    }
    if (stage) d->give_stage(stage, stage_bytes);
  };
  if (nthreads == 1) {
    work();
  } else {
    std::vector<std::thread> pool;
    pool.reserve(nthreads - 1);
    for (int t = 1; t < nthreads; ++t) pool.emplace_back(work);
    work();
    for (auto& t : pool) t.join();
  }
  if (faulted.load()) d->bounce_pool.store(host_pool, std::memory_order_relaxed);
  d->last_bounced.store(direct && !(in_place && !faulted.load()), std::memory_order_relaxed);
  if (const int err = first_errno.load())
    return fail(KVC_ERR_IO, "%s: %s of %s failed: %s", fn, to_disk ? "write" : "read", d->path.c_str(),
                strerror(err));
  return KVC_OK;
}

}  // namespace

extern "C" {

int kvc_disk_open(const char* path, const char* descr, int64_t num_blocks, int64_t num_layers,
                  int64_t block_elems, int elem_bytes, int flags, kvc_disk** out) {
  if (!out) return fail(KVC_ERR_INVALID_ARG, "kvc_disk_open: null output");
  *out = nullptr;
  if (!path || !descr || !*path || !*descr) return fail(KVC_ERR_INVALID_ARG, "kvc_disk_open: null or empty string");
  if (num_blocks <= 0 || num_layers <= 0 || block_elems <= 0 || elem_bytes <= 0)
    return fail(KVC_ERR_INVALID_ARG, "kvc_disk_open: sizes must be positive");
  if (strlen(descr) > 16 || strchr(descr, '\''))
    return fail(KVC_ERR_INVALID_ARG, "kvc_disk_open: bad dtype string");
  const int64_t row_bytes = num_layers * block_elems * elem_bytes;
  const int64_t payload = num_blocks * row_bytes;

  std::unique_ptr<kvc_disk> holder(new kvc_disk);
  kvc_disk& d = *holder;
  d.path = path;
  d.num_blocks = num_blocks;
  d.row_bytes = row_bytes;

  // reuse a file whose stored shape and dtype match and which holds all its rows
  int fd = open(path, O_RDWR | O_CLOEXEC);
  if (fd >= 0) {
    std::string have_descr;
    std::vector<int64_t> shape;
    int64_t off = 0;
    struct stat st;
    const bool ok = parse_npy(fd, &have_descr, &shape, &off) && have_descr == descr && shape.size() == 3 &&
                    shape[0] == num_blocks && shape[1] == num_layers && shape[2] == block_elems &&
                    fstat(fd, &st) == 0 && (int64_t)st.st_size >= off + payload;
    if (ok) {
      d.fd = fd;
      d.data_offset = off;
    } else {
      close(fd);
      if (unlink(path) != 0 && errno != ENOENT)
        return fail(KVC_ERR_IO, "kvc_disk_open: cannot remove stale %s: %s", path, strerror(errno));
    }
  } else if (errno != ENOENT) {
    return fail(KVC_ERR_IO, "kvc_disk_open: cannot open %s: %s", path, strerror(errno));
  }
  if (d.fd < 0) {
    fd = open(path, O_RDWR | O_CREAT | O_EXCL | O_CLOEXEC, 0644);
    if (fd < 0) return fail(KVC_ERR_IO, "kvc_disk_open: cannot create %s: %s", path, strerror(errno));
    const std::string h = npy_header(descr, num_blocks, num_layers, block_elems, (size_t)kAlign);
    int err = write_all(fd, h.data(), (int64_t)h.size(), 0);
    if (!err && ftruncate(fd, (off_t)(kAlign + payload)) != 0) err = errno;  // sparse, like open_memmap
    // reserve the blocks now: later writes then meet no allocation in the file
    // system and cannot run out of space half-way
    if (!err && (flags & KVC_DISK_PREALLOCATE)) err = posix_fallocate(fd, 0, (off_t)(kAlign + payload));
    if (err) {
      close(fd);
      unlink(path);
      return fail(KVC_ERR_IO, "kvc_disk_open: cannot size %s: %s", path, strerror(err));
    }
    d.fd = fd;
    d.data_offset = kAlign;
    d.created = true;
  }
  d.aligned = d.data_offset % kAlign == 0 && row_bytes % kAlign == 0;
  if ((flags & KVC_DISK_DIRECT) && d.aligned) d.fd_direct = open(path, O_RDWR | O_DIRECT | O_CLOEXEC);
  *out = holder.release();
  return KVC_OK;
}

int kvc_disk_close(kvc_disk* d) {
  if (!d) return KVC_OK;
  int rc = KVC_OK;
  if (d->fd_direct >= 0) close(d->fd_direct);
  if (d->fd >= 0 && close(d->fd) != 0) rc = fail(KVC_ERR_IO, "kvc_disk_close: %s", strerror(errno));
  delete d;
  return rc;
}

int kvc_disk_sync(kvc_disk* d) {
  if (!d || d->fd < 0) return fail(KVC_ERR_INVALID_ARG, "kvc_disk_sync: disk tier is not open");
  if (fdatasync(d->fd) != 0) return fail(KVC_ERR_IO, "kvc_disk_sync: %s", strerror(errno));
  return KVC_OK;
}

int64_t kvc_disk_info(const kvc_disk* d, int what) {
  if (!d) return -1;
  switch (what) {
    case KVC_DISK_INFO_DATA_OFFSET: return d->data_offset;
    case KVC_DISK_INFO_DIRECT: return d->fd_direct >= 0 ? 1 : 0;
    case KVC_DISK_INFO_CREATED: return d->created ? 1 : 0;
    case KVC_DISK_INFO_ROW_BYTES: return d->row_bytes;
    case KVC_DISK_INFO_NUM_BLOCKS: return d->num_blocks;
    case KVC_DISK_INFO_BOUNCED: return d->last_bounced.load(std::memory_order_relaxed) ? 1 : 0;
    default: return -1;
  }
}

int kvc_disk_save_blocks(kvc_disk* d, const void* host_pool, int64_t num_host_blocks,
                         const int64_t* src_host_ids, const int64_t* dst_disk_ids, int64_t n,
                         int threads) {
  return run_io("kvc_disk_save_blocks", d, true, const_cast<char*>(static_cast<const char*>(host_pool)),
                num_host_blocks, src_host_ids, dst_disk_ids, n, threads);
}

int kvc_disk_load_blocks(kvc_disk* d, void* host_pool, int64_t num_host_blocks,
                         const int64_t* src_disk_ids, const int64_t* dst_host_ids, int64_t n,
                         int threads) {
  return run_io("kvc_disk_load_blocks", d, false, static_cast<char*>(host_pool), num_host_blocks,
                dst_host_ids, src_disk_ids, n, threads);
}

}  // extern "C"

// Host-only driver for sanitizer builds of the disk tier (csrc/disk_tier.cpp):
// a new block file, scattered and consecutive saves and loads on several threads,
// buffered and O_DIRECT descriptors, aligned and unaligned host pools, a reopen
// that reuses the file and one that recreates it, ids out of range. No GPU.
// Built and run by tests/test_host_sanitizers.py; argv[1] = directory for the
// file; exits with the number of wrong results.
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "kvcache.h"

namespace kvc {
// the library's error recorder lives in the GPU source file; this build has only the host file
int fail(int code, const char* fmt, ...) { (void)fmt; return code; }
}

static void fill(std::vector<uint16_t>& v, uint32_t seed) {
  for (size_t i = 0; i < v.size(); ++i) v[i] = (uint16_t)((i * 2654435761u + seed) >> 7);
}

int main(int argc, char** argv) {
  if (argc < 2) return 100;
  const std::string path = std::string(argv[1]) + "/blocks.npy";
  const int64_t nblk = 48, L = 3, elems = 2048, nhb = 32;   // 4 KiB per layer row, 12 KiB per block
  const int64_t row = L * elems;
  int bad = 0;
  for (int flags : {0, (int)KVC_DISK_DIRECT, (int)(KVC_DISK_DIRECT | KVC_DISK_PREALLOCATE)}) {
    for (int misalign : {0, 1}) {
      kvc_disk* d = nullptr;
      std::remove(path.c_str());
      if (kvc_disk_open(path.c_str(), "<u2", nblk, L, elems, 2, flags, &d) != KVC_OK || !d) { ++bad; continue; }
      if (kvc_disk_info(d, KVC_DISK_INFO_CREATED) != 1) ++bad;
      // host pool: 4096-aligned, or off by two bytes
      void* raw = nullptr;
      if (posix_memalign(&raw, 4096, (size_t)(nhb * row * 2 + 4096)) != 0) return 101;
      uint16_t* pool = (uint16_t*)raw + misalign;
      std::vector<uint16_t> image((size_t)(nhb * row));
      fill(image, 17u + (uint32_t)flags);
      std::memcpy(pool, image.data(), image.size() * 2);
      // save: a consecutive run and scattered pairs
      std::vector<int64_t> src, dst;
      for (int64_t i = 0; i < 12; ++i) { src.push_back(4 + i); dst.push_back(20 + i); }
      for (int64_t i = 0; i < 10; ++i) { src.push_back((i * 7 + 1) % nhb); dst.push_back((i * 3 + 1) % 20); }
      if (kvc_disk_save_blocks(d, pool, nhb, src.data(), dst.data(), (int64_t)src.size(), 4) != KVC_OK) ++bad;
      if (kvc_disk_sync(d) != KVC_OK) ++bad;
      // load them back into other host blocks and compare
      std::vector<int64_t> back;
      std::memset(pool, 0, image.size() * 2);
      for (size_t i = 0; i < src.size(); ++i) back.push_back((int64_t)((i * 3 + 2) % nhb));
      // distinct destinations: 22 entries, stride 3 modulo 32 is a permutation prefix
      if (kvc_disk_load_blocks(d, pool, nhb, dst.data(), back.data(), (int64_t)dst.size(), 3) != KVC_OK) ++bad;
      for (size_t i = 0; i < src.size(); ++i)
        if (std::memcmp(pool + back[i] * row, image.data() + src[i] * row, (size_t)row * 2) != 0) { ++bad; break; }
      // ids out of range are refused before any I/O
      int64_t bad_src[1] = {nhb}, ok_dst[1] = {0}, bad_dst[1] = {nblk};
      if (kvc_disk_save_blocks(d, pool, nhb, bad_src, ok_dst, 1, 1) != KVC_ERR_OUT_OF_RANGE) ++bad;
      if (kvc_disk_save_blocks(d, pool, nhb, ok_dst, bad_dst, 1, 1) != KVC_ERR_OUT_OF_RANGE) ++bad;
      if (kvc_disk_close(d) != KVC_OK) ++bad;
      // same shape: reused; another shape: recreated
      if (kvc_disk_open(path.c_str(), "<u2", nblk, L, elems, 2, flags, &d) != KVC_OK) { ++bad; free(raw); continue; }
      if (kvc_disk_info(d, KVC_DISK_INFO_CREATED) != 0) ++bad;
      std::memset(pool, 0, image.size() * 2);
      if (kvc_disk_load_blocks(d, pool, nhb, dst.data(), back.data(), 1, 1) != KVC_OK) ++bad;
      if (std::memcmp(pool + back[0] * row, image.data() + src[0] * row, (size_t)row * 2) != 0) ++bad;
      kvc_disk_close(d);
      if (kvc_disk_open(path.c_str(), "<u2", nblk + 1, L, elems, 2, flags, &d) != KVC_OK) { ++bad; free(raw); continue; }
      if (kvc_disk_info(d, KVC_DISK_INFO_CREATED) != 1) ++bad;
      kvc_disk_close(d);
      free(raw);
    }
  }
  std::remove(path.c_str());
  std::printf("bad=%d\n", bad);
  return bad;
}

// kx_load.hip -- checkpoint files -> HBM (see kx_load.h).
//
// Each reader thread owns one pinned staging buffer and one stream.  It takes the next piece (at
// most 32 MiB of a tensor's 4096-aligned extent), reads it with pread, and copies the part that is
// tensor data to the tensor's place in the arena; while one thread waits for the disk another
// one's copy is on the bus.  The router bias, bf16 in the checkpoint, is widened to f32 on the way.
// Direct I/O cannot target HIP's pinned memory (the kernel refuses to pin those pages again, EFAULT),
// so a file opened with O_DIRECT is read into an ordinary page-aligned buffer and moved to the pinned
// one by the CPU -- the copy a buffered read makes inside the kernel, without filling the page cache
// with a checkpoint that is read once.
#ifndef _GNU_SOURCE
#define _GNU_SOURCE  // O_DIRECT
#endif
#include <errno.h>
#include <fcntl.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>
#include <atomic>
#include <chrono>
#include <mutex>
#include <thread>
#include "kx_load.h"

namespace {

constexpr uint64_t PIECE = 32ull << 20;       // bytes of file per read
constexpr uint64_t WIDEN_MAX = 1ull << 20;    // largest tensor widened on the host
constexpr uint64_t SLOT = PIECE + 2 * WIDEN_MAX;

struct Piece {
  int fd;
  bool direct;       // fd was opened with O_DIRECT
  uint64_t at, len;  // file range read, both multiples of the extent's alignment
  uint64_t d0, d1;   // file range of the tensor data inside it
  char *dst;
  bool widen;
  const KxTensorRec *t;
};

struct Shared {
  std::vector<Piece> pieces;
  std::atomic<size_t> next{0};
  std::atomic<bool> failed{false};
  std::atomic<uint64_t> copied{0};
  std::mutex mu;
  std::string error;
  int device = 0;
  void fail(const std::string &msg) {
    std::lock_guard<std::mutex> g(mu);
    if (!failed.exchange(true)) error = msg;
  }
};

void reader(Shared *sh) {
  char *slot = nullptr, *bounce = nullptr;
  hipStream_t st = nullptr;
  auto hip_ok = [&](hipError_t e, const char *what) {
    if (e == hipSuccess) return true;
    sh->fail(std::string("kx_model_load: ") + what + ": " + hipGetErrorString(e));
    return false;
  };
  if (!hip_ok(hipSetDevice(sh->device), "hipSetDevice")) return;
  if (!hip_ok(hipHostMalloc((void **)&slot, SLOT, hipHostMallocDefault), "hipHostMalloc")) return;
  if (hip_ok(hipStreamCreate(&st), "hipStreamCreate")) {
    for (;;) {
      const size_t i = sh->next.fetch_add(1);
      if (i >= sh->pieces.size() || sh->failed.load()) break;
      const Piece &p = sh->pieces[i];
      uint64_t got = 0;
      bool io_ok = true;
      if (p.direct && !bounce && posix_memalign((void **)&bounce, 4096, PIECE)) {
        bounce = nullptr;
        sh->fail("kx_model_load: out of host memory for a read buffer");
        break;
      }
      char *into = p.direct ? bounce : slot;
      while (got < p.len && p.at + got < p.d1) {
        const ssize_t r = pread(p.fd, into + got, p.len - got, (off_t)(p.at + got));
        if (r < 0) {
          if (errno == EINTR) continue;
          if (errno == EINVAL && got % 4096) break;  // a direct read past a short last block: end of file
          sh->fail("kx_model_load: read of " + p.t->file + " failed: " + strerror(errno));
          io_ok = false;
          break;
        }
        if (r == 0) break;  // end of file
        got += (uint64_t)r;
      }
      if (!io_ok) break;
      if (p.at + got < p.d1) {
        sh->fail("kx_model_load: " + p.t->file + " ends inside tensor " + p.t->name);
        break;
      }
      uint64_t n = p.d1 - p.d0;
      if (p.direct) memcpy(slot + (p.d0 - p.at), bounce + (p.d0 - p.at), n);
      const char *src = slot + (p.d0 - p.at);
      if (p.widen) {  // bf16 -> f32: the bit pattern moves to the upper half of the word
        const uint16_t *h = (const uint16_t *)src;
        uint32_t *w = (uint32_t *)(slot + PIECE);
        for (uint64_t k = 0; k < n / 2; ++k) w[k] = (uint32_t)h[k] << 16;
        src = (const char *)w;
        n *= 2;
      }
      if (!hip_ok(hipMemcpyAsync(p.dst, src, n, hipMemcpyHostToDevice, st), "hipMemcpyAsync")) break;
      if (!hip_ok(hipStreamSynchronize(st), "hipStreamSynchronize")) break;  // the slot is reused by the next piece
      sh->copied.fetch_add(p.d1 - p.d0);
    }
    (void)hipStreamDestroy(st);
  }
  (void)hipHostFree(slot);
  free(bounce);
}

}  // namespace

int kx_load_run(const std::vector<KxLoadItem> &items, uint64_t *bytes, double *seconds) {
  const auto t0 = std::chrono::steady_clock::now();
  Shared sh;
  KX_HIP(hipGetDevice(&sh.device));
  const char *env_direct = getenv("KX_LOAD_DIRECT");
  const bool want_direct = !(env_direct && env_direct[0] == '0');
  std::unordered_map<std::string, std::pair<int, bool>> fds;  // descriptor, opened with O_DIRECT
  auto close_all = [&]() {
    for (auto &kv : fds) close(kv.second.first);
  };
  for (const KxLoadItem &it : items) {
    const KxTensorRec &t = *it.t;
    auto found = fds.find(t.file);
    if (found == fds.end()) {
      int fd = want_direct ? open(t.file.c_str(), O_RDONLY | O_DIRECT | O_CLOEXEC) : -1;
      const bool direct = fd >= 0;
      if (fd < 0) fd = open(t.file.c_str(), O_RDONLY | O_CLOEXEC);  // e.g. tmpfs has no O_DIRECT
      if (fd < 0) {
        kx_set_error("kx_model_load: cannot open %s: %s", t.file.c_str(), strerror(errno));
        close_all();
        return KX_ERR_ARG;
      }
      found = fds.emplace(t.file, std::make_pair(fd, direct)).first;
    }
    if (it.widen && (t.data_bytes > WIDEN_MAX || t.data + t.data_bytes - t.off > PIECE || t.data_bytes % 2)) {
      kx_set_error("kx_model_load: %s is too large to widen on the host", t.name.c_str());
      close_all();
      return KX_ERR_ARG;
    }
    // pieces of the aligned extent that hold tensor data (the extent was validated with the index)
    const uint64_t d_end = t.data + t.data_bytes;
    for (uint64_t at = t.off; at < t.off + t.bytes && at < d_end; at += PIECE) {
      const uint64_t len = t.off + t.bytes - at < PIECE ? t.off + t.bytes - at : PIECE;
      if (at + len <= t.data) continue;
      Piece p;
      p.fd = found->second.first;
      p.direct = found->second.second;
      p.at = at;
      p.len = len;
      p.d0 = at > t.data ? at : t.data;
      p.d1 = at + len < d_end ? at + len : d_end;
      p.dst = it.dst + (p.d0 - t.data) * (it.widen ? 2 : 1);
      p.widen = it.widen;
      p.t = &t;
      sh.pieces.push_back(p);
    }
  }
  int n_threads = 8;
  if (const char *e = getenv("KX_LOAD_THREADS")) n_threads = atoi(e);
  n_threads = n_threads < 1 ? 1 : n_threads > 16 ? 16 : n_threads;
  if ((size_t)n_threads > sh.pieces.size()) n_threads = sh.pieces.empty() ? 1 : (int)sh.pieces.size();
  std::vector<std::thread> pool;
  for (int i = 0; i < n_threads; ++i) pool.emplace_back(reader, &sh);
  for (auto &th : pool) th.join();
  close_all();
  (void)hipSetDevice(sh.device);
  if (sh.failed.load()) {
    kx_set_error("%s", sh.error.c_str());
    return KX_ERR_STATE;
  }
  if (bytes) *bytes = sh.copied.load();
  if (seconds) *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  return KX_OK;
}

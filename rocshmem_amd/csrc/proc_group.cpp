// One process per PE: the shared-file rendezvous (see proc_group.hpp).
#include "proc_group.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>

namespace rocshmem {
namespace runtime {

namespace {
ProcGroup g_procs;

uint64_t set_key(int start, int stride, int size) {
  // never zero: size >= 1
  return (static_cast<uint64_t>(start) << 42) | (static_cast<uint64_t>(stride) << 21) |
         static_cast<uint64_t>(size);
}

double now_s() {
  using clock = std::chrono::steady_clock;
  return std::chrono::duration<double>(clock::now().time_since_epoch()).count();
}

// Short spins first (a meeting of processes that are all running takes
// microseconds), then sleeps that do not hold a core.
void pause_for(unsigned spins) {
  if (spins < 2000) {
    std::this_thread::yield();
  } else {
    std::this_thread::sleep_for(std::chrono::microseconds(spins < 20000 ? 50 : 500));
  }
}
}  // namespace

ProcGroup &procs() { return g_procs; }

int ProcGroup::attach(const char *path, int nprocs, int rank) {
  if (shared_ || !path || nprocs < 1 || nprocs > kMaxProcs || rank < 0 || rank >= nprocs) return -1;
  const int fd = open(path, O_RDWR);
  if (fd < 0) return -1;
  struct stat st;
  if (fstat(fd, &st) != 0 || static_cast<size_t>(st.st_size) < sizeof(ProcShared)) {
    close(fd);
    return -1;
  }
  void *p = mmap(nullptr, sizeof(ProcShared), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (p == MAP_FAILED) return -1;
  shared_ = static_cast<ProcShared *>(p);
  nprocs_ = nprocs;
  rank_ = rank;
  shared_->attached.fetch_add(1, std::memory_order_acq_rel);
  if (const char *t = getenv("ROCSHMEM_EMU_RDV_TIMEOUT_S")) {
    const double v = atof(t);
    if (v > 0) timeout_s = v;
  }
  return 0;
}

bool ProcGroup::attach_from_env() {
  if (shared_) return true;
  const char *n = getenv("ROCSHMEM_EMU_PROCS");
  if (!n || !*n) return false;
  const char *r = getenv("ROCSHMEM_EMU_RANK");
  const char *path = getenv("ROCSHMEM_EMU_RDV");
  if (!r || !path || attach(path, atoi(n), atoi(r)) != 0) {
    fprintf(stderr,
            "rocshmem: ROCSHMEM_EMU_PROCS is set, so this process is one PE of a job, but "
            "ROCSHMEM_EMU_RANK / ROCSHMEM_EMU_RDV do not name a rank below it and a rendezvous file "
            "of at least %zu bytes (python -m rocshmem_amd.launch sets all three)\n",
            sizeof(ProcShared));
    fflush(nullptr);
    _Exit(EXIT_FAILURE);
  }
  return true;
}

void ProcGroup::detach() {
  if (!shared_) return;
  munmap(shared_, sizeof(ProcShared));
  shared_ = nullptr;
  nprocs_ = 0;
  rank_ = -1;
}

int ProcGroup::barrier(int start, int stride, int size) {
  if (!shared_ || size < 1 || stride < 1 || start < 0) return -1;
  if (size == 1) return 0;
  if (abort_requested() >= 0) return -1;
  // Find or claim the slot of this PE set: open addressing from a hash of the key.
  const uint64_t key = set_key(start, stride, size);
  ProcShared::Barrier *slot = nullptr;
  const size_t home = static_cast<size_t>((key * 0x9E3779B97F4A7C15ull) >> 40) % kBarrierSlots;
  for (int probe = 0; probe < kBarrierSlots && !slot; ++probe) {
    ProcShared::Barrier &b = shared_->barriers[(home + probe) % kBarrierSlots];
    uint64_t seen = b.key.load(std::memory_order_acquire);
    if (seen == 0 && b.key.compare_exchange_strong(seen, key, std::memory_order_acq_rel)) seen = key;
    if (seen == key) slot = &b;
  }
  if (!slot) {
    fprintf(stderr, "rocshmem: more than %d different PE sets have met in this job\n", kBarrierSlots);
    return -1;
  }
  const uint32_t round = slot->round.load(std::memory_order_acquire);
  if (slot->count.fetch_add(1, std::memory_order_acq_rel) + 1 == static_cast<uint32_t>(size)) {
    slot->count.store(0, std::memory_order_relaxed);
    slot->round.store(round + 1, std::memory_order_release);
    return 0;
  }
  const double t0 = now_s();
  for (unsigned spins = 0; slot->round.load(std::memory_order_acquire) == round; ++spins) {
    pause_for(spins);
    if ((spins & 255u) == 255u) {
      if (abort_requested() >= 0) return -1;
      if (now_s() - t0 > timeout_s) {
        fprintf(stderr,
                "rocshmem: PE %d waited %.0f s at a meeting of PEs (%d, stride %d, %d of them): "
                "giving up\n",
                rank_, timeout_s, start, stride, size);
        return -1;
      }
    }
  }
  return 0;
}

int ProcGroup::publish(const void *bytes, size_t n) {
  if (!shared_ || n > kBlobBytes || !bytes) return -1;
  ProcShared::Blob &b = shared_->blobs[rank_];
  memcpy(b.bytes, bytes, n);
  b.version.fetch_add(1, std::memory_order_release);
  return 0;
}

int ProcGroup::fetch(int rank, void *bytes, size_t n) const {
  if (!shared_ || rank < 0 || rank >= nprocs_ || n > kBlobBytes || !bytes) return -1;
  const ProcShared::Blob &b = shared_->blobs[rank];
  (void)b.version.load(std::memory_order_acquire);
  memcpy(bytes, b.bytes, n);
  return 0;
}

void ProcGroup::request_abort(int status) {
  if (!shared_) return;
  int32_t none = 0;
  // (a status of -1 would read as "none": it travels as 255, what a shell shows for it)
  shared_->abort_status_plus_one.compare_exchange_strong(none, (status == -1 ? 255 : status) + 1,
                                                         std::memory_order_acq_rel);
}

int ProcGroup::abort_requested() const {
  if (!shared_) return -1;
  return shared_->abort_status_plus_one.load(std::memory_order_acquire) - 1;
}

}  // namespace runtime
}  // namespace rocshmem

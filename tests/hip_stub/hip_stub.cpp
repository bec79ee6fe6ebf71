// A stand-in for the HIP runtime library, for tests of HOST LOGIC on a machine
// without a GPU.  Test infrastructure only: the product never loads it, and
// nothing computed under it counts as a result of the library.
//
// tests/test_host_logic_without_gpu.py puts this file's shared object in front
// of the real libamdhip64 for child processes that load the product library
// unchanged.  "Device memory" is host memory (blocks of 1 MiB and more are
// memfd mappings, so that hipIpcGetMemHandle / hipIpcOpenMemHandle map them
// into another process at another address, as the real calls do), copies and
// fills are memcpy / memset, events read the clock.  Kernels do NOT run: a
// launch is counted and dropped — with one exception, the whole-GPU copy
// kernel behind the host's rocshmem_putmem / getmem, whose single argument
// {dst, src, nbytes} is carried out with memcpy after both ranges have been
// checked against the blocks this process has allocated or mapped (a range
// that leaves them ends the process with a message: on a GPU it would be a
// memory fault).  What this lets a CPU test see: rocshmem_init between
// processes (handle exchange, layout check, peer table, contexts), the
// allocator, team bookkeeping, address resolution, host-initiated copies.
#include <hip/hip_runtime_api.h>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>

namespace {

struct Block {
  size_t bytes;
  int fd;       // memfd behind the block, -1 for plain host memory
  bool mapped;  // opened from another process's handle
};
std::mutex g_lock;
std::map<uintptr_t, Block> g_blocks;           // by base address
std::map<const void *, std::string> g_kernels;  // host stub address -> device name
unsigned long long g_launches = 0, g_copies_run = 0, g_alloc_calls = 0;
thread_local hipError_t g_last = hipSuccess;

constexpr size_t kShareFrom = size_t{1} << 20;

struct Handle {  // what travels in hipIpcMemHandle_t::reserved
  int pid, fd;
  unsigned long long bytes;
  char tag[8];
};
static_assert(sizeof(Handle) <= sizeof(hipIpcMemHandle_t), "handle does not fit");

// The block that holds [p, p + n), or nullptr.
const Block *holder(const void *p, size_t n, uintptr_t *base_out = nullptr) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  auto it = g_blocks.upper_bound(a);
  if (it == g_blocks.begin()) return nullptr;
  --it;
  if (a < it->first || a - it->first > it->second.bytes || n > it->second.bytes - (a - it->first))
    return nullptr;
  if (base_out) *base_out = it->first;
  return &it->second;
}

hipError_t allocate(void **ptr, size_t bytes) {
  {
    std::lock_guard<std::mutex> guard(g_lock);
    ++g_alloc_calls;
  }
  if (!ptr) return hipErrorInvalidValue;
  if (!bytes) {
    *ptr = nullptr;
    return hipSuccess;
  }
  void *p = nullptr;
  int fd = -1;
  if (bytes >= kShareFrom) {
    fd = static_cast<int>(syscall(SYS_memfd_create, "rocshmem_hip_stub", 0u));
    if (fd < 0 || ftruncate(fd, static_cast<off_t>(bytes)) != 0) return hipErrorOutOfMemory;
    p = mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    if (p == MAP_FAILED) {
      close(fd);
      return hipErrorOutOfMemory;
    }
  } else {
    if (posix_memalign(&p, 256, (bytes + 255) / 256 * 256) != 0) return hipErrorOutOfMemory;
    memset(p, 0xCD, bytes);  // device memory is not zeroed
  }
  std::lock_guard<std::mutex> guard(g_lock);
  g_blocks[reinterpret_cast<uintptr_t>(p)] = Block{bytes, fd, false};
  *ptr = p;
  return hipSuccess;
}

[[noreturn]] void out_of_bounds(const char *what, const void *p, size_t n) {
  fprintf(stderr,
          "hip stub: %s [%p, +%zu) is not inside memory this process has allocated or mapped "
          "(on a GPU: a memory access fault)\n", what, p, n);
  fflush(nullptr);
  _Exit(97);
}

}  // namespace

extern "C" {

// ---- what the compiler's registration code calls -----------------------------
void **__hipRegisterFatBinary(const void *) {
  static void *dummy[1];
  return dummy;
}
void __hipUnregisterFatBinary(void **) {}
void __hipRegisterFunction(void **, const void *host_function, char *, const char *device_name,
                           unsigned int, void *, void *, dim3 *, dim3 *, int *) {
  std::lock_guard<std::mutex> guard(g_lock);
  g_kernels[host_function] = device_name ? device_name : "";
}
void __hipRegisterVar(void **, void *, char *, char *, int, size_t, int, int) {}

struct CallConfig {
  dim3 grid, block;
  size_t shared;
  hipStream_t stream;
};
static thread_local CallConfig g_config;
hipError_t __hipPushCallConfiguration(dim3 grid, dim3 block, size_t shared, hipStream_t stream) {
  g_config = CallConfig{grid, block, shared, stream};
  return hipSuccess;
}
hipError_t __hipPopCallConfiguration(dim3 *grid, dim3 *block, size_t *shared, hipStream_t *stream) {
  *grid = g_config.grid;
  *block = g_config.block;
  *shared = g_config.shared;
  *stream = g_config.stream;
  return hipSuccess;
}

// ---- launches ----------------------------------------------------------------
hipError_t hipLaunchKernel(const void *function, dim3, dim3, void **args, size_t, hipStream_t) {
  std::string name;
  {
    std::lock_guard<std::mutex> guard(g_lock);
    ++g_launches;
    auto it = g_kernels.find(function);
    if (it != g_kernels.end()) name = it->second;
  }
  if (name.find("bulk_copy_kernel") != std::string::npos && args && args[0]) {
    struct BulkArgs {
      char *dst;
      const char *src;
      size_t nbytes;
    } a;
    memcpy(&a, args[0], sizeof(a));
    {
      std::lock_guard<std::mutex> guard(g_lock);
      if (!holder(a.dst, a.nbytes)) out_of_bounds("the destination of a copy kernel", a.dst, a.nbytes);
      if (!holder(a.src, a.nbytes)) out_of_bounds("the source of a copy kernel", a.src, a.nbytes);
      ++g_copies_run;
    }
    memmove(a.dst, a.src, a.nbytes);
  }
  return hipSuccess;
}
// Launches seen, and how many of them were copy kernels that were carried out.
void hip_stub_counts(unsigned long long *launches, unsigned long long *copies_run) {
  std::lock_guard<std::mutex> guard(g_lock);
  if (launches) *launches = g_launches;
  if (copies_run) *copies_run = g_copies_run;
}

// Calls of hipMalloc / hipExtMallocWithFlags / hipHostMalloc / hipFree / hipHostFree so far.
unsigned long long hip_stub_alloc_calls(void) {
  std::lock_guard<std::mutex> guard(g_lock);
  return g_alloc_calls;
}

// ---- device, errors ----------------------------------------------------------
hipError_t hipGetDeviceCount(int *n) {
  *n = 1;
  return hipSuccess;
}
hipError_t hipGetDevice(int *d) {
  *d = 0;
  return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) { return hipSuccess; }
hipError_t hipGetLastError(void) {
  const hipError_t e = g_last;
  g_last = hipSuccess;
  return e;
}
const char *hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "error (hip stub)"; }
hipError_t hipDeviceGetAttribute(int *value, hipDeviceAttribute_t attr, int) {
  switch (attr) {
    case hipDeviceAttributeMultiprocessorCount: *value = 256; break;
    case hipDeviceAttributeMaxSharedMemoryPerMultiprocessor: *value = 163840; break;
    case hipDeviceAttributeWallClockRate: *value = 100000; break;
    default: *value = 1; break;
  }
  return hipSuccess;
}
hipError_t hipOccupancyMaxActiveBlocksPerMultiprocessor(int *blocks, const void *, int, size_t) {
  *blocks = 8;
  return hipSuccess;
}
hipError_t hipMemGetInfo(size_t *free_bytes, size_t *total_bytes) {
  *free_bytes = *total_bytes = size_t{288} << 30;
  return hipSuccess;
}

// ---- memory --------------------------------------------------------------------
hipError_t hipMalloc(void **ptr, size_t bytes) { return allocate(ptr, bytes); }
hipError_t hipExtMallocWithFlags(void **ptr, size_t bytes, unsigned int) { return allocate(ptr, bytes); }
hipError_t hipHostMalloc(void **ptr, size_t bytes, unsigned int) {
  {
    std::lock_guard<std::mutex> guard(g_lock);
    ++g_alloc_calls;
  }
  *ptr = calloc(1, bytes ? bytes : 1);
  return *ptr ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipHostFree(void *ptr) {
  {
    std::lock_guard<std::mutex> guard(g_lock);
    ++g_alloc_calls;
  }
  free(ptr);
  return hipSuccess;
}
hipError_t hipFree(void *ptr) {
  std::lock_guard<std::mutex> guard(g_lock);
  ++g_alloc_calls;
  if (!ptr) return hipSuccess;
  auto it = g_blocks.find(reinterpret_cast<uintptr_t>(ptr));
  if (it == g_blocks.end()) return hipErrorInvalidValue;
  if (it->second.fd >= 0 || it->second.mapped) {
    munmap(ptr, it->second.bytes);
    if (it->second.fd >= 0) close(it->second.fd);
  } else {
    free(ptr);
  }
  g_blocks.erase(it);
  return hipSuccess;
}
hipError_t hipMemcpy(void *dst, const void *src, size_t n, hipMemcpyKind) {
  if (n) memmove(dst, src, n);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t n, hipMemcpyKind kind, hipStream_t) {
  return hipMemcpy(dst, src, n, kind);
}
hipError_t hipMemset(void *dst, int value, size_t n) {
  if (n) {
    std::lock_guard<std::mutex> guard(g_lock);
    if (!holder(dst, n)) out_of_bounds("the range of a memset", dst, n);
  }
  if (n) memset(dst, value, n);
  return hipSuccess;
}
hipError_t hipMemsetAsync(void *dst, int value, size_t n, hipStream_t) { return hipMemset(dst, value, n); }
// A __device__ / __constant__ variable is its host-side shadow here.
hipError_t hipMemcpyToSymbol(const void *symbol, const void *src, size_t n, size_t offset, hipMemcpyKind) {
  memcpy(static_cast<char *>(const_cast<void *>(symbol)) + offset, src, n);
  return hipSuccess;
}
hipError_t hipGetSymbolAddress(void **ptr, const void *symbol) {
  *ptr = const_cast<void *>(symbol);
  return hipSuccess;
}
hipError_t hipPointerGetAttributes(hipPointerAttribute_t *attributes, const void *ptr) {
  std::lock_guard<std::mutex> guard(g_lock);
  if (!holder(ptr, 0)) return g_last = hipErrorInvalidValue;
  memset(attributes, 0, sizeof(*attributes));
  attributes->type = hipMemoryTypeDevice;
  attributes->devicePointer = const_cast<void *>(ptr);
  return hipSuccess;
}

// ---- sharing between processes ---------------------------------------------------
hipError_t hipIpcGetMemHandle(hipIpcMemHandle_t *handle, void *ptr) {
  std::lock_guard<std::mutex> guard(g_lock);
  auto it = g_blocks.find(reinterpret_cast<uintptr_t>(ptr));
  if (it == g_blocks.end() || it->second.fd < 0) return g_last = hipErrorInvalidValue;
  memset(handle, 0, sizeof(*handle));
  Handle h{static_cast<int>(getpid()), it->second.fd, it->second.bytes, "stubmem"};
  memcpy(handle, &h, sizeof(h));
  return hipSuccess;
}
hipError_t hipIpcOpenMemHandle(void **ptr, hipIpcMemHandle_t handle, unsigned int) {
  Handle h;
  memcpy(&h, &handle, sizeof(h));
  if (memcmp(h.tag, "stubmem", 8) != 0 || h.pid == static_cast<int>(getpid())) return g_last = hipErrorInvalidValue;
  char path[64];
  snprintf(path, sizeof(path), "/proc/%d/fd/%d", h.pid, h.fd);
  const int fd = open(path, O_RDWR);
  if (fd < 0) return g_last = hipErrorInvalidValue;
  void *p = mmap(nullptr, h.bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (p == MAP_FAILED) return g_last = hipErrorOutOfMemory;
  std::lock_guard<std::mutex> guard(g_lock);
  g_blocks[reinterpret_cast<uintptr_t>(p)] = Block{static_cast<size_t>(h.bytes), -1, true};
  *ptr = p;
  return hipSuccess;
}

// ---- streams and events ------------------------------------------------------------
hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned int) {
  *stream = reinterpret_cast<hipStream_t>(calloc(1, 8));
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
struct StubEvent {
  double at;
};
static double now_ms() {
  return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
hipError_t hipEventCreate(hipEvent_t *event) {
  *event = reinterpret_cast<hipEvent_t>(new StubEvent{0.0});
  return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t event) {
  delete reinterpret_cast<StubEvent *>(event);
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t event, hipStream_t) {
  reinterpret_cast<StubEvent *>(event)->at = now_ms();
  return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t start, hipEvent_t stop) {
  *ms = static_cast<float>(reinterpret_cast<StubEvent *>(stop)->at - reinterpret_cast<StubEvent *>(start)->at);
  return hipSuccess;
}

}  // extern "C"

// Drivers for atomics, put-with-signal, point-to-point waits, the ping-pong
// and MoE-dispatch patterns, and context lifecycle.
#include <mutex>

#include "drv_common.hpp"
#include "rocshmem_amd.h"

#include <algorithm>
#include <vector>

namespace rocshmem {
namespace drv {

// ---------------------------------------------------------------------------
// Atomic memory operations.
// ---------------------------------------------------------------------------
template <typename T>
struct AmoArgs {
  T *counters;  // address on my_pe
  uint32_t n_slots;
  const uint32_t *ids;
  const T *values;
  const T *conds;
  T *fetched;
  size_t n_ops;
  rocshmem_ctx_t ctx;
};

template <typename T>
__device__ __host__ inline T zero_of() {
  return static_cast<T>(0);
}

// Public entry points for element type T.
template <typename T>
struct PublicAmo;
#define DRV_AMO_STD(T, TN)                                                                 \
  __device__ static T fetch_add(rocshmem_ctx_t c, T *d, T v, int pe) {                     \
    return rocshmem_ctx_##TN##_atomic_fetch_add(c, d, v, pe);                              \
  }                                                                                        \
  __device__ static void add(rocshmem_ctx_t c, T *d, T v, int pe) {                        \
    rocshmem_ctx_##TN##_atomic_add(c, d, v, pe);                                           \
  }                                                                                        \
  __device__ static T fetch_inc(rocshmem_ctx_t c, T *d, int pe) {                          \
    return rocshmem_ctx_##TN##_atomic_fetch_inc(c, d, pe);                                 \
  }                                                                                        \
  __device__ static void inc(rocshmem_ctx_t c, T *d, int pe) {                             \
    rocshmem_ctx_##TN##_atomic_inc(c, d, pe);                                              \
  }                                                                                        \
  __device__ static T compare_swap(rocshmem_ctx_t c, T *d, T cond, T v, int pe) {          \
    return rocshmem_ctx_##TN##_atomic_compare_swap(c, d, cond, v, pe);                     \
  }
#define DRV_AMO_EXT(T, TN)                                                                 \
  __device__ static T fetch(rocshmem_ctx_t c, T *d, int pe) {                              \
    return rocshmem_ctx_##TN##_atomic_fetch(c, d, pe);                                     \
  }                                                                                        \
  __device__ static void set(rocshmem_ctx_t c, T *d, T v, int pe) {                        \
    rocshmem_ctx_##TN##_atomic_set(c, d, v, pe);                                           \
  }                                                                                        \
  __device__ static T swap(rocshmem_ctx_t c, T *d, T v, int pe) {                          \
    return rocshmem_ctx_##TN##_atomic_swap(c, d, v, pe);                                   \
  }
#define DRV_AMO_BIT(T, TN)                                                                 \
  __device__ static T fetch_and(rocshmem_ctx_t c, T *d, T v, int pe) {                     \
    return rocshmem_ctx_##TN##_atomic_fetch_and(c, d, v, pe);                              \
  }                                                                                        \
  __device__ static T fetch_or(rocshmem_ctx_t c, T *d, T v, int pe) {                      \
    return rocshmem_ctx_##TN##_atomic_fetch_or(c, d, v, pe);                               \
  }                                                                                        \
  __device__ static T fetch_xor(rocshmem_ctx_t c, T *d, T v, int pe) {                     \
    return rocshmem_ctx_##TN##_atomic_fetch_xor(c, d, v, pe);                              \
  }
#define DRV_NO_STD(T)                                                                      \
  __device__ static T fetch_add(rocshmem_ctx_t, T *, T, int) { return zero_of<T>(); }               \
  __device__ static void add(rocshmem_ctx_t, T *, T, int) {}                               \
  __device__ static T fetch_inc(rocshmem_ctx_t, T *, int) { return zero_of<T>(); }                  \
  __device__ static void inc(rocshmem_ctx_t, T *, int) {}                                  \
  __device__ static T compare_swap(rocshmem_ctx_t, T *, T, T, int) { return zero_of<T>(); }
#define DRV_NO_BIT(T)                                                                      \
  __device__ static T fetch_and(rocshmem_ctx_t, T *, T, int) { return zero_of<T>(); }               \
  __device__ static T fetch_or(rocshmem_ctx_t, T *, T, int) { return zero_of<T>(); }                \
  __device__ static T fetch_xor(rocshmem_ctx_t, T *, T, int) { return zero_of<T>(); }

template <> struct PublicAmo<int> {
  static constexpr bool kStd = true, kBit = false;
  DRV_AMO_STD(int, int) DRV_AMO_EXT(int, int) DRV_NO_BIT(int)
};
template <> struct PublicAmo<long> {
  static constexpr bool kStd = true, kBit = false;
  DRV_AMO_STD(long, long) DRV_AMO_EXT(long, long) DRV_NO_BIT(long)
};
template <> struct PublicAmo<long long> {
  static constexpr bool kStd = true, kBit = false;
  DRV_AMO_STD(long long, longlong) DRV_AMO_EXT(long long, longlong) DRV_NO_BIT(long long)
};
template <> struct PublicAmo<unsigned int> {
  static constexpr bool kStd = true, kBit = true;
  DRV_AMO_STD(unsigned int, uint) DRV_AMO_EXT(unsigned int, uint) DRV_AMO_BIT(unsigned int, uint)
};
template <> struct PublicAmo<unsigned long> {
  static constexpr bool kStd = true, kBit = true;
  DRV_AMO_STD(unsigned long, ulong) DRV_AMO_EXT(unsigned long, ulong) DRV_AMO_BIT(unsigned long, ulong)
};
template <> struct PublicAmo<unsigned long long> {
  static constexpr bool kStd = true, kBit = true;
  DRV_AMO_STD(unsigned long long, ulonglong) DRV_AMO_EXT(unsigned long long, ulonglong)
  DRV_AMO_BIT(unsigned long long, ulonglong)
};
template <> struct PublicAmo<float> {
  static constexpr bool kStd = false, kBit = false;
  DRV_NO_STD(float) DRV_AMO_EXT(float, float) DRV_NO_BIT(float)
};
template <> struct PublicAmo<double> {
  static constexpr bool kStd = false, kBit = false;
  DRV_NO_STD(double) DRV_AMO_EXT(double, double) DRV_NO_BIT(double)
};

template <typename T, int kAmo>
__global__ void amo_kernel(AmoArgs<T> a) {
  using P = PublicAmo<T>;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < a.n_ops;
       i += stride) {
    const uint32_t id = a.ids[i];
    const int pe = static_cast<int>(id / a.n_slots);
    T *target = a.counters + (id % a.n_slots);
    const T v = a.values ? a.values[i] : static_cast<T>(1);
    T out = zero_of<T>();
    if constexpr (kAmo == ROCSHMEM_AMD_AMO_FETCH_ADD) out = P::fetch_add(a.ctx, target, v, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_ADD) P::add(a.ctx, target, v, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_FETCH_INC) out = P::fetch_inc(a.ctx, target, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_INC) P::inc(a.ctx, target, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_COMPARE_SWAP)
      out = P::compare_swap(a.ctx, target, a.conds[i], v, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_FETCH) out = P::fetch(a.ctx, target, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_SET) P::set(a.ctx, target, v, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_SWAP) out = P::swap(a.ctx, target, v, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_FETCH_AND) out = P::fetch_and(a.ctx, target, v, pe);
    else if constexpr (kAmo == ROCSHMEM_AMD_AMO_FETCH_OR) out = P::fetch_or(a.ctx, target, v, pe);
    else out = P::fetch_xor(a.ctx, target, v, pe);
    if (a.fetched) a.fetched[i] = out;
  }
}

template <typename T>
int launch_amo(int amo_op, const AmoArgs<T> &a, int n_wgs, int wg_size, hipStream_t s) {
  using P = PublicAmo<T>;
  const dim3 g(n_wgs), b(wg_size);
  const bool std_op = amo_op <= ROCSHMEM_AMD_AMO_COMPARE_SWAP;
  const bool bit_op = amo_op >= ROCSHMEM_AMD_AMO_FETCH_AND;
  if ((std_op && !P::kStd) || (bit_op && !P::kBit)) return -1;
  switch (amo_op) {
#define DRV_AMO_CASE(OP) \
  case OP: hipLaunchKernelGGL((amo_kernel<T, OP>), g, b, 0, s, a); break;
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_FETCH_ADD)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_ADD)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_FETCH_INC)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_INC)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_COMPARE_SWAP)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_FETCH)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_SET)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_SWAP)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_FETCH_AND)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_FETCH_OR)
    DRV_AMO_CASE(ROCSHMEM_AMD_AMO_FETCH_XOR)
#undef DRV_AMO_CASE
    default: return -1;
  }
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

// ---------------------------------------------------------------------------
// put-with-signal
// ---------------------------------------------------------------------------
struct SignalArgs {
  char *dest;
  const char *source;
  size_t nbytes;
  size_t tile;
  uint64_t *sig_addr;
  uint64_t signal;
  int sig_op;
  rocshmem_ctx_t ctx;
  int pe;
  int calls;
};

template <int kGran>
__global__ void put_signal_kernel(SignalArgs a) {
  size_t group;
  const size_t tid = threadIdx.x, bs = blockDim.x;
  if constexpr (kGran == ROCSHMEM_AMD_WG) group = blockIdx.x;
  else if constexpr (kGran == ROCSHMEM_AMD_WAVE) group = blockIdx.x * ((bs + 63) / 64) + tid / 64;
  else group = blockIdx.x * bs + tid;
  const size_t off = group * a.tile;
  // A group whose tile starts past the end has nothing to send: a zero-length
  // call, which leaves the signal untouched.
  const size_t len = off >= a.nbytes ? 0 : (a.nbytes - off < a.tile ? a.nbytes - off : a.tile);
  for (int k = 0; k < a.calls; ++k) {
    if constexpr (kGran == ROCSHMEM_AMD_WG)
      rocshmem_ctx_putmem_signal_wg(a.ctx, a.dest + off, a.source + off, len, a.sig_addr,
                                    a.signal, a.sig_op, a.pe);
    else if constexpr (kGran == ROCSHMEM_AMD_WAVE)
      rocshmem_ctx_putmem_signal_wave(a.ctx, a.dest + off, a.source + off, len, a.sig_addr,
                                      a.signal, a.sig_op, a.pe);
    else
      rocshmem_ctx_putmem_signal(a.ctx, a.dest + off, a.source + off, len, a.sig_addr,
                                 a.signal, a.sig_op, a.pe);
  }
}

template <int kGran>
__global__ void signal_fetch_kernel(const uint64_t *sig, uint64_t *out) {
  uint64_t v;
  if constexpr (kGran == ROCSHMEM_AMD_WG) v = rocshmem_signal_fetch_wg(sig);
  else if constexpr (kGran == ROCSHMEM_AMD_WAVE) v = rocshmem_signal_fetch_wave(sig);
  else v = rocshmem_signal_fetch(sig);
  // Every thread must have received the value.
  if (v != *reinterpret_cast<const volatile uint64_t *>(sig)) atomicAdd(reinterpret_cast<unsigned long long *>(out + 1), 1ull);
  if (threadIdx.x == 0) out[0] = v;
}

// ---------------------------------------------------------------------------
// ping-pong between two work-groups acting as two PEs
// ---------------------------------------------------------------------------
struct PingPongArgs {
  char *buf_a;      // address on pe_a
  uint64_t *sig_a;  // address on pe_a
  size_t nbytes;
  size_t slot_bytes;  // distance between the buffers of consecutive pairs
  int iters;
  int pe_a, pe_b;
  uint64_t pe_stride;
  detail::Context *ctx_row;
  detail::Team *world_row;
  unsigned long long *ticks;  // [pairs]
};

__global__ void pingpong_kernel(PingPongArgs a) {
  // Work-groups 2k and 2k+1 are the two ends of pair k.
  const bool is_a = (blockIdx.x & 1) == 0;
  const size_t pair = blockIdx.x >> 1;
  const int me = is_a ? a.pe_a : a.pe_b;
  const int peer = is_a ? a.pe_b : a.pe_a;
  const int64_t shift = static_cast<int64_t>(me - a.pe_a) * static_cast<int64_t>(a.pe_stride);
  char *buf = a.buf_a + shift + pair * a.slot_bytes;
  uint64_t *sig = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(a.sig_a) + shift) + pair;
  rocshmem_ctx_t ctx{a.ctx_row + me, &a.world_row[me].wrt_world};
  const unsigned long long t0 = wall_clock64();
  for (int r = 1; r <= a.iters; ++r) {
    if (is_a) {
      rocshmem_ctx_putmem_signal_wg(ctx, buf, buf, a.nbytes, sig, static_cast<uint64_t>(r),
                                    ROCSHMEM_SIGNAL_SET, peer);
      if (threadIdx.x == 0)
        rocshmem_ulong_wait_until(reinterpret_cast<unsigned long *>(sig), ROCSHMEM_CMP_EQ,
                                  static_cast<unsigned long>(r));
      __syncthreads();
    } else {
      if (threadIdx.x == 0)
        rocshmem_ulong_wait_until(reinterpret_cast<unsigned long *>(sig), ROCSHMEM_CMP_EQ,
                                  static_cast<unsigned long>(r));
      __syncthreads();
      rocshmem_ctx_putmem_signal_wg(ctx, buf, buf, a.nbytes, sig, static_cast<uint64_t>(r),
                                    ROCSHMEM_SIGNAL_SET, peer);
    }
  }
  const unsigned long long t1 = wall_clock64();
  if (is_a && threadIdx.x == 0) a.ticks[pair] = t1 - t0;
}

// ---------------------------------------------------------------------------
// put + quiet + flag, checked by the receiver inside the same kernel
// ---------------------------------------------------------------------------
struct PutFlagArgs {
  char *data_a;          // [pairs][nbytes], address on pe_a
  int64_t a_to_b;        // bytes from pe_a's slice to pe_b's
  uint64_t *flag_b;      // [pairs] on pe_b : round announced by the producer
  uint64_t *ack_a;       // [pairs] on pe_a : round consumed by the receiver
  uint32_t *staging;     // [pairs][nbytes/4] producer-side source, plain device memory
  size_t nbytes;         // per pair, multiple of 4
  int rounds;
  int pe_a, pe_b;
  int with_signal;       // 0: putmem_wg, quiet, relaxed flag store; 1: putmem_signal_wg;
                         // 2 / 3: putmem_nbi_wave / putmem_nbi pieces, quiet by all, flag;
                         // 4 / 5: as 0 / 1 with the source in the producer's LDS
  unsigned spin_limit;
  rocshmem_ctx_t ctx_a;
  unsigned long long *mismatches;
  int *timed_out;
};

__device__ __forceinline__ uint32_t put_flag_word(int pair, int round, size_t i) {
  return static_cast<uint32_t>(i) * 2654435761u + static_cast<uint32_t>(round) * 40503u +
         static_cast<uint32_t>(pair);
}

// Waits (thread 0, bounded) until *word == round; false when the limit ran out.
__device__ __forceinline__ bool put_flag_wait(uint64_t *word, uint64_t round, unsigned limit,
                                              int *timed_out) {
  __shared__ int ok;
  if (threadIdx.x == 0) {
    ok = 0;
    for (unsigned spin = 0; spin < limit; ++spin) {
      if (detail::load_through(word) == round) {
        ok = 1;
        break;
      }
      if (detail::load_through(timed_out)) break;
      __builtin_amdgcn_s_sleep(2);
    }
    if (ok) detail::fence_acquire();
    else detail::store_through(timed_out, 1);
  }
  __syncthreads();
  const bool r = ok != 0;
  __syncthreads();
  return r;
}

// Even work-groups produce for pe_a, odd ones consume for pe_b.  The flag and
// the acknowledgement are relaxed write-through stores: the only thing that
// orders the payload before the flag is the context's quiet.
__global__ void put_flag_kernel(PutFlagArgs a) {
  const int pair = blockIdx.x >> 1;
  const bool producer = (blockIdx.x & 1) == 0;
  const size_t nwords = a.nbytes / 4;
  char *data = a.data_a + static_cast<size_t>(pair) * a.nbytes;
  extern __shared__ __attribute__((aligned(16))) uint32_t put_flag_lds[];
  const bool from_lds = a.with_signal >= 4;
  uint32_t *stage = from_lds ? put_flag_lds : a.staging + static_cast<size_t>(pair) * nwords;
  // Own-PE views of the two control words.
  uint64_t *flag_on_b = a.flag_b + pair;
  uint64_t *ack_on_a = a.ack_a + pair;
  for (int r = 1; r <= a.rounds; ++r) {
    if (producer) {
      for (size_t i = threadIdx.x; i < nwords; i += blockDim.x) stage[i] = put_flag_word(pair, r, i);
      __syncthreads();
      if (a.with_signal == 1 || a.with_signal == 5) {
        // flag_on_b is pe_b's address; the call wants pe_a's.
        uint64_t *flag_sym = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(flag_on_b) - a.a_to_b);
        rocshmem_ctx_putmem_signal_wg(a.ctx_a, data, stage, a.nbytes, flag_sym,
                                      static_cast<uint64_t>(r), ROCSHMEM_SIGNAL_SET, a.pe_b);
      } else if (a.with_signal == 2 || a.with_signal == 3) {
        // Non-blocking puts in pieces (four per wavefront, or 12 bytes per call
        // per thread), completed by the quiet of whoever issued them.
        if (a.with_signal == 2) {
          const size_t waves = (blockDim.x + 63) / 64, w = threadIdx.x / 64;
          const size_t piece = ((a.nbytes + waves * 4 - 1) / (waves * 4) + 3) & ~size_t{3};
          for (size_t k = w; k * piece < a.nbytes; k += waves) {
            const size_t off = k * piece;
            const size_t len = a.nbytes - off < piece ? a.nbytes - off : piece;
            rocshmem_ctx_putmem_nbi_wave(a.ctx_a, data + off, reinterpret_cast<char *>(stage) + off,
                                         len, a.pe_b);
          }
        } else {
          for (size_t off = threadIdx.x * size_t{12}; off < a.nbytes; off += blockDim.x * size_t{12}) {
            const size_t len = a.nbytes - off < 12 ? a.nbytes - off : 12;
            rocshmem_ctx_putmem_nbi(a.ctx_a, data + off, reinterpret_cast<char *>(stage) + off, len,
                                    a.pe_b);
          }
        }
        rocshmem_ctx_quiet(a.ctx_a);
        __syncthreads();
        if (threadIdx.x == 0) detail::store_through(flag_on_b, static_cast<uint64_t>(r));
      } else {
        rocshmem_ctx_putmem_wg(a.ctx_a, data, stage, a.nbytes, a.pe_b);
        if (threadIdx.x == 0) {
          rocshmem_ctx_quiet(a.ctx_a);
          detail::store_through(flag_on_b, static_cast<uint64_t>(r));
        }
      }
      if (!put_flag_wait(ack_on_a, static_cast<uint64_t>(r), a.spin_limit, a.timed_out)) return;
    } else {
      if (!put_flag_wait(flag_on_b, static_cast<uint64_t>(r), a.spin_limit, a.timed_out)) return;
      unsigned bad = 0;
      const uint32_t *got = reinterpret_cast<const uint32_t *>(data + a.a_to_b);
      for (size_t i = threadIdx.x; i < nwords; i += blockDim.x)
        bad += got[i] != put_flag_word(pair, r, i);
      if (bad) atomicAdd(a.mismatches, static_cast<unsigned long long>(bad));
      __syncthreads();
      if (threadIdx.x == 0) detail::store_through(ack_on_a, static_cast<uint64_t>(r));
    }
  }
}

// ---------------------------------------------------------------------------
// MoE-style dispatch with put_signal
// ---------------------------------------------------------------------------
struct DispatchArgs {
  char *recv0;          // addresses on PE 0
  const char *send0;
  uint64_t *sig0;
  const uint32_t *count, *send_row, *recv_row;
  const uint2 *calls;   // [n_calls] {pair, first row of the call within the pair}
  size_t row_bytes;
  uint64_t pe_stride;
  int np;
  uint32_t rows_per_call;
  uint32_t n_calls;
  detail::Context *ctx_row;
  detail::Team *world_row;
  uint64_t *expect;     // [P*P], [d*P+s]: what d's signal word s has been waited up to; may be null
};

// Work-groups walk the list of all calls (a call = up to rows_per_call rows of
// one (source, destination) pair), so a skewed routing table still keeps every
// CU busy; the last P work-groups are the receivers.
__global__ void dispatch_kernel(DispatchArgs a) {
  const int P = a.np;
  const unsigned senders = gridDim.x - P;
  if (blockIdx.x < senders) {
    // The routing tables are read-only while the kernel runs and indexed by
    // work-group-uniform values: through the constant address space they come
    // as scalar loads instead of vector loads behind the bulk traffic.
    typedef const __attribute__((address_space(4))) uint32_t *Table;
    const Table calls = (Table)a.calls, count = (Table)a.count;          // NOLINT
    const Table send_row = (Table)a.send_row, recv_row = (Table)a.recv_row;  // NOLINT
    for (uint32_t c = blockIdx.x; c < a.n_calls; c += senders) {
      const int pair = static_cast<int>(calls[2 * c]), s = pair / P, d = pair % P;
      const uint32_t first = calls[2 * c + 1];
      const uint32_t cnt = count[pair];
      const uint32_t rows = cnt - first < a.rows_per_call ? cnt - first : a.rows_per_call;
      rocshmem_ctx_t ctx{a.ctx_row + s, &a.world_row[s].wrt_world};
      char *recv_s = a.recv0 + static_cast<uint64_t>(s) * a.pe_stride;
      const char *send_s = a.send0 + static_cast<uint64_t>(s) * a.pe_stride;
      uint64_t *sig_s = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(a.sig0) +
                                                     static_cast<uint64_t>(s) * a.pe_stride);
      rocshmem_ctx_putmem_signal_wg(
          ctx, recv_s + (static_cast<size_t>(recv_row[pair]) + first) * a.row_bytes,
          send_s + (static_cast<size_t>(send_row[pair]) + first) * a.row_bytes,
          static_cast<size_t>(rows) * a.row_bytes, sig_s + s, static_cast<uint64_t>(rows),
          ROCSHMEM_SIGNAL_ADD, d);
    }
  } else {
    const int d = blockIdx.x - senders;
    uint64_t *sig_d = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(a.sig0) +
                                                   static_cast<uint64_t>(d) * a.pe_stride);
    // Lane s of the receiver waits for sender s.  The signal words only ever
    // grow: with `expect` the receiver keeps, per word, the total it has
    // waited for so far, as an application that dispatches every step would,
    // and nobody has to clear the words between dispatches.
    for (int s = threadIdx.x; s < P; s += blockDim.x) {
      unsigned long target = a.count[s * P + d];
      if (a.expect) {
        target += a.expect[d * P + s];
        a.expect[d * P + s] = target;
      }
      rocshmem_ulong_wait_until(reinterpret_cast<unsigned long *>(sig_d + s), ROCSHMEM_CMP_GE, target);
    }
  }
}

// ---------------------------------------------------------------------------
// wait / test
// ---------------------------------------------------------------------------
template <typename T>
struct PublicWait;
#define DRV_WAIT(T, TN)                                                                    \
  template <>                                                                              \
  struct PublicWait<T> {                                                                   \
    __device__ static int test(T *p, int c, T v) { return rocshmem_##TN##_test(p, c, v); } \
    __device__ static void wait(T *p, int c, T v) { rocshmem_##TN##_wait_until(p, c, v); } \
    __device__ static size_t any(T *p, size_t n, const int *s, int c, T v) {               \
      return rocshmem_##TN##_wait_until_any(p, n, s, c, v);                                \
    }                                                                                      \
    __device__ static void all(T *p, size_t n, const int *s, int c, T v) {                 \
      rocshmem_##TN##_wait_until_all(p, n, s, c, v);                                       \
    }                                                                                      \
    __device__ static size_t some(T *p, size_t n, size_t *idx, const int *s, int c, T v) { \
      return rocshmem_##TN##_wait_until_some(p, n, idx, s, c, v);                          \
    }                                                                                      \
  };
DRV_WAIT(short, short)
DRV_WAIT(int, int)
DRV_WAIT(long, long)
DRV_WAIT(long long, longlong)
DRV_WAIT(float, float)
DRV_WAIT(double, double)
DRV_WAIT(unsigned int, uint)
DRV_WAIT(unsigned long, ulong)
DRV_WAIT(unsigned long long, ulonglong)

// A wait with an end: rocshmem_<T>_test polled up to max_polls times.
template <typename T>
__global__ void poll_until_kernel(T *ivar, int cmp, T value, unsigned long long max_polls,
                                  unsigned long long *result) {
  unsigned long long polls = 0;
  int seen = 0;
  while (polls < max_polls) {
    ++polls;
    if (PublicWait<T>::test(ivar, cmp, value)) {
      seen = 1;
      break;
    }
    __builtin_amdgcn_s_sleep(8);
  }
  result[0] = static_cast<unsigned long long>(seen);
  result[1] = polls;
}

template <typename T>
struct WaitArgs {
  int fn;
  T *ivars;
  size_t nelems;
  const int *status;
  int cmp;
  T value;
  size_t *ret;
  size_t *indices;
  // waker
  int woken;
  size_t wake_index;
  T wake_value;
  unsigned long long delay_ticks;
};

template <typename T>
__global__ void wait_kernel(WaitArgs<T> a) {
  using P = PublicWait<T>;
  if (blockIdx.x == 0) {
    if (threadIdx.x != 0) return;
    size_t r = 0;
    switch (a.fn) {
      case ROCSHMEM_AMD_TEST: r = static_cast<size_t>(P::test(a.ivars, a.cmp, a.value)); break;
      case ROCSHMEM_AMD_WAIT_UNTIL: P::wait(a.ivars, a.cmp, a.value); break;
      case ROCSHMEM_AMD_WAIT_UNTIL_ANY: r = P::any(a.ivars, a.nelems, a.status, a.cmp, a.value); break;
      case ROCSHMEM_AMD_WAIT_UNTIL_ALL: P::all(a.ivars, a.nelems, a.status, a.cmp, a.value); break;
      default: r = P::some(a.ivars, a.nelems, a.indices, a.status, a.cmp, a.value); break;
    }
    *a.ret = r;
  } else if (a.woken && threadIdx.x == 0) {
    const unsigned long long t0 = wall_clock64();
    while (wall_clock64() - t0 < a.delay_ticks) __builtin_amdgcn_s_sleep(8);
    detail::amo_set(a.ivars + a.wake_index, a.wake_value);
  }
}

// ---------------------------------------------------------------------------
// context lifecycle
// ---------------------------------------------------------------------------
struct CtxCycleArgs {
  rocshmem_team_t team;  // may be null
  int per_wg;
  int *status, *pe, *npes;
};

__global__ void ctx_cycle_kernel(CtxCycleArgs a) {
  constexpr int kMaxPerWg = 64;
  __shared__ rocshmem_ctx_t ctxs[kMaxPerWg];
  rocshmem_wg_init();
  for (int k = 0; k < a.per_wg; ++k) {
    int rc;
    if (a.team) rc = rocshmem_wg_team_create_ctx(a.team, 0, &ctxs[k]);
    else rc = rocshmem_wg_ctx_create(0, &ctxs[k]);
    if (threadIdx.x == 0) {
      const int slot = blockIdx.x * a.per_wg + k;
      a.status[slot] = rc;
      a.pe[slot] = rc == 0 ? rocshmem_ctx_my_pe(ctxs[k]) : -2;
      a.npes[slot] = rc == 0 ? rocshmem_ctx_n_pes(ctxs[k]) : -2;
    }
  }
  __syncthreads();
  for (int k = 0; k < a.per_wg; ++k) {
    if (ctxs[k].ctx_opaque) rocshmem_wg_ctx_destroy(&ctxs[k]);
  }
  rocshmem_wg_finalize();
}

template <typename Fn>
bool for_amo_dtype(int dtype, Fn &&fn) {
  switch (dtype) {
    case ROCSHMEM_AMD_INT: fn(static_cast<int *>(nullptr)); return true;
    case ROCSHMEM_AMD_LONG: fn(static_cast<long *>(nullptr)); return true;
    case ROCSHMEM_AMD_LONGLONG: fn(static_cast<long long *>(nullptr)); return true;
    case ROCSHMEM_AMD_UINT: fn(static_cast<unsigned int *>(nullptr)); return true;
    case ROCSHMEM_AMD_ULONG: fn(static_cast<unsigned long *>(nullptr)); return true;
    case ROCSHMEM_AMD_ULONGLONG: fn(static_cast<unsigned long long *>(nullptr)); return true;
    case ROCSHMEM_AMD_FLOAT: fn(static_cast<float *>(nullptr)); return true;
    case ROCSHMEM_AMD_DOUBLE: fn(static_cast<double *>(nullptr)); return true;
    default: return false;
  }
}
template <typename Fn>
bool for_wait_dtype(int dtype, Fn &&fn) {
  if (dtype == ROCSHMEM_AMD_SHORT) {
    fn(static_cast<short *>(nullptr));
    return true;
  }
  return for_amo_dtype(dtype, fn);
}

// Comparator table of rocshmem_<T>_test on the host (src/context_tmpl_device.hpp:337-377).
template <typename T>
bool host_compare(T x, int cmp, T val) {
  switch (cmp) {
    case ROCSHMEM_CMP_EQ: return x == val;
    case ROCSHMEM_CMP_NE: return x != val;
    case ROCSHMEM_CMP_GT: return x > val;
    case ROCSHMEM_CMP_GE: return x >= val;
    case ROCSHMEM_CMP_LT: return x < val;
    case ROCSHMEM_CMP_LE: return x <= val;
    default: return false;
  }
}

// Would the blocking call return without anybody changing ivars?  Read on the
// host from the values as they are now.
template <typename T>
bool wait_already_satisfied(int wait_fn, const T *ivars_dev, size_t nelems, const int *status,
                            int cmp, T value) {
  const size_t n = wait_fn == ROCSHMEM_AMD_WAIT_UNTIL ? 1 : nelems;
  if (!n) return true;  // the vector forms return at once for an empty vector
  std::vector<T> now(n);
  DRV_CHECK_HIP(hipMemcpy(now.data(), ivars_dev, n * sizeof(T), hipMemcpyDeviceToHost));
  if (wait_fn == ROCSHMEM_AMD_WAIT_UNTIL) return host_compare(now[0], cmp, value);
  size_t unmasked = 0, holding = 0;
  for (size_t i = 0; i < n; ++i) {
    if (status && status[i]) continue;
    ++unmasked;
    holding += host_compare(now[i], cmp, value) ? 1 : 0;
  }
  if (!unmasked) return true;
  return wait_fn == ROCSHMEM_AMD_WAIT_UNTIL_ALL ? holding == unmasked : holding > 0;
}

template <typename T>
int run_wait(int wait_fn, void *ivars, size_t nelems, const int *status, int cmp,
             const void *value, int woken, size_t wake_index, const void *wake_value,
             uint64_t delay_ticks, size_t *ret_out, size_t *indices_out) {
  if (!local_ok(ivars, (nelems ? nelems : 1) * sizeof(T))) return -1;
  // A blocking form with nobody to wake it would spin for ever on a condition
  // that does not hold yet: refused, nothing launched — unless the runtime's
  // waits give up after a limit.
  if (!woken && wait_fn != ROCSHMEM_AMD_TEST && runtime::rt().state.spin_limit == 0 &&
      !wait_already_satisfied<T>(wait_fn, static_cast<const T *>(ivars), nelems, status, cmp,
                                 *static_cast<const T *>(value)))
    return -2;
  if (woken && !grid_fits(wait_kernel<T>, 2, 64)) return -1;
  WaitArgs<T> a;
  a.fn = wait_fn;
  a.ivars = static_cast<T *>(ivars);
  a.nelems = nelems;
  a.cmp = cmp;
  a.value = *static_cast<const T *>(value);
  a.woken = woken;
  a.wake_index = wake_index;
  a.wake_value = woken ? *static_cast<const T *>(wake_value) : zero_of<T>();
  a.delay_ticks = delay_ticks;
  int *d_status = nullptr;
  size_t *d_ret, *d_idx;
  const size_t nidx = nelems ? nelems : 1;
  if (status) {
    DRV_CHECK_HIP(hipMalloc(&d_status, nidx * sizeof(int)));
    DRV_CHECK_HIP(hipMemcpy(d_status, status, nelems * sizeof(int), hipMemcpyHostToDevice));
  }
  DRV_CHECK_HIP(hipMalloc(&d_ret, sizeof(size_t)));
  DRV_CHECK_HIP(hipMalloc(&d_idx, nidx * sizeof(size_t)));
  DRV_CHECK_HIP(hipMemset(d_ret, 0, sizeof(size_t)));
  DRV_CHECK_HIP(hipMemset(d_idx, 0xff, nidx * sizeof(size_t)));
  a.status = d_status;
  a.ret = d_ret;
  a.indices = d_idx;
  hipLaunchKernelGGL(wait_kernel<T>, dim3(woken ? 2 : 1), dim3(64), 0, 0, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipDeviceSynchronize());
  if (ret_out) DRV_CHECK_HIP(hipMemcpy(ret_out, d_ret, sizeof(size_t), hipMemcpyDeviceToHost));
  if (indices_out && nelems)
    DRV_CHECK_HIP(hipMemcpy(indices_out, d_idx, nelems * sizeof(size_t), hipMemcpyDeviceToHost));
  if (d_status) DRV_CHECK_HIP(hipFree(d_status));
  DRV_CHECK_HIP(hipFree(d_ret));
  DRV_CHECK_HIP(hipFree(d_idx));
  return 0;
}

// ---------------------------------------------------------------------------
// A loop that polls with gets must see a value another PE has put
// ---------------------------------------------------------------------------
struct PollGetArgs {
  uint64_t *word_a;      // [pairs][8] words on pe_a (the call's symmetric address)
  int64_t a_to_b;        // bytes from pe_a's slice to pe_b's
  uint64_t *ready_a;     // [pairs] on pe_a: round the poller has read the old value in
  int rounds;
  int pe_a, pe_b;
  int kind;              // 0: rocshmem_ctx_uint64_g, 1: getmem, 2: getmem_wave (64 bytes)
  unsigned spin_limit;
  rocshmem_ctx_t ctx_a, ctx_b;
  int *timed_out;
};

// Even work-groups act for pe_a and put; odd ones act for pe_b and poll their
// own copy of the word with gets from themselves — no wait_until, no fence:
// what ends the loop is that a get reads memory, not a cached line.  Every
// wait is bounded.
__global__ void poll_get_kernel(PollGetArgs a) {
  const int pair = blockIdx.x >> 1;
  const bool putter = (blockIdx.x & 1) == 0;
  uint64_t *word = a.word_a + 8 * pair;  // pe_a's address of the pair's eight words
  uint64_t *word_on_b = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(word) + a.a_to_b);
  uint64_t *ready = a.ready_a + pair;
  __shared__ uint64_t got[8];
  for (int r = 1; r <= a.rounds; ++r) {
    if (putter) {
      // the poller has the old value in its caches: now change it
      if (!put_flag_wait(ready, static_cast<uint64_t>(r), a.spin_limit, a.timed_out)) return;
      if (threadIdx.x < 8)
        rocshmem_ctx_uint64_p(a.ctx_a, word + threadIdx.x, static_cast<uint64_t>(r), a.pe_b);
    } else {
      __shared__ int seen;
      int outcome = 0;
      if (threadIdx.x == 0) seen = 0;
      __syncthreads();
      for (unsigned spin = 0; spin < a.spin_limit; ++spin) {
        if (a.kind == 0) {
          if (threadIdx.x == 0) got[7] = rocshmem_ctx_uint64_g(a.ctx_b, word_on_b + 7, a.pe_b);
        } else if (a.kind == 1) {
          if (threadIdx.x == 0) rocshmem_ctx_getmem(a.ctx_b, got, word_on_b, 64, a.pe_b);
        } else {
          if (threadIdx.x < 64) rocshmem_ctx_getmem_wave(a.ctx_b, got, word_on_b, 64, a.pe_b);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
          if (got[7] == static_cast<uint64_t>(r)) seen = 1;
          // first look of the round done: let the putter go
          if (spin == 0) detail::store_through(reinterpret_cast<uint64_t *>(
                                                   reinterpret_cast<char *>(ready)), static_cast<uint64_t>(r));
          if (detail::load_through(a.timed_out)) seen = 2;
        }
        __syncthreads();
        outcome = seen;
        __syncthreads();  // everybody has read it before anybody can write it again
        if (outcome) break;
        __builtin_amdgcn_s_sleep(4);
      }
      if (outcome != 1) {
        if (threadIdx.x == 0) detail::store_through(a.timed_out, 1);
        return;
      }
    }
  }
}

}  // namespace drv
}  // namespace rocshmem

using namespace rocshmem;
using namespace rocshmem::drv;

extern "C" {

int rocshmem_amd_amo(int amo_op, int dtype, void *counters, uint32_t n_slots,
                     const uint32_t *ids, const void *values, const void *conds, void *fetched,
                     size_t n_ops, int my_pe, int n_wgs, int wg_size,
                     rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !valid_launch(n_wgs, wg_size) || !n_slots || !ids) return -1;
  if (amo_op == ROCSHMEM_AMD_AMO_COMPARE_SWAP && !conds) return -1;
  {
    const size_t es = (dtype == ROCSHMEM_AMD_INT || dtype == ROCSHMEM_AMD_UINT ||
                       dtype == ROCSHMEM_AMD_FLOAT) ? 4 : 8;
    if (!sym_ok_on(counters, es * n_slots, my_pe)) return -1;
  }
  int rc = -1;
  const bool known = for_amo_dtype(dtype, [&](auto *tag) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    AmoArgs<T> a;
    a.counters = static_cast<T *>(counters);
    a.n_slots = n_slots;
    a.ids = ids;
    a.values = static_cast<const T *>(values);
    a.conds = static_cast<const T *>(conds);
    a.fetched = static_cast<T *>(fetched);
    a.n_ops = n_ops;
    a.ctx = runtime::rt().driver_ctx_handle(my_pe);
    rc = launch_amo<T>(amo_op, a, n_wgs, wg_size, as_stream(stream));
  });
  return known ? rc : -1;
}

int rocshmem_amd_put_signal(int gran, void *dest, const void *source, size_t nbytes,
                            uint64_t *sig_addr, uint64_t signal, int sig_op, int my_pe, int pe,
                            int n_wgs, int wg_size, int calls, rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !valid_pe(pe) || !valid_launch(n_wgs, wg_size) || calls < 0) return -1;
  if (gran < ROCSHMEM_AMD_THREAD || gran > ROCSHMEM_AMD_WG) return -1;
  if (!sym_ok_on(dest, nbytes, my_pe) || !local_ok(source, nbytes) ||
      !sym_ok_on(sig_addr, 8, my_pe))
    return -1;
  size_t groups = n_wgs;
  if (gran == ROCSHMEM_AMD_WAVE) groups *= (wg_size + 63) / 64;
  if (gran == ROCSHMEM_AMD_THREAD) groups *= wg_size;
  SignalArgs a;
  a.dest = static_cast<char *>(dest);
  a.source = static_cast<const char *>(source);
  a.nbytes = nbytes;
  a.tile = auto_tile(nbytes, groups);
  a.sig_addr = sig_addr;
  a.signal = signal;
  a.sig_op = sig_op;
  a.ctx = runtime::rt().driver_ctx_handle(my_pe);
  a.pe = pe;
  a.calls = calls;
  hipStream_t s = as_stream(stream);
  const dim3 g(n_wgs), b(wg_size);
  if (gran == ROCSHMEM_AMD_WG) hipLaunchKernelGGL(put_signal_kernel<ROCSHMEM_AMD_WG>, g, b, 0, s, a);
  else if (gran == ROCSHMEM_AMD_WAVE) hipLaunchKernelGGL(put_signal_kernel<ROCSHMEM_AMD_WAVE>, g, b, 0, s, a);
  else hipLaunchKernelGGL(put_signal_kernel<ROCSHMEM_AMD_THREAD>, g, b, 0, s, a);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_signal_fetch(int gran, const uint64_t *sig_addr, int my_pe, uint64_t *value_out) {
  if (!valid_actor(my_pe) || !value_out || !sym_ok_on(sig_addr, 8, my_pe)) return -1;
  uint64_t *d_out;
  DRV_CHECK_HIP(hipMalloc(&d_out, 2 * sizeof(uint64_t)));
  DRV_CHECK_HIP(hipMemset(d_out, 0, 2 * sizeof(uint64_t)));
  const dim3 g(1), b(gran == ROCSHMEM_AMD_THREAD ? 1 : (gran == ROCSHMEM_AMD_WAVE ? 64 : 256));
  if (gran == ROCSHMEM_AMD_WG) hipLaunchKernelGGL(signal_fetch_kernel<ROCSHMEM_AMD_WG>, g, b, 0, 0, sig_addr, d_out);
  else if (gran == ROCSHMEM_AMD_WAVE) hipLaunchKernelGGL(signal_fetch_kernel<ROCSHMEM_AMD_WAVE>, g, b, 0, 0, sig_addr, d_out);
  else if (gran == ROCSHMEM_AMD_THREAD) hipLaunchKernelGGL(signal_fetch_kernel<ROCSHMEM_AMD_THREAD>, g, b, 0, 0, sig_addr, d_out);
  else { DRV_CHECK_HIP(hipFree(d_out)); return -1; }
  DRV_CHECK_HIP(hipGetLastError());
  uint64_t out[2];
  DRV_CHECK_HIP(hipMemcpy(out, d_out, sizeof(out), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d_out));
  *value_out = out[0];
  return out[1] == 0 ? 0 : -2;
}

int rocshmem_amd_pingpong(void *buf, uint64_t *sig, size_t nbytes, int iters, int pairs,
                          int pe_a, int pe_b, int wg_size, uint64_t *ticks_out,
                          double *tick_hz_out, rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  if (!valid_pe(pe_a) || !valid_pe(pe_b) || pe_a == pe_b || pairs < 1 || pairs > 128 ||
      !valid_launch(2 * pairs, wg_size) || iters < 0 || nbytes == 0)
    return -1;
  const size_t slot = (nbytes + 255) / 256 * 256;
  if (!sym_ok_on(buf, slot * (pairs - 1) + nbytes, pe_a) || !sym_ok_on(sig, 8u * pairs, pe_a))
    return -1;
  if (!grid_fits(pingpong_kernel, 2L * pairs, wg_size)) return -1;
  auto &r = runtime::rt();
  unsigned long long *d_ticks;
  DRV_CHECK_HIP(hipMalloc(&d_ticks, sizeof(unsigned long long) * pairs));
  DRV_CHECK_HIP(hipMemset(d_ticks, 0, sizeof(unsigned long long) * pairs));
  PingPongArgs a;
  a.buf_a = static_cast<char *>(buf);
  a.sig_a = sig;
  a.nbytes = nbytes;
  a.slot_bytes = slot;
  a.iters = iters;
  a.pe_a = pe_a;
  a.pe_b = pe_b;
  a.pe_stride = r.pe_stride;
  a.ctx_row = r.driver_ctx_row();
  a.world_row = r.d_teams;
  a.ticks = d_ticks;
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL(pingpong_kernel, dim3(2 * pairs), dim3(wg_size), 0, s, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  std::vector<unsigned long long> ticks(pairs);
  DRV_CHECK_HIP(hipMemcpy(ticks.data(), d_ticks, sizeof(unsigned long long) * pairs,
                          hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d_ticks));
  // The slowest pair: all pairs run the same number of round trips at once.
  if (ticks_out) *ticks_out = *std::max_element(ticks.begin(), ticks.end());
  if (tick_hz_out) {
    int khz = 0, dev = 0;
    DRV_CHECK_HIP(hipGetDevice(&dev));
    DRV_CHECK_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    *tick_hz_out = static_cast<double>(khz) * 1e3;
  }
  return 0;
}

int rocshmem_amd_poll_with_gets(uint64_t *words, uint64_t *ready, int pairs, int rounds, int pe_a,
                                int pe_b, int kind, int wg_size, int *timed_out_out,
                                rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  auto &r = runtime::rt();
  if (!valid_pe(pe_a) || !valid_pe(pe_b) || pe_a == pe_b || pairs < 1 || pairs > 128 ||
      !valid_launch(2 * pairs, wg_size) || wg_size < 64 || rounds < 0 || kind < 0 || kind > 2 ||
      !timed_out_out)
    return -1;
  if (!sym_ok_on(words, 64u * pairs, pe_a) || !sym_ok_on(ready, 8u * pairs, pe_a)) return -1;
  if (!grid_fits(poll_get_kernel, 2L * pairs, wg_size)) return -1;
  const int64_t a_to_b = static_cast<int64_t>(pe_b - pe_a) * static_cast<int64_t>(r.pe_stride);
  int *d_timed_out;
  hipStream_t s = as_stream(stream);
  DRV_CHECK_HIP(hipMalloc(&d_timed_out, sizeof(int)));
  DRV_CHECK_HIP(hipMemsetAsync(d_timed_out, 0, sizeof(int), s));
  DRV_CHECK_HIP(hipMemsetAsync(reinterpret_cast<char *>(words) + a_to_b, 0, 64u * pairs, s));
  DRV_CHECK_HIP(hipMemsetAsync(ready, 0, 8u * pairs, s));
  PollGetArgs a;
  a.word_a = words;
  a.a_to_b = a_to_b;
  a.ready_a = ready;
  a.rounds = rounds;
  a.pe_a = pe_a;
  a.pe_b = pe_b;
  a.kind = kind;
  a.spin_limit = 1u << 20;
  a.ctx_a = r.driver_ctx_handle(pe_a);
  a.ctx_b = r.driver_ctx_handle(pe_b);
  a.timed_out = d_timed_out;
  hipLaunchKernelGGL(poll_get_kernel, dim3(2 * pairs), dim3(wg_size), 0, s, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  int timed_out = 0;
  DRV_CHECK_HIP(hipMemcpy(&timed_out, d_timed_out, sizeof(timed_out), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d_timed_out));
  *timed_out_out = timed_out;
  return 0;
}

int rocshmem_amd_put_flag_check(void *data, uint64_t *flags, size_t nbytes, int pairs, int rounds,
                                int pe_a, int pe_b, int wg_size, int with_signal,
                                uint64_t *mismatches_out, int *timed_out_out,
                                rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  auto &r = runtime::rt();
  if (!valid_pe(pe_a) || !valid_pe(pe_b) || pe_a == pe_b || pairs < 1 || pairs > 128 ||
      !valid_launch(2 * pairs, wg_size) || rounds < 0 || nbytes == 0 || (nbytes & 3) ||
      with_signal < 0 || with_signal > 5)
    return -1;
  // Modes 4 and 5 stage the message in the producer's LDS.
  const size_t lds_bytes = with_signal >= 4 ? nbytes : 0;
  if (lds_bytes > (size_t{64} << 10)) return -1;
  const size_t total = nbytes * static_cast<size_t>(pairs);
  if (!sym_ok_on(data, total, pe_a) || !sym_ok_on(flags, 16u * pairs, pe_a)) return -1;
  if (!mismatches_out || !timed_out_out) return -1;
  if (!grid_fits(put_flag_kernel, 2L * pairs, wg_size, lds_bytes)) return -1;
  const int64_t a_to_b = static_cast<int64_t>(pe_b - pe_a) * static_cast<int64_t>(r.pe_stride);
  uint32_t *staging;
  unsigned long long *d_bad;
  int *d_timed_out;
  hipStream_t s = as_stream(stream);
  DRV_CHECK_HIP(hipMalloc(&staging, total));
  DRV_CHECK_HIP(hipMalloc(&d_bad, sizeof(unsigned long long)));
  DRV_CHECK_HIP(hipMalloc(&d_timed_out, sizeof(int)));
  DRV_CHECK_HIP(hipMemsetAsync(d_bad, 0, sizeof(unsigned long long), s));
  DRV_CHECK_HIP(hipMemsetAsync(d_timed_out, 0, sizeof(int), s));
  // Both control arrays start at zero on both PEs.
  DRV_CHECK_HIP(hipMemsetAsync(flags, 0, 16u * pairs, s));
  DRV_CHECK_HIP(hipMemsetAsync(reinterpret_cast<char *>(flags) + a_to_b, 0, 16u * pairs, s));
  PutFlagArgs a;
  a.data_a = static_cast<char *>(data);
  a.a_to_b = a_to_b;
  a.flag_b = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(flags) + a_to_b);
  a.ack_a = flags + pairs;
  a.staging = staging;
  a.nbytes = nbytes;
  a.rounds = rounds;
  a.pe_a = pe_a;
  a.pe_b = pe_b;
  a.with_signal = with_signal;
  a.spin_limit = 1u << 22;
  a.ctx_a = r.driver_ctx_handle(pe_a);
  a.mismatches = d_bad;
  a.timed_out = d_timed_out;
  hipLaunchKernelGGL(put_flag_kernel, dim3(2 * pairs), dim3(wg_size), lds_bytes, s, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  unsigned long long bad = 0;
  int timed_out = 0;
  DRV_CHECK_HIP(hipMemcpy(&bad, d_bad, sizeof(bad), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipMemcpy(&timed_out, d_timed_out, sizeof(timed_out), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(staging));
  DRV_CHECK_HIP(hipFree(d_bad));
  DRV_CHECK_HIP(hipFree(d_timed_out));
  *mismatches_out = bad;
  *timed_out_out = timed_out;
  return 0;
}

// Device copy of the last routing tables seen, so that a dispatch repeated
// with the same tables only launches.
namespace {
struct DispatchTables {
  std::mutex lock;             // one caller at a time rebuilds or reads the tables
  std::vector<uint32_t> host;  // count | send_row | recv_row | calls {pair, first row}
  uint32_t *dev = nullptr;
  size_t pp = 0;
  uint32_t rows_per_call = 0;
  uint32_t n_calls = 0;
  size_t max_send = 0, max_recv = 0;
};
DispatchTables g_tables;
}  // namespace

int rocshmem_amd_dispatch_put_signal(void *recv, const void *send, uint64_t *sig,
                                     const uint32_t *count, const uint32_t *send_row,
                                     const uint32_t *recv_row, size_t row_bytes,
                                     int rows_per_call, int wg_size, uint64_t *expect,
                                     rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  auto &r = runtime::rt();
  if (!r.live || rows_per_call < 1 || !valid_launch(1, wg_size) || !row_bytes) return -1;
  if (expect && !local_ok(expect, 8 * static_cast<size_t>(r.npes) * r.npes)) return -1;
  if (!count || !send_row || !recv_row) return -1;
  const size_t pp = static_cast<size_t>(r.npes) * r.npes;
  DispatchTables &t = g_tables;
  std::lock_guard<std::mutex> guard(t.lock);
  std::vector<uint32_t> h(3 * pp);
  std::copy(count, count + pp, h.begin());
  std::copy(send_row, send_row + pp, h.begin() + pp);
  std::copy(recv_row, recv_row + pp, h.begin() + 2 * pp);
  const bool same = t.dev && t.pp == pp && t.rows_per_call == static_cast<uint32_t>(rows_per_call) &&
                    std::equal(h.begin(), h.begin() + 3 * pp, t.host.begin());
  if (!same) {
    // Bounds of every pair's rows and the list of calls.
    t.max_send = t.max_recv = 0;
    uint32_t calls = 0;
    for (size_t i = 0; i < pp; ++i) {
      t.max_send = std::max<size_t>(t.max_send, static_cast<size_t>(h[pp + i]) + h[i]);
      t.max_recv = std::max<size_t>(t.max_recv, static_cast<size_t>(h[2 * pp + i]) + h[i]);
      for (uint32_t first = 0; first < h[i]; first += static_cast<uint32_t>(rows_per_call)) {
        h.push_back(static_cast<uint32_t>(i));
        h.push_back(first);
        ++calls;
      }
    }
    DRV_CHECK_HIP(hipDeviceSynchronize());  // nobody is reading the old tables any more
    if (t.dev) DRV_CHECK_HIP(hipFree(t.dev));
    DRV_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&t.dev), h.size() * 4));
    DRV_CHECK_HIP(hipMemcpy(t.dev, h.data(), h.size() * 4, hipMemcpyHostToDevice));
    t.host = h;
    t.pp = pp;
    t.rows_per_call = static_cast<uint32_t>(rows_per_call);
    t.n_calls = calls;
  }
  if (!sym_ok_on(send, t.max_send * row_bytes, 0) || !sym_ok_on(recv, t.max_recv * row_bytes, 0) ||
      !sym_ok_on(sig, 8 * static_cast<size_t>(r.npes), 0))
    return -1;
  DispatchArgs a;
  a.recv0 = static_cast<char *>(recv);
  a.send0 = static_cast<const char *>(send);
  a.sig0 = sig;
  a.count = t.dev;
  a.send_row = t.dev + pp;
  a.recv_row = t.dev + 2 * pp;
  a.calls = reinterpret_cast<const uint2 *>(t.dev + 3 * pp);
  a.row_bytes = row_bytes;
  a.pe_stride = r.pe_stride;
  a.np = r.npes;
  a.rows_per_call = static_cast<uint32_t>(rows_per_call);
  a.n_calls = t.n_calls;
  a.ctx_row = r.driver_ctx_row();
  a.world_row = r.d_teams;
  a.expect = expect;
  // One call per work-group where the grid allows it: work-groups start in
  // call order, so the senders sweep each pair's rows together (6.3 TB/s
  // against 6.1 when 16384 work-groups loop over 32768 calls).
  const uint32_t max_senders = 1u << 20;
  const uint32_t senders = a.n_calls < max_senders ? (a.n_calls ? a.n_calls : 1) : max_senders;
  hipLaunchKernelGGL(dispatch_kernel, dim3(senders + r.npes), dim3(wg_size), 0, as_stream(stream), a);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_wait_test(int wait_fn, int dtype, void *ivars, size_t nelems, const int *status,
                           int cmp, const void *value, size_t *ret_out, size_t *indices_out) {
  if (!runtime::rt().live || !ivars || !value) return -1;
  if (wait_fn < ROCSHMEM_AMD_TEST || wait_fn > ROCSHMEM_AMD_WAIT_UNTIL_SOME) return -1;
  int rc = -1;
  const bool known = for_wait_dtype(dtype, [&](auto *tag) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    rc = run_wait<T>(wait_fn, ivars, nelems, status, cmp, value, 0, 0, nullptr, 0, ret_out,
                     indices_out);
  });
  return known ? rc : -1;
}

int rocshmem_amd_wait_test_woken(int wait_fn, int dtype, void *ivars, size_t nelems,
                                 const int *status, int cmp, const void *value,
                                 size_t wake_index, const void *wake_value,
                                 uint64_t delay_ticks, size_t *ret_out, size_t *indices_out) {
  DRV_ONE_PROCESS_ONLY();
  if (!runtime::rt().live || !ivars || !value || !wake_value) return -1;
  if (wait_fn < ROCSHMEM_AMD_WAIT_UNTIL || wait_fn > ROCSHMEM_AMD_WAIT_UNTIL_SOME) return -1;
  if (wake_index >= (nelems ? nelems : 1)) return -1;
  int rc = -1;
  const bool known = for_wait_dtype(dtype, [&](auto *tag) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    rc = run_wait<T>(wait_fn, ivars, nelems, status, cmp, value, 1, wake_index, wake_value,
                     delay_ticks, ret_out, indices_out);
  });
  return known ? rc : -1;
}

int rocshmem_amd_poll_until(int dtype, void *ivar, int cmp, const void *value, uint64_t max_polls,
                            uint64_t *result_dev, rocshmem_amd_stream_t stream) {
  if (!runtime::rt().live || !ivar || !value || !result_dev || !max_polls) return -1;
  if (!local_ok(ivar, 8) || !local_ok(result_dev, 16)) return -1;
  hipStream_t s = as_stream(stream);
  const bool known = for_wait_dtype(dtype, [&](auto *tag) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    hipLaunchKernelGGL(poll_until_kernel<T>, dim3(1), dim3(1), 0, s, static_cast<T *>(ivar), cmp,
                       *static_cast<const T *>(value), static_cast<unsigned long long>(max_polls),
                       reinterpret_cast<unsigned long long *>(result_dev));
  });
  if (!known) return -1;
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_ctx_cycle(rocshmem_amd_team_t team, int n_wgs, int wg_size, int per_wg,
                           int *status_out, int *pe_out, int *npes_out) {
  DRV_ONE_PROCESS_ONLY();
  if (!runtime::rt().live || !valid_launch(n_wgs, wg_size) || per_wg < 1 || per_wg > 64)
    return -1;
  if (!status_out || !pe_out || !npes_out) return -1;
  const size_t n = static_cast<size_t>(n_wgs) * per_wg;
  int *d;
  DRV_CHECK_HIP(hipMalloc(&d, 3 * n * sizeof(int)));
  DRV_CHECK_HIP(hipMemset(d, 0xff, 3 * n * sizeof(int)));
  CtxCycleArgs a{static_cast<rocshmem_team_t>(team), per_wg, d, d + n, d + 2 * n};
  hipLaunchKernelGGL(ctx_cycle_kernel, dim3(n_wgs), dim3(wg_size), 0, 0, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipDeviceSynchronize());
  DRV_CHECK_HIP(hipMemcpy(status_out, d, n * sizeof(int), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipMemcpy(pe_out, d + n, n * sizeof(int), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipMemcpy(npes_out, d + 2 * n, n * sizeof(int), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d));
  return 0;
}

}  // extern "C"

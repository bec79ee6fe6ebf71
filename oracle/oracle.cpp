// CPU oracle for the symmetric-heap data-movement path.
//
// TEST INFRASTRUCTURE ONLY.  This file restates, on the CPU, what the
// reference library computes on the path this repository implements for the
// GPU.  Only tests/, the smoke check and the cpu_baseline leg of bench.py may
// build, load or call it; the product never does.
//
// Every function cites the reference source it follows.  Where this repository
// deliberately defines behaviour the reference lacks or leaves open (ascending
// PE order for floating-point sums, bf16), the function says so.
//
// What pins each function (see tests/test_oracle_*.py):
//   allocator      the reference's own allocator headers compiled into
//                  oracle/_ref (random request sequences) + the known answers
//                  of tests/unit_tests/{single_heap,pow2_bins,binner}_gtest.cpp
//   PE/team math   closed forms + tests/sos_tests/shmem_team_translate.cpp
//   copy           identity (memcmp) — nothing to pin
//   coalesce       the worked example in src/wf_coal_policy.cpp:41-53 + brute
//                  force against an independent run-length formulation
//   reductions     closed forms of examples/rocshmem_allreduce_test.cc,
//                  tests/sos_tests/to_all.cpp, numpy for integer ops;
//                  floating-point sums: the ascending order is this
//                  repository's definition, cross-checked against the
//                  reference-order model below to (P-1) ulp
//   bf16           parity unpinned by the reference (it has no bf16); pinned
//                  by exhaustive comparison with an independent formulation
//   alltoall etc.  index identities + example/test vectors of the reference
//   atomics        sum invariants + tests/functional_tests/amo_*_tester.cpp
//   waits          comparator truth table by brute force
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <stack>
#include <thread>
#include <type_traits>
#include <vector>

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

// ----------------------------------------------------------------------------
// dtype / op codes (same numbering as include/rocshmem_amd.h)
// ----------------------------------------------------------------------------
enum { DT_SHORT, DT_INT, DT_LONG, DT_LONGLONG, DT_FLOAT, DT_DOUBLE, DT_BF16, DT_UINT, DT_ULONG,
       DT_ULONGLONG, DT_CHAR, DT_SCHAR, DT_UCHAR, DT_USHORT };
enum { OP_SUM, OP_MAX, OP_MIN, OP_PROD, OP_AND, OP_OR, OP_XOR };

inline float bf16_to_f32(uint16_t b) {
  uint32_t u = static_cast<uint32_t>(b) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// dst = dst op src, element-wise: OpWrap<Op>::Calc, src/rocshmem_calc.hpp:43-97.
// Integer + and * wrap (two's complement), as on the device.
template <typename T>
inline T combine(int op, T acc, T x) {
  if constexpr (std::is_integral<T>::value) {
    using U = typename std::make_unsigned<T>::type;
    switch (op) {
      case OP_SUM: return static_cast<T>(static_cast<U>(static_cast<U>(acc) + static_cast<U>(x)));
      case OP_PROD: return static_cast<T>(static_cast<U>(static_cast<U>(acc) * static_cast<U>(x)));
      case OP_MAX: return acc < x ? x : acc;
      case OP_MIN: return x < acc ? x : acc;
      case OP_AND: return static_cast<T>(acc & x);
      case OP_OR: return static_cast<T>(acc | x);
      default: return static_cast<T>(acc ^ x);
    }
  } else {
    switch (op) {
      case OP_SUM: return acc + x;
      case OP_PROD: return acc * x;
      case OP_MAX: return std::fmax(acc, x);  // HIP max(float,float) is fmaxf
      default: return std::fmin(acc, x);
    }
  }
}

template <typename Fn>
void parallel_for(size_t n, int nthreads, Fn fn) {
  if (nthreads <= 1 || n < 2) {
    fn(size_t{0}, n, 0);
    return;
  }
  std::vector<std::thread> pool;
  const size_t per = (n + nthreads - 1) / nthreads;
  for (int t = 0; t < nthreads; ++t) {
    const size_t lo = std::min(n, per * t), hi = std::min(n, lo + per);
    if (lo == hi) break;
    pool.emplace_back([=] { fn(lo, hi, t); });
  }
  for (auto &th : pool) th.join();
}

// Ascending-PE left fold of elements [lo, hi): this repository's contract for
// the all-reduce result (bit-exact definition for floating-point sums).  For
// integers, bitwise ops and min/max it equals any order, hence the reference.
template <typename T>
void fold_range(int op, int P, const T *const *srcs, T *const *dsts, int ndst, size_t lo, size_t hi) {
  for (size_t i = lo; i < hi; ++i) {
    T acc = srcs[0][i];
    for (int p = 1; p < P; ++p) acc = combine<T>(op, acc, srcs[p][i]);
    for (int d = 0; d < ndst; ++d) dsts[d][i] = acc;
  }
}
void fold_range_bf16(int P, const uint16_t *const *srcs, uint16_t *const *dsts, int ndst, size_t lo,
                     size_t hi) {
  for (size_t i = lo; i < hi; ++i) {
    float acc = bf16_to_f32(srcs[0][i]);
    for (int p = 1; p < P; ++p) acc = acc + bf16_to_f32(srcs[p][i]);
    const uint16_t out = f32_to_bf16(acc);
    for (int d = 0; d < ndst; ++d) dsts[d][i] = out;
  }
}

template <typename T>
int to_all_typed(int op, int P, size_t n, const void *const *srcs, void *const *dsts, int ndst,
                 int nthreads) {
  if (!std::is_integral<T>::value && op > OP_PROD) return -1;
  parallel_for(n, nthreads, [&](size_t lo, size_t hi, int) {
    fold_range<T>(op, P, reinterpret_cast<const T *const *>(srcs),
                  reinterpret_cast<T *const *>(dsts), ndst, lo, hi);
  });
  return 0;
}

}  // namespace

// ============================================================================
// Seeded inputs.  Counter-based: value i of stream `stream` depends only on
// (seed, stream, i).  (Workload definition of this repository; no reference
// counterpart.)
// ============================================================================
static inline uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}
static inline uint64_t draw(uint64_t seed, uint64_t stream, uint64_t i) {
  return splitmix64(splitmix64(seed * 0x100000001B3ull + stream) + i);
}

ORC_API uint64_t orc_draw(uint64_t seed, uint64_t stream, uint64_t i) { return draw(seed, stream, i); }

ORC_API void orc_fill_u8(uint8_t *buf, size_t n, uint64_t seed, uint64_t stream) {
  for (size_t i = 0; i < n; ++i) buf[i] = static_cast<uint8_t>(draw(seed, stream, i >> 3) >> ((i & 7) * 8));
}
ORC_API void orc_fill_u64(uint64_t *buf, size_t n, uint64_t seed, uint64_t stream) {
  for (size_t i = 0; i < n; ++i) buf[i] = draw(seed, stream, i);
}
// Uniform integer in [-1000, 1000].
ORC_API void orc_fill_i32_pm1000(int32_t *buf, size_t n, uint64_t seed, uint64_t stream) {
  for (size_t i = 0; i < n; ++i) buf[i] = static_cast<int32_t>(draw(seed, stream, i) % 2001u) - 1000;
}
// N(0,1): Box-Muller on two 24-bit uniforms, computed in float.
ORC_API void orc_fill_normal_f32(float *buf, size_t n, uint64_t seed, uint64_t stream) {
  for (size_t i = 0; i < n; ++i) {
    const uint64_t r = draw(seed, stream, i);
    const float u1 = (static_cast<float>((r >> 40) & 0xFFFFFFu) + 1.0f) * (1.0f / 16777216.0f);
    const float u2 = static_cast<float>((r >> 8) & 0xFFFFFFu) * (1.0f / 16777216.0f);
    buf[i] = std::sqrt(-2.0f * std::log(u1)) * std::cos(6.28318530717958647692f * u2);
  }
}
ORC_API void orc_f32_to_bf16(const float *in, uint16_t *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = f32_to_bf16(in[i]);
}
ORC_API void orc_bf16_to_f32(const uint16_t *in, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = bf16_to_f32(in[i]);
}
// Zipf(s) over K items (item 0 most likely) by inverse CDF built in double.
ORC_API void orc_fill_zipf_u32(uint32_t *buf, size_t n, uint64_t seed, uint64_t stream, uint32_t K,
                               double s) {
  std::vector<double> cdf(K);
  double z = 0;
  for (uint32_t k = 0; k < K; ++k) z += 1.0 / std::pow(static_cast<double>(k + 1), s);
  double acc = 0;
  for (uint32_t k = 0; k < K; ++k) {
    acc += 1.0 / std::pow(static_cast<double>(k + 1), s) / z;
    cdf[k] = acc;
  }
  cdf[K - 1] = 1.0;
  for (size_t i = 0; i < n; ++i) {
    const double u = static_cast<double>(draw(seed, stream, i) >> 11) * (1.0 / 9007199254740992.0);
    buf[i] = static_cast<uint32_t>(std::lower_bound(cdf.begin(), cdf.end(), u) - cdf.begin());
    if (buf[i] >= K) buf[i] = K - 1;
  }
}

// ============================================================================
// H1  Symmetric-heap allocator.
// Follows src/memory/pow2_bins.hpp:90-152,264-287 (alloc / free / split),
// binner.hpp:109-231 (bin set, head alignment, largest-first carving),
// bin.hpp:41-77 (a bin is a stack), address_record.hpp:83-98 (split in
// halves), single_heap.cpp:39-62 (size 0 -> null, free(null) ignored, used =
// sum of handed-out block sizes).  Addresses are plain integers here.
// ============================================================================
namespace {
struct Record {
  uint64_t addr = 0;
  uint64_t size = 0;
};
struct OrcHeap {
  std::map<uint64_t, std::stack<Record>> bins;
  std::map<uint64_t, Record> proffered;
  uint64_t heap_size = 0;
};
constexpr uint64_t kAlignment = 128;  // src/constants.hpp:39

void split_larger_bin(OrcHeap &h, std::map<uint64_t, std::stack<Record>>::iterator it) {
  auto next = std::next(it);
  if (next == h.bins.end()) return;
  if (next->second.empty()) split_larger_bin(h, next);
  if (next->second.empty()) return;
  Record r = next->second.top();
  next->second.pop();
  const uint64_t half = r.size >> 1;
  it->second.push(Record{r.addr + half, half});  // "larger" address first ...
  it->second.push(Record{r.addr, half});         // ... so the lower one is on top
}
}  // namespace

ORC_API void *orc_heap_create(uint64_t base_addr, uint64_t heap_size) {
  OrcHeap *h = new OrcHeap;
  h->heap_size = heap_size;
  if (heap_size < kAlignment) return h;
  // Binner ctor: one bin per power of two from 2^7 to 2^msb(heap_size).
  int msb = 63;
  while (!((heap_size >> msb) & 1)) --msb;
  for (int b = 7; b <= msb; ++b) h->bins[uint64_t{1} << b];
  // ignore_unaligned_heap_memory
  uint64_t addr = base_addr, size = heap_size;
  if (addr % kAlignment) {
    const uint64_t skip = kAlignment - addr % kAlignment;
    addr += skip;
    size -= skip;
  }
  // assign_heap_memory_to_bins / assign_heap_chunk
  while (true) {
    auto rit = h->bins.rbegin();
    while (rit != h->bins.rend() && size < rit->first) ++rit;
    if (rit == h->bins.rend()) break;
    rit->second.push(Record{addr, rit->first});
    addr += rit->first;
    size -= rit->first;
  }
  return h;
}
ORC_API void orc_heap_destroy(void *hp) { delete static_cast<OrcHeap *>(hp); }
// Returns the block address, or 0 for "nullptr".
ORC_API uint64_t orc_heap_alloc(void *hp, uint64_t request) {
  OrcHeap &h = *static_cast<OrcHeap *>(hp);
  if (!request) return 0;
  auto attempt = [&](std::map<uint64_t, std::stack<Record>>::iterator it) -> uint64_t {
    if (it == h.bins.end()) return 0;
    if (it->second.empty()) split_larger_bin(h, it);
    if (it->second.empty()) return 0;
    Record r = it->second.top();
    it->second.pop();
    if (r.addr) h.proffered[r.addr] = r;
    return r.addr;
  };
  const uint64_t exact = attempt(h.bins.find(request));
  if (exact) return exact;
  return attempt(h.bins.lower_bound(request));
}
ORC_API int orc_heap_free(void *hp, uint64_t addr) {
  OrcHeap &h = *static_cast<OrcHeap *>(hp);
  if (!addr) return 0;
  auto it = h.proffered.find(addr);
  if (it == h.proffered.end()) return -1;
  h.bins[it->second.size].push(it->second);
  h.proffered.erase(it);
  return 0;
}
ORC_API uint64_t orc_heap_used(void *hp) {
  uint64_t s = 0;
  for (auto &kv : static_cast<OrcHeap *>(hp)->proffered) s += kv.second.size;
  return s;
}
ORC_API uint64_t orc_heap_avail(void *hp) {
  return static_cast<OrcHeap *>(hp)->heap_size - orc_heap_used(hp);
}
ORC_API uint64_t orc_heap_num_bins(void *hp) { return static_cast<OrcHeap *>(hp)->bins.size(); }
ORC_API uint64_t orc_heap_bin_population(void *hp, uint64_t block_size) {
  auto &b = static_cast<OrcHeap *>(hp)->bins;
  auto it = b.find(block_size);
  return it == b.end() ? 0 : it->second.size();
}

// ============================================================================
// H2  PE / team arithmetic.  src/team.cpp:51-111, src/rocshmem_gpu.cpp:267-274,
// :606-635, src/rocshmem.cpp:209-262.
// ============================================================================
ORC_API int orc_pe_in_world(int pe_start, int stride, int pe_in_team) {
  return pe_start + stride * pe_in_team;
}
ORC_API int orc_pe_in_team(int pe_start, int stride, int size, int pe_in_world) {
  if (pe_in_world < pe_start) return -1;
  if ((pe_in_world - pe_start) % stride) return -1;
  const int rel = (pe_in_world - pe_start) / stride;
  return rel >= size ? -1 : rel;
}
// team_translate_pe with both teams given by their world triples; a team with
// size <= 0 stands for ROCSHMEM_TEAM_INVALID.
ORC_API int orc_team_translate_pe(int s_start, int s_stride, int s_size, int src_pe, int d_start,
                                  int d_stride, int d_size) {
  if (s_size <= 0 || d_size <= 0) return -1;
  return orc_pe_in_team(d_start, d_stride, d_size, orc_pe_in_world(s_start, s_stride, src_pe));
}
// rocshmem_team_split_strided argument checks and world triple
// (src/rocshmem.cpp:243-262).  Returns 0 and fills out[3] = {start, stride,
// size} wrt world, or -1.  `strict` = 1 also rejects a last member beyond the
// last PE, which the reference's `>` comparison lets through.
ORC_API int orc_split_strided(int p_start, int p_stride, int p_size, int npes, int start, int stride,
                              int size, int strict, int *out) {
  if (start < 0 || start >= p_size || size < 1 || size > p_size || stride < 1) return -1;
  const int start_w = p_start + p_stride * start;
  const int stride_w = stride * p_stride;
  const int end_w = start_w + stride_w * (size - 1);
  if (end_w > npes) return -1;
  if (strict && end_w >= npes) return -1;
  out[0] = start_w;
  out[1] = stride_w;
  out[2] = size;
  return 0;
}

// H3  Address translation: ipc_bases[pe] + (dest - ipc_bases[my_pe])
// (src/ipc/context_ipc_device.cpp:62-69).
ORC_API uint64_t orc_translate(const uint64_t *ipc_bases, uint64_t dest, int my_pe, int pe) {
  return ipc_bases[pe] + (dest - ipc_bases[my_pe]);
}

// ============================================================================
// C1-C3  Copy.  The contract is a byte-exact copy.
// ============================================================================
ORC_API void orc_copy(void *dst, const void *src, size_t n) { memmove(dst, src, n); }

// Lane-by-lane model of the reference's memcpy_wg / memcpy_wave loop
// (src/util.hpp:188-262) with `lanes` cooperating lanes, INCLUDING its tail
// defect: the final one-byte move uses the pointers lane 0 last formed inside
// the 8/4/2-byte loops instead of the advanced base, so for odd n >= 3 it
// re-copies an earlier byte and the last byte is never written.
ORC_API void orc_ref_memcpy_lanes_model(uint8_t *dst, const uint8_t *src, size_t size, int lanes) {
  uint8_t *dst_def = dst;
  const uint8_t *src_def = src;
  // per-lane "dst_bytes/src_bytes" as left by the loops; only lane 0's matter
  uint8_t *lane0_dst = dst;
  const uint8_t *lane0_src = src;
  for (int j = 8; j > 1; j >>= 1) {
    const int cpy = static_cast<int>(size / j);
    for (int lane = 0; lane < lanes; ++lane) {
      for (int i = lane; i < cpy; i += lanes) {
        memcpy(dst_def + static_cast<size_t>(i) * j, src_def + static_cast<size_t>(i) * j, j);
        if (lane == 0) {
          lane0_dst = dst_def + static_cast<size_t>(i) * j;
          lane0_src = src_def + static_cast<size_t>(i) * j;
        }
      }
    }
    size -= static_cast<size_t>(cpy) * j;
    dst_def += static_cast<size_t>(cpy) * j;
    src_def += static_cast<size_t>(cpy) * j;
  }
  if (size == 1) *lane0_dst = *lane0_src;
}

// Threaded memcpy: the CPU baseline of the bulk copy.
ORC_API void orc_copy_threaded(void *dst, const void *src, size_t n, int nthreads) {
  parallel_for(n, nthreads, [&](size_t lo, size_t hi, int) {
    memcpy(static_cast<char *>(dst) + lo, static_cast<const char *>(src) + lo, hi - lo);
  });
}

// ============================================================================
// C4  Wavefront coalescing.  Lane simulator of WfCoalOn::coalesce,
// src/wf_coal_policy.cpp:119-171.
// ============================================================================
ORC_API void orc_wf_coalesce(const int *pe, const uint64_t *src, const uint64_t *dst,
                             const uint64_t *size, uint64_t active_mask, int *sends,
                             uint64_t *size_out) {
  bool coal[64];
  for (int l = 0; l < 64; ++l) {
    coal[l] = false;
    if (!((active_mask >> l) & 1)) continue;
    // __shfl_up(x, 1): lane 0 receives its own value.
    const int lo = l == 0 ? 0 : l - 1;
    const uint64_t lower_size = static_cast<uint32_t>(size[lo]);
    coal[l] = l != 0 && ((active_mask >> (l - 1)) & 1) && lower_size == size[l] &&
              src[lo] + size[l] == src[l] && dst[lo] + size[l] == dst[l] && pe[l] == pe[lo];
  }
  uint64_t ballot = 0;
  for (int l = 0; l < 64; ++l)
    if (coal[l]) ballot |= uint64_t{1} << l;
  for (int l = 0; l < 64; ++l) {
    if (!((active_mask >> l) & 1)) continue;
    sends[l] = !coal[l];
    size_out[l] = size[l];
    if (!coal[l]) {
      const uint64_t above = l == 63 ? 0 : ballot >> (l + 1);
      const int first_zero = __builtin_ffsll(static_cast<long long>(~above));  // 1-based
      if (first_zero) size_out[l] = size[l] + size[l] * static_cast<uint64_t>(first_zero - 1);
    }
  }
}

// ============================================================================
// R  All-reduce.
// ============================================================================
// Result of the all-reduce over P sources, written to `ndst` destinations.
// Order: ascending PE, (((x0 op x1) op x2) ...) — this repository's contract
// (the reference's order is modelled separately below).  bf16: widen to fp32,
// fold in fp32, round to nearest even once.  nthreads > 1 splits the index
// range; this is also the threaded CPU baseline.
ORC_API int orc_to_all(int dtype, int op, int P, size_t n, const void *const *srcs,
                       void *const *dsts, int ndst, int nthreads) {
  if (P < 1) return -1;
  switch (dtype) {
    case DT_SHORT: return to_all_typed<int16_t>(op, P, n, srcs, dsts, ndst, nthreads);
    case DT_INT: return to_all_typed<int32_t>(op, P, n, srcs, dsts, ndst, nthreads);
    case DT_LONG:
    case DT_LONGLONG: return to_all_typed<int64_t>(op, P, n, srcs, dsts, ndst, nthreads);
    case DT_FLOAT: return to_all_typed<float>(op, P, n, srcs, dsts, ndst, nthreads);
    case DT_DOUBLE: return to_all_typed<double>(op, P, n, srcs, dsts, ndst, nthreads);
    case DT_BF16:
      if (op != OP_SUM) return -1;
      parallel_for(n, nthreads, [&](size_t lo, size_t hi, int) {
        fold_range_bf16(P, reinterpret_cast<const uint16_t *const *>(srcs),
                        reinterpret_cast<uint16_t *const *>(dsts), ndst, lo, hi);
      });
      return 0;
    default: return -1;
  }
}

// Which algorithm the reference's IPCContext::reduce picks and with what
// geometry (src/ipc/context_ipc_tmpl_device.hpp:361-418).
// out = {status, algo (0 direct, 1 ring), n_seg, seg_size, chunk_size,
//        has_remainder_ring, p_count, p_chunk, tail_direct_count}
ORC_API void orc_reduce_plan(int P, int nreduce, int *out) {
  for (int i = 0; i < 9; ++i) out[i] = 0;
  const size_t direct_pWrk = static_cast<size_t>(P) * nreduce;
  const size_t provided_pWrk = std::max<size_t>(nreduce / 2 + 1, 1024);
  if (provided_pWrk >= direct_pWrk && 256 >= static_cast<size_t>(P)) {
    out[1] = 0;
    return;
  }
  if (static_cast<size_t>(2 * P) > 256) {
    out[0] = 1;  // ROCSHMEM_ERROR
    return;
  }
  out[1] = 1;
  int chunk = 1024 / P;
  const int seg = chunk * P;
  int n_seg = nreduce / seg;
  const int n_seg_up = (nreduce - 1) / seg + 1;
  chunk = seg / P;
  if (n_seg == 0) n_seg = 1;
  out[2] = n_seg;
  out[3] = seg;
  out[4] = chunk;
  if (n_seg_up > n_seg) {
    out[5] = 1;
    const int p_count = nreduce - n_seg * seg;
    const int p_chunk = p_count / P;
    out[6] = p_count;
    out[7] = p_chunk;
    if (p_chunk * P < p_count) out[8] = p_count - p_chunk * P;
  }
}

// Floating-point sum in the ORDER the reference would use, for element index i
// as seen by PE `pe` (float only; used to bound the difference from the
// ascending order).  direct: own value first, then the others ascending
// (context_ipc_tmpl_device.hpp:183-215).  ring: chunk c of a segment is folded
// starting at PE c-1 and going up cyclically, and every PE receives that one
// result (:308-352).
ORC_API void orc_reduce_f32_sum_reference_order(int P, int nreduce, const float *const *srcs, int pe,
                                                float *dst) {
  int plan[9];
  orc_reduce_plan(P, nreduce, plan);
  auto direct = [&](int lo, int count) {
    for (int i = lo; i < lo + count; ++i) {
      float acc = srcs[pe][i];
      for (int q = 0; q < P; ++q)
        if (q != pe) acc += srcs[q][i];
      dst[i] = acc;
    }
  };
  auto ring = [&](int lo, int n_seg, int seg, int chunk) {
    for (int s = 0; s < n_seg; ++s)
      for (int c = 0; c < P; ++c)
        for (int k = 0; k < chunk; ++k) {
          const int i = lo + s * seg + c * chunk + k;
          // For 1024/P < nreduce < 1024 the reference still walks a whole
          // 1024-element segment and so touches memory past nreduce; the
          // elements below nreduce are what this model reports.
          if (i >= nreduce) continue;
          float acc = srcs[(c - 1 + P) % P][i];
          for (int step = 0; step < P - 1; ++step) acc = srcs[(c + step) % P][i] + acc;
          dst[i] = acc;
        }
  };
  if (plan[0]) return;
  if (plan[1] == 0) {
    direct(0, nreduce);
    return;
  }
  ring(0, plan[2], plan[3], plan[4]);
  if (plan[5]) {
    const int base = plan[2] * plan[3];
    if (plan[7] > 0) ring(base, 1, plan[7] * P, plan[7]);
    if (plan[8]) direct(base + plan[7] * P, plan[8]);
  }
}

// ============================================================================
// A2A / FC / BC  (src/ipc/context_ipc_tmpl_device.hpp:420-531)
//   alltoall : dst_j[i*n + k] = src_i[j*n + k]      for all i, j (self included)
//   fcollect : dst_j[i*n + k] = src_i[k]
//   broadcast: dst_j[k] = src_root[k] for j != root; root's dst untouched
// n in bytes.  Threaded over (i, j) blocks.
// ============================================================================
ORC_API void orc_alltoall(int P, size_t n, const void *const *srcs, void *const *dsts, int nthreads) {
  parallel_for(static_cast<size_t>(P) * P, nthreads, [&](size_t lo, size_t hi, int) {
    for (size_t b = lo; b < hi; ++b) {
      const int i = static_cast<int>(b / P), j = static_cast<int>(b % P);
      memcpy(static_cast<char *>(dsts[j]) + i * n, static_cast<const char *>(srcs[i]) + j * n, n);
    }
  });
}
ORC_API void orc_fcollect(int P, size_t n, const void *const *srcs, void *const *dsts, int nthreads) {
  parallel_for(static_cast<size_t>(P) * P, nthreads, [&](size_t lo, size_t hi, int) {
    for (size_t b = lo; b < hi; ++b) {
      const int i = static_cast<int>(b / P), j = static_cast<int>(b % P);
      memcpy(static_cast<char *>(dsts[j]) + i * n, srcs[i], n);
    }
  });
}
ORC_API void orc_broadcast(int P, size_t n, int root, const void *const *srcs, void *const *dsts) {
  for (int j = 0; j < P; ++j)
    if (j != root) memcpy(dsts[j], srcs[root], n);
}

// ============================================================================
// A1  Atomic memory operations: one serialisation (program order of the op
// list) of the RMWs of src/ipc_policy.hpp:69-99.  counters: all P*n_slots
// counters laid out PE-major.  Element type int64 / uint64 (bit patterns).
// ops as in include/rocshmem_amd.h.
// ============================================================================
ORC_API int orc_amo_i64(int amo_op, int64_t *counters, const uint32_t *ids, const int64_t *values,
                        const int64_t *conds, int64_t *fetched, size_t n_ops) {
  for (size_t i = 0; i < n_ops; ++i) {
    int64_t &c = counters[ids[i]];
    const int64_t v = values ? values[i] : 1;
    const int64_t old = c;
    switch (amo_op) {
      case 0: case 1: c = static_cast<int64_t>(static_cast<uint64_t>(c) + static_cast<uint64_t>(v)); break;
      case 2: case 3: c = static_cast<int64_t>(static_cast<uint64_t>(c) + 1u); break;
      case 4: if (c == conds[i]) c = v; break;
      case 5: break;
      case 6: case 7: c = v; break;
      case 8: c &= v; break;
      case 9: c |= v; break;
      case 10: c ^= v; break;
      default: return -1;
    }
    if (fetched) fetched[i] = old;
  }
  return 0;
}
// Threaded fetch_add on std::atomic (seq_cst): the CPU baseline of the AMO
// workload.  Returns elapsed seconds.
ORC_API double orc_amo_fetch_add_threaded(int64_t *counters, const uint32_t *ids, const int64_t *values,
                                          int64_t *fetched, size_t n_ops, int nthreads) {
  static_assert(sizeof(std::atomic<int64_t>) == sizeof(int64_t), "atomic layout");
  auto *a = reinterpret_cast<std::atomic<int64_t> *>(counters);
  const auto t0 = std::chrono::steady_clock::now();
  parallel_for(n_ops, nthreads, [&](size_t lo, size_t hi, int) {
    for (size_t i = lo; i < hi; ++i) {
      const int64_t old = a[ids[i]].fetch_add(values ? values[i] : 1);
      if (fetched) fetched[i] = old;
    }
  });
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

// ============================================================================
// S1 / W1  Signals and waits.
// ============================================================================
// putmem_signal: payload, then SET (store) or ADD on the 64-bit word; unknown
// op leaves the word; zero length does nothing at all
// (src/ipc/context_ipc_device.cpp:221-259, src/context_device.cpp:251-262).
ORC_API void orc_put_signal(void *dst, const void *src, size_t n, uint64_t *sig, uint64_t signal,
                            int sig_op) {
  if (n == 0) return;
  memcpy(dst, src, n);
  if (sig_op == 0) *sig = signal;
  else if (sig_op == 1) *sig += signal;
}

namespace {
template <typename T>
int cmp_typed(int cmp, const void *x, const void *v) {
  T a, b;
  memcpy(&a, x, sizeof(T));
  memcpy(&b, v, sizeof(T));
  switch (cmp) {  // src/context_tmpl_device.hpp:342-375
    case 0: return a == b;
    case 1: return a != b;
    case 2: return a > b;
    case 3: return a >= b;
    case 4: return a < b;
    case 5: return a <= b;
    default: return 0;
  }
}
size_t dtype_size(int dtype) {
  switch (dtype) {
    case DT_CHAR: case DT_SCHAR: case DT_UCHAR: return 1;
    case DT_SHORT: case DT_BF16: case DT_USHORT: return 2;
    case DT_INT: case DT_FLOAT: case DT_UINT: return 4;
    default: return 8;
  }
}
}  // namespace

// Context::test on a value.
ORC_API int orc_test(int dtype, int cmp, const void *x, const void *val) {
  switch (dtype) {
    case DT_SHORT: return cmp_typed<int16_t>(cmp, x, val);
    case DT_INT: return cmp_typed<int32_t>(cmp, x, val);
    case DT_LONG: case DT_LONGLONG: return cmp_typed<int64_t>(cmp, x, val);
    case DT_FLOAT: return cmp_typed<float>(cmp, x, val);
    case DT_DOUBLE: return cmp_typed<double>(cmp, x, val);
    case DT_UINT: return cmp_typed<uint32_t>(cmp, x, val);
    case DT_ULONG: case DT_ULONGLONG: return cmp_typed<uint64_t>(cmp, x, val);
    // The wait types only the host side has (include/rocshmem/rocshmem_P2P_SYNC.hpp:
    // char, schar, uchar, ushort); plain char is signed on this platform.
    case DT_CHAR: case DT_SCHAR: return cmp_typed<int8_t>(cmp, x, val);
    case DT_UCHAR: return cmp_typed<uint8_t>(cmp, x, val);
    case DT_USHORT: return cmp_typed<uint16_t>(cmp, x, val);
    default: return 0;
  }
}
// wait_until_any / _some on a frozen array (src/context_tmpl_device.hpp:
// 220-310): what the call returns if the values never change.  Returns
// SIZE_MAX-1 when the call would block forever.
ORC_API size_t orc_wait_until_any(int dtype, const void *ivars, size_t nelems, const int *status,
                                  int cmp, const void *val) {
  if (!nelems) return SIZE_MAX;
  size_t pos = 0;
  while (pos < nelems && status && status[pos]) ++pos;
  if (pos == nelems) return SIZE_MAX;
  const size_t es = dtype_size(dtype);
  for (size_t i = pos; i < nelems; ++i) {
    if (status && status[i]) continue;
    if (orc_test(dtype, cmp, static_cast<const char *>(ivars) + i * es, val)) return i;
  }
  return SIZE_MAX - 1;
}
ORC_API size_t orc_wait_until_some(int dtype, const void *ivars, size_t nelems, size_t *indices,
                                   const int *status, int cmp, const void *val) {
  if (!nelems) return 0;
  size_t pos = 0;
  while (pos < nelems && status && status[pos]) ++pos;
  if (pos == nelems) return 0;
  const size_t es = dtype_size(dtype);
  size_t done = 0;
  for (size_t i = pos; i < nelems; ++i) {
    if (status && status[i]) continue;
    if (orc_test(dtype, cmp, static_cast<const char *>(ivars) + i * es, val)) indices[done++] = i;
  }
  return done ? done : SIZE_MAX - 1;
}

// Two-thread ping-pong: payload memcpy + release store / acquire spin on a
// 64-bit word, the CPU baseline of the put_signal / wait_until exchange.
// Returns seconds for `iters` round trips.
ORC_API double orc_pingpong_threaded(size_t nbytes, int iters) {
  std::vector<char> buf_a(nbytes, 1), buf_b(nbytes, 2);
  alignas(64) std::atomic<uint64_t> sig_a{0};
  alignas(64) std::atomic<uint64_t> sig_b{0};
  const auto t0 = std::chrono::steady_clock::now();
  std::thread b([&] {
    for (int r = 1; r <= iters; ++r) {
      while (sig_b.load(std::memory_order_acquire) != static_cast<uint64_t>(r)) {}
      memcpy(buf_a.data(), buf_b.data(), nbytes);
      sig_a.store(r, std::memory_order_release);
    }
  });
  for (int r = 1; r <= iters; ++r) {
    memcpy(buf_b.data(), buf_a.data(), nbytes);
    sig_b.store(r, std::memory_order_release);
    while (sig_a.load(std::memory_order_acquire) != static_cast<uint64_t>(r)) {}
  }
  b.join();
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

ORC_API int orc_hardware_threads() { return static_cast<int>(std::thread::hardware_concurrency()); }

// Element-wise combine behind the all-reduce ("to_all" / wg_reduce) path.
//
// The reference combines with OpWrap<Op>::Calc, dst[i] = dst[i] op src[i]
// (src/rocshmem_calc.hpp:43-97), applied chunk by chunk as data travels round
// a ring through a 1024-element work buffer
// (src/ipc/context_ipc_tmpl_device.hpp:282-359).  Here every output element is
// produced in one pass: the P source values are loaded (16 bytes per lane per
// source, all P loads in flight), folded in registers in ASCENDING team-PE
// order  (((x0 op x1) op x2) ...), and the result is stored to all P
// destinations.  For integers, bitwise ops and min/max this equals the
// reference for any order; for floating-point sums it differs from the
// reference's cyclic order by rounding only.
//
// bf16 (no counterpart in the reference): operands are widened to fp32
// exactly, folded in fp32, and rounded to nearest-even once at the end.
#ifndef ROCSHMEM_AMD_DETAIL_REDUCE_ENGINE_HPP_
#define ROCSHMEM_AMD_DETAIL_REDUCE_ENGINE_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <type_traits>

#include "../rocshmem_common.hpp"
#include "copy_engine.hpp"

namespace rocshmem {

// Storage type of a bfloat16 element (1 sign, 8 exponent, 7 mantissa bits).
struct rocshmem_bf16 {
  uint16_t bits;
};

namespace detail {

__host__ __device__ inline float bf16_to_f32(uint16_t b) {
  union { uint32_t u; float f; } c;
  c.u = static_cast<uint32_t>(b) << 16;
  return c.f;
}

// Round-to-nearest-even; NaNs keep their sign and become quiet.
__host__ __device__ inline uint16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } c;
  c.f = f;
  uint32_t u = c.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// acc op x for one element.  Integer sums and products wrap (computed in the
// unsigned type), as the reference's += / *= do on the device.
template <typename T, ROCSHMEM_OP Op>
__host__ __device__ inline T combine(T acc, T x) {
  if constexpr (Op == ROCSHMEM_SUM) {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      return static_cast<T>(static_cast<U>(static_cast<U>(acc) + static_cast<U>(x)));
    } else {
      return acc + x;
    }
  } else if constexpr (Op == ROCSHMEM_PROD) {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      return static_cast<T>(static_cast<U>(static_cast<U>(acc) * static_cast<U>(x)));
    } else {
      return acc * x;
    }
  } else if constexpr (Op == ROCSHMEM_MAX) {
    if constexpr (std::is_same<T, float>::value) return fmaxf(acc, x);
    else if constexpr (std::is_same<T, double>::value) return fmax(acc, x);
    else return acc < x ? x : acc;
  } else if constexpr (Op == ROCSHMEM_MIN) {
    if constexpr (std::is_same<T, float>::value) return fminf(acc, x);
    else if constexpr (std::is_same<T, double>::value) return fmin(acc, x);
    else return x < acc ? x : acc;
  } else if constexpr (Op == ROCSHMEM_AND) {
    return static_cast<T>(acc & x);
  } else if constexpr (Op == ROCSHMEM_OR) {
    return static_cast<T>(acc | x);
  } else {
    static_assert(Op == ROCSHMEM_XOR, "unsupported reduction op");
    return static_cast<T>(acc ^ x);
  }
}

#if defined(__HIPCC__)

typedef uint32_t r_u32x4 __attribute__((ext_vector_type(4)));
typedef r_u32x4 r_u32x4_any __attribute__((aligned(1)));

// 16 bytes of elements viewed as T[16/sizeof(T)].
template <typename T>
union Pack {
  r_u32x4 raw;
  T e[16 / sizeof(T)];
};

// Element type tag for bf16 storage with fp32 accumulation.
struct Bf16Tag {};

template <typename T>
struct ElemTraits {
  using storage = T;
  using accum = T;
  static constexpr int kPerVec = 16 / sizeof(T);
  __device__ static accum widen(storage s) { return s; }
  __device__ static storage narrow(accum a) { return a; }
};
template <>
struct ElemTraits<Bf16Tag> {
  using storage = uint16_t;
  using accum = float;
  static constexpr int kPerVec = 8;
  __device__ static float widen(uint16_t s) { return bf16_to_f32(s); }
  __device__ static uint16_t narrow(float a) { return f32_to_bf16(a); }
};

// One element of 2, 4 or 8 bytes as a write-through buffer store.
template <typename S>
__device__ __forceinline__ void store_elem(__amdgpu_buffer_rsrc_t w, uint32_t off, S v) {
  if constexpr (sizeof(S) == 2) {
    uint16_t b;
    __builtin_memcpy(&b, &v, 2);
    __builtin_amdgcn_raw_buffer_store_b16(b, w, static_cast<int>(off), 0, kAuxWriteThrough);
  } else if constexpr (sizeof(S) == 4) {
    uint32_t b;
    __builtin_memcpy(&b, &v, 4);
    __builtin_amdgcn_raw_buffer_store_b32(b, w, static_cast<int>(off), 0, kAuxWriteThrough);
  } else {
    typedef uint32_t b64_t __attribute__((ext_vector_type(2)));
    b64_t b;
    __builtin_memcpy(&b, &v, 8);
    __builtin_amdgcn_raw_buffer_store_b64(b, w, static_cast<int>(off), 0, kAuxWriteThrough);
  }
}

// Vectors (16 bytes each) per block when several groups share one range: the
// unit in which team members take turns through the arrays.  A constant, so
// that the split does not depend on how many lanes each group brings (team
// members may run work-groups of different sizes); 1024 keeps every lane of
// the largest work-group busy.
constexpr size_t kShareVectors = 1024;

// Fold elements [lo, hi) across P team members and store the result on all P.
//   src0 / dst0 : the buffers on team member 0
//   hop         : bytes from one team member's buffer to the next member's
//   kP          : P when known at compile time (loads fully unrolled), 0 when
//                 only `np` is known
// `lane` of `nlanes` dense cooperating lanes (a work-group or a whole grid);
// (hi - lo) * sizeof(element) must not exceed kWindowBytes.  Results leave as
// write-through buffer stores, one resource per destination.
//
// With kShared == SHARE_BLOCKS the range is shared by `nparts` such groups (the
// members of a team, one work-group each, of any sizes): group `part` takes the blocks
// part, part + nparts, ... of kShareVectors vectors each and strides through
// a block with its own lanes, so the groups work side by side through the
// arrays.  Group 0 also takes the unaligned head, the last group the tail.
// (Measured on MI355X, P = 8 x 64 Mi fp32, 256-1024 work-groups that loop:
// 6.3-6.4 TB/s for this split and for contiguous chunks alike, against 6.45
// for one-vector work-groups; issuing a lane's next loads ahead of its stores
// gained nothing and cost 20-40 registers.)
//
// With kShared == SHARE_TICKETS the groups do not split the vectors by rule:
// every wavefront draws the next block of kTicketVectors vectors from a
// counter that all groups share (`tickets`, zero when the first draw is made),
// so the blocks are taken in index order whatever the pace of each group, and
// at any moment the groups together work on one narrow stretch of every array.
// (Work-groups that loop over a fixed share drift apart; on MI355X the P = 8
// fp32 fold then runs at 6.2 TB/s against 6.55 for work-groups that are started
// in index order.)  Each wavefront draws its next block before it loads the
// current one, so the draw travels with the block's loads.
enum ShareKind : int { SHARE_NONE = 0, SHARE_BLOCKS = 1, SHARE_TICKETS = 2 };
constexpr size_t kTicketVectors = 256;

template <typename E, ROCSHMEM_OP Op, int kP, bool kNonTemporal, int kShared = SHARE_NONE>
__device__ __forceinline__ void fold_window(
    typename ElemTraits<E>::storage *dst0,
    const typename ElemTraits<E>::storage *src0, int64_t hop, int np,
    size_t lo, size_t hi, size_t lane, size_t nlanes, size_t part = 0, size_t nparts = 1,
    unsigned long long *tickets = nullptr) {
  using Tr = ElemTraits<E>;
  using S = typename Tr::storage;
  using A = typename Tr::accum;
  constexpr int V = Tr::kPerVec;
  const int P = kP ? kP : np;
  const size_t win_bytes = (hi - lo) * sizeof(S);

  auto src_at = [&](int p, size_t i) -> const S * {
    return reinterpret_cast<const S *>(reinterpret_cast<const char *>(src0 + i) + p * hop);
  };
  auto dst_window = [&](int p) {
    return window_of(reinterpret_cast<char *>(dst0 + lo) + p * hop, win_bytes);
  };
  auto scalar_one = [&](size_t i) {
    A acc = Tr::widen(*src_at(0, i));
    for (int p = 1; p < P; ++p) acc = combine<A, Op>(acc, Tr::widen(*src_at(p, i)));
    const S out = Tr::narrow(acc);
    for (int p = 0; p < P; ++p)
      store_elem<S>(dst_window(p), static_cast<uint32_t>((i - lo) * sizeof(S)), out);
  };

  // Elements before the first 16-byte boundary of the destination.
  const uintptr_t mis = reinterpret_cast<uintptr_t>(dst0 + lo) & 15u;
  size_t head = mis ? (16u - mis) / sizeof(S) : 0;
  if (head > hi - lo) head = hi - lo;
  if (part == 0)
    for (size_t k = lane; k < head; k += nlanes) scalar_one(lo + k);
  const size_t vlo = lo + head;
  const size_t nvec = (hi - vlo) / V;
  // Vector v of the window sits 16 * v bytes after element vlo in every source
  // and destination.  Each source is a global-memory base in scalar registers
  // plus that one 32-bit offset, each destination a buffer resource built once.
  const char *const first_src = reinterpret_cast<const char *>(src0 + vlo);
  char *const first_dst = reinterpret_cast<char *>(dst0 + vlo);
  const size_t vec_bytes = nvec << 4;
  auto load_vec = [&](GlobalBytes base, uint32_t off) -> r_u32x4 {
    return load16<kNonTemporal>(base, off);
  };
  // Calls body(v) for every vector index this lane owns.
  auto for_my_vectors = [&](auto &&body) {
    if constexpr (kShared == SHARE_TICKETS) {
      unsigned count;
      const unsigned rank = active_lane_rank(&count);
      // The lowest active lane draws; the others learn the block from it.
      auto draw = [&]() -> unsigned long long {
        unsigned long long t = 0;
        if (rank == 0)
          t = __hip_atomic_fetch_add(tickets, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return t;
      };
      auto drawn = [&](unsigned long long t) -> size_t {
        const uint32_t tl = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(t));
        const uint32_t th = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(t >> 32));
        return ((static_cast<size_t>(th) << 32) | tl) * kTicketVectors;
      };
      size_t b = drawn(draw());
      while (b < nvec) {
        const unsigned long long next = draw();
        const size_t bend = b + kTicketVectors < nvec ? b + kTicketVectors : nvec;
        for (size_t v = b + rank; v < bend; v += count) body(v);
        b = drawn(next);
      }
    } else if constexpr (kShared == SHARE_BLOCKS) {
      for (size_t b = part * kShareVectors; b < nvec; b += nparts * kShareVectors) {
        const size_t bend = b + kShareVectors < nvec ? b + kShareVectors : nvec;
        for (size_t v = b + lane; v < bend; v += nlanes) body(v);
      }
    } else {
      for (size_t v = lane; v < nvec; v += nlanes) body(v);
    }
  };

  if constexpr (kP != 0) {
    GlobalBytes from[kP];
    __amdgpu_buffer_rsrc_t to[kP];
#pragma unroll
    for (int p = 0; p < kP; ++p) {
      from[p] = wave_uniform_global(first_src + p * hop);
      to[p] = window_of(first_dst + p * hop, vec_bytes);
    }
    for_my_vectors([&](size_t v) {
      const uint32_t off = static_cast<uint32_t>(v << 4);
      Pack<S> in[kP], out;
#pragma unroll
      for (int p = 0; p < kP; ++p) in[p].raw = load_vec(from[p], off);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        A acc = Tr::widen(in[0].e[e]);
#pragma unroll
        for (int p = 1; p < kP; ++p) acc = combine<A, Op>(acc, Tr::widen(in[p].e[e]));
        out.e[e] = Tr::narrow(acc);
      }
#pragma unroll
      for (int p = 0; p < kP; ++p) store16<kNonTemporal>(to[p], off, out.raw);
    });
  } else {
    for_my_vectors([&](size_t v) {
      const uint32_t off = static_cast<uint32_t>(v << 4);
      A acc[V];
      Pack<S> in, out;
      in.raw = load_vec(wave_uniform_global(first_src), off);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = Tr::widen(in.e[e]);
      for (int p = 1; p < P; ++p) {
        in.raw = load_vec(wave_uniform_global(first_src + p * hop), off);
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = combine<A, Op>(acc[e], Tr::widen(in.e[e]));
      }
#pragma unroll
      for (int e = 0; e < V; ++e) out.e[e] = Tr::narrow(acc[e]);
      for (int p = 0; p < P; ++p)
        store16<kNonTemporal>(window_of(first_dst + p * hop, vec_bytes), off, out.raw);
    });
  }

  const size_t tlo = vlo + nvec * V;
  if (part == nparts - 1)
    for (size_t k = tlo + lane; k < hi; k += nlanes) scalar_one(k);
}

// Any range: windows of at most kWindowBytes.  A range whose blocks are drawn
// from a counter must fit one window (the counter counts from zero once).
template <typename E, ROCSHMEM_OP Op, int kP, bool kNonTemporal, int kShared = SHARE_NONE>
__device__ __forceinline__ void fold_span(
    typename ElemTraits<E>::storage *dst0,
    const typename ElemTraits<E>::storage *src0, int64_t hop, int np,
    size_t lo, size_t hi, size_t lane, size_t nlanes, size_t part = 0, size_t nparts = 1,
    unsigned long long *tickets = nullptr) {
  constexpr size_t kWin = kWindowBytes / sizeof(typename ElemTraits<E>::storage);
  if constexpr (kShared != SHARE_TICKETS) {
    while (hi - lo > kWin) {
      fold_window<E, Op, kP, kNonTemporal, kShared>(dst0, src0, hop, np, lo, lo + kWin, lane, nlanes,
                                                    part, nparts);
      lo += kWin;
    }
  }
  fold_window<E, Op, kP, kNonTemporal, kShared>(dst0, src0, hop, np, lo, hi, lane, nlanes, part,
                                                nparts, tickets);
}

// Dispatch on the team size so the common sizes get fully unrolled loads.
template <typename E, ROCSHMEM_OP Op, bool kNonTemporal, int kShared = SHARE_NONE>
__device__ __forceinline__ void fold_span_any(
    typename ElemTraits<E>::storage *dst0,
    const typename ElemTraits<E>::storage *src0, int64_t hop, int np,
    size_t lo, size_t hi, size_t lane, size_t nlanes, size_t part = 0, size_t nparts = 1,
    unsigned long long *tickets = nullptr) {
#define ROCSHMEM_AMD_FOLD_CASE(KP)                                                               \
  fold_span<E, Op, KP, kNonTemporal, kShared>(dst0, src0, hop, np, lo, hi, lane, nlanes, part, \
                                              nparts, tickets)
  switch (np) {
    case 2: ROCSHMEM_AMD_FOLD_CASE(2); break;
    case 4: ROCSHMEM_AMD_FOLD_CASE(4); break;
    case 8: ROCSHMEM_AMD_FOLD_CASE(8); break;
    default: ROCSHMEM_AMD_FOLD_CASE(0); break;
  }
#undef ROCSHMEM_AMD_FOLD_CASE
}

#endif  // __HIPCC__

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_REDUCE_ENGINE_HPP_

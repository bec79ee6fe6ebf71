// Power-of-two binned allocator for one slice of the symmetric heap.
//
// Behavioural restatement of the reference's SingleHeap / Pow2Bins / Binner
// (src/memory/single_heap.cpp:29-64, pow2_bins.hpp:90-152,264-287,
// binner.hpp:109-231): bins for every power of two from 128 bytes up to the
// largest power of two that fits the heap; the heap is carved largest-first
// into initial blocks after skipping an unaligned head; a request takes a
// block from the smallest bin that is >= the request, splitting a block of
// the next non-empty larger bin in halves on demand (lower half handed out
// first); freed blocks go back to their own bin (last freed, first reused)
// and are never merged; size 0 and exhaustion give "no block".
//
// Works on offsets from the slice base so one instance serves every PE: the
// same call sequence yields the same offset on all of them.
#ifndef ROCSHMEM_AMD_POW2_ALLOCATOR_HPP_
#define ROCSHMEM_AMD_POW2_ALLOCATOR_HPP_

#include <cstddef>
#include <cstdint>
#include <map>
#include <vector>

namespace rocshmem {
namespace runtime {

class Pow2Allocator {
 public:
  static constexpr uint64_t kMinBlock = 128;
  static constexpr uint64_t kNoBlock = ~uint64_t{0};

  Pow2Allocator() = default;
  // base_address is only used for its alignment (the reference skips bytes
  // until the first 128-byte boundary).
  Pow2Allocator(uint64_t base_address, uint64_t heap_bytes) { reset(base_address, heap_bytes); }

  void reset(uint64_t base_address, uint64_t heap_bytes) {
    bins_.clear();
    handed_out_.clear();
    heap_bytes_ = heap_bytes;
    if (heap_bytes < kMinBlock) return;
    // One bin per power of two in [128, 2^floor(log2(heap_bytes))].
    for (uint64_t s = kMinBlock; s <= heap_bytes && s != 0; s <<= 1) bins_[s];
    uint64_t off = 0, left = heap_bytes;
    const uint64_t mis = base_address % kMinBlock;
    if (mis) {
      off = kMinBlock - mis;
      left -= off;
    }
    // Largest-first carving: each step takes the biggest bin size that fits.
    for (;;) {
      auto it = bins_.upper_bound(left);
      if (it == bins_.begin()) break;
      --it;
      it->second.push_back(off);
      off += it->first;
      left -= it->first;
    }
  }

  // Offset of the block, or kNoBlock.
  uint64_t alloc(uint64_t request) {
    if (!request) return kNoBlock;
    auto it = bins_.lower_bound(request);
    if (it == bins_.end()) return kNoBlock;
    if (it->second.empty()) refill(it);
    if (it->second.empty()) return kNoBlock;
    const uint64_t off = it->second.back();
    it->second.pop_back();
    handed_out_[off] = it->first;
    return off;
  }

  // Returns false when `off` was not handed out.
  bool free(uint64_t off) {
    auto it = handed_out_.find(off);
    if (it == handed_out_.end()) return false;
    bins_[it->second].push_back(off);
    handed_out_.erase(it);
    return true;
  }

  uint64_t used() const {
    uint64_t s = 0;
    for (const auto &kv : handed_out_) s += kv.second;
    return s;
  }
  uint64_t size() const { return heap_bytes_; }
  uint64_t avail() const { return heap_bytes_ - used(); }
  size_t num_bins() const { return bins_.size(); }
  // Blocks currently sitting in the bin of exactly `block_size` bytes.
  size_t bin_population(uint64_t block_size) const {
    auto it = bins_.find(block_size);
    return it == bins_.end() ? 0 : it->second.size();
  }
  uint64_t block_size_of(uint64_t off) const {
    auto it = handed_out_.find(off);
    return it == handed_out_.end() ? 0 : it->second;
  }

 private:
  using Bins = std::map<uint64_t, std::vector<uint64_t>>;

  // Make `it`'s bin non-empty by halving one block of the next larger bin,
  // refilling that one first if it is empty too.
  void refill(Bins::iterator it) {
    auto next = std::next(it);
    if (next == bins_.end()) return;
    if (next->second.empty()) refill(next);
    if (next->second.empty()) return;
    const uint64_t off = next->second.back();
    next->second.pop_back();
    it->second.push_back(off + it->first);  // upper half, handed out second
    it->second.push_back(off);              // lower half, handed out first
  }

  Bins bins_;
  std::map<uint64_t, uint64_t> handed_out_;  // offset -> block size
  uint64_t heap_bytes_ = 0;
};

}  // namespace runtime
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_POW2_ALLOCATOR_HPP_

// Test infrastructure: C entry points around the REFERENCE's own allocator
// classes, included from the reference tree where it lies (nothing is copied
// into this repository).  Built into oracle/_ref/libref_allocator.so by
// oracle/Makefile and used only by the tests that pin the oracle's allocator.
//
// Pow2Bins is a class template over the heap-memory type; the one used here is
// a plain address range owned by this harness, so no GPU is needed.
#include <cstddef>
#include <cstdint>

#include "memory/address_record.hpp"
#include "memory/pow2_bins.hpp"

namespace {
struct RangeHeap {
  char *ptr;
  size_t size;
  char *get_ptr() { return ptr; }
  size_t get_size() { return size; }
};
using RefStrategy = rocshmem::Pow2Bins<rocshmem::AddressRecord, RangeHeap>;
struct RefHeap {
  RangeHeap range;
  RefStrategy *strat;
};
}  // namespace

extern "C" {
__attribute__((visibility("default"))) void *ref_heap_create(uint64_t base_addr, uint64_t size) {
  RefHeap *h = new RefHeap;
  h->range = RangeHeap{reinterpret_cast<char *>(base_addr), static_cast<size_t>(size)};
  h->strat = new RefStrategy(&h->range);
  return h;
}
__attribute__((visibility("default"))) void ref_heap_destroy(void *hp) {
  RefHeap *h = static_cast<RefHeap *>(hp);
  delete h->strat;
  delete h;
}
__attribute__((visibility("default"))) uint64_t ref_heap_alloc(void *hp, uint64_t request) {
  char *p = nullptr;
  static_cast<RefHeap *>(hp)->strat->alloc(&p, static_cast<size_t>(request));
  return reinterpret_cast<uint64_t>(p);
}
__attribute__((visibility("default"))) void ref_heap_free(void *hp, uint64_t addr) {
  if (!addr) return;  // SingleHeap::free ignores nullptr (src/memory/single_heap.cpp:45-50)
  static_cast<RefHeap *>(hp)->strat->free(reinterpret_cast<char *>(addr));
}
__attribute__((visibility("default"))) uint64_t ref_heap_used(void *hp) {
  return static_cast<RefHeap *>(hp)->strat->amount_proffered();
}
__attribute__((visibility("default"))) uint64_t ref_heap_num_bins(void *hp) {
  return static_cast<RefHeap *>(hp)->strat->get_bins()->size();
}
__attribute__((visibility("default"))) uint64_t ref_heap_bin_population(void *hp, uint64_t block) {
  auto *bins = static_cast<RefHeap *>(hp)->strat->get_bins();
  auto it = bins->find(static_cast<size_t>(block));
  return it == bins->end() ? 0 : it->second.size();
}
}

// C entry points around the reference's own symmetric-heap allocator
// (Pow2Bins<AddressRecord, HM_T>, library/src/memory/pow2_bins.hpp with
// binner.hpp, bin.hpp, address_record.hpp), compiled from the reference tree
// where it lies; nothing of it is copied here.  Test infrastructure only: the
// CPU oracle's allocator (oracle/alloc.c) and the library's are checked
// against it.  HM_T is the template's own extension point; this one describes
// an address range that is never dereferenced (the allocator only does
// arithmetic on addresses).
#include <cstddef>
#include <cstdint>

#include "src/memory/address_record.hpp"
#include "src/memory/pow2_bins.hpp"

namespace {

class AddressRange {
 public:
  AddressRange(char *base, size_t bytes) : base_(base), bytes_(bytes) {}
  char *get_ptr() { return base_; }
  size_t get_size() { return bytes_; }

 private:
  char *base_;
  size_t bytes_;
};

struct RefAllocator {
  AddressRange range;
  rocshmem::Pow2Bins<rocshmem::AddressRecord, AddressRange> bins;
  RefAllocator(char *base, size_t bytes) : range(base, bytes), bins(&range) {}
};

// Any non-null, suitably aligned address will do as the start of the range.
char *const kBase = reinterpret_cast<char *>(uintptr_t{1} << 40);

}  // namespace

extern "C" {

void *ref_alloc_create(size_t heap_bytes) { return new RefAllocator(kBase, heap_bytes); }

void ref_alloc_destroy(void *a) { delete static_cast<RefAllocator *>(a); }

// Offset of the block inside the heap, or (size_t)-1 when the request cannot be met.
size_t ref_alloc_alloc(void *a, size_t request) {
  char *p = nullptr;
  static_cast<RefAllocator *>(a)->bins.alloc(&p, request);
  return p ? static_cast<size_t>(p - kBase) : static_cast<size_t>(-1);
}

void ref_alloc_free(void *a, size_t offset) {
  static_cast<RefAllocator *>(a)->bins.free(kBase + offset);
}

size_t ref_alloc_in_use(void *a) { return static_cast<RefAllocator *>(a)->bins.amount_proffered(); }

}  // extern "C"

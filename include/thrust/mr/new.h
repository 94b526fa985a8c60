// thrust::mr::new_delete_resource: host memory from operator new / delete
// (thrust/mr/new.h).  The bookkeeper of the disjoint pools by default.
#pragma once
#include <cstddef>
#include <cstdlib>
#include <new>

#include <thrust/mr/memory_resource.h>

namespace thrust {
namespace mr {

class new_delete_resource final : public memory_resource<void*> {
 protected:
  // alignments beyond that of operator new come from posix_memalign (and go back through free)
  void* do_allocate(std::size_t bytes, std::size_t alignment) override {
    if (alignment <= alignof(std::max_align_t)) return ::operator new(bytes ? bytes : 1);
    void* p = nullptr;
    if (posix_memalign(&p, alignment, bytes ? bytes : 1) != 0) throw std::bad_alloc();
    return p;
  }
  void do_deallocate(void* p, std::size_t, std::size_t alignment) override {
    if (alignment <= alignof(std::max_align_t)) ::operator delete(p);
    else std::free(p);
  }
  bool do_is_equal(const memory_resource<void*>& other) const noexcept override {
    return dynamic_cast<const new_delete_resource*>(&other) != nullptr;
  }
};

}  // namespace mr
}  // namespace thrust

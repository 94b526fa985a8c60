// thrust::mr::unsynchronized_pool_resource: a caching layer over another resource.
//
// Requests are rounded up to size classes (powers of two from smallest_block_size up to
// largest_block_size); a block given back is kept and handed out again for the next request
// of its class, so steady-state allocation touches the upstream resource (hipMalloc is a
// device-wide synchronisation point) only for new high-water marks.  Requests above
// largest_block_size go straight to the upstream resource.  release() returns every cached
// block; the destructor does the same.  Not thread-safe, like its namesake
// (thrust/mr/pool.h:70-500 and pool_options.h of the reference, whose pool keeps chunked
// free lists; this one keeps whole blocks, which is what device temporary storage and
// vectors ask for).  Memory handed out must come back before the resource is destroyed.
#pragma once
#include <cstddef>
#include <map>
#include <new>
#include <vector>

#include <thrust/mr/memory_resource.h>

namespace thrust {
namespace mr {

struct pool_options {
  std::size_t smallest_block_size;  // requests are rounded up to at least this, a power of two
  std::size_t largest_block_size;   // larger requests are not cached
  pool_options() : smallest_block_size(256), largest_block_size((std::size_t)1 << 30) {}
};

template <typename Upstream>
class unsynchronized_pool_resource : public memory_resource<typename Upstream::pointer> {
 public:
  typedef typename Upstream::pointer pointer;
  explicit unsynchronized_pool_resource(Upstream* upstream, pool_options options = pool_options())
      : upstream_(upstream), options_(options), upstream_calls_(0), cached_bytes_(0) {}
  unsynchronized_pool_resource(const unsynchronized_pool_resource&) = delete;
  unsynchronized_pool_resource& operator=(const unsynchronized_pool_resource&) = delete;
  ~unsynchronized_pool_resource() { release(); }

  // Returns every cached block to the upstream resource.
  void release() {
    for (auto& kv : free_)
      for (auto& p : kv.second) upstream_->deallocate(p, kv.first, block_alignment);
    free_.clear();
    cached_bytes_ = 0;
  }
  Upstream* upstream_resource() const { return upstream_; }
  std::size_t upstream_allocations() const { return upstream_calls_; }  // how often the upstream resource was asked
  std::size_t cached_bytes() const { return cached_bytes_; }

 protected:
  static const std::size_t block_alignment = 256;
  pointer do_allocate(std::size_t bytes, std::size_t alignment) override {
    if (alignment > block_alignment) throw std::bad_alloc();
    const std::size_t cls = size_class(bytes);
    if (cls == 0) {  // too large to cache
      ++upstream_calls_;
      return upstream_->allocate(bytes, block_alignment);
    }
    auto it = free_.find(cls);
    if (it != free_.end() && !it->second.empty()) {
      pointer p = it->second.back();
      it->second.pop_back();
      cached_bytes_ -= cls;
      return p;
    }
    ++upstream_calls_;
    return upstream_->allocate(cls, block_alignment);
  }
  void do_deallocate(pointer p, std::size_t bytes, std::size_t) override {
    const std::size_t cls = size_class(bytes);
    if (cls == 0) {
      upstream_->deallocate(p, bytes, block_alignment);
      return;
    }
    free_[cls].push_back(p);
    cached_bytes_ += cls;
  }

 private:
  std::size_t size_class(std::size_t bytes) const {
    if (bytes > options_.largest_block_size) return 0;
    std::size_t c = options_.smallest_block_size ? options_.smallest_block_size : 1;
    while (c < bytes) c <<= 1;
    return c;
  }
  Upstream* upstream_;
  pool_options options_;
  std::map<std::size_t, std::vector<pointer> > free_;
  std::size_t upstream_calls_, cached_bytes_;
};

}  // namespace mr
}  // namespace thrust

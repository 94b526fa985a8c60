// thrust::mr::disjoint_synchronized_pool_resource: the disjoint pool behind a mutex
// (thrust/mr/disjoint_sync_pool.h:44-118).
#pragma once
#include <mutex>

#include <thrust/mr/disjoint_pool.h>

namespace thrust {
namespace mr {

template <typename Upstream, typename Bookkeeper = new_delete_resource>
class disjoint_synchronized_pool_resource : public memory_resource<typename Upstream::pointer> {
 public:
  typedef typename Upstream::pointer pointer;
  typedef disjoint_unsynchronized_pool_resource<Upstream, Bookkeeper> unsync_pool;
  static disjoint_pool_options get_default_options() { return disjoint_pool_options(); }
  disjoint_synchronized_pool_resource(Upstream* upstream, Bookkeeper* bookkeeper,
                                      disjoint_pool_options options = get_default_options())
      : pool_(upstream, bookkeeper, options) {}
  explicit disjoint_synchronized_pool_resource(disjoint_pool_options options = get_default_options())
      : pool_(get_global_resource<Upstream>(), get_global_resource<Bookkeeper>(), options) {}
  void release() {
    std::lock_guard<std::mutex> lock(mutex_);
    pool_.release();
  }
  std::size_t upstream_allocations() const {
    std::lock_guard<std::mutex> lock(mutex_);
    return pool_.upstream_allocations();
  }

 protected:
  pointer do_allocate(std::size_t bytes, std::size_t alignment) override {
    std::lock_guard<std::mutex> lock(mutex_);
    return pool_.allocate(bytes, alignment);
  }
  void do_deallocate(pointer p, std::size_t bytes, std::size_t alignment) override {
    std::lock_guard<std::mutex> lock(mutex_);
    pool_.deallocate(p, bytes, alignment);
  }

 private:
  mutable std::mutex mutex_;
  unsync_pool pool_;
};

}  // namespace mr
}  // namespace thrust

// thrust::mr::synchronized_pool_resource: unsynchronized_pool_resource behind a mutex, for a
// pool shared by several host threads (thrust/mr/sync_pool.h:43-110).
#pragma once
#include <mutex>

#include <thrust/mr/pool.h>

namespace thrust {
namespace mr {

template <typename Upstream>
class synchronized_pool_resource : public memory_resource<typename Upstream::pointer> {
 public:
  typedef typename Upstream::pointer pointer;
  typedef unsynchronized_pool_resource<Upstream> unsync_pool;
  static pool_options get_default_options() { return pool_options(); }
  explicit synchronized_pool_resource(Upstream* upstream, pool_options options = get_default_options())
      : pool_(upstream, options) {}
  explicit synchronized_pool_resource(pool_options options = get_default_options())
      : pool_(get_global_resource<Upstream>(), options) {}
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

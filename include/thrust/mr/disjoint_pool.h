// thrust::mr::disjoint_unsynchronized_pool_resource: a pool whose bookkeeping never touches
// the memory it hands out (thrust/mr/disjoint_pool.h:40-490 of the reference).
//
// A pool normally threads its free lists through the free blocks themselves; that needs the
// pooled memory to be addressable by the host.  Device memory is not, so this pool keeps all
// of its bookkeeping in memory from a second resource, the bookkeeper (host memory).
//   * requests up to largest_block_size are rounded to a power-of-two block size; blocks are
//     carved from chunks obtained upstream, min_blocks_per_chunk at first and twice as many
//     for every further chunk of that size, up to max_blocks_per_chunk / max_bytes_per_chunk;
//   * larger ("oversized") requests go upstream one by one and, with cache_oversized, are kept
//     when they come back and reused for requests of at most cached_size_cutoff_factor times
//     less;
//   * release() gives every chunk and cached oversized block back; so does the destructor.
// Not thread-safe; thrust/mr/disjoint_sync_pool.h wraps it in a mutex.
#pragma once
#include <cstddef>
#include <cstring>
#include <new>

#include <thrust/mr/memory_resource.h>
#include <thrust/device_ptr.h>
#include <thrust/mr/new.h>
#include <thrust/mr/pool.h>

namespace thrust {
namespace mr {

namespace detail {
// A grow-only array of trivially copyable records in memory from a bookkeeper resource.
template <typename T, typename Bookkeeper>
class book_vector {
 public:
  explicit book_vector(Bookkeeper* b) : book_(b), data_(nullptr), size_(0), cap_(0) {}
  book_vector(const book_vector&) = delete;
  book_vector& operator=(const book_vector&) = delete;
  ~book_vector() { clear_storage(); }
  std::size_t size() const { return size_; }
  bool empty() const { return size_ == 0; }
  T& operator[](std::size_t i) { return data_[i]; }
  const T& operator[](std::size_t i) const { return data_[i]; }
  T& back() { return data_[size_ - 1]; }
  void pop_back() { --size_; }
  void push_back(const T& v) {
    if (size_ == cap_) grow();
    data_[size_++] = v;
  }
  void erase(std::size_t i) {
    for (std::size_t k = i + 1; k < size_; ++k) data_[k - 1] = data_[k];
    --size_;
  }
  void clear() { size_ = 0; }
  void clear_storage() {
    if (data_) book_->deallocate(data_, cap_ * sizeof(T), alignof(T));
    data_ = nullptr;
    size_ = cap_ = 0;
  }

 private:
  void grow() {
    const std::size_t ncap = cap_ ? cap_ * 2 : 16;
    T* nd = static_cast<T*>(book_->allocate(ncap * sizeof(T), alignof(T)));
    if (size_) std::memcpy(static_cast<void*>(nd), static_cast<const void*>(data_), size_ * sizeof(T));
    if (data_) book_->deallocate(data_, cap_ * sizeof(T), alignof(T));
    data_ = nd;
    cap_ = ncap;
  }
  Bookkeeper* book_;
  T* data_;
  std::size_t size_, cap_;
};

// device_ptr<void> and void* both: the address as a char pointer of the same kind
template <typename P> struct pool_pointer;
template <> struct pool_pointer<void*> {
  static void* advance(void* p, std::size_t bytes) { return static_cast<char*>(p) + bytes; }
  static bool same(void* a, void* b) { return a == b; }
};
template <typename T> struct pool_pointer<thrust::device_ptr<T> > {
  static bool same(thrust::device_ptr<T> a, thrust::device_ptr<T> b) { return a.get() == b.get(); }
  static thrust::device_ptr<T> advance(thrust::device_ptr<T> p, std::size_t bytes) {
    return thrust::device_ptr<T>(reinterpret_cast<T*>(reinterpret_cast<char*>(p.get()) + bytes));
  }
};
}  // namespace detail

struct disjoint_pool_options : pool_options {
  std::size_t min_blocks_per_chunk, max_blocks_per_chunk, min_bytes_per_chunk, max_bytes_per_chunk;
  bool cache_oversized;
  std::size_t cached_size_cutoff_factor;
  disjoint_pool_options()
      : min_blocks_per_chunk(16), max_blocks_per_chunk((std::size_t)1 << 20), min_bytes_per_chunk(1024),
        max_bytes_per_chunk((std::size_t)1 << 30), cache_oversized(true), cached_size_cutoff_factor(16) {
    smallest_block_size = 256;
    largest_block_size = (std::size_t)1 << 20;
  }
};

template <typename Upstream, typename Bookkeeper = new_delete_resource>
class disjoint_unsynchronized_pool_resource final : public memory_resource<typename Upstream::pointer> {
 public:
  typedef typename Upstream::pointer pointer;
  static disjoint_pool_options get_default_options() { return disjoint_pool_options(); }

  disjoint_unsynchronized_pool_resource(Upstream* upstream, Bookkeeper* bookkeeper,
                                        disjoint_pool_options options = get_default_options())
      : upstream_(upstream), book_(bookkeeper), options_(options), pools_(bookkeeper), chunks_(bookkeeper),
        cached_oversized_(bookkeeper), oversized_(bookkeeper), upstream_calls_(0) {
    init_pools();
  }
  explicit disjoint_unsynchronized_pool_resource(disjoint_pool_options options = get_default_options())
      : upstream_(get_global_resource<Upstream>()), book_(get_global_resource<Bookkeeper>()), options_(options),
        pools_(book_), chunks_(book_), cached_oversized_(book_), oversized_(book_), upstream_calls_(0) {
    init_pools();
  }
  disjoint_unsynchronized_pool_resource(const disjoint_unsynchronized_pool_resource&) = delete;
  disjoint_unsynchronized_pool_resource& operator=(const disjoint_unsynchronized_pool_resource&) = delete;
  ~disjoint_unsynchronized_pool_resource() {
    release();
    for (std::size_t i = 0; i < pools_.size(); ++i) {
      pools_[i].free_blocks->~free_list();
      book_->deallocate(pools_[i].free_blocks, sizeof(free_list), alignof(free_list));
    }
  }

  // Gives every chunk and every cached oversized block back to the upstream resource.  Blocks
  // still handed out become invalid, as with the reference's pool.
  void release() {
    for (std::size_t i = 0; i < pools_.size(); ++i) {
      pools_[i].free_blocks->clear();
      pools_[i].previous_allocated_count = 0;
    }
    for (std::size_t i = 0; i < chunks_.size(); ++i) upstream_->deallocate(chunks_[i].ptr, chunks_[i].bytes, block_alignment);
    chunks_.clear();
    for (std::size_t i = 0; i < cached_oversized_.size(); ++i)
      upstream_->deallocate(cached_oversized_[i].ptr, cached_oversized_[i].bytes, block_alignment);
    cached_oversized_.clear();
    oversized_.clear();
  }
  Upstream* upstream_resource() const { return upstream_; }
  std::size_t upstream_allocations() const { return upstream_calls_; }  // how often the upstream resource was asked
  std::size_t chunks() const { return chunks_.size(); }
  std::size_t cached_oversized_blocks() const { return cached_oversized_.size(); }

 protected:
  static const std::size_t block_alignment = 256;

  pointer do_allocate(std::size_t bytes, std::size_t alignment) override {
    if (alignment > block_alignment) throw std::bad_alloc();
    if (bytes == 0) bytes = 1;
    if (bytes > options_.largest_block_size) return allocate_oversized(bytes);
    const std::size_t idx = pool_index(bytes);
    pool_t& p = pools_[idx];
    if (p.free_blocks->empty()) refill(idx);
    const pointer block = p.free_blocks->back();
    p.free_blocks->pop_back();
    return block;
  }

  void do_deallocate(pointer ptr, std::size_t bytes, std::size_t) override {
    if (bytes == 0) bytes = 1;
    if (bytes > options_.largest_block_size) {
      for (std::size_t i = 0; i < oversized_.size(); ++i) {
        if (detail::pool_pointer<pointer>::same(oversized_[i].ptr, ptr)) {
          const block_t b = oversized_[i];
          oversized_.erase(i);
          if (options_.cache_oversized) cached_oversized_.push_back(b);
          else upstream_->deallocate(b.ptr, b.bytes, block_alignment);
          return;
        }
      }
      throw std::bad_alloc();  // not one of ours
    }
    pools_[pool_index(bytes)].free_blocks->push_back(ptr);
  }

 private:
  typedef detail::book_vector<pointer, Bookkeeper> free_list;
  struct pool_t {
    free_list* free_blocks;
    std::size_t previous_allocated_count;
  };
  struct block_t {
    pointer ptr;
    std::size_t bytes;
  };

  void init_pools() {
    std::size_t smallest = options_.smallest_block_size ? options_.smallest_block_size : 1;
    smallest_log2_ = 0;
    while (((std::size_t)1 << smallest_log2_) < smallest) ++smallest_log2_;
    std::size_t largest_log2 = smallest_log2_;
    while (((std::size_t)1 << largest_log2) < options_.largest_block_size) ++largest_log2;
    for (std::size_t l = smallest_log2_; l <= largest_log2; ++l) {
      void* mem = book_->allocate(sizeof(free_list), alignof(free_list));
      pool_t p = {new (mem) free_list(book_), 0};
      pools_.push_back(p);
    }
  }
  std::size_t pool_index(std::size_t bytes) const {
    std::size_t l = smallest_log2_;
    while (((std::size_t)1 << l) < bytes) ++l;
    return l - smallest_log2_;
  }
  // a new chunk for pool idx: twice as many blocks as the last one, within the options' limits
  void refill(std::size_t idx) {
    pool_t& p = pools_[idx];
    const std::size_t block = (std::size_t)1 << (idx + smallest_log2_);
    std::size_t count = p.previous_allocated_count ? p.previous_allocated_count * 2 : options_.min_blocks_per_chunk;
    if (count * block < options_.min_bytes_per_chunk) count = (options_.min_bytes_per_chunk + block - 1) / block;
    if (count > options_.max_blocks_per_chunk) count = options_.max_blocks_per_chunk;
    if (count * block > options_.max_bytes_per_chunk) count = options_.max_bytes_per_chunk / block;
    if (count == 0) count = 1;
    // blocks keep the chunk's alignment: every block size is a power of two, rounded to it
    const std::size_t stride = block < block_alignment ? block_alignment : block;
    const std::size_t bytes = count * stride;
    ++upstream_calls_;
    const pointer chunk = upstream_->allocate(bytes, block_alignment);
    const block_t c = {chunk, bytes};
    chunks_.push_back(c);
    p.previous_allocated_count = count;
    for (std::size_t i = count; i-- > 0;) p.free_blocks->push_back(detail::pool_pointer<pointer>::advance(chunk, i * stride));
  }
  pointer allocate_oversized(std::size_t bytes) {
    if (options_.cache_oversized) {
      // smallest cached block that is large enough and not wastefully larger
      std::size_t best = cached_oversized_.size();
      for (std::size_t i = 0; i < cached_oversized_.size(); ++i) {
        const std::size_t have = cached_oversized_[i].bytes;
        if (have >= bytes && have / options_.cached_size_cutoff_factor <= bytes &&
            (best == cached_oversized_.size() || have < cached_oversized_[best].bytes))
          best = i;
      }
      if (best != cached_oversized_.size()) {
        const block_t b = cached_oversized_[best];
        cached_oversized_.erase(best);
        oversized_.push_back(b);
        return b.ptr;
      }
    }
    ++upstream_calls_;
    const block_t b = {upstream_->allocate(bytes, block_alignment), bytes};
    oversized_.push_back(b);
    return b.ptr;
  }

  Upstream* upstream_;
  Bookkeeper* book_;
  disjoint_pool_options options_;
  std::size_t smallest_log2_;
  detail::book_vector<pool_t, Bookkeeper> pools_;
  detail::book_vector<block_t, Bookkeeper> chunks_;
  detail::book_vector<block_t, Bookkeeper> cached_oversized_;
  detail::book_vector<block_t, Bookkeeper> oversized_;
  std::size_t upstream_calls_;
};

}  // namespace mr
}  // namespace thrust

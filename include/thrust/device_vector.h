// thrust::device_vector<T, Alloc>: a resizable array in device memory.
//
// The subset of the reference's vector_base that code on the sort / scan / reduce /
// select / merge path uses (thrust/device_vector.h:54-64, thrust/detail/vector_base.inl):
// construction from a size, a size and a value, a host range, a std::vector / host_vector
// or another device_vector; begin/end/data/size/resize/clear/swap; operator[] / front /
// back through device_reference; assignment across systems.  Elements must be trivially
// copy-constructible and destructible: storage is raw device memory, filled and copied by the device system.  Storage
// comes from Alloc (default thrust::device_allocator<T>: the device system's malloc); any
// allocator whose allocate(n) yields a device_ptr<T> or a raw device pointer will do, e.g.
// thrust::mr::allocator<T, Pool> over a pool resource (thrust/mr/pool.h).
#pragma once
#include <algorithm>
#include <cstring>
#include <new>
#include <stdexcept>
#include <cstddef>
#include <iterator>
#include <type_traits>
#include <utility>
#include <vector>

#include <thrust/device_allocator.h>
#include <thrust/device_ptr.h>
#include <thrust/host_vector.h>

namespace thrust {

template <typename T, typename Alloc = device_allocator<T> >
class device_vector {
  // (a type may still define its own assignment: elements are never assigned on the device
  // side of this class, only copied as bytes)
  static_assert(std::is_trivially_copy_constructible<T>::value && std::is_trivially_destructible<T>::value,
                "thrust::device_vector: elements must be trivially copy-constructible and destructible");

 public:
  typedef T value_type;
  typedef Alloc allocator_type;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  typedef device_ptr<T> pointer;
  typedef device_ptr<const T> const_pointer;
  typedef device_ptr<T> iterator;
  typedef device_ptr<const T> const_iterator;
  typedef device_reference<T> reference;
  typedef device_reference<const T> const_reference;
  typedef std::reverse_iterator<iterator> reverse_iterator;
  typedef std::reverse_iterator<const_iterator> const_reverse_iterator;

  device_vector() : data_(nullptr), size_(0), capacity_(0), alloc_() {}
  explicit device_vector(const Alloc& alloc) : data_(nullptr), size_(0), capacity_(0), alloc_(alloc) {}
  explicit device_vector(size_type n, const Alloc& alloc = Alloc()) : device_vector(alloc) { resize(n); }
  device_vector(size_type n, const T& value, const Alloc& alloc = Alloc()) : device_vector(alloc) { resize(n, value); }
  device_vector(const device_vector& o) : device_vector(o.alloc_) { assign_device(o.data_, o.size_); }
  template <typename A2>
  device_vector(const device_vector<T, A2>& o, const Alloc& alloc = Alloc()) : device_vector(alloc) {
    assign_device(o.data_, o.size_);
  }
  device_vector(device_vector&& o) noexcept
      : data_(o.data_), size_(o.size_), capacity_(o.capacity_), alloc_(o.alloc_) {
    o.data_ = nullptr;
    o.size_ = o.capacity_ = 0;
  }
  template <typename A>
  device_vector(const std::vector<T, A>& h, const Alloc& alloc = Alloc()) : device_vector(alloc) {
    assign_std_vector(h, std::is_same<T, bool>());
  }
  // host_vector<bool>: an array of bool
  device_vector(const detail::contiguous_vector<T>& h, const Alloc& alloc = Alloc()) : device_vector(alloc) {
    assign_host(h.data(), h.size());
  }
  template <typename InputIterator,
            typename = typename std::iterator_traits<InputIterator>::iterator_category>
  device_vector(InputIterator first, InputIterator last, const Alloc& alloc = Alloc()) : device_vector(alloc) {
    assign(first, last);
  }
  ~device_vector() { release(); }

  device_vector& operator=(const device_vector& o) {
    if (this != &o) assign_device(o.data_, o.size_);
    return *this;
  }
  device_vector& operator=(device_vector&& o) noexcept {
    swap(o);
    return *this;
  }
  template <typename A>
  device_vector& operator=(const std::vector<T, A>& h) {
    assign_std_vector(h, std::is_same<T, bool>());
    return *this;
  }
  device_vector& operator=(const detail::contiguous_vector<T>& h) {
    assign_host(h.data(), h.size());
    return *this;
  }

  template <typename InputIterator>
  void assign(InputIterator first, InputIterator last) { assign_range(first, last, 0); }
  void assign(size_type n, const T& value) {
    size_ = 0;
    resize(n, value);
  }

  iterator begin() { return iterator(data_); }
  iterator end() { return iterator(data_ + size_); }
  const_iterator begin() const { return const_iterator(data_); }
  const_iterator end() const { return const_iterator(data_ + size_); }
  const_iterator cbegin() const { return begin(); }
  const_iterator cend() const { return end(); }
  reverse_iterator rbegin() { return reverse_iterator(end()); }
  reverse_iterator rend() { return reverse_iterator(begin()); }
  const_reverse_iterator rbegin() const { return const_reverse_iterator(end()); }
  const_reverse_iterator rend() const { return const_reverse_iterator(begin()); }
  const_reverse_iterator crbegin() const { return rbegin(); }
  const_reverse_iterator crend() const { return rend(); }
  pointer data() { return pointer(data_); }
  const_pointer data() const { return const_pointer(data_); }
  size_type size() const { return size_; }
  size_type capacity() const { return capacity_; }
  bool empty() const { return size_ == 0; }

  reference operator[](size_type i) { return reference(data_ + i); }
  const_reference operator[](size_type i) const { return const_reference(data_ + i); }
  reference front() { return reference(data_); }
  reference back() { return reference(data_ + size_ - 1); }
  const_reference front() const { return const_reference(data_); }
  const_reference back() const { return const_reference(data_ + size_ - 1); }
  reference at(size_type i) {
    if (i >= size_) throw std::out_of_range("thrust::device_vector::at");
    return reference(data_ + i);
  }
  const_reference at(size_type i) const {
    if (i >= size_) throw std::out_of_range("thrust::device_vector::at");
    return const_reference(data_ + i);
  }
  size_type max_size() const { return (~size_type(0)) / sizeof(T); }

  allocator_type get_allocator() const { return alloc_; }
  void reserve(size_type n) {
    if (n <= capacity_) return;
    T* fresh = allocate(n);
    if (size_) copy_raw(fresh, data_, size_, THRUST_AMD_D2D);
    sync();
    free_raw(data_, capacity_);
    data_ = fresh;
    capacity_ = n;
  }
  void resize(size_type n) { resize(n, T()); }
  void resize(size_type n, const T& value) {
    if (n > capacity_) reserve(n);
    if (n > size_) {
      if (sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8) {
        system::hip::detail::throw_on_error(
            thrust_amd_fill(data_ + size_, n - size_, sizeof(T), &value, nullptr), "device_vector fill");
      } else {
        // the fill kernel moves items of 1, 2, 4 or 8 bytes; wider elements are laid out on
        // the host, a piece at a time, and copied
        const size_type piece = (size_type)((std::size_t)(1 << 20) / sizeof(T) + 1);
        const size_type count = (n - size_) < piece ? (n - size_) : piece;
        T* staged = static_cast<T*>(::operator new((std::size_t)count * sizeof(T)));
        for (size_type i = 0; i < count; ++i) std::memcpy(static_cast<void*>(staged + i), &value, sizeof(T));
        for (size_type done = size_; done < n; done += count)
          copy_raw(data_ + done, staged, (n - done) < count ? (n - done) : count, THRUST_AMD_H2D);
        sync();
        ::operator delete(staged);
      }
      sync();
    }
    size_ = n;
  }
  void clear() { size_ = 0; }
  void shrink_to_fit() {
    if (size_ == capacity_) return;
    device_vector tmp(*this);
    swap(tmp);
  }
  void push_back(const T& v) {
    if (size_ == capacity_) reserve(capacity_ ? 2 * capacity_ : 16);
    copy_raw(data_ + size_, &v, 1, THRUST_AMD_H2D);
    ++size_;
  }
  void pop_back() { --size_; }
  iterator erase(iterator position) { return erase(position, position + 1); }
  // Inserts before `position`; returns the first inserted element.  The elements behind the
  // insertion point move through a temporary copy (device memory cannot be shifted onto itself).
  iterator insert(iterator position, const T& value) { return insert(position, (size_type)1, value); }
  iterator insert(iterator position, size_type n, const T& value) {
    const size_type at = (size_type)(position - begin());
    open_gap(at, n);
    if (n) {
      device_vector fill(n, value);
      copy_raw(data_ + at, fill.data_, n, THRUST_AMD_D2D);
      sync();
    }
    return begin() + at;
  }
  template <typename InputIterator,
            typename = typename std::iterator_traits<InputIterator>::iterator_category>
  iterator insert(iterator position, InputIterator first, InputIterator last) {
    const size_type at = (size_type)(position - begin());
    device_vector added(first, last);  // (also when the range lies in this vector)
    open_gap(at, added.size());
    if (added.size()) {
      copy_raw(data_ + at, added.data_, added.size(), THRUST_AMD_D2D);
      sync();
    }
    return begin() + at;
  }
  iterator erase(iterator first, iterator last) {
    const size_type tail = end() - last;
    if (tail && first != last) {
      // overlapping move towards the front: stage through a copy of the tail
      device_vector tmp(last, end());
      copy_raw(first.get(), tmp.data_, tail, THRUST_AMD_D2D);
      sync();
    }
    size_ -= (last - first);
    return first;
  }
  void swap(device_vector& o) noexcept {
    std::swap(data_, o.data_);
    std::swap(size_, o.size_);
    std::swap(capacity_, o.capacity_);
    std::swap(alloc_, o.alloc_);
  }

  // Host copy of the contents.
  void copy_to_host(T* dst) const {
    if (size_) copy_raw(dst, data_, size_, THRUST_AMD_D2H);
  }

 private:
  template <typename U, typename A2> friend class device_vector;

  static T* to_raw(T* p) { return p; }
  template <typename P>
  static T* to_raw(const P& p) { return p.get(); }
  T* allocate(size_type n) {
    if (n == 0) return nullptr;
    if (n > (~size_type(0)) / sizeof(T)) throw system::detail::bad_alloc("device_vector: size overflow");
    return to_raw(alloc_.allocate(n));
  }
  void free_raw(T* p, size_type n) {
    typedef decltype(std::declval<Alloc&>().allocate(size_type())) alloc_pointer;
    if (p) alloc_.deallocate(alloc_pointer(p), n);
  }
  static void sync() {
    system::hip::detail::throw_on_error(thrust_amd_stream_synchronize(nullptr), "device_vector synchronize");
  }
  static void copy_raw(T* dst, const T* src, size_type n, int kind) {
    system::hip::detail::throw_on_error(thrust_amd_memcpy(dst, src, n * sizeof(T), kind, nullptr),
                                        "device_vector copy");
  }
  // Makes room for n elements at index `at`: the tail moves n places back, the size grows by n.
  // The capacity grows only when it has to, and then to exactly the new size.
  void open_gap(size_type at, size_type n) {
    if (n == 0) return;
    const size_type tail = size_ - at;
    device_vector moved;
    if (tail) moved.assign_device(data_ + at, tail);
    if (size_ + n > capacity_) reserve(size_ + n);
    if (tail) {
      copy_raw(data_ + at + n, moved.data_, tail, THRUST_AMD_D2D);
      sync();
    }
    size_ += n;
  }
  void release() {
    free_raw(data_, capacity_);
    data_ = nullptr;
    size_ = capacity_ = 0;
  }
  void assign_host(const T* src, size_type n) {
    size_ = 0;
    if (n > capacity_) reserve(n);
    if (n) copy_raw(data_, src, n, THRUST_AMD_H2D);
    size_ = n;
  }
  void assign_device(const T* src, size_type n) {
    size_ = 0;
    if (n > capacity_) reserve(n);
    if (n) {
      copy_raw(data_, src, n, THRUST_AMD_D2D);
      sync();
    }
    size_ = n;
  }
  // device range
  template <typename U>
  void assign_range(device_ptr<U> first, device_ptr<U> last, int) {
    static_assert(std::is_same<typename std::remove_const<U>::type, T>::value,
                  "device_vector: element types of a device range must match");
    assign_device(first.get(), (size_type)(last - first));
  }
  // host range (any input iterator)
  template <typename It>
  void assign_range(It first, It last, long) {
    detail::staging_vector<T> staged(first, last);
    assign_host(staged.data(), staged.size());
  }
  template <typename A>
  void assign_std_vector(const std::vector<T, A>& h, std::false_type) { assign_host(h.data(), h.size()); }
  // std::vector<bool> is bit-packed: through an array of bool
  template <typename A>
  void assign_std_vector(const std::vector<T, A>& h, std::true_type) { assign_range(h.begin(), h.end(), 0L); }

  T* data_;
  size_type size_, capacity_;
  Alloc alloc_;
};

template <typename T, typename DA>
inline void swap(device_vector<T, DA>& a, device_vector<T, DA>& b) { a.swap(b); }

template <typename T, typename Alloc>
template <typename DA>
host_vector<T, Alloc>::host_vector(const device_vector<T, DA>& d) : base(d.size()) {
  d.copy_to_host(this->data());
}
template <typename T, typename Alloc>
template <typename DA>
host_vector<T, Alloc>& host_vector<T, Alloc>::operator=(const device_vector<T, DA>& d) {
  this->resize(d.size());
  d.copy_to_host(this->data());
  return *this;
}

template <typename T, typename Alloc>
template <typename U>
host_vector<T, Alloc>::host_vector(device_ptr<U> first, device_ptr<U> last) : base((std::size_t)(last - first)) {
  typedef typename std::remove_const<U>::type V;
  const std::size_t n = this->size();
  if (n == 0) return;
  if (std::is_same<V, T>::value) {
    system::hip::detail::throw_on_error(
        thrust_amd_memcpy(this->data(), first.get(), n * sizeof(V), THRUST_AMD_D2H, nullptr), "host_vector copy");
  } else {
    detail::staging_vector<V> staged(n);
    system::hip::detail::throw_on_error(
        thrust_amd_memcpy(staged.data(), first.get(), n * sizeof(V), THRUST_AMD_D2H, nullptr), "host_vector copy");
    for (std::size_t i = 0; i < n; ++i) (*this)[i] = static_cast<T>(staged[i]);
  }
}

// Comparisons between device_vector, host_vector and std::vector, in either order
// (thrust/detail/vector_base.inl:1190-1320): the device side is copied to the host once.
template <typename T, typename DA, typename DB>
inline bool operator==(const device_vector<T, DA>& a, const device_vector<T, DB>& b) {
  if (a.size() != b.size()) return false;
  return host_vector<T>(a) == host_vector<T>(b);
}
template <typename T, typename DA, typename A>
inline bool operator==(const device_vector<T, DA>& a, const std::vector<T, A>& b) {
  if (a.size() != b.size()) return false;
  const host_vector<T> h(a);
  return std::equal(h.begin(), h.end(), b.begin());
}
template <typename T, typename DA, typename A>
inline bool operator==(const std::vector<T, A>& a, const device_vector<T, DA>& b) { return b == a; }
template <typename T, typename DA>
inline bool operator==(const device_vector<T, DA>& a, const detail::contiguous_vector<T>& b) {
  if (a.size() != b.size()) return false;
  const host_vector<T> h(a);
  return std::equal(h.begin(), h.end(), b.begin());
}
template <typename T, typename DA>
inline bool operator==(const detail::contiguous_vector<T>& a, const device_vector<T, DA>& b) { return b == a; }
template <typename T, typename DA, typename DB>
inline bool operator!=(const device_vector<T, DA>& a, const device_vector<T, DB>& b) { return !(a == b); }
template <typename T, typename DA, typename A>
inline bool operator!=(const device_vector<T, DA>& a, const std::vector<T, A>& b) { return !(a == b); }
template <typename T, typename DA, typename A>
inline bool operator!=(const std::vector<T, A>& a, const device_vector<T, DA>& b) { return !(b == a); }
template <typename T, typename DA>
inline bool operator!=(const device_vector<T, DA>& a, const detail::contiguous_vector<T>& b) { return !(a == b); }
template <typename T, typename DA>
inline bool operator!=(const detail::contiguous_vector<T>& a, const device_vector<T, DA>& b) { return !(b == a); }

}  // namespace thrust

// Programs written for the reference reach these through its vector headers
// (thrust/detail/vector_base.inl:19-40 includes the algorithms the container is built from).
#include <thrust/advance.h>
#include <thrust/copy.h>
#include <thrust/distance.h>
#include <thrust/equal.h>
#include <thrust/fill.h>
#include <thrust/reduce.h>
#include <thrust/swap.h>

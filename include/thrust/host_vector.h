// thrust::host_vector<T>: a std::vector whose iterators belong to the host system.
// host_vector<bool> is an array of bool like the reference's (thrust/host_vector.h:56-66 over
// thrust/detail/vector_base.h: contiguous storage whatever the element type), not the
// bit-packed std::vector<bool>: its elements have addresses, so it can be copied to and from
// device memory as a block and its iterators are plain pointers.
#pragma once
#include <algorithm>
#include <cstddef>
#include <initializer_list>
#include <iterator>
#include <memory>
#include <stdexcept>
#include <vector>

#include <thrust/detail/config.h>

namespace thrust {

template <typename T> class device_allocator;
template <typename T, typename Alloc> class device_vector;
template <typename T> class device_ptr;

namespace detail {

// The part of std::vector's interface that host code of this API uses, over one contiguous
// array of T.  Only instantiated for bool.
template <typename T>
class contiguous_vector {
 public:
  typedef T value_type;
  typedef std::size_t size_type;
  typedef std::ptrdiff_t difference_type;
  typedef T& reference;
  typedef const T& const_reference;
  typedef T* pointer;
  typedef const T* const_pointer;
  typedef T* iterator;
  typedef const T* const_iterator;
  typedef std::reverse_iterator<iterator> reverse_iterator;
  typedef std::reverse_iterator<const_iterator> const_reverse_iterator;

  contiguous_vector() : data_(nullptr), size_(0), capacity_(0) {}
  explicit contiguous_vector(size_type n) : contiguous_vector() { resize(n); }
  contiguous_vector(size_type n, const T& value) : contiguous_vector() { resize(n, value); }
  contiguous_vector(const contiguous_vector& o) : contiguous_vector() { assign(o.begin(), o.end()); }
  contiguous_vector(contiguous_vector&& o) noexcept : data_(o.data_), size_(o.size_), capacity_(o.capacity_) {
    o.data_ = nullptr;
    o.size_ = o.capacity_ = 0;
  }
  contiguous_vector(std::initializer_list<T> l) : contiguous_vector() { assign(l.begin(), l.end()); }
  template <typename A>
  contiguous_vector(const std::vector<T, A>& v) : contiguous_vector() { assign(v.begin(), v.end()); }
  template <typename InputIterator, typename = typename std::iterator_traits<InputIterator>::iterator_category>
  contiguous_vector(InputIterator first, InputIterator last) : contiguous_vector() { assign(first, last); }
  ~contiguous_vector() { delete[] data_; }

  contiguous_vector& operator=(const contiguous_vector& o) {
    if (this != &o) assign(o.begin(), o.end());
    return *this;
  }
  contiguous_vector& operator=(contiguous_vector&& o) noexcept {
    swap(o);
    return *this;
  }

  iterator begin() { return data_; }
  iterator end() { return data_ + size_; }
  const_iterator begin() const { return data_; }
  const_iterator end() const { return data_ + size_; }
  const_iterator cbegin() const { return data_; }
  const_iterator cend() const { return data_ + size_; }
  reverse_iterator rbegin() { return reverse_iterator(end()); }
  reverse_iterator rend() { return reverse_iterator(begin()); }
  const_reverse_iterator rbegin() const { return const_reverse_iterator(end()); }
  const_reverse_iterator rend() const { return const_reverse_iterator(begin()); }
  size_type size() const { return size_; }
  size_type capacity() const { return capacity_; }
  bool empty() const { return size_ == 0; }
  T* data() { return data_; }
  const T* data() const { return data_; }
  reference operator[](size_type i) { return data_[i]; }
  const_reference operator[](size_type i) const { return data_[i]; }
  reference at(size_type i) {
    if (i >= size_) throw std::out_of_range("thrust::host_vector::at");
    return data_[i];
  }
  const_reference at(size_type i) const {
    if (i >= size_) throw std::out_of_range("thrust::host_vector::at");
    return data_[i];
  }
  reference front() { return data_[0]; }
  const_reference front() const { return data_[0]; }
  reference back() { return data_[size_ - 1]; }
  const_reference back() const { return data_[size_ - 1]; }

  void reserve(size_type n) {
    if (n <= capacity_) return;
    T* fresh = new T[n]();
    std::copy(data_, data_ + size_, fresh);
    delete[] data_;
    data_ = fresh;
    capacity_ = n;
  }
  void resize(size_type n, const T& value = T()) {
    if (n > capacity_) reserve(std::max(n, 2 * capacity_));
    if (n > size_) std::fill(data_ + size_, data_ + n, value);
    size_ = n;
  }
  void clear() { size_ = 0; }
  void shrink_to_fit() {}
  void push_back(const T& value) {
    const T copy = value;  // value may live in this vector
    resize(size_ + 1, copy);
  }
  void pop_back() { --size_; }
  void assign(size_type n, const T& value) {
    clear();
    resize(n, value);
  }
  template <typename InputIterator, typename = typename std::iterator_traits<InputIterator>::iterator_category>
  void assign(InputIterator first, InputIterator last) {
    clear();
    for (; first != last; ++first) push_back(static_cast<T>(*first));
  }
  iterator erase(const_iterator pos) { return erase(pos, pos + 1); }
  iterator erase(const_iterator first, const_iterator last) {
    iterator f = data_ + (first - data_), l = data_ + (last - data_);
    std::copy(l, end(), f);
    size_ -= (size_type)(l - f);
    return f;
  }
  iterator insert(const_iterator pos, const T& value) { return insert(pos, (size_type)1, value); }
  iterator insert(const_iterator pos, size_type n, const T& value) {
    const size_type at = (size_type)(pos - data_), old = size_;
    const T copy = value;
    resize(old + n);
    std::copy_backward(data_ + at, data_ + old, data_ + old + n);
    std::fill(data_ + at, data_ + at + n, copy);
    return data_ + at;
  }
  template <typename InputIterator, typename = typename std::iterator_traits<InputIterator>::iterator_category>
  iterator insert(const_iterator pos, InputIterator first, InputIterator last) {
    const contiguous_vector added(first, last);
    const size_type at = (size_type)(pos - data_), old = size_, n = added.size();
    resize(old + n);
    std::copy_backward(data_ + at, data_ + old, data_ + old + n);
    std::copy(added.begin(), added.end(), data_ + at);
    return data_ + at;
  }
  void swap(contiguous_vector& o) noexcept {
    std::swap(data_, o.data_);
    std::swap(size_, o.size_);
    std::swap(capacity_, o.capacity_);
  }

 private:
  T* data_;
  size_type size_, capacity_;
};

template <typename T>
inline bool operator==(const contiguous_vector<T>& a, const contiguous_vector<T>& b) {
  return a.size() == b.size() && std::equal(a.begin(), a.end(), b.begin());
}
template <typename T>
inline bool operator!=(const contiguous_vector<T>& a, const contiguous_vector<T>& b) { return !(a == b); }
template <typename T, typename A>
inline bool operator==(const contiguous_vector<T>& a, const std::vector<T, A>& b) {
  return a.size() == b.size() && std::equal(a.begin(), a.end(), b.begin());
}
template <typename T, typename A>
inline bool operator==(const std::vector<T, A>& a, const contiguous_vector<T>& b) { return b == a; }
template <typename T>
inline void swap(contiguous_vector<T>& a, contiguous_vector<T>& b) noexcept { a.swap(b); }

// What holds a host_vector's elements, and host-side staging copies of element type T.
template <typename T, typename Alloc = std::allocator<T> >
struct host_storage { typedef std::vector<T, Alloc> type; };
template <typename Alloc>
struct host_storage<bool, Alloc> { typedef contiguous_vector<bool> type; };
template <typename T>
using staging_vector = typename host_storage<T>::type;

}  // namespace detail

template <typename T, typename Alloc = std::allocator<T> >
class host_vector : public detail::host_storage<T, Alloc>::type {
  typedef typename detail::host_storage<T, Alloc>::type base;

 public:
  using base::base;
  host_vector() : base() {}
  host_vector(const base& v) : base(v) {}
  host_vector(const host_vector&) = default;
  host_vector(host_vector&&) = default;
  host_vector& operator=(const host_vector&) = default;
  host_vector& operator=(host_vector&&) = default;
  template <typename DA>
  host_vector(const device_vector<T, DA>& d);             // defined in device_vector.h
  template <typename DA>
  host_vector& operator=(const device_vector<T, DA>& d);  // defined in device_vector.h
  // a range of device memory: one copy for the whole range, not one per element
  template <typename U>
  host_vector(device_ptr<U> first, device_ptr<U> last);   // defined in device_vector.h
};

}  // namespace thrust

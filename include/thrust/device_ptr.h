// thrust::device_ptr<T>, thrust::device_reference<T>, raw_pointer_cast, device_pointer_cast,
// device_malloc / device_free.
//
// A device_ptr is a typed pointer tagged with the device system: algorithms given
// device_ptr iterators (device_vector::iterator is one) run on the GPU without an
// explicit policy.  Dereferencing on the host yields a device_reference, a proxy whose
// reads and writes are one-element copies across the bus -- the reference's
// tagged_reference over get_value / assign_value
// (thrust/system/cuda/detail/get_value.h:35-92, assign_value.h:32-100).
#pragma once
#include <cstddef>
#include <iterator>
#include <type_traits>

#include <thrust/detail/config.h>
#include <thrust/detail/execution_policy.h>
#include <thrust/system_error.h>

namespace thrust {

template <typename T> class device_ptr;

template <typename T>
class device_reference {
 public:
  typedef typename std::remove_const<T>::type value_type;
  typedef device_ptr<T> pointer;
  __host__ __device__ explicit device_reference(T* p) : ptr_(p) {}
  __host__ __device__ explicit device_reference(const device_ptr<T>& p);  // defined below device_ptr
  device_reference(const device_reference&) = default;
  // a reference to const from a reference to non-const
  template <typename U, typename = typename std::enable_if<std::is_same<const U, T>::value>::type>
  __host__ __device__ device_reference(const device_reference<U>& o) : ptr_((&o).get()) {}

  // (in device code the referent is ordinary memory: a functor handed device_vector iterators
  // may dereference them, thrust/detail/reference.h of the reference)
  __host__ __device__ operator value_type() const {
#if defined(__HIP_DEVICE_COMPILE__)
    return *ptr_;
#else
    value_type v;
    system::hip::detail::throw_on_error(
        thrust_amd_memcpy(static_cast<void*>(&v), ptr_, sizeof(value_type), THRUST_AMD_D2H, nullptr), "device_reference read");
    return v;
#endif
  }
  __host__ __device__ device_reference& operator=(const value_type& v) {
#if defined(__HIP_DEVICE_COMPILE__)
    *const_cast<value_type*>(ptr_) = v;
#else
    system::hip::detail::throw_on_error(
        thrust_amd_memcpy(const_cast<value_type*>(ptr_), &v, sizeof(value_type), THRUST_AMD_H2D, nullptr),
        "device_reference write");
#endif
    return *this;
  }
  __host__ __device__ device_reference& operator=(const device_reference& other) { return *this = (value_type)other; }
  // from a reference to another element type: converted on the way
  template <typename U>
  __host__ __device__ device_reference& operator=(const device_reference<U>& other) {
    return *this = static_cast<value_type>((typename device_reference<U>::value_type)other);
  }
  __host__ __device__ device_ptr<T> operator&() const { return device_ptr<T>(ptr_); }
  // exchanges the two referents
  __host__ __device__ void swap(device_reference& other) {
    const value_type mine = *this, theirs = other;
    *this = theirs;
    other = mine;
  }
#define THRUST_AMD_REF_COMPOUND(OP)                               \
  __host__ __device__ device_reference& operator OP##=(const value_type& v) {         \
    value_type t = *this;                                         \
    t OP##= v;                                                    \
    return *this = t;                                             \
  }
  THRUST_AMD_REF_COMPOUND(+) THRUST_AMD_REF_COMPOUND(-) THRUST_AMD_REF_COMPOUND(*) THRUST_AMD_REF_COMPOUND(/)
  THRUST_AMD_REF_COMPOUND(%) THRUST_AMD_REF_COMPOUND(<<) THRUST_AMD_REF_COMPOUND(>>) THRUST_AMD_REF_COMPOUND(&)
  THRUST_AMD_REF_COMPOUND(|) THRUST_AMD_REF_COMPOUND(^)
#undef THRUST_AMD_REF_COMPOUND
  __host__ __device__ device_reference& operator++() { return *this += value_type(1); }
  __host__ __device__ device_reference& operator--() { return *this -= value_type(1); }
  __host__ __device__ value_type operator++(int) {
    const value_type before = *this;
    *this = before + value_type(1);
    return before;
  }
  __host__ __device__ value_type operator--(int) {
    const value_type before = *this;
    *this = before - value_type(1);
    return before;
  }

 private:
  T* ptr_;
};
// thrust::swap of two references exchanges what they refer to (the references are proxies, taken by value)
template <typename T>
__host__ __device__ inline void swap(device_reference<T> a, device_reference<T> b) { a.swap(b); }

template <typename T>
class device_ptr {
 public:
  typedef std::random_access_iterator_tag iterator_category;
  typedef typename std::remove_const<T>::type value_type;
  typedef std::ptrdiff_t difference_type;
  typedef device_ptr pointer;
  typedef device_reference<T> reference;
  typedef T element_type;
  typedef thrust::device_system_tag system_tag;

  __host__ __device__ device_ptr() : ptr_(nullptr) {}
  __host__ __device__ device_ptr(std::nullptr_t) : ptr_(nullptr) {}
  __host__ __device__ explicit device_ptr(T* p) : ptr_(p) {}
  template <typename U, typename = typename std::enable_if<std::is_convertible<U*, T*>::value>::type>
  __host__ __device__ device_ptr(const device_ptr<U>& o) : ptr_(o.get()) {}

  __host__ __device__ T* get() const { return ptr_; }
  __host__ __device__ reference operator*() const { return reference(ptr_); }
  __host__ __device__ reference operator[](difference_type i) const { return reference(ptr_ + i); }
  __host__ __device__ T* operator->() const { return ptr_; }
  __host__ __device__ explicit operator bool() const { return ptr_ != nullptr; }

  __host__ __device__ device_ptr& operator++() { ++ptr_; return *this; }
  __host__ __device__ device_ptr operator++(int) { device_ptr t(*this); ++ptr_; return t; }
  __host__ __device__ device_ptr& operator--() { --ptr_; return *this; }
  __host__ __device__ device_ptr operator--(int) { device_ptr t(*this); --ptr_; return t; }
  __host__ __device__ device_ptr& operator=(std::nullptr_t) { ptr_ = nullptr; return *this; }
  // (templates on the integer type: an unsigned or 64-bit offset would otherwise be ambiguous
  // between the offset form and the conversion of the offset to a pointer difference)
  template <typename I, typename = typename std::enable_if<std::is_integral<I>::value>::type>
  __host__ __device__ device_ptr& operator+=(I n) { ptr_ += (difference_type)n; return *this; }
  template <typename I, typename = typename std::enable_if<std::is_integral<I>::value>::type>
  __host__ __device__ device_ptr& operator-=(I n) { ptr_ -= (difference_type)n; return *this; }
  template <typename I, typename = typename std::enable_if<std::is_integral<I>::value>::type>
  __host__ __device__ device_ptr operator+(I n) const { return device_ptr(ptr_ + (difference_type)n); }
  template <typename I, typename = typename std::enable_if<std::is_integral<I>::value>::type>
  __host__ __device__ device_ptr operator-(I n) const { return device_ptr(ptr_ - (difference_type)n); }
  __host__ __device__ difference_type operator-(const device_ptr& o) const { return ptr_ - o.ptr_; }
  __host__ __device__ bool operator==(const device_ptr& o) const { return ptr_ == o.ptr_; }
  __host__ __device__ bool operator!=(const device_ptr& o) const { return ptr_ != o.ptr_; }
  __host__ __device__ bool operator<(const device_ptr& o) const { return ptr_ < o.ptr_; }
  __host__ __device__ bool operator>(const device_ptr& o) const { return ptr_ > o.ptr_; }
  __host__ __device__ bool operator<=(const device_ptr& o) const { return ptr_ <= o.ptr_; }
  __host__ __device__ bool operator>=(const device_ptr& o) const { return ptr_ >= o.ptr_; }
  __host__ __device__ bool operator==(std::nullptr_t) const { return ptr_ == nullptr; }
  __host__ __device__ bool operator!=(std::nullptr_t) const { return ptr_ != nullptr; }

 private:
  T* ptr_;
};
template <typename T>
__host__ __device__ inline bool operator==(std::nullptr_t, const device_ptr<T>& p) { return p.get() == nullptr; }
template <typename T>
__host__ __device__ inline bool operator!=(std::nullptr_t, const device_ptr<T>& p) { return p.get() != nullptr; }
template <typename T>
__host__ __device__ inline device_reference<T>::device_reference(const device_ptr<T>& p) : ptr_(p.get()) {}

template <>
class device_ptr<void> {
 public:
  __host__ __device__ device_ptr() : ptr_(nullptr) {}
  __host__ __device__ explicit device_ptr(void* p) : ptr_(p) {}
  __host__ __device__ void* get() const { return ptr_; }

 private:
  void* ptr_;
};

template <typename T>
__host__ __device__ inline device_ptr<T> operator+(std::ptrdiff_t n, const device_ptr<T>& p) { return p + n; }

template <typename T>
__host__ __device__ inline device_ptr<T> device_pointer_cast(T* p) { return device_ptr<T>(p); }
template <typename T>
__host__ __device__ inline device_ptr<T> device_pointer_cast(const device_ptr<T>& p) { return p; }

template <typename T>
__host__ __device__ inline T* raw_pointer_cast(const device_ptr<T>& p) { return p.get(); }
template <typename T>
__host__ __device__ inline T* raw_pointer_cast(T* p) { return p; }
template <typename T>
__host__ __device__ inline T* raw_pointer_cast(const device_reference<T>& r) { return (&r).get(); }

// Allocation through the device system (cuda_cub::malloc / free in the reference,
// thrust/system/cuda/detail/malloc_and_free.h:51-100).
inline device_ptr<void> device_malloc(std::size_t bytes) {
  void* p = nullptr;
  const int rc = thrust_amd_malloc(&p, bytes);
  if (rc != 0) throw system::detail::bad_alloc(thrust_amd_error_string(rc));
  return device_ptr<void>(p);
}
template <typename T>
inline device_ptr<T> device_malloc(std::size_t n) {
  return device_ptr<T>(static_cast<T*>(device_malloc(n * sizeof(T)).get()));
}
template <typename T>
inline void device_free(device_ptr<T> p) {
  system::hip::detail::throw_on_error(thrust_amd_free(const_cast<void*>(static_cast<const void*>(p.get()))),
                                      "device_free");
}

}  // namespace thrust

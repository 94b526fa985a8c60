// thrust::host_vector<T>: a std::vector whose iterators belong to the host system.
#pragma once
#include <vector>

#include <thrust/detail/config.h>

namespace thrust {

template <typename T> class device_allocator;
template <typename T, typename Alloc> class device_vector;
template <typename T> class device_ptr;

template <typename T, typename Alloc = std::allocator<T> >
class host_vector : public std::vector<T, Alloc> {
  typedef std::vector<T, Alloc> base;

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

// thrust::device_event, thrust::device_future<T> and the policies that order asynchronous
// work: device.on(stream), device.after(dependencies...), device(alloc).
//
// An asynchronous algorithm (thrust/async/*.h) enqueues its kernels on a stream and returns
// at once.  What it returns owns everything the work needs until it has finished: the
// stream, the temporary storage, and for a future the device slot of the value.
//   event.wait()            blocks until the work has finished
//   event.ready()           asks without blocking
//   event.stream()          the stream the work runs on (native_handle() = hipStream_t as void*)
//   future.get() / extract() waits and returns the value
// Which stream the work runs on follows the reference (thrust/system/cuda/detail/future.inl,
// thrust/detail/execute_with_dependencies.h; tested by testing/async_reduce.cu:773-990):
// the stream given with .on(stream); else the stream of the first dependency given with
// .after(...); else a new stream of its own.  The work starts only after every dependency
// has finished; a dependency stays usable (its stream is shared, not taken away).
#pragma once
#include <atomic>
#include <cstddef>
#include <memory>
#include <utility>
#include <vector>

#include <thrust/execution_policy.h>
#include <thrust/system/hip/detail/backend.h>

namespace thrust {
namespace system {
namespace hip {

namespace detail {
// enqueued counts the pieces of work the library has put on the stream, synced how many of
// them a host-side wait has seen finished: an event whose number is not above `synced` is
// complete without asking the runtime (which, after a wait on an idle stream's event, can go
// on answering "not ready" for a stream that has been synchronised).
struct stream_state {
  void* stream;
  bool owned;
  std::atomic<unsigned long long> enqueued, synced;
  stream_state(void* s, bool o) : stream(s), owned(o), enqueued(0), synced(0) {}
  void mark_synced(unsigned long long upto) {
    unsigned long long seen = synced.load();
    while (seen < upto && !synced.compare_exchange_weak(seen, upto)) {}
  }
  ~stream_state() {
    if (owned && stream) {
      (void)thrust_amd_stream_synchronize(stream);
      (void)thrust_amd_stream_destroy(stream);
    }
  }
  stream_state(const stream_state&) = delete;
  stream_state& operator=(const stream_state&) = delete;
};
// What a piece of asynchronous work keeps alive: resources are released in reverse order of
// their registration, the stream last.
struct keep_alive {
  std::shared_ptr<stream_state> stream;
  unsigned long long ticket = 0;  // the work's number on its stream (stream_state::enqueued)
  std::vector<std::shared_ptr<void> > resources;
  ~keep_alive() {
    while (!resources.empty()) resources.pop_back();
  }
};
}  // namespace detail

// Handle to a stream; copies share it.
class unique_stream {
 public:
  unique_stream() {}
  explicit unique_stream(std::shared_ptr<detail::stream_state> s) : state_(std::move(s)) {}
  static unique_stream create() {
    void* s = nullptr;
    detail::throw_on_error(thrust_amd_stream_create(&s), "stream creation failed");
    return unique_stream(std::make_shared<detail::stream_state>(s, true));
  }
  static unique_stream borrow(void* s) { return unique_stream(std::make_shared<detail::stream_state>(s, false)); }
  bool valid() const { return (bool)state_; }
  void* native_handle() const { return state_ ? state_->stream : nullptr; }
  const std::shared_ptr<detail::stream_state>& state() const { return state_; }

 private:
  std::shared_ptr<detail::stream_state> state_;
};

class unique_eager_event {
 public:
  unique_eager_event() {}
  explicit unique_eager_event(std::shared_ptr<detail::keep_alive> k) : keep_(std::move(k)), stream_(keep_->stream) {}
  unique_eager_event(unique_eager_event&&) = default;
  unique_eager_event& operator=(unique_eager_event&&) = default;
  unique_eager_event(const unique_eager_event&) = delete;
  unique_eager_event& operator=(const unique_eager_event&) = delete;

  bool valid_stream() const { return stream_.valid(); }
  unique_stream& stream() { return stream_; }
  const unique_stream& stream() const { return stream_; }
  // Once the work has been seen complete it stays complete, whatever is enqueued on the
  // (shared) stream afterwards; the runtime is only asked while that is not yet known.
  bool ready() const {
    if (!valid_stream() || complete()) return true;
    int done = 0;
    detail::throw_on_error(thrust_amd_stream_query(stream_.native_handle(), &done), "stream query failed");
    if (done) done_ = true;
    return done != 0;
  }
  void wait() const {
    if (!valid_stream() || complete()) return;
    const std::shared_ptr<detail::stream_state>& st = stream_.state();
    const unsigned long long upto = st->enqueued.load();  // everything enqueued before the wait
    detail::throw_on_error(thrust_amd_stream_synchronize(stream_.native_handle()), "waiting for asynchronous work failed");
    st->mark_synced(upto);
    done_ = true;
  }
  const std::shared_ptr<detail::keep_alive>& keep() const { return keep_; }

 protected:
  std::shared_ptr<detail::keep_alive> keep_;
  unique_stream stream_;
  mutable bool done_ = false;

 private:
  bool complete() const {
    if (done_) return true;
    if (keep_ && keep_->ticket != 0 && keep_->ticket <= stream_.state()->synced.load()) done_ = true;
    return done_;
  }
};

template <typename T>
class unique_eager_future : public unique_eager_event {
 public:
  unique_eager_future() : d_value_(nullptr) {}
  unique_eager_future(std::shared_ptr<detail::keep_alive> k, const T* d_value)
      : unique_eager_event(std::move(k)), d_value_(d_value) {}
  unique_eager_future(unique_eager_future&&) = default;
  unique_eager_future& operator=(unique_eager_future&&) = default;

  bool valid_content() const { return d_value_ != nullptr; }
  // Waits for the work and returns the value; may be called more than once.
  T get() const {
    if (!d_value_) throw thrust::system_error(1, "thrust::future: no value to get");
    return detail::read_scalar<T>(d_value_, stream_.native_handle(), "future: value copy");  // the copy waits for the stream
  }
  T extract() { return get(); }
  const T* raw_data() const { return d_value_; }

 private:
  const T* d_value_;
};

// ------------------------------------------------------------------ dependencies
// device.after(a, b, ...): each argument is an event or a future; what is kept of it is
// its stream (shared) and whatever it keeps alive.
struct dependency_list {
  std::vector<std::shared_ptr<detail::keep_alive> > items;
  void add(const unique_eager_event& e) {
    if (e.valid_stream()) items.push_back(e.keep());
  }
};

struct after_policy : execution_policy<after_policy> {
  void* stream;        // from .on(stream); null = not given
  bool has_stream;
  dependency_list deps;
  after_policy() : stream(nullptr), has_stream(false) {}
  after_policy on(void* s) const {
    after_policy p(*this);
    p.stream = s;
    p.has_stream = true;
    return p;
  }
  template <typename... Events>
  after_policy after(const Events&... events) const {
    after_policy p(*this);
    const int dummy[] = {0, (p.deps.add(events), 0)...};
    (void)dummy;
    return p;
  }
};
// A synchronous algorithm called with such a policy waits for the dependencies on the host
// and then runs on the stream the rules above name (the null stream when there is none).
inline void* get_stream(const after_policy& p) {
  for (const auto& d : p.deps.items) (void)thrust_amd_stream_synchronize(d->stream->stream);
  if (p.has_stream) return p.stream;
  return p.deps.items.empty() ? nullptr : p.deps.items.front()->stream->stream;
}

template <typename... Events>
inline after_policy stream_policy::after(const Events&... events) const {
  return after_policy().on(stream).after(events...);
}
template <typename... Events>
inline after_policy par_t::after(const Events&... events) const {
  return after_policy().after(events...);
}

namespace detail {
// The launch context of one asynchronous call: where it runs and what it must keep alive.
struct async_context {
  std::shared_ptr<keep_alive> keep;
  void* stream() const { return keep->stream->stream; }
};

inline void wait_for(void* stream, const std::shared_ptr<keep_alive>& dep) {
  void* other = dep->stream->stream;
  if (other == stream) return;  // same stream: ordered already
  void* ev = nullptr;
  throw_on_error(thrust_amd_event_create(&ev), "event creation failed");
  int rc = thrust_amd_event_record(ev, other);
  if (rc == 0) rc = thrust_amd_stream_wait_event(stream, ev);
  (void)thrust_amd_event_destroy(ev);  // the runtime keeps a recorded event until it has fired
  throw_on_error(rc, "ordering asynchronous work failed");
}

inline async_context make_context(void* on_stream, bool has_stream, const dependency_list* deps) {
  async_context ctx;
  ctx.keep = std::make_shared<keep_alive>();
  if (has_stream) ctx.keep->stream = std::make_shared<stream_state>(on_stream, false);
  else if (deps && !deps->items.empty()) ctx.keep->stream = deps->items.front()->stream;
  else ctx.keep->stream = unique_stream::create().state();
  ctx.keep->ticket = ++ctx.keep->stream->enqueued;
  if (deps)
    for (const auto& d : deps->items) {
      wait_for(ctx.stream(), d);
      ctx.keep->resources.push_back(d);  // a dependency's resources outlive the work that follows it
    }
  return ctx;
}

// Policies an asynchronous algorithm accepts: any policy of this system.  Those without a
// stream of their own (device, par) get a new stream; par.on(s) runs on s.
template <typename Derived>
inline async_context context_of(execution_policy<Derived>& p, ...) {
  return make_context(nullptr, false, nullptr);
}
inline async_context context_of(execution_policy<stream_policy>& p, int) {
  return make_context(thrust::detail::derived_cast(p).stream, true, nullptr);
}
inline async_context context_of(execution_policy<after_policy>& p, int) {
  after_policy& a = thrust::detail::derived_cast(p);
  return make_context(a.stream, a.has_stream, &a.deps);
}
template <typename Alloc>
inline async_context context_of(execution_policy<allocator_policy<Alloc> >& p, int) {
  allocator_policy<Alloc>& a = thrust::detail::derived_cast(p);
  return a.stream ? make_context(a.stream, true, nullptr) : make_context(nullptr, false, nullptr);
}

// Temporary storage of an asynchronous call: taken like the synchronous algorithms take it
// and handed to the context, which gives it back when the work's owner goes away (the
// arena's release is stream-ordered; a user allocator's memory returns after the stream
// has drained -- temp_storage does both).
inline std::shared_ptr<temp_storage> async_temp(async_context& ctx, const temp_source& source) {
  std::shared_ptr<temp_storage> t = std::make_shared<temp_storage>(ctx.stream(), source);
  ctx.keep->resources.push_back(t);
  return t;
}
}  // namespace detail

}  // namespace hip
}  // namespace system

namespace detail {
template <typename... Events>
inline system::hip::after_policy device_t::after(const Events&... events) const {
  return system::hip::after_policy().after(events...);
}
}  // namespace detail

typedef system::hip::unique_eager_event device_event;
typedef system::hip::unique_eager_event device_unique_eager_event;
template <typename T>
using device_future = system::hip::unique_eager_future<T>;
template <typename T>
using device_unique_eager_future = system::hip::unique_eager_future<T>;

// Waits for every event or future given.
template <typename... Events>
inline void when_all_wait(const Events&... events) {
  const int dummy[] = {0, (events.wait(), 0)...};
  (void)dummy;
}

// when_all(a, b, ...): an event that is complete once every event or future given is
// (thrust/system/cuda/detail/future.inl:1350-1362).  No work is enqueued: the result lives on
// the first argument's stream, which is made to wait for the others on the device, and keeps
// alive what they keep alive.  With no arguments the event is complete at once.
template <typename... Events>
inline device_event when_all(const Events&... events) {
  system::hip::dependency_list deps;
  const int dummy[] = {0, (deps.add(events), 0)...};
  (void)dummy;
  if (deps.items.empty()) return device_event();
  system::hip::detail::async_context ctx = system::hip::detail::make_context(nullptr, false, &deps);
  return device_event(ctx.keep);
}

}  // namespace thrust

// thrust::mr::polymorphic_adaptor_resource: any resource with the right pointer type behind one
// class, so that containers of one type can draw from resources chosen at run time
// (thrust/mr/polymorphic_adaptor.h:25-55; examples/mr_basic.cu).
#pragma once
#include <thrust/mr/memory_resource.h>

namespace thrust {
namespace mr {
template <typename Pointer = void*>
class polymorphic_adaptor_resource final : public memory_resource<Pointer> {
 public:
  polymorphic_adaptor_resource(memory_resource<Pointer>* upstream) : upstream_(upstream) {}
  memory_resource<Pointer>* upstream_resource() const { return upstream_; }

 protected:
  Pointer do_allocate(std::size_t bytes, std::size_t alignment) override { return upstream_->allocate(bytes, alignment); }
  void do_deallocate(Pointer p, std::size_t bytes, std::size_t alignment) override {
    upstream_->deallocate(p, bytes, alignment);
  }
  bool do_is_equal(const memory_resource<Pointer>& other) const noexcept override {
    const polymorphic_adaptor_resource* o = dynamic_cast<const polymorphic_adaptor_resource*>(&other);
    return upstream_->is_equal(o ? *o->upstream_ : other);
  }

 private:
  memory_resource<Pointer>* upstream_;
};
}  // namespace mr
}  // namespace thrust

// rmm::device_async_resource_ref as it appears in the nvtext signatures: a non-owning reference to a
// stream-ordered device memory resource.  The default resource uses hipMallocAsync / hipFreeAsync.
#pragma once
#include <cuda/stream_ref>

#include <cstddef>

#include <nvtext_amd.h>

namespace rmm {
namespace mr {

class device_memory_resource {
 public:
  virtual ~device_memory_resource() = default;
  // return nullptr on failure
  virtual void* allocate_async(std::size_t bytes, cuda::stream_ref stream)                  = 0;
  virtual void deallocate_async(void* ptr, std::size_t bytes, cuda::stream_ref stream) noexcept = 0;
};

}  // namespace mr

class device_async_resource_ref {
 public:
  device_async_resource_ref() = default;  // the library's default: hipMallocAsync / hipFreeAsync
  device_async_resource_ref(mr::device_memory_resource& r) : _r{&r} {}
  device_async_resource_ref(mr::device_memory_resource* r) : _r{r} {}

  // The C-ABI view of this resource; `storage` must outlive the call it is passed to.
  const nvtext_amd_allocator* c_allocator(nvtext_amd_allocator& storage) const
  {
    if (!_r) return nullptr;
    storage.ctx      = _r;
    storage.allocate = [](void* ctx, size_t bytes, void* stream) -> void* {
      return static_cast<mr::device_memory_resource*>(ctx)->allocate_async(bytes, cuda::stream_ref{stream});
    };
    storage.deallocate = [](void* ctx, void* ptr, size_t bytes, void* stream) {
      static_cast<mr::device_memory_resource*>(ctx)->deallocate_async(ptr, bytes, cuda::stream_ref{stream});
    };
    return &storage;
  }

 private:
  mr::device_memory_resource* _r{nullptr};
};

}  // namespace rmm

namespace cudf {
inline cuda::stream_ref get_default_stream() { return cuda::stream_ref{}; }
inline rmm::device_async_resource_ref get_current_device_resource_ref() { return rmm::device_async_resource_ref{}; }
}  // namespace cudf

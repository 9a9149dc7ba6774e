// cudf::column (cpp/include/cudf/column/column.hpp:37): owning column.  Buffers are released through the
// memory resource and stream they were allocated with.
#pragma once
#include <cudf/column/column_view.hpp>
#include <rmm/resource_ref.hpp>

#include <memory>
#include <utility>
#include <vector>

namespace cudf {

// Owning device allocation (the role of rmm::device_buffer).
class device_buffer {
 public:
  device_buffer() = default;
  device_buffer(void* ptr, std::size_t bytes, cuda::stream_ref stream, rmm::device_async_resource_ref mr)
    : _ptr{ptr}, _bytes{bytes}, _stream{stream}, _mr{mr} {}
  device_buffer(device_buffer&& o) noexcept { *this = std::move(o); }
  device_buffer& operator=(device_buffer&& o) noexcept
  {
    if (this != &o) {
      release();
      _ptr = o._ptr; _bytes = o._bytes; _stream = o._stream; _mr = o._mr;
      o._ptr = nullptr; o._bytes = 0;
    }
    return *this;
  }
  device_buffer(device_buffer const&)            = delete;
  device_buffer& operator=(device_buffer const&) = delete;
  ~device_buffer() { release(); }
  [[nodiscard]] void* data() const noexcept { return _ptr; }
  [[nodiscard]] std::size_t size() const noexcept { return _bytes; }

 private:
  void release() noexcept
  {
    if (!_ptr) return;
    nvtext_amd_list_column tmp{};
    tmp.child       = _ptr;
    tmp.child_bytes = _bytes;
    nvtext_amd_allocator storage{};
    nvtext_amd_list_column_free(&tmp, _stream.get(), _mr.c_allocator(storage));
    _ptr = nullptr;
  }
  void* _ptr{nullptr};
  std::size_t _bytes{0};
  cuda::stream_ref _stream{};
  rmm::device_async_resource_ref _mr{};
};

class column {
 public:
  column(data_type type, size_type size, device_buffer&& data, device_buffer&& null_mask, size_type null_count,
         std::vector<std::unique_ptr<column>>&& children = {})
    : _type{type}, _size{size}, _data{std::move(data)}, _null_mask{std::move(null_mask)}, _null_count{null_count},
      _children{std::move(children)} {}

  [[nodiscard]] data_type type() const noexcept { return _type; }
  [[nodiscard]] size_type size() const noexcept { return _size; }
  [[nodiscard]] size_type null_count() const noexcept { return _null_count; }
  [[nodiscard]] bool nullable() const noexcept { return _null_mask.size() > 0; }
  [[nodiscard]] bool has_nulls() const noexcept { return _null_count > 0; }
  [[nodiscard]] size_type num_children() const noexcept { return static_cast<size_type>(_children.size()); }
  [[nodiscard]] column const& child(size_type i) const { return *_children.at(static_cast<std::size_t>(i)); }

  [[nodiscard]] column_view view() const
  {
    std::vector<column_view> kids;
    for (auto const& c : _children) kids.push_back(c->view());
    return column_view{_type, _size, _data.data(), static_cast<bitmask_type const*>(_null_mask.data()), _null_count, 0, kids};
  }
  operator column_view() const { return view(); }

 private:
  data_type _type{};
  size_type _size{0};
  device_buffer _data{};
  device_buffer _null_mask{};
  size_type _null_count{0};
  std::vector<std::unique_ptr<column>> _children{};
};

}  // namespace cudf

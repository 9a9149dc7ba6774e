// cudf::column_view (cpp/include/cudf/column/column_view.hpp:44-293, 317-471): non-owning, immutable
// view of device memory as a column.
#pragma once
#include <cudf/types.hpp>
#include <cudf/utilities/error.hpp>
#include <cudf/utilities/span.hpp>

#include <vector>

namespace cudf {

class column_view {
 public:
  column_view() = default;
  column_view(data_type type, size_type size, void const* data, bitmask_type const* null_mask, size_type null_count,
              size_type offset = 0, std::vector<column_view> const& children = {})
    : _type{type}, _size{size}, _data{data}, _null_mask{null_mask}, _null_count{null_count}, _offset{offset}, _children{children}
  {
    CUDF_EXPECTS(size >= 0, "Column size cannot be negative.");
    CUDF_EXPECTS(offset >= 0, "Invalid offset.");
    if (null_count > 0) CUDF_EXPECTS(null_mask != nullptr, "Invalid null mask for non-zero null count.");
  }

  [[nodiscard]] data_type type() const noexcept { return _type; }
  [[nodiscard]] size_type size() const noexcept { return _size; }
  [[nodiscard]] bool is_empty() const noexcept { return _size == 0; }
  [[nodiscard]] size_type offset() const noexcept { return _offset; }
  [[nodiscard]] size_type null_count() const noexcept { return _null_count; }
  [[nodiscard]] bool nullable() const noexcept { return _null_mask != nullptr; }
  [[nodiscard]] bool has_nulls() const noexcept { return _null_count > 0; }
  [[nodiscard]] bitmask_type const* null_mask() const noexcept { return _null_mask; }
  [[nodiscard]] size_type num_children() const noexcept { return static_cast<size_type>(_children.size()); }
  [[nodiscard]] column_view const& child(size_type i) const { return _children.at(static_cast<std::size_t>(i)); }

  // head<T>() ignores the offset, data<T>() applies it (column_view.hpp:70-113)
  template <typename T = void>
  [[nodiscard]] T const* head() const noexcept { return static_cast<T const*>(_data); }
  template <typename T>
  [[nodiscard]] T const* data() const noexcept { return head<T>() + _offset; }

  // column_view.hpp:445-452: implicit view of a fixed-width column as a device_span; throws
  // cudf::logic_error on a type mismatch or a nullable column.
  template <typename T>
  [[nodiscard]] operator device_span<T const>() const
  {
    CUDF_EXPECTS(type() == data_type{type_to_id<std::remove_const_t<T>>()}, "Device span type must match column view type.");
    CUDF_EXPECTS(!nullable(), "A nullable column view cannot be converted to a device span.");
    return device_span<T const>(data<T>(), static_cast<std::size_t>(size()));
  }

 private:
  data_type _type{};
  size_type _size{0};
  void const* _data{nullptr};
  bitmask_type const* _null_mask{nullptr};
  size_type _null_count{0};
  size_type _offset{0};
  std::vector<column_view> _children{};
};

}  // namespace cudf

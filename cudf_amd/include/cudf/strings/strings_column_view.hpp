// cudf::strings_column_view (cpp/include/cudf/strings/strings_column_view.hpp:27-114): a STRING column is
// parent{data = chars, null_mask, offset, size} with child[0] = offsets (INT32 or INT64).
#pragma once
#include <cudf/column/column_view.hpp>
#include <nvtext_amd.h>

namespace cudf {

class strings_column_view : private column_view {
 public:
  strings_column_view(column_view strings_column) : column_view(strings_column)
  {
    CUDF_EXPECTS(type().id() == type_id::STRING, "strings_column_view only supports strings");
  }
  static constexpr size_type offsets_column_index{0};

  using column_view::has_nulls;
  using column_view::is_empty;
  using column_view::null_count;
  using column_view::null_mask;
  using column_view::nullable;
  using column_view::offset;
  using column_view::size;

  [[nodiscard]] column_view parent() const { return static_cast<column_view>(*this); }
  [[nodiscard]] column_view offsets() const
  {
    CUDF_EXPECTS(num_children() > 0, "strings column has no children");
    return child(offsets_column_index);
  }
  [[nodiscard]] char const* chars_begin() const noexcept { return head<char>(); }

  // the C-ABI descriptor of this view
  [[nodiscard]] nvtext_amd_strings_column c_view() const
  {
    nvtext_amd_strings_column c{};
    c.chars      = head<char>();
    c.null_mask  = null_mask();
    c.size       = size();
    c.offset     = offset();
    c.null_count = null_count();
    if (num_children() > 0) {
      column_view const o = child(offsets_column_index);
      CUDF_EXPECTS(o.type().id() == type_id::INT32 || o.type().id() == type_id::INT64, "offsets must be INT32 or INT64");
      c.offsets          = o.head<void>();
      c.offsets_is_int64 = o.type().id() == type_id::INT64 ? 1 : 0;
    } else {
      CUDF_EXPECTS(size() == 0, "a strings column with rows needs an offsets child");
    }
    return c;
  }
};

}  // namespace cudf

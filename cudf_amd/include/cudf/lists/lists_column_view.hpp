// cudf::lists_column_view (cpp/include/cudf/lists/lists_column_view.hpp:54-55): children = [offsets INT32, child].
#pragma once
#include <cudf/column/column_view.hpp>
#include <cudf/strings/strings_column_view.hpp>

namespace cudf {

class lists_column_view : private column_view {
 public:
  lists_column_view(column_view const& lists_column) : column_view(lists_column)
  {
    CUDF_EXPECTS(type().id() == type_id::LIST, "lists_column_view only supports lists");
  }
  static constexpr size_type offsets_column_index{0};
  static constexpr size_type child_column_index{1};
  using column_view::has_nulls;
  using column_view::null_count;
  using column_view::null_mask;
  using column_view::num_children;
  using column_view::offset;
  using column_view::size;
  [[nodiscard]] column_view parent() const { return static_cast<column_view>(*this); }
  [[nodiscard]] column_view offsets() const { return column_view::child(offsets_column_index); }
  [[nodiscard]] column_view child() const { return column_view::child(child_column_index); }

  // the C-ABI descriptor of this view when the elements are strings
  [[nodiscard]] nvtext_amd_list_strings_column c_list_strings_view() const
  {
    nvtext_amd_list_strings_column c{};
    c.null_mask  = null_mask();
    c.size       = size();
    c.offset     = offset();
    c.null_count = null_count();
    if (num_children() > 1) {
      CUDF_EXPECTS(offsets().type().id() == type_id::INT32, "list offsets must be INT32");
      c.offsets = offsets().head<int32_t>();
      c.child   = strings_column_view(child()).c_view();
    } else {
      CUDF_EXPECTS(size() == 0, "a lists column with rows needs offsets and a child");
    }
    return c;
  }
};

}  // namespace cudf

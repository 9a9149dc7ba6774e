// nvtext::jaccard_index with the reference's signature (cpp/include/nvtext/jaccard.hpp:66-71), implemented over the
// C ABI in include/nvtext_amd.h.
#pragma once
#include <cudf/strings/strings_column_view.hpp>
#include <nvtext/detail_result.hpp>

namespace nvtext {

/**
 * Jaccard similarity of corresponding rows: the sets are the hashed `width`-character windows of each row,
 * output[row] = |A n B| / |A u B| as FLOAT32.  A row that is null in either input is null in the output.
 * Throws std::invalid_argument if width < 2 or the columns differ in size.
 */
inline std::unique_ptr<cudf::column> jaccard_index(cudf::strings_column_view const& input1, cudf::strings_column_view const& input2,
                                                   cudf::size_type width, cuda::stream_ref stream = cudf::get_default_stream(),
                                                   rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_strings_column const c1 = input1.c_view();
  nvtext_amd_strings_column const c2 = input2.c_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_fixed_column out{};
  detail::throw_on_error(nvtext_amd_jaccard_index(&c1, &c2, width, stream.get(), mr.c_allocator(storage), &out));
  return detail::make_fixed_result(out, stream, mr);
}

}  // namespace nvtext

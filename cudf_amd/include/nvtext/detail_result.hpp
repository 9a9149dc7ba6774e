// Shared by the nvtext entry points: status -> exception, C-ABI result -> cudf::column.
#pragma once
#include <cudf/column/column.hpp>
#include <cudf/utilities/error.hpp>

#include <new>
#include <stdexcept>
#include <string>

namespace nvtext::detail {

// cpp/include/cudf/utilities/error.hpp: the exception types of the reference's surface
inline void throw_on_error(nvtext_amd_status st)
{
  if (st == NVTEXT_AMD_SUCCESS) return;
  std::string const msg = nvtext_amd_last_error();
  switch (st) {
    case NVTEXT_AMD_INVALID_ARGUMENT: throw std::invalid_argument(msg);
    case NVTEXT_AMD_OVERFLOW: throw std::overflow_error(msg);
    case NVTEXT_AMD_LOGIC_ERROR: throw cudf::logic_error(msg);
    case NVTEXT_AMD_ALLOC_FAILED: throw std::bad_alloc();
    default: throw cudf::cuda_error(msg);
  }
}

// cudf::make_lists_column (cpp/src/lists/lists_column_factories.cu:106-129): LIST parent without data,
// children [offsets INT32, child].
inline std::unique_ptr<cudf::column> make_list_result(nvtext_amd_list_column const& r, cuda::stream_ref stream,
                                                      rmm::device_async_resource_ref mr)
{
  using namespace cudf;
  auto offsets = std::make_unique<column>(data_type{type_id::INT32}, r.offsets_size,
                                          device_buffer{r.offsets, r.offsets_bytes, stream, mr}, device_buffer{}, 0);
  auto child   = std::make_unique<column>(data_type{static_cast<type_id>(r.child_type)}, static_cast<size_type>(r.child_size),
                                          device_buffer{r.child, r.child_bytes, stream, mr}, device_buffer{}, 0);
  std::vector<std::unique_ptr<column>> kids;
  kids.push_back(std::move(offsets));
  kids.push_back(std::move(child));
  return std::make_unique<column>(data_type{type_id::LIST}, r.size, device_buffer{},
                                  device_buffer{r.null_mask, r.null_mask_bytes, stream, mr}, r.null_count, std::move(kids));
}

// cudf::make_numeric_column with the null mask set afterwards (cpp/src/text/jaccard.cu:458-476)
inline std::unique_ptr<cudf::column> make_fixed_result(nvtext_amd_fixed_column const& r, cuda::stream_ref stream,
                                                       rmm::device_async_resource_ref mr)
{
  using namespace cudf;
  return std::make_unique<column>(data_type{static_cast<type_id>(r.type)}, r.size, device_buffer{r.data, r.data_bytes, stream, mr},
                                  device_buffer{r.null_mask, r.null_mask_bytes, stream, mr}, r.null_count);
}

}  // namespace nvtext::detail

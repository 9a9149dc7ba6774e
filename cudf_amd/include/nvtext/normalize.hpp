// nvtext::character_normalizer, create_character_normalizer and normalize_characters with the reference's
// signatures (cpp/include/nvtext/normalize.hpp:81-160), implemented over the C ABI in include/nvtext_amd.h.
#pragma once
#include <cudf/strings/strings_column_view.hpp>
#include <nvtext/detail_result.hpp>

namespace nvtext {

/** Holds the per-code-point tables and the special tokens on the device.  Immutable; reusable across calls. */
struct character_normalizer {
  /** Throws std::invalid_argument if special_tokens has nulls. */
  character_normalizer(bool do_lower_case, cudf::strings_column_view const& special_tokens, cuda::stream_ref stream = cudf::get_default_stream(),
                       rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref());
  ~character_normalizer();

  struct character_normalizer_impl;
  std::unique_ptr<character_normalizer_impl> _impl;
};

/** Owns the handle of the C ABI and, with it, the allocator struct that the handle's tables go back to. */
struct character_normalizer::character_normalizer_impl {
  nvtext_amd_allocator storage{};
  nvtext_amd_character_normalizer* handle{nullptr};
  character_normalizer_impl()                                            = default;
  character_normalizer_impl(character_normalizer_impl const&)            = delete;
  character_normalizer_impl& operator=(character_normalizer_impl const&) = delete;
  ~character_normalizer_impl() { nvtext_amd_character_normalizer_destroy(handle); }
};

inline character_normalizer::character_normalizer(bool do_lower_case, cudf::strings_column_view const& special_tokens, cuda::stream_ref stream,
                                                  rmm::device_async_resource_ref mr)
  : _impl(std::make_unique<character_normalizer_impl>())
{
  nvtext_amd_strings_column const c = special_tokens.c_view();
  detail::throw_on_error(
    nvtext_amd_character_normalizer_create(do_lower_case ? 1 : 0, &c, stream.get(), mr.c_allocator(_impl->storage), &_impl->handle));
}

// defined where character_normalizer_impl is complete, as the owner of a unique_ptr to it must be
inline character_normalizer::~character_normalizer() = default;

namespace detail {
// an empty STRING column view, the default of create_character_normalizer's special_tokens
inline cudf::strings_column_view no_special_tokens()
{
  return cudf::strings_column_view(cudf::column_view{cudf::data_type{cudf::type_id::STRING}, 0, nullptr, nullptr, 0});
}

// cudf::make_strings_column: STRING parent owning the chars, child[0] = INT32 (INT64 for large strings) offsets
inline std::unique_ptr<cudf::column> make_strings_result(nvtext_amd_strings_result const& r, cuda::stream_ref stream,
                                                         rmm::device_async_resource_ref mr)
{
  using namespace cudf;
  std::vector<std::unique_ptr<column>> kids;
  if (r.offsets_size > 0) {
    kids.push_back(std::make_unique<column>(data_type{r.offsets_is_int64 ? type_id::INT64 : type_id::INT32}, r.offsets_size, device_buffer{r.offsets, r.offsets_bytes, stream, mr},
                                            device_buffer{}, 0));
  }
  return std::make_unique<column>(data_type{type_id::STRING}, r.size, device_buffer{r.chars, r.chars_bytes, stream, mr},
                                  device_buffer{r.null_mask, r.null_mask_bytes, stream, mr}, r.null_count, std::move(kids));
}
}  // namespace detail

inline std::unique_ptr<character_normalizer> create_character_normalizer(
  bool do_lower_case, cudf::strings_column_view const& special_tokens = detail::no_special_tokens(),
  cuda::stream_ref stream = cudf::get_default_stream(), rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  return std::make_unique<character_normalizer>(do_lower_case, special_tokens, stream, mr);
}

/**
 * Normalizes the characters of every row for tokenizing: punctuation and CJK ideographs padded with spaces,
 * whitespace replaced by a space, control characters removed and, when the normalizer lower-cases, characters
 * lower-cased with their accents stripped.  The normalizer's special tokens keep their brackets and case.
 */
inline std::unique_ptr<cudf::column> normalize_characters(cudf::strings_column_view const& input, character_normalizer const& normalizer,
                                                          cuda::stream_ref stream           = cudf::get_default_stream(),
                                                          rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_strings_column const c = input.c_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_strings_result out{};
  detail::throw_on_error(nvtext_amd_normalize_characters(&c, normalizer._impl->handle, stream.get(), mr.c_allocator(storage), &out));
  return detail::make_strings_result(out, stream, mr);
}

}  // namespace nvtext

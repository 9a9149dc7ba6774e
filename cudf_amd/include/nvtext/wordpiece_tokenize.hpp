// nvtext::wordpiece_vocabulary, load_wordpiece_vocabulary and wordpiece_tokenize with the reference's
// signatures (cpp/include/nvtext/wordpiece_tokenize.hpp:26-111), implemented over the C ABI.
#pragma once
#include <cudf/strings/strings_column_view.hpp>
#include <nvtext/detail_result.hpp>

namespace nvtext {

/** Vocabulary object: token id = row index of the entry.  Immutable; may be shared by concurrent calls. */
struct wordpiece_vocabulary {
  /** Throws std::invalid_argument if `input` is empty or has nulls. */
  wordpiece_vocabulary(cudf::strings_column_view const& input, cuda::stream_ref stream = cudf::get_default_stream(),
                       rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref());
  ~wordpiece_vocabulary();

  struct wordpiece_vocabulary_impl;
  std::unique_ptr<wordpiece_vocabulary_impl> _impl;
};

/** Owns the handle of the C ABI and, with it, the allocator struct that the handle's tables go back to. */
struct wordpiece_vocabulary::wordpiece_vocabulary_impl {
  nvtext_amd_allocator storage{};
  nvtext_amd_wordpiece_vocabulary* handle{nullptr};
  wordpiece_vocabulary_impl()                                            = default;
  wordpiece_vocabulary_impl(wordpiece_vocabulary_impl const&)            = delete;
  wordpiece_vocabulary_impl& operator=(wordpiece_vocabulary_impl const&) = delete;
  ~wordpiece_vocabulary_impl() { nvtext_amd_wordpiece_vocabulary_destroy(handle); }
};

inline wordpiece_vocabulary::wordpiece_vocabulary(cudf::strings_column_view const& input, cuda::stream_ref stream,
                                                  rmm::device_async_resource_ref mr)
  : _impl(std::make_unique<wordpiece_vocabulary_impl>())
{
  nvtext_amd_strings_column const c = input.c_view();
  detail::throw_on_error(nvtext_amd_wordpiece_vocabulary_create(&c, stream.get(), mr.c_allocator(_impl->storage), &_impl->handle));
}

// defined where wordpiece_vocabulary_impl is complete, as the owner of a unique_ptr to it must be
inline wordpiece_vocabulary::~wordpiece_vocabulary() = default;

inline std::unique_ptr<wordpiece_vocabulary> load_wordpiece_vocabulary(
  cudf::strings_column_view const& input, cuda::stream_ref stream = cudf::get_default_stream(),
  rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  return std::make_unique<wordpiece_vocabulary>(input, stream, mr);
}

/**
 * Token ids of every row as LIST<INT32>.  max_words_per_row == 0 tokenizes every word; > 0 only the first
 * words of each row.  Throws std::invalid_argument if max_words_per_row < 0, std::overflow_error if the
 * tokens exceed the column size limit.
 */
inline std::unique_ptr<cudf::column> wordpiece_tokenize(cudf::strings_column_view const& input, wordpiece_vocabulary const& vocabulary,
                                                        cudf::size_type max_words_per_row = 0,
                                                        cuda::stream_ref stream           = cudf::get_default_stream(),
                                                        rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_strings_column const c = input.c_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_list_column out{};
  detail::throw_on_error(nvtext_amd_wordpiece_tokenize(&c, vocabulary._impl->handle, max_words_per_row, stream.get(), mr.c_allocator(storage), &out));
  return detail::make_list_result(out, stream, mr);
}

}  // namespace nvtext

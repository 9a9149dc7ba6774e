// nvtext::minhash / minhash64 / minhash_ngrams / minhash64_ngrams with the reference's signatures
// (cpp/include/nvtext/minhash.hpp:62-69, 109-116, 156-163, 203-210), implemented over the C ABI in include/nvtext_amd.h.
#pragma once
#include <cudf/lists/lists_column_view.hpp>
#include <cudf/strings/strings_column_view.hpp>
#include <cudf/utilities/span.hpp>
#include <nvtext/detail_result.hpp>

namespace nvtext {

/**
 * Minhash of every row: MurmurHash3_x86_32(seed) over each `width`-character window, permuted with
 * (hash * a + b) for every (a, b) pair, minimum per pair.  Returns LIST<UINT32>.
 * Throws std::invalid_argument if width < 2, if the parameters are empty or differ in size;
 * std::overflow_error if rows * parameters reaches the column size limit.
 */
inline std::unique_ptr<cudf::column> minhash(cudf::strings_column_view const& input, uint32_t seed,
                                             cudf::device_span<uint32_t const> parameter_a,
                                             cudf::device_span<uint32_t const> parameter_b, cudf::size_type width,
                                             cuda::stream_ref stream           = cudf::get_default_stream(),
                                             rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_strings_column const c = input.c_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_list_column out{};
  detail::throw_on_error(nvtext_amd_minhash(&c, seed, parameter_a.data(), parameter_b.data(), static_cast<int64_t>(parameter_a.size()),
                                            static_cast<int64_t>(parameter_b.size()), width, stream.get(), mr.c_allocator(storage), &out));
  return detail::make_list_result(out, stream, mr);
}

/** As minhash, with MurmurHash3_x64_128(seed) (first 64-bit word) and ((hash*a+b) mod 2^64) % (2^61-1). Returns LIST<UINT64>. */
inline std::unique_ptr<cudf::column> minhash64(cudf::strings_column_view const& input, uint64_t seed,
                                               cudf::device_span<uint64_t const> parameter_a,
                                               cudf::device_span<uint64_t const> parameter_b, cudf::size_type width,
                                               cuda::stream_ref stream           = cudf::get_default_stream(),
                                               rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_strings_column const c = input.c_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_list_column out{};
  detail::throw_on_error(nvtext_amd_minhash64(&c, seed, parameter_a.data(), parameter_b.data(), static_cast<int64_t>(parameter_a.size()),
                                              static_cast<int64_t>(parameter_b.size()), width, stream.get(), mr.c_allocator(storage), &out));
  return detail::make_list_result(out, stream, mr);
}

/**
 * Minhash of every row of a LIST<STRING> column: MurmurHash3_x86_32(seed) over runs of consecutive strings of the row
 * (`ngrams` sets the run length), permuted and reduced as in minhash.  Returns LIST<UINT32>.
 * Throws std::invalid_argument if ngrams < 2, if the parameters are empty or differ in size;
 * std::overflow_error if rows * parameters reaches the column size limit.
 */
inline std::unique_ptr<cudf::column> minhash_ngrams(cudf::lists_column_view const& input, cudf::size_type ngrams, uint32_t seed,
                                                    cudf::device_span<uint32_t const> parameter_a,
                                                    cudf::device_span<uint32_t const> parameter_b,
                                                    cuda::stream_ref stream           = cudf::get_default_stream(),
                                                    rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_list_strings_column const c = input.c_list_strings_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_list_column out{};
  detail::throw_on_error(nvtext_amd_minhash_ngrams(&c, ngrams, seed, parameter_a.data(), parameter_b.data(),
                                                   static_cast<int64_t>(parameter_a.size()), static_cast<int64_t>(parameter_b.size()),
                                                   stream.get(), mr.c_allocator(storage), &out));
  return detail::make_list_result(out, stream, mr);
}

/** As minhash_ngrams, with MurmurHash3_x64_128(seed) (first 64-bit word) and the minhash64 permutation. Returns LIST<UINT64>. */
inline std::unique_ptr<cudf::column> minhash64_ngrams(cudf::lists_column_view const& input, cudf::size_type ngrams, uint64_t seed,
                                                      cudf::device_span<uint64_t const> parameter_a,
                                                      cudf::device_span<uint64_t const> parameter_b,
                                                      cuda::stream_ref stream           = cudf::get_default_stream(),
                                                      rmm::device_async_resource_ref mr = cudf::get_current_device_resource_ref())
{
  nvtext_amd_list_strings_column const c = input.c_list_strings_view();
  nvtext_amd_allocator storage{};
  nvtext_amd_list_column out{};
  detail::throw_on_error(nvtext_amd_minhash64_ngrams(&c, ngrams, seed, parameter_a.data(), parameter_b.data(),
                                                     static_cast<int64_t>(parameter_a.size()), static_cast<int64_t>(parameter_b.size()),
                                                     stream.get(), mr.c_allocator(storage), &out));
  return detail::make_list_result(out, stream, mr);
}

}  // namespace nvtext

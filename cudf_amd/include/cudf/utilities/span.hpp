// cudf::device_span (cpp/include/cudf/utilities/span.hpp:300): pointer + element count over device memory.
#pragma once
#include <cstddef>

namespace cudf {

template <typename T>
class device_span {
 public:
  constexpr device_span() noexcept = default;
  constexpr device_span(T* data, std::size_t size) noexcept : _data{data}, _size{size} {}
  [[nodiscard]] constexpr T* data() const noexcept { return _data; }
  [[nodiscard]] constexpr std::size_t size() const noexcept { return _size; }
  [[nodiscard]] constexpr bool empty() const noexcept { return _size == 0; }

 private:
  T* _data{nullptr};
  std::size_t _size{0};
};

}  // namespace cudf

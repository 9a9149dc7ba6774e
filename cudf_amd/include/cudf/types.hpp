// Minimal restatement of the libcudf vocabulary types that appear in the nvtext signatures
// (cpp/include/cudf/types.hpp:76-80 size_type / bitmask_type, :185-217 type_id, :230-290 data_type).
#pragma once
#include <cstdint>

namespace cudf {

using size_type    = int32_t;
using bitmask_type = uint32_t;

enum class type_id : int32_t {
  EMPTY, INT8, INT16, INT32, INT64, UINT8, UINT16, UINT32, UINT64, FLOAT32, FLOAT64, BOOL8,
  TIMESTAMP_DAYS, TIMESTAMP_SECONDS, TIMESTAMP_MILLISECONDS, TIMESTAMP_MICROSECONDS, TIMESTAMP_NANOSECONDS,
  DURATION_DAYS, DURATION_SECONDS, DURATION_MILLISECONDS, DURATION_MICROSECONDS, DURATION_NANOSECONDS,
  DICTIONARY32, STRING, LIST, DECIMAL32, DECIMAL64, DECIMAL128, STRUCT, NUM_TYPE_IDS
};

class data_type {
 public:
  data_type() = default;
  explicit constexpr data_type(type_id id) : _id{id} {}
  [[nodiscard]] constexpr type_id id() const noexcept { return _id; }
  constexpr bool operator==(data_type const& o) const noexcept { return _id == o._id; }
  constexpr bool operator!=(data_type const& o) const noexcept { return _id != o._id; }

 private:
  type_id _id{type_id::EMPTY};
};

template <typename T> constexpr type_id type_to_id() { return type_id::EMPTY; }
template <> constexpr type_id type_to_id<int32_t>() { return type_id::INT32; }
template <> constexpr type_id type_to_id<int64_t>() { return type_id::INT64; }
template <> constexpr type_id type_to_id<uint32_t>() { return type_id::UINT32; }
template <> constexpr type_id type_to_id<uint64_t>() { return type_id::UINT64; }
template <> constexpr type_id type_to_id<uint8_t>() { return type_id::UINT8; }

constexpr std::size_t size_of(data_type t)
{
  switch (t.id()) {
    case type_id::INT8: case type_id::UINT8: case type_id::BOOL8: return 1;
    case type_id::INT16: case type_id::UINT16: return 2;
    case type_id::INT32: case type_id::UINT32: case type_id::FLOAT32: return 4;
    case type_id::INT64: case type_id::UINT64: case type_id::FLOAT64: return 8;
    default: return 0;
  }
}

}  // namespace cudf

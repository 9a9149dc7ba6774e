// Exception types of the nvtext surface (cpp/include/cudf/utilities/error.hpp:35-103, 182-199, 280-284).
#pragma once
#include <stdexcept>
#include <string>

namespace cudf {

struct logic_error : public std::logic_error {
  using std::logic_error::logic_error;
};

// Device runtime failure (the reference's cudf::cuda_error; the runtime here is HIP).
struct cuda_error : public std::runtime_error {
  using std::runtime_error::runtime_error;
};

}  // namespace cudf

#define CUDF_EXPECTS_3(cond, reason, exception_type) \
  do {                                               \
    if (!(cond)) throw exception_type{reason};       \
  } while (0)
#define CUDF_EXPECTS_2(cond, reason) CUDF_EXPECTS_3(cond, reason, cudf::logic_error)
#define CUDF_GET_EXPECTS(_1, _2, _3, NAME, ...) NAME
#define CUDF_EXPECTS(...) CUDF_GET_EXPECTS(__VA_ARGS__, CUDF_EXPECTS_3, CUDF_EXPECTS_2)(__VA_ARGS__)

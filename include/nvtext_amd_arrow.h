/* Arrow C Device Data Interface for the columns of nvtext_amd.h.
 *
 * Replaces, for the column types this library takes and returns, what a caller of the reference does with
 * cudf::from_arrow_device_column (cpp/include/cudf/interop.hpp:841-876: a non-owning view over an
 * ArrowDeviceArray, waiting on its sync_event) and cudf::to_arrow_device (cpp/include/cudf/interop.hpp:500-533:
 * the result's buffers move into an ArrowDeviceArray that the consumer releases).  Zero copies either way.
 *
 * The struct definitions below are the published Arrow ABI (arrow/c/abi.h), under the same include guards, so
 * this header can sit next to Arrow's own.
 */
#ifndef NVTEXT_AMD_ARROW_H
#define NVTEXT_AMD_ARROW_H

#include "nvtext_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

#ifndef ARROW_C_DATA_INTERFACE
#define ARROW_C_DATA_INTERFACE

#define ARROW_FLAG_DICTIONARY_ORDERED 1
#define ARROW_FLAG_NULLABLE 2
#define ARROW_FLAG_MAP_KEYS_SORTED 4

struct ArrowSchema {
  const char* format;
  const char* name;
  const char* metadata;
  int64_t flags;
  int64_t n_children;
  struct ArrowSchema** children;
  struct ArrowSchema* dictionary;
  void (*release)(struct ArrowSchema*);
  void* private_data;
};

struct ArrowArray {
  int64_t length;
  int64_t null_count;
  int64_t offset;
  int64_t n_buffers;
  int64_t n_children;
  const void** buffers;
  struct ArrowArray** children;
  struct ArrowArray* dictionary;
  void (*release)(struct ArrowArray*);
  void* private_data;
};

#endif /* ARROW_C_DATA_INTERFACE */

#ifndef ARROW_C_DEVICE_DATA_INTERFACE
#define ARROW_C_DEVICE_DATA_INTERFACE

typedef int32_t ArrowDeviceType;
#define ARROW_DEVICE_CPU 1
#define ARROW_DEVICE_CUDA 2
#define ARROW_DEVICE_CUDA_HOST 3
#define ARROW_DEVICE_ROCM 10
#define ARROW_DEVICE_ROCM_HOST 11

struct ArrowDeviceArray {
  struct ArrowArray array;
  int64_t device_id;
  ArrowDeviceType device_type;
  void* sync_event; /* for ARROW_DEVICE_ROCM: hipEvent_t* or NULL */
  int64_t reserved[3];
};

#endif /* ARROW_C_DEVICE_DATA_INTERFACE */

/* Non-owning view of an Arrow utf8 ("u") or large_utf8 ("U") device array as a strings column
 * (from_arrow_device_column, cpp/include/cudf/interop.hpp:841-876).  The array must stay alive while the view
 * is used.  device_type must be ARROW_DEVICE_ROCM or ARROW_DEVICE_ROCM_HOST (INVALID_ARGUMENT otherwise);
 * a length above INT32_MAX gives OVERFLOW.  If sync_event is set, `stream` waits on it (no host wait).
 * An unknown null count (-1) is counted on the device, which synchronises `stream` once. */
nvtext_amd_status nvtext_amd_strings_from_arrow_device(const struct ArrowSchema* schema,
                                                       const struct ArrowDeviceArray* input,
                                                       void* stream,
                                                       nvtext_amd_strings_column* out);

/* As above for a list ("+l") of utf8 / large_utf8: the input of nvtext_amd_minhash_ngrams. */
nvtext_amd_status nvtext_amd_list_strings_from_arrow_device(const struct ArrowSchema* schema,
                                                            const struct ArrowDeviceArray* input,
                                                            void* stream,
                                                            nvtext_amd_list_strings_column* out);

/* Moves a LIST result into an ArrowDeviceArray + ArrowSchema (to_arrow_device, cpp/include/cudf/interop.hpp:529-533):
 * format "+l" with one child "element" of "I" (uint32), "L" (uint64) or "i" (int32), device_type ARROW_DEVICE_ROCM,
 * sync_event = an event recorded on `stream` after the producing work.  `col` is emptied; the buffers are
 * returned to `mr` (which must outlive the array, together with its ctx) when the consumer calls
 * out_array->array.release.  out_schema is released separately by its consumer. */
nvtext_amd_status nvtext_amd_list_to_arrow_device(nvtext_amd_list_column* col,
                                                  void* stream,
                                                  const nvtext_amd_allocator* mr,
                                                  struct ArrowSchema* out_schema,
                                                  struct ArrowDeviceArray* out_array);

/* As above for a fixed-width result ("f" for FLOAT32). */
nvtext_amd_status nvtext_amd_fixed_to_arrow_device(nvtext_amd_fixed_column* col,
                                                   void* stream,
                                                   const nvtext_amd_allocator* mr,
                                                   struct ArrowSchema* out_schema,
                                                   struct ArrowDeviceArray* out_array);

/* As above for a strings result: "u" (utf8, int32 offsets) or "U" (large_utf8, int64 offsets), buffers
 * [validity, offsets, data].  An empty result gets the single offset an Arrow string array of length 0 holds. */
nvtext_amd_status nvtext_amd_strings_to_arrow_device(nvtext_amd_strings_result* col,
                                                     void* stream,
                                                     const nvtext_amd_allocator* mr,
                                                     struct ArrowSchema* out_schema,
                                                     struct ArrowDeviceArray* out_array);

#ifdef __cplusplus
}
#endif

#endif /* NVTEXT_AMD_ARROW_H */

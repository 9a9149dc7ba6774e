// Arrow C Device Data Interface adaptors for the column structs of the C ABI: zero-copy views of incoming
// ArrowDeviceArrays and hand-over of result buffers to outgoing ones.
#include "common.cuh"

#include "../../include/nvtext_amd_arrow.h"

#include <cstdlib>
#include <cstring>
#include <limits>

namespace nvtext_amd {
namespace {

// Zero bits among `bits` bits of `mask` starting at bit `begin`, added to *zeros.
__global__ void count_unset_bits_kernel(const uint32_t* __restrict__ mask, int64_t begin, int64_t bits, uint32_t* __restrict__ zeros)
{
  int64_t const stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  uint32_t mine        = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < bits; i += stride) {
    int64_t const b = begin + i;
    mine += ((mask[b >> 5] >> (b & 31)) & 1u) ^ 1u;
  }
  uint32_t const total = wave_bcast(wave_inclusive_scan(mine), kWave - 1);
  if (lane_id() == 0 && total) atomicAdd(zeros, total);
}

bool on_this_kind_of_device(const ArrowDeviceArray* a) { return a->device_type == ARROW_DEVICE_ROCM || a->device_type == ARROW_DEVICE_ROCM_HOST; }

nvtext_amd_status wait_for_producer(const ArrowDeviceArray* a, hipStream_t stream)
{
  if (a->sync_event) {
    hipEvent_t const ev = *static_cast<hipEvent_t*>(a->sync_event);
    if (hipStreamWaitEvent(stream, ev, 0) != hipSuccess) return fail(NVTEXT_AMD_DEVICE_ERROR, "hipStreamWaitEvent on the array's sync_event failed");
  }
  return NVTEXT_AMD_SUCCESS;
}

// The true null count of an array whose producer left it unknown (-1).
nvtext_amd_status resolve_null_count(const ArrowArray& a, hipStream_t stream, int32_t* out)
{
  const void* validity = a.n_buffers > 0 ? a.buffers[0] : nullptr;
  if (!validity || a.null_count == 0 || a.length == 0) {
    *out = 0;
    return NVTEXT_AMD_SUCCESS;
  }
  if (a.null_count > 0) {
    *out = static_cast<int32_t>(a.null_count);
    return NVTEXT_AMD_SUCCESS;
  }
  uint32_t* d_zeros = nullptr;
  NVTEXT_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&d_zeros), sizeof(uint32_t), stream));
  launch_fill_u32(d_zeros, 0u, 1, stream);
  int64_t blocks = (a.length + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(count_unset_bits_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, static_cast<const uint32_t*>(validity), a.offset,
                     a.length, d_zeros);
  uint32_t zeros = 0;
  hipError_t e   = hipMemcpyAsync(&zeros, d_zeros, sizeof(zeros), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFreeAsync(d_zeros, stream);
  if (e != hipSuccess) return fail(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
  *out = static_cast<int32_t>(zeros);
  return NVTEXT_AMD_SUCCESS;
}

nvtext_amd_status strings_view(const ArrowSchema* schema, const ArrowArray& a, hipStream_t stream, nvtext_amd_strings_column* out)
{
  bool const large = std::strcmp(schema->format, "U") == 0;
  if (!large && std::strcmp(schema->format, "u") != 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "expected a utf8 (u) or large_utf8 (U) array");
  if (a.n_buffers != 3) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "a utf8 array has three buffers");
  if (a.length > std::numeric_limits<int32_t>::max() || a.offset > std::numeric_limits<int32_t>::max() - a.length)
    return fail(NVTEXT_AMD_OVERFLOW, "the array exceeds the column size limit");
  *out                  = nvtext_amd_strings_column{};
  out->null_mask        = static_cast<const uint32_t*>(a.buffers[0]);
  out->offsets          = a.buffers[1];
  out->offsets_is_int64 = large ? 1 : 0;
  out->chars            = static_cast<const char*>(a.buffers[2]);
  out->size             = static_cast<int32_t>(a.length);
  out->offset           = static_cast<int32_t>(a.offset);
  return resolve_null_count(a, stream, &out->null_count);
}

// ---- outgoing arrays: everything the release callbacks need lives in one heap block
struct Exported {
  nvtext_amd_allocator mr;
  bool has_mr;
  hipStream_t stream;
  hipEvent_t event;
  bool has_event;
  void* buffers_to_free[3];
  size_t bytes_to_free[3];
  const void* parent_buffers[3];
  const void* child_buffers[2];
  ArrowArray child;
  ArrowArray* children[1];
};

void release_child_array(ArrowArray* a) { a->release = nullptr; }

void release_exported_array(ArrowArray* a)
{
  if (!a || !a->release) return;
  auto* x = static_cast<Exported*>(a->private_data);
  Mr m{x->has_mr ? &x->mr : nullptr, x->stream};
  for (int i = 0; i < 3; ++i) m.deallocate(x->buffers_to_free[i], x->bytes_to_free[i]);
  if (x->has_event) (void)hipEventDestroy(x->event);
  if (a->n_children == 1 && x->child.release) x->child.release(&x->child);
  delete x;
  a->release = nullptr;
}

struct ExportedSchema {
  ArrowSchema child;
  ArrowSchema* children[1];
};

void release_child_schema(ArrowSchema* s) { s->release = nullptr; }

void release_exported_schema(ArrowSchema* s)
{
  if (!s || !s->release) return;
  auto* x = static_cast<ExportedSchema*>(s->private_data);
  if (s->n_children == 1 && x->child.release) x->child.release(&x->child);
  delete x;
  s->release = nullptr;
}

const char* format_of(int32_t type)
{
  switch (type) {
    case NVTEXT_AMD_TYPE_INT32: return "i";
    case NVTEXT_AMD_TYPE_UINT32: return "I";
    case NVTEXT_AMD_TYPE_UINT64: return "L";
    case NVTEXT_AMD_TYPE_FLOAT32: return "f";
    default: return nullptr;
  }
}

// Fills the device part of an outgoing array: current device, an event recorded on the stream.
nvtext_amd_status finish_device_array(Exported* x, hipStream_t stream, ArrowDeviceArray* out)
{
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return fail(NVTEXT_AMD_DEVICE_ERROR, "hipGetDevice failed");
  if (hipEventCreateWithFlags(&x->event, hipEventDisableTiming) != hipSuccess) return fail(NVTEXT_AMD_DEVICE_ERROR, "hipEventCreate failed");
  x->has_event = true;
  if (hipEventRecord(x->event, stream) != hipSuccess) return fail(NVTEXT_AMD_DEVICE_ERROR, "hipEventRecord failed");
  out->device_id   = device;
  out->device_type = ARROW_DEVICE_ROCM;
  out->sync_event  = &x->event;
  std::memset(out->reserved, 0, sizeof(out->reserved));
  return NVTEXT_AMD_SUCCESS;
}

Exported* new_exported(void* stream, const nvtext_amd_allocator* mr)
{
  auto* x = new Exported{};
  if (mr) x->mr = *mr;
  x->has_mr = mr != nullptr;
  x->stream = static_cast<hipStream_t>(stream);
  return x;
}

}  // namespace
}  // namespace nvtext_amd

extern "C" {

nvtext_amd_status nvtext_amd_strings_from_arrow_device(const ArrowSchema* schema, const ArrowDeviceArray* input, void* stream_,
                                                       nvtext_amd_strings_column* out)
{
  using namespace nvtext_amd;
  if (!schema || !input || !out || !schema->format) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  if (!on_this_kind_of_device(input)) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "the array is not in ROCm device or pinned host memory");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  nvtext_amd_status st = wait_for_producer(input, stream);
  if (st != NVTEXT_AMD_SUCCESS) return st;
  return strings_view(schema, input->array, stream, out);
}

nvtext_amd_status nvtext_amd_list_strings_from_arrow_device(const ArrowSchema* schema, const ArrowDeviceArray* input, void* stream_,
                                                            nvtext_amd_list_strings_column* out)
{
  using namespace nvtext_amd;
  if (!schema || !input || !out || !schema->format) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  if (!on_this_kind_of_device(input)) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "the array is not in ROCm device or pinned host memory");
  if (std::strcmp(schema->format, "+l") != 0 || schema->n_children != 1 || input->array.n_children != 1 || input->array.n_buffers != 2)
    return fail(NVTEXT_AMD_INVALID_ARGUMENT, "expected a list (+l) array with one child");
  ArrowArray const& a = input->array;
  if (a.length > std::numeric_limits<int32_t>::max() || a.offset > std::numeric_limits<int32_t>::max() - a.length)
    return fail(NVTEXT_AMD_OVERFLOW, "the array exceeds the column size limit");
  hipStream_t stream   = static_cast<hipStream_t>(stream_);
  nvtext_amd_status st = wait_for_producer(input, stream);
  if (st != NVTEXT_AMD_SUCCESS) return st;
  *out           = nvtext_amd_list_strings_column{};
  out->null_mask = static_cast<const uint32_t*>(a.buffers[0]);
  out->offsets   = static_cast<const int32_t*>(a.buffers[1]);
  out->size      = static_cast<int32_t>(a.length);
  out->offset    = static_cast<int32_t>(a.offset);
  st             = resolve_null_count(a, stream, &out->null_count);
  if (st != NVTEXT_AMD_SUCCESS) return st;
  return strings_view(schema->children[0], *a.children[0], stream, &out->child);
}

nvtext_amd_status nvtext_amd_list_to_arrow_device(nvtext_amd_list_column* col, void* stream, const nvtext_amd_allocator* mr, ArrowSchema* out_schema,
                                                  ArrowDeviceArray* out_array)
{
  using namespace nvtext_amd;
  if (!col || !out_schema || !out_array) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  const char* child_format = format_of(col->child_type);
  if (!child_format) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "the column is not a list result of this library");

  Exported* x = new_exported(stream, mr);
  nvtext_amd_status st = finish_device_array(x, x->stream, out_array);
  if (st != NVTEXT_AMD_SUCCESS) {
    if (x->has_event) (void)hipEventDestroy(x->event);
    delete x;
    return st;
  }
  x->buffers_to_free[0] = col->offsets;
  x->bytes_to_free[0]   = col->offsets_bytes;
  x->buffers_to_free[1] = col->child;
  x->bytes_to_free[1]   = col->child_bytes;
  x->buffers_to_free[2] = col->null_mask;
  x->bytes_to_free[2]   = col->null_mask_bytes;
  x->parent_buffers[0]  = col->null_mask;
  x->parent_buffers[1]  = col->offsets;
  x->child_buffers[0]   = nullptr;
  x->child_buffers[1]   = col->child;
  x->child              = ArrowArray{col->child_size, 0, 0, 2, 0, x->child_buffers, nullptr, nullptr, release_child_array, nullptr};
  x->children[0]        = &x->child;
  out_array->array      = ArrowArray{col->size, col->null_count, 0, 2, 1, x->parent_buffers, x->children, nullptr, release_exported_array, x};

  auto* s        = new ExportedSchema{};
  s->child       = ArrowSchema{child_format, "element", nullptr, 0, 0, nullptr, nullptr, release_child_schema, nullptr};
  s->children[0] = &s->child;
  *out_schema    = ArrowSchema{"+l", "", nullptr, col->null_mask ? ARROW_FLAG_NULLABLE : 0, 1, s->children, nullptr, release_exported_schema, s};
  std::memset(col, 0, sizeof(*col));
  return NVTEXT_AMD_SUCCESS;
}

nvtext_amd_status nvtext_amd_fixed_to_arrow_device(nvtext_amd_fixed_column* col, void* stream, const nvtext_amd_allocator* mr, ArrowSchema* out_schema,
                                                   ArrowDeviceArray* out_array)
{
  using namespace nvtext_amd;
  if (!col || !out_schema || !out_array) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  const char* format = format_of(col->type);
  if (!format) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "the column is not a fixed-width result of this library");
  Exported* x = new_exported(stream, mr);
  nvtext_amd_status st = finish_device_array(x, x->stream, out_array);
  if (st != NVTEXT_AMD_SUCCESS) {
    if (x->has_event) (void)hipEventDestroy(x->event);
    delete x;
    return st;
  }
  x->buffers_to_free[0] = col->data;
  x->bytes_to_free[0]   = col->data_bytes;
  x->buffers_to_free[1] = col->null_mask;
  x->bytes_to_free[1]   = col->null_mask_bytes;
  x->parent_buffers[0]  = col->null_mask;
  x->parent_buffers[1]  = col->data;
  out_array->array      = ArrowArray{col->size, col->null_count, 0, 2, 0, x->parent_buffers, nullptr, nullptr, release_exported_array, x};
  auto* s               = new ExportedSchema{};
  *out_schema = ArrowSchema{format, "", nullptr, col->null_mask ? ARROW_FLAG_NULLABLE : 0, 0, nullptr, nullptr, release_exported_schema, s};
  *col        = nvtext_amd_fixed_column{};
  return NVTEXT_AMD_SUCCESS;
}

nvtext_amd_status nvtext_amd_strings_to_arrow_device(nvtext_amd_strings_result* col, void* stream, const nvtext_amd_allocator* mr,
                                                     ArrowSchema* out_schema, ArrowDeviceArray* out_array)
{
  using namespace nvtext_amd;
  if (!col || !out_schema || !out_array) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  Exported* x = new_exported(stream, mr);
  auto give_up = [&](nvtext_amd_status st) {
    if (x->has_event) (void)hipEventDestroy(x->event);
    delete x;
    return st;
  };
  if (col->size == 0 && !col->offsets) {
    // the canonical empty column has no offsets child; an Arrow string array holds length + 1 of them
    Mr m{mr, x->stream};
    col->offsets_bytes    = sizeof(int32_t);
    col->offsets          = m.allocate(col->offsets_bytes);
    col->offsets_is_int64 = 0;
    if (!col->offsets) return give_up(fail(NVTEXT_AMD_ALLOC_FAILED, "offsets allocation failed"));
    launch_fill_u32(static_cast<uint32_t*>(col->offsets), 0u, 1, x->stream);
  }
  nvtext_amd_status st = finish_device_array(x, x->stream, out_array);
  if (st != NVTEXT_AMD_SUCCESS) return give_up(st);
  x->buffers_to_free[0] = col->offsets;
  x->bytes_to_free[0]   = col->offsets_bytes;
  x->buffers_to_free[1] = col->chars;
  x->bytes_to_free[1]   = col->chars_bytes;
  x->buffers_to_free[2] = col->null_mask;
  x->bytes_to_free[2]   = col->null_mask_bytes;
  x->parent_buffers[0]  = col->null_mask;
  x->parent_buffers[1]  = col->offsets;
  x->parent_buffers[2]  = col->chars;
  out_array->array      = ArrowArray{col->size, col->null_count, 0, 3, 0, x->parent_buffers, nullptr, nullptr, release_exported_array, x};
  auto* s               = new ExportedSchema{};
  *out_schema = ArrowSchema{col->offsets_is_int64 ? "U" : "u", "", nullptr, col->null_mask ? ARROW_FLAG_NULLABLE : 0, 0, nullptr, nullptr,
                            release_exported_schema, s};
  *col        = nvtext_amd_strings_result{};
  return NVTEXT_AMD_SUCCESS;
}

}  // extern "C"

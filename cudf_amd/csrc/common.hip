// Host-side plumbing shared by the entry points: status text, allocator adaptor,
// bitmask copy, fills, the middle stage of the device-wide scan and the small
// C-ABI utilities (version, last error, result release).
#include "common.cuh"

#include <cstring>
#include <mutex>
#include <vector>

#include <dlfcn.h>

namespace nvtext_amd {

namespace {
thread_local std::string g_last_error;

struct ProfileRecord {
  const char* name;
  hipEvent_t begin;
  hipEvent_t end;
};
bool g_profile_on   = false;
bool g_profile_open = false;  // the last profile_mark_begin made a record
std::vector<ProfileRecord> g_profile;
}  // namespace

bool profiling_on() { return g_profile_on; }

void profile_mark_begin(const char* name, hipStream_t stream)
{
  ProfileRecord r{name, nullptr, nullptr};
  g_profile_open = false;
  if (hipEventCreate(&r.begin) != hipSuccess) return;
  if (hipEventCreate(&r.end) != hipSuccess) {
    (void)hipEventDestroy(r.begin);
    return;
  }
  (void)hipEventRecord(r.begin, stream);
  g_profile.push_back(r);
  g_profile_open = true;
}

void profile_mark_end(hipStream_t stream)
{
  // only the record that the matching begin made: a begin that failed leaves nothing to close
  if (g_profile_open) (void)hipEventRecord(g_profile.back().end, stream);
  g_profile_open = false;
}

namespace {
using RangePushFn = int (*)(const char*);
using RangePopFn  = int (*)();
RangePushFn g_range_push = nullptr;
RangePopFn g_range_pop   = nullptr;
std::once_flag g_range_once;
void find_marker_library()
{
  // rocprofv3 listens to the first; the second is the older tracer's
  for (const char* lib : {"librocprofiler-sdk-roctx.so.1", "libroctx64.so.4"}) {
    void* const h = dlopen(lib, RTLD_NOW | RTLD_LOCAL);
    if (!h) continue;
    auto const push = reinterpret_cast<RangePushFn>(dlsym(h, "roctxRangePushA"));
    auto const pop  = reinterpret_cast<RangePopFn>(dlsym(h, "roctxRangePop"));
    if (push && pop) {
      g_range_push = push;
      g_range_pop  = pop;
      return;
    }
  }
}
}  // namespace

EntryScope::EntryScope(const char* name)
{
  (void)hipGetLastError();
  std::call_once(g_range_once, find_marker_library);
  if (g_range_push) (void)g_range_push(name);
}

EntryScope::~EntryScope()
{
  if (g_range_pop) (void)g_range_pop();
}

void set_last_error(const char* msg) { g_last_error = msg ? msg : ""; }

nvtext_amd_status fail(nvtext_amd_status st, const char* msg)
{
  set_last_error(msg);
  return st;
}

void* Mr::allocate(size_t bytes) const
{
  if (bytes == 0) return nullptr;
  if (a && a->allocate) return a->allocate(a->ctx, bytes, stream);
  void* p = nullptr;
  if (hipMallocAsync(&p, bytes, stream) != hipSuccess) return nullptr;
  return p;
}

void Mr::deallocate(void* p, size_t bytes) const
{
  if (!p) return;
  if (a && a->deallocate) {
    a->deallocate(a->ctx, p, bytes, stream);
    return;
  }
  (void)hipFreeAsync(p, stream);
}

__global__ void __launch_bounds__(kScanThreads) scan_tile_offsets_kernel(uint64_t* tile_sums, int64_t ntiles)
{
  __shared__ uint64_t lds[kScanThreads / kWave + 1];
  uint64_t carry = 0;
  for (int64_t base = 0; base < ntiles; base += kScanThreads) {
    int64_t const i  = base + threadIdx.x;
    uint64_t const v = (i < ntiles) ? tile_sums[i] : 0;
    uint64_t total;
    uint64_t const ex = block_exclusive_scan64<kScanThreads>(v, lds, &total);
    if (i < ntiles) tile_sums[i] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) tile_sums[ntiles] = carry;
}

namespace {
__global__ void copy_bitmask_kernel(uint32_t* dst, const uint32_t* src, int32_t begin_bit, int32_t bits, int32_t words)
{
  int32_t const w = blockIdx.x * blockDim.x + threadIdx.x;
  if (w >= words) return;
  int64_t const first = static_cast<int64_t>(begin_bit) + static_cast<int64_t>(w) * 32;
  int64_t const sw    = first >> 5;
  int const sh        = static_cast<int>(first & 31);
  int64_t const last_src_word = (static_cast<int64_t>(begin_bit) + bits - 1) >> 5;
  uint32_t v = src[sw] >> sh;
  if (sh != 0 && sw + 1 <= last_src_word) v |= src[sw + 1] << (32 - sh);
  int32_t const remaining = bits - w * 32;
  if (remaining < 32) v &= (1u << remaining) - 1u;
  dst[w] = v;
}

__global__ void fill_u32_kernel(uint32_t* dst, uint32_t value, int64_t count)
{
  int64_t const stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = value;
}
}  // namespace

namespace {
__global__ void read_two_offsets_kernel(const void* offsets, int is64, int64_t first_index, int64_t last_index, uint64_t* dst)
{
  int64_t const i = threadIdx.x == 0 ? first_index : last_index;
  dst[threadIdx.x] = static_cast<uint64_t>(is64 ? static_cast<const int64_t*>(offsets)[i] : static_cast<int64_t>(static_cast<const int32_t*>(offsets)[i]));
}
}  // namespace

uint64_t* host_scalars()
{
  struct Slot {
    uint64_t* p = nullptr;
    bool tried  = false;
  };
  thread_local Slot slot;
  if (!slot.tried) {
    slot.tried = true;
    void* p    = nullptr;
    // portable: usable whichever device the thread has current at a later call
    if (hipHostMalloc(&p, kHostScalarBytes, hipHostMallocPortable) == hipSuccess) slot.p = static_cast<uint64_t*>(p);
    else (void)hipGetLastError();
  }
  return slot.p;
}

void launch_read_two_offsets(const void* offsets, int is64, int64_t first_index, int64_t last_index, uint64_t* dst, hipStream_t stream)
{
  hipLaunchKernelGGL(read_two_offsets_kernel, dim3(1), dim3(2), 0, stream, offsets, is64, first_index, last_index, dst);
}

void launch_copy_bitmask(uint32_t* dst, const uint32_t* src, int32_t begin_bit, int32_t bits, hipStream_t stream)
{
  int32_t const words = (bits + 31) / 32;
  if (words == 0) return;
  hipLaunchKernelGGL(copy_bitmask_kernel, dim3((words + 255) / 256), dim3(256), 0, stream, dst, src, begin_bit, bits, words);
}

void launch_fill_u32(uint32_t* dst, uint32_t value, int64_t count, hipStream_t stream)
{
  if (count <= 0) return;
  int64_t blocks = (count + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, dst, value, count);
}

}  // namespace nvtext_amd

extern "C" {

int32_t nvtext_amd_version(void) { return 100; }

void nvtext_amd_profile_enable(int32_t on)
{
  nvtext_amd::g_profile_on = on != 0;
}

int32_t nvtext_amd_profile_read(const char** names, float* milliseconds, int32_t capacity)
{
  int32_t n = 0;
  for (auto& r : nvtext_amd::g_profile) {
    float ms = 0.f;
    if (r.begin && r.end && hipEventSynchronize(r.end) == hipSuccess && hipEventElapsedTime(&ms, r.begin, r.end) == hipSuccess &&
        n < capacity) {
      names[n]        = r.name;
      milliseconds[n] = ms;
      ++n;
    }
    if (r.begin) (void)hipEventDestroy(r.begin);
    if (r.end) (void)hipEventDestroy(r.end);
  }
  nvtext_amd::g_profile.clear();
  return n;
}

const char* nvtext_amd_last_error(void) { return nvtext_amd::g_last_error.c_str(); }

void nvtext_amd_list_column_free(nvtext_amd_list_column* col, void* stream, const nvtext_amd_allocator* mr)
{
  if (!col) return;
  nvtext_amd::Mr m{mr, static_cast<hipStream_t>(stream)};
  m.deallocate(col->offsets, col->offsets_bytes);
  m.deallocate(col->child, col->child_bytes);
  m.deallocate(col->null_mask, col->null_mask_bytes);
  std::memset(col, 0, sizeof(*col));
}

}  // extern "C"

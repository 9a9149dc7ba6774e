// Shared host/device helpers for the gfx950 nvtext kernels: status reporting,
// stream-ordered temporaries, the device view of an Arrow strings column,
// wavefront (64-lane) DPP scans, workgroup scans and a device-wide exclusive scan.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <utility>
#include <vector>

#include "../../include/nvtext_amd.h"
#include "../../include/nvtext_amd_profile.h"

namespace nvtext_amd {

constexpr int kWave = 64;

// ------------------------------------------------------------------ status
void set_last_error(const char* msg);
nvtext_amd_status fail(nvtext_amd_status st, const char* msg);
// What every entry point does first.  (1) hipGetLastError keeps the last error of the calling thread until somebody
// reads it, whoever made the failing call (a device query of another library, long before): it is read away before the
// entry point's own launches, which are checked with the same call, so that it reports no error but its own.  (2) A
// named range around the call, as CUDF_FUNC_RANGE() puts an NVTX range around the reference's entry points
// (cpp/include/cudf/detail/nvtx/ranges.hpp; wordpiece_tokenize.cu:291,897, minhash.cu:699,724): rocprofv3
// --marker-trace shows it.  The marker library (rocTX) is looked up at first use and left alone when it is absent;
// the library does not link it.
struct EntryScope {
  explicit EntryScope(const char* name);
  ~EntryScope();
  EntryScope(const EntryScope&)            = delete;
  EntryScope& operator=(const EntryScope&) = delete;
};

#define NVTEXT_HIP_TRY(expr)                                                          \
  do {                                                                                \
    hipError_t _e = (expr);                                                           \
    if (_e != hipSuccess) {                                                           \
      std::string _m = std::string(#expr) + ": " + hipGetErrorString(_e);             \
      return ::nvtext_amd::fail(NVTEXT_AMD_DEVICE_ERROR, _m.c_str());                 \
    }                                                                                 \
  } while (0)

// The same once the result has buffers: `release` hands them back before the error is returned.
#define NVTEXT_HIP_TRY_OR(expr, release)                                              \
  do {                                                                                \
    hipError_t _e = (expr);                                                           \
    if (_e != hipSuccess) {                                                           \
      release;                                                                        \
      std::string _m = std::string(#expr) + ": " + hipGetErrorString(_e);             \
      return ::nvtext_amd::fail(NVTEXT_AMD_DEVICE_ERROR, _m.c_str());                 \
    }                                                                                 \
  } while (0)

// ------------------------------------------------------------------ kernel timing (benchmarks)
bool profiling_on();
void profile_mark_begin(const char* name, hipStream_t stream);
void profile_mark_end(hipStream_t stream);

// Brackets one kernel launch with HIP events when profiling is enabled.
struct ProfileScope {
  hipStream_t stream;
  bool on;
  ProfileScope(const char* name, hipStream_t s) : stream(s), on(profiling_on())
  {
    if (on) profile_mark_begin(name, stream);
  }
  ~ProfileScope()
  {
    if (on) profile_mark_end(stream);
  }
};

// ------------------------------------------------------------------ memory
// Stream-ordered allocation through the caller's allocator (or hipMallocAsync).
struct Mr {
  const nvtext_amd_allocator* a;
  hipStream_t stream;
  void* allocate(size_t bytes) const;
  void deallocate(void* p, size_t bytes) const;
};

// Device memory that an object keeps for as long as it lives.  With an allocator it comes from there and goes back
// there on the stream of creation (a copy of the struct is kept: its ctx and that stream must outlive the object,
// as a memory resource must outlive what it allocated); without one it is plain hipMalloc / hipFree.
struct DeviceStore {
  nvtext_amd_allocator alloc{};
  bool has_alloc     = false;
  hipStream_t stream = nullptr;
  std::vector<std::pair<void*, size_t>> held;

  void bind(const nvtext_amd_allocator* a, hipStream_t s)
  {
    has_alloc = a && a->allocate && a->deallocate;
    if (has_alloc) alloc = *a;
    stream = s;
  }
  void* allocate(size_t bytes)
  {
    void* p = nullptr;
    if (has_alloc) {
      p = alloc.allocate(alloc.ctx, bytes, stream);
    } else if (hipMalloc(&p, bytes) != hipSuccess) {
      p = nullptr;
    }
    if (p) held.emplace_back(p, bytes);
    return p;
  }
  template <typename T>
  bool allocate(T** out, size_t count)
  {
    *out = static_cast<T*>(allocate(count * sizeof(T)));
    return *out != nullptr;
  }
  void release()
  {
    for (auto const& h : held) {
      if (has_alloc)
        alloc.deallocate(alloc.ctx, h.first, h.second, stream);
      else
        (void)hipFree(h.first);
    }
    held.clear();
  }
  DeviceStore() = default;
  ~DeviceStore() { release(); }
  DeviceStore(const DeviceStore&)            = delete;
  DeviceStore& operator=(const DeviceStore&) = delete;
};

// Temporary released (stream-ordered) when it goes out of scope.
struct Temp {
  Mr mr;
  void* ptr   = nullptr;
  size_t size = 0;
  Temp(Mr m, size_t bytes) : mr(m), size(bytes)
  {
    if (bytes) ptr = mr.allocate(bytes);
  }
  ~Temp()
  {
    if (ptr) mr.deallocate(ptr, size);
  }
  Temp(const Temp&)            = delete;
  Temp& operator=(const Temp&) = delete;
  bool ok() const { return size == 0 || ptr != nullptr; }
  template <typename T>
  T* as() const
  {
    return static_cast<T*>(ptr);
  }
};

// Several temporaries in ONE allocation (a call to the caller's allocator can cost tens of microseconds: from Python
// it is a callback into the interpreter), each part 256-byte aligned.
template <int N>
struct TempParts {
  size_t at[N + 1];
  Temp whole;
  static size_t total(const size_t (&bytes)[N])
  {
    size_t sum = 0;
    for (int i = 0; i < N; ++i) sum += (bytes[i] + 255) & ~static_cast<size_t>(255);
    return sum;
  }
  TempParts(Mr m, const size_t (&bytes)[N]) : whole(m, total(bytes))
  {
    at[0] = 0;
    for (int i = 0; i < N; ++i) at[i + 1] = at[i] + ((bytes[i] + 255) & ~static_cast<size_t>(255));
  }
  bool ok() const { return whole.ok(); }
  template <typename T>
  T* part(int i) const
  {
    return reinterpret_cast<T*>(static_cast<char*>(whole.ptr) + at[i]);
  }
};

inline size_t mask_alloc_bytes(int64_t bits)
{
  // libcudf pads bitmask allocations to 64 bytes (cpp/include/cudf/null_mask.hpp:56-57)
  size_t const bytes = static_cast<size_t>((bits + 7) / 8);
  return (bytes + 63) / 64 * 64;
}

// ------------------------------------------------------------------ column view on the device
struct ColView {
  const uint8_t* chars;
  const void* offsets;
  const uint32_t* mask;
  int32_t size;
  int32_t offset;
  int32_t is64;
  int32_t use_mask;  // 1 when validity must be consulted (mask present and null_count > 0)

  __device__ __forceinline__ int64_t off(int64_t i) const
  {
    return is64 ? static_cast<const int64_t*>(offsets)[i + offset]
                : static_cast<int64_t>(static_cast<const int32_t*>(offsets)[i + offset]);
  }
  __device__ __forceinline__ bool valid(int64_t i) const
  {
    if (!use_mask) return true;
    int64_t const b = i + offset;
    return (mask[b >> 5] >> (b & 31)) & 1u;
  }
};

inline ColView make_view(const nvtext_amd_strings_column& c)
{
  ColView v;
  v.chars    = reinterpret_cast<const uint8_t*>(c.chars);
  v.offsets  = c.offsets;
  v.mask     = c.null_mask;
  v.size     = c.size;
  v.offset   = c.offset;
  v.is64     = c.offsets_is_int64 ? 1 : 0;
  v.use_mask = (c.null_mask != nullptr && c.null_count > 0) ? 1 : 0;
  return v;
}

// ------------------------------------------------------------------ UTF-8
// cpp/include/cudf/strings/detail/utf8.hpp:23-27, 84-90
__device__ __forceinline__ bool is_utf8_continuation(uint32_t b) { return (b & 0xC0u) == 0x80u; }
__device__ __forceinline__ int bytes_in_utf8_byte(uint32_t b)
{
  return 1 + int((b & 0xF0u) == 0xF0u) + int((b & 0xE0u) == 0xE0u) + int((b & 0xC0u) == 0xC0u) -
         int((b & 0xC0u) == 0x80u);
}

// ------------------------------------------------------------------ wavefront primitives (wave64, DPP)
// Loads and stores for data that is touched once: the non-temporal hint lets the caches drop these lines
// first, so that tables which are probed again and again stay resident.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream(const uint4* p)
{
  u32x4_t const v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_stream(uint4* p, uint4 v)
{
  u32x4_t w;
  w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w;
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(p));
}
__device__ __forceinline__ uint32_t load_stream(const uint32_t* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_stream(uint32_t* p, uint32_t v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void store_stream(int32_t* p, int32_t v) { __builtin_nontemporal_store(v, p); }

__device__ __forceinline__ int lane_id() { return static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))); }

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_zero(uint32_t v)
{
  // lanes without a source (or masked-out rows) read 0
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, ROW_MASK, 0xf, false));
}

// Inclusive prefix sum across the 64 lanes: four row_shr steps inside each row of 16,
// then row_bcast:15 / row_bcast:31 carry the row totals forward.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v)
{
  v += dpp_zero<0x111, 0xf>(v);  // row_shr:1
  v += dpp_zero<0x112, 0xf>(v);  // row_shr:2
  v += dpp_zero<0x114, 0xf>(v);  // row_shr:4
  v += dpp_zero<0x118, 0xf>(v);  // row_shr:8
  v += dpp_zero<0x142, 0xa>(v);  // row_bcast:15 -> rows 1,3
  v += dpp_zero<0x143, 0xc>(v);  // row_bcast:31 -> rows 2,3
  return v;
}

__device__ __forceinline__ uint64_t wave_inclusive_scan64(uint64_t v)
{
#define NVTEXT_DPP64(CTRL, RM)                                                                  \
  {                                                                                             \
    uint32_t lo = dpp_zero<CTRL, RM>(static_cast<uint32_t>(v));                                 \
    uint32_t hi = dpp_zero<CTRL, RM>(static_cast<uint32_t>(v >> 32));                           \
    v += (static_cast<uint64_t>(hi) << 32) | lo;                                                \
  }
  NVTEXT_DPP64(0x111, 0xf)
  NVTEXT_DPP64(0x112, 0xf)
  NVTEXT_DPP64(0x114, 0xf)
  NVTEXT_DPP64(0x118, 0xf)
  NVTEXT_DPP64(0x142, 0xa)
  NVTEXT_DPP64(0x143, 0xc)
#undef NVTEXT_DPP64
  return v;
}

__device__ __forceinline__ uint32_t wave_bcast(uint32_t v, int lane) { return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), lane)); }
__device__ __forceinline__ uint64_t wave_bcast64(uint64_t v, int lane)
{
  uint32_t lo = wave_bcast(static_cast<uint32_t>(v), lane);
  uint32_t hi = wave_bcast(static_cast<uint32_t>(v >> 32), lane);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

__device__ __forceinline__ uint64_t ballot64(bool p) { return __builtin_amdgcn_ballot_w64(p); }
__device__ __forceinline__ uint32_t lanes_below(uint64_t mask)
{
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

// Workgroup exclusive scan of one uint32 per thread.  `lds` needs (blockDim/64 + 1) words.
// Returns the exclusive prefix; *total receives the workgroup sum (same value on every thread).
template <int THREADS>
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* lds, uint32_t* total)
{
  constexpr int W  = THREADS / kWave;
  int const lane   = lane_id();
  int const wave   = threadIdx.x / kWave;
  uint32_t const i = wave_inclusive_scan(v);
  __syncthreads();  // protect lds reuse between calls
  if (lane == kWave - 1) lds[wave] = i;
  __syncthreads();
  uint32_t base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    uint32_t const t = lds[w];
    if (w < wave) base += t;
    sum += t;
  }
  *total = sum;
  return base + i - v;
}

// Workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight (a __syncthreads()
// waits for them).  For kernels whose lanes exchange data through LDS alone.
__device__ __forceinline__ void lds_barrier()
{
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// block_exclusive_scan with lds_barrier() in place of __syncthreads().
template <int THREADS>
__device__ __forceinline__ uint32_t block_exclusive_scan_lds(uint32_t v, uint32_t* lds, uint32_t* total)
{
  constexpr int W  = THREADS / kWave;
  int const lane   = lane_id();
  int const wave   = threadIdx.x / kWave;
  uint32_t const i = wave_inclusive_scan(v);
  lds_barrier();  // protect lds reuse between calls
  if (lane == kWave - 1) lds[wave] = i;
  lds_barrier();
  uint32_t base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    uint32_t const t = lds[w];
    if (w < wave) base += t;
    sum += t;
  }
  *total = sum;
  return base + i - v;
}

template <int THREADS>
__device__ __forceinline__ uint64_t block_exclusive_scan64(uint64_t v, uint64_t* lds, uint64_t* total)
{
  constexpr int W  = THREADS / kWave;
  int const lane   = lane_id();
  int const wave   = threadIdx.x / kWave;
  uint64_t const i = wave_inclusive_scan64(v);
  __syncthreads();
  if (lane == kWave - 1) lds[wave] = i;
  __syncthreads();
  uint64_t base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    uint64_t const t = lds[w];
    if (w < wave) base += t;
    sum += t;
  }
  *total = sum;
  return base + i - v;
}

// ------------------------------------------------------------------ device-wide exclusive scan
// out[i] = sum_{j<i} f(j) for i in [0, n]  (n+1 entries; out[n] is the total).
// Three launches: per-tile sums, scan of the tile sums (one workgroup), rescan + add; one launch for a few thousand values.
constexpr int kScanThreads = 256;
constexpr int kScanItems   = 8;
constexpr int kScanTile    = kScanThreads * kScanItems;

template <typename F>
__global__ void __launch_bounds__(kScanThreads) scan_tile_sums_kernel(F f, int64_t n, uint64_t* tile_sums)
{
  __shared__ uint64_t lds[kScanThreads / kWave + 1];
  int64_t const base = static_cast<int64_t>(blockIdx.x) * kScanTile + static_cast<int64_t>(threadIdx.x) * kScanItems;
  uint64_t s         = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    int64_t const i = base + k;
    if (i < n) s += f(i);
  }
  uint64_t total;
  block_exclusive_scan64<kScanThreads>(s, lds, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// exclusive scan of tile_sums in place; tile_sums[ntiles] = grand total
__global__ void __launch_bounds__(kScanThreads) scan_tile_offsets_kernel(uint64_t* tile_sums, int64_t ntiles);

template <typename F, typename OutT>
__global__ void __launch_bounds__(kScanThreads) scan_apply_kernel(F f, int64_t n, const uint64_t* tile_offsets, OutT* out)
{
  __shared__ uint64_t lds[kScanThreads / kWave + 1];
  int64_t const base = static_cast<int64_t>(blockIdx.x) * kScanTile + static_cast<int64_t>(threadIdx.x) * kScanItems;
  uint64_t vals[kScanItems];
  uint64_t s = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    int64_t const i = base + k;
    vals[k]         = (i < n) ? static_cast<uint64_t>(f(i)) : 0;
    s += vals[k];
  }
  uint64_t total;
  uint64_t run = block_exclusive_scan64<kScanThreads>(s, lds, &total) + tile_offsets[blockIdx.x];
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    int64_t const i = base + k;
    if (i < n) out[i] = static_cast<OutT>(run);
    run += vals[k];
    if (i == n - 1) out[n] = static_cast<OutT>(run);
  }
}

// The whole scan by one workgroup, for the few thousand values of a small call: one launch instead of three.
// tile_sums[tiles] receives the grand total, as scan_tile_offsets_kernel leaves it.
constexpr int64_t kScanSmallTiles = 4;
template <typename F, typename OutT>
__global__ void __launch_bounds__(kScanThreads) scan_small_kernel(F f, int64_t n, uint64_t* total_out, OutT* out)
{
  __shared__ uint64_t lds[kScanThreads / kWave + 1];
  uint64_t carry = 0;
  for (int64_t tile = 0; tile * kScanTile < n; ++tile) {
    int64_t const base = tile * kScanTile + static_cast<int64_t>(threadIdx.x) * kScanItems;
    uint64_t vals[kScanItems];
    uint64_t s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      int64_t const i = base + k;
      vals[k]         = (i < n) ? static_cast<uint64_t>(f(i)) : 0;
      s += vals[k];
    }
    uint64_t total;
    uint64_t run = block_exclusive_scan64<kScanThreads>(s, lds, &total) + carry;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      int64_t const i = base + k;
      if (i < n) out[i] = static_cast<OutT>(run);
      run += vals[k];
    }
    carry += total;
  }
  if (threadIdx.x == 0) {
    out[n]     = static_cast<OutT>(carry);
    *total_out = carry;
  }
}

inline int64_t scan_tiles(int64_t n) { return (n + kScanTile - 1) / kScanTile; }
inline size_t scan_temp_bytes(int64_t n) { return static_cast<size_t>(scan_tiles(n) + 1) * sizeof(uint64_t); }

// `temp` holds scan_temp_bytes(n) bytes; temp[ntiles] receives the grand total (uint64).
// n must be > 0.
template <typename F, typename OutT>
void device_exclusive_scan(F f, int64_t n, OutT* out, uint64_t* temp, hipStream_t stream)
{
  int64_t const tiles = scan_tiles(n);
  if (tiles <= kScanSmallTiles) {
    hipLaunchKernelGGL(HIP_KERNEL_NAME(scan_small_kernel<F, OutT>), dim3(1), dim3(kScanThreads), 0, stream, f, n, temp + tiles, out);
    return;
  }
  hipLaunchKernelGGL(HIP_KERNEL_NAME(scan_tile_sums_kernel<F>), dim3(static_cast<unsigned>(tiles)), dim3(kScanThreads), 0, stream, f, n, temp);
  hipLaunchKernelGGL(scan_tile_offsets_kernel, dim3(1), dim3(kScanThreads), 0, stream, temp, tiles);
  hipLaunchKernelGGL(HIP_KERNEL_NAME(scan_apply_kernel<F, OutT>), dim3(static_cast<unsigned>(tiles)), dim3(kScanThreads), 0, stream, f, n, temp, out);
}

// ------------------------------------------------------------------ scalars for the host
// A few KB of pinned host memory that kernels write and the host reads once the stream is synchronised (a copy of a
// few bytes into ordinary host memory goes through a staging buffer and costs ten microseconds and more): eight 64-bit
// words, and behind them room for kHostSampleWords 32-bit words.  One buffer per host thread, allocated at the thread's
// first call and kept until the process ends; nullptr when the allocation failed (the callers then copy).
constexpr size_t kHostSampleWords = 3 * 512;
constexpr size_t kHostScalarBytes = 8 * sizeof(uint64_t) + kHostSampleWords * sizeof(uint32_t);
uint64_t* host_scalars();
// dst[0] = offsets[first_index], dst[1] = offsets[last_index] (offsets of 32 or 64 bits)
void launch_read_two_offsets(const void* offsets, int is64, int64_t first_index, int64_t last_index, uint64_t* dst, hipStream_t stream);

// ------------------------------------------------------------------ bitmask copy
// dst bit i = src bit (i + begin_bit); bits past `bits` are cleared
// (cpp/src/bitmask/null_mask.cu:332-347).
void launch_copy_bitmask(uint32_t* dst, const uint32_t* src, int32_t begin_bit, int32_t bits, hipStream_t stream);

void launch_fill_u32(uint32_t* dst, uint32_t value, int64_t count, hipStream_t stream);

}  // namespace nvtext_amd

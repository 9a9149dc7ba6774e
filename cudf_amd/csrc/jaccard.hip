// jaccard_index for gfx950.
//
// The reference (cpp/src/text/jaccard.cu) hashes the character windows of both columns into two
// chars-sized temporaries, sorts each row's hashes with a device-wide segmented sort, and counts unique
// and common values with a warp per row (66-170, 196-400).
//
// Here a workgroup takes a row pair and needs no sort and no temporary: the window hashes of both rows go
// into ONE open-addressing set in LDS (load <= 2/3) with two membership bits per slot, "seen in row 1" and
// "seen in row 2".  |A|, |B| and |A n B| are then population counts of the two bit arrays and of their
// AND.  The launches cover the pairs by size: an 8 KiB set per WAVEFRONT (each wavefront its own pair, nothing
// shared, so that many short pairs are in flight per CU) for pairs of up to 1365 bytes together, a 32 KiB set
// (four workgroups per CU) up to 5461 bytes, a 64 KiB set (two workgroups of eight wavefronts per CU) up to 10922
// bytes, a 128 KiB set (one workgroup per CU) up to 21845 bytes; the few longer pairs are done by a last kernel
// with the same code over a set in global memory.
// Each kernel lists the pairs that are too large for it for the next one.
#include "common.cuh"
#include "murmur.cuh"
#include "windows.cuh"

#include <limits>

namespace nvtext_amd {
namespace {

constexpr uint32_t kTinySlots   = 2048;   // slots of a wavefront's own LDS set
constexpr uint32_t kSmallSlots  = 8192;   // slots of the small LDS set
constexpr uint32_t kMidSlots    = 16384;  // slots of the 64 KiB LDS set
constexpr uint32_t kMediumSlots = 32768;  // slots of the large LDS set
constexpr int kMediumWaves      = 8;

// An insert-only set of non-zero uint32 values with two membership bits per slot.
struct PairSet {
  uint32_t* slots;   // 0 = empty
  uint32_t* in1;     // bit s: the value in slot s occurs in row 1
  uint32_t* in2;     // bit s: ... in row 2
  uint32_t mask;     // slots - 1 (a power of two)
  uint32_t shift;    // 32 - log2(slots)

  __device__ __forceinline__ void insert(uint32_t h, int which) const
  {
    uint32_t s = (h * 0x9E3779B1u) >> shift;
    for (;;) {
      uint32_t const old = atomicCAS(&slots[s], 0u, h);
      if (old == 0u || old == h) break;
      s = (s + 1u) & mask;
    }
    atomicOr(which == 0 ? &in1[s >> 5] : &in2[s >> 5], 1u << (s & 31u));
  }
};

// Hashes the windows of one row (jaccard.cu:249-292) and inserts the non-zero hashes into the set.
// The wavefronts of the workgroup take the tiles of the row in turn.
__device__ __forceinline__ void insert_row(const uint8_t* row, int64_t n, int32_t width, PairSet const& set, int which, uint32_t* stage,
                                           int wave, int nwaves, int lane)
{
  if (static_cast<int64_t>(width) * 4 <= kHalo) {
    uint32_t const halo = static_cast<uint32_t>(width) * 4u;
    for (int64_t base = static_cast<int64_t>(wave) * kTile; base < n; base += static_cast<int64_t>(nwaves) * kTile) {
      uint32_t const cnt = static_cast<uint32_t>(min(static_cast<int64_t>(kTile), n - base));
      uint32_t const len = static_cast<uint32_t>(min(n - base, static_cast<int64_t>(cnt + halo)));
      bool all_ascii;
      uint32_t const mis = stage_bytes(row, base, len, stage, lane, &all_ascii);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      for (uint32_t q = 0; q < cnt; q += kWave) {
        uint32_t const p = q + lane;
        if (p < cnt) {
          int64_t const gpos = base + p;
          WordSrc const src{stage, mis + p};
          uint32_t hlen;
          if (window_at(src, row + gpos, n - gpos, len - p, gpos == 0, all_ascii, width, &hlen)) {
            uint32_t const hv = murmur3_x86_32(src, hlen, 0u);  // jaccard.cu:258: seed 0
            if (hv != 0u) set.insert(hv, which);                // 282-286: zero hashes are dropped
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  } else {
    // very wide windows: bytes straight from global memory
    for (int64_t gpos = static_cast<int64_t>(wave) * kWave + lane; gpos < n; gpos += nwaves * kWave) {
      int64_t const remaining = n - gpos;
      BoundedSrc const src{row + gpos, remaining};
      uint32_t hlen;
      uint32_t const readable = static_cast<uint32_t>(min(remaining, static_cast<int64_t>(width) * 4));
      if (window_at(src, row + gpos, remaining, readable, gpos == 0, false, width, &hlen)) {
        uint32_t const hv = murmur3_x86_32(src, hlen, 0u);
        if (hv != 0u) set.insert(hv, which);
      }
    }
  }
}

template <int WAVES>
struct PairScratch {
  uint32_t stage[WAVES][kTileWords];  // per wavefront: the bytes of the tile being hashed
  uint32_t sums[3][WAVES];
};

// One row pair with a set of `slots` slots (a power of two, at least 64): clears the set, inserts both
// rows, counts, writes the index (jaccard.cu:414-425).
template <int WAVES>
__device__ __forceinline__ void jaccard_pair(ColView const& c1, ColView const& c2, int64_t r, int32_t width, uint32_t* slots, uint32_t* in1,
                                             uint32_t* in2, uint32_t nslots, PairScratch<WAVES>& scratch, float* out)
{
  constexpr uint32_t kPairThreads = WAVES * kWave;
  int const lane = lane_id();
  int const wave = threadIdx.x / kWave;
  // (nslots is a power of two of at least 64 and the arrays are 16-byte aligned: whole uint4 stores)
  for (uint32_t i = threadIdx.x; i < nslots / 4; i += kPairThreads) reinterpret_cast<uint4*>(slots)[i] = make_uint4(0u, 0u, 0u, 0u);
  for (uint32_t i = threadIdx.x; i < nslots / 32; i += kPairThreads) {
    in1[i] = 0u;
    in2[i] = 0u;
  }
  __syncthreads();
  PairSet const set{slots, in1, in2, nslots - 1u, static_cast<uint32_t>(__builtin_clz(nslots)) + 1u};
  // 211-220: null rows and empty rows have no hashes
  if (c1.valid(r)) {
    int64_t const o = c1.off(r);
    insert_row(c1.chars + o, c1.off(r + 1) - o, width, set, 0, scratch.stage[wave], wave, WAVES, lane);
  }
  if (c2.valid(r)) {
    int64_t const o = c2.off(r);
    insert_row(c2.chars + o, c2.off(r + 1) - o, width, set, 1, scratch.stage[wave], wave, WAVES, lane);
  }
  __syncthreads();
  uint32_t u1 = 0, u2 = 0, both = 0;
  for (uint32_t i = threadIdx.x; i < nslots / 32; i += kPairThreads) {
    uint32_t const a = in1[i], b = in2[i];
    u1 += __builtin_popcount(a);
    u2 += __builtin_popcount(b);
    both += __builtin_popcount(a & b);
  }
  u1   = wave_bcast(wave_inclusive_scan(u1), kWave - 1);
  u2   = wave_bcast(wave_inclusive_scan(u2), kWave - 1);
  both = wave_bcast(wave_inclusive_scan(both), kWave - 1);
  if (lane == 0) {
    scratch.sums[0][wave] = u1;
    scratch.sums[1][wave] = u2;
    scratch.sums[2][wave] = both;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t count1 = 0, count2 = 0, intersects = 0;
    for (int w = 0; w < WAVES; ++w) {
      count1 += static_cast<int32_t>(scratch.sums[0][w]);
      count2 += static_cast<int32_t>(scratch.sums[1][w]);
      intersects += static_cast<int32_t>(scratch.sums[2][w]);
    }
    int32_t const unions = count1 + count2 - intersects;
    out[r]               = unions ? static_cast<float>(intersects) / static_cast<float>(unions) : 0.f;
  }
  __syncthreads();
}

// Window starts of the pair are at most the bytes of both rows.
__device__ __forceinline__ int64_t pair_bytes(ColView const& c1, ColView const& c2, int64_t r)
{
  int64_t n = 0;
  if (c1.valid(r)) n += c1.off(r + 1) - c1.off(r);
  if (c2.valid(r)) n += c2.off(r + 1) - c2.off(r);
  return n;
}

// Slots a pair needs: a power of two that keeps the load at or below 2/3 (window starts <= bytes).  This decides
// the kernel that takes the pair; where that kernel's set has room it uses twice as many (shorter probe runs).
__device__ __host__ __forceinline__ uint64_t slots_for(int64_t bytes)
{
  uint64_t s = 64;
  while (2 * s < 3 * static_cast<uint64_t>(bytes)) s <<= 1;
  return s;
}

// Work lists in `lists`: a header of 8 words -- [0] = pairs listed for the global-memory kernel, [1] = for the
// 128 KiB kernel, [2..3] = the most bytes a pair of the first list has (64 bits), [4] = pairs listed for the 32 KiB
// kernel, [5] = for the 64 KiB kernel -- then `rows` entries for each of these four lists, in the order 0, 1, [4], [5].
constexpr int kListHeader = 8;
__device__ __forceinline__ uint32_t* list_count(uint32_t* lists, int which) { return &lists[which >= 2 ? which + 2 : which]; }
__device__ __forceinline__ uint32_t* list_entries(uint32_t* lists, int which, int64_t rows) { return lists + kListHeader + which * rows; }
__device__ __forceinline__ void list_pair(uint32_t* lists, int which, int64_t rows, int64_t r, int64_t bytes)
{
  uint32_t const at                  = atomicAdd(list_count(lists, which), 1u);
  list_entries(lists, which, rows)[at] = static_cast<uint32_t>(r);
  if (which == 0) atomicMax(reinterpret_cast<unsigned long long*>(&lists[2]), static_cast<unsigned long long>(bytes));
}

struct TinyLds {
  alignas(16) uint32_t slots[kTinySlots];
  uint32_t in1[kTinySlots / 32], in2[kTinySlots / 32];
  uint32_t stage[kTileWords];  // the bytes of the tile being hashed
};

// Every wavefront on its own: it sizes 64 consecutive pairs at once (lanes <-> pairs, coalesced offset loads), lists
// those that need more than kTinySlots for the small kernel with one atomic, and does the others one after the
// other with its own set.  No workgroup barrier anywhere.
__global__ void __launch_bounds__(kThreads) jaccard_tiny_kernel(ColView c1, ColView c2, int32_t width, float* __restrict__ out,
                                                                uint32_t* __restrict__ lists)
{
  __shared__ TinyLds lds_all[kWaves];
  int const lane       = lane_id();
  TinyLds& lds         = lds_all[threadIdx.x / kWave];
  int64_t const rows   = c1.size;
  int64_t const nwaves = static_cast<int64_t>(gridDim.x) * kWaves;
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  for (int64_t base = (static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave) * kWave; base < rows; base += nwaves * kWave) {
    int64_t const r = base + lane;
    int64_t o1 = 0, n1 = 0, o2 = 0, n2 = 0;  // 211-220: null rows and empty rows have no hashes
    if (r < rows) {
      if (c1.valid(r)) {
        o1 = c1.off(r);
        n1 = c1.off(r + 1) - o1;
      }
      if (c2.valid(r)) {
        o2 = c2.off(r);
        n2 = c2.off(r + 1) - o2;
      }
    }
    uint64_t const need = slots_for(n1 + n2);
    bool const mine     = r < rows && need <= kTinySlots;
    uint64_t const later = ballot64(r < rows && !mine);
    if (later != 0) {
      uint32_t at = 0;
      if (lane == 0) at = atomicAdd(list_count(lists, 2), static_cast<uint32_t>(__builtin_popcountll(later)));
      at = wave_bcast(at, 0);
      if (r < rows && !mine) list_entries(lists, 2, rows)[at + lanes_below(later)] = static_cast<uint32_t>(r);
    }
    for (uint64_t todo = ballot64(mine); todo != 0; todo &= todo - 1) {
      int const b           = __builtin_ctzll(todo);
      uint32_t const nslots = min(kTinySlots, 2u * static_cast<uint32_t>(wave_bcast64(need, b)));
      int64_t const ro1 = static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(o1), b)), rn1 = static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(n1), b));
      int64_t const ro2 = static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(o2), b)), rn2 = static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(n2), b));
      for (uint32_t i = lane; i < nslots / 4; i += kWave) reinterpret_cast<uint4*>(lds.slots)[i] = make_uint4(0u, 0u, 0u, 0u);
      if (static_cast<uint32_t>(lane) < nslots / 32) {
        lds.in1[lane] = 0u;
        lds.in2[lane] = 0u;
      }
      wave_sync();
      PairSet const set{lds.slots, lds.in1, lds.in2, nslots - 1u, static_cast<uint32_t>(__builtin_clz(nslots)) + 1u};
      if (rn1 > 0) insert_row(c1.chars + ro1, rn1, width, set, 0, lds.stage, 0, 1, lane);
      if (rn2 > 0) insert_row(c2.chars + ro2, rn2, width, set, 1, lds.stage, 0, 1, lane);
      wave_sync();
      uint32_t u1 = 0, u2 = 0, both = 0;
      if (static_cast<uint32_t>(lane) < nslots / 32) {  // at most 64 words of bits
        uint32_t const a = lds.in1[lane], bb = lds.in2[lane];
        u1   = __builtin_popcount(a);
        u2   = __builtin_popcount(bb);
        both = __builtin_popcount(a & bb);
      }
      int32_t const count1     = static_cast<int32_t>(wave_bcast(wave_inclusive_scan(u1), kWave - 1));
      int32_t const count2     = static_cast<int32_t>(wave_bcast(wave_inclusive_scan(u2), kWave - 1));
      int32_t const intersects = static_cast<int32_t>(wave_bcast(wave_inclusive_scan(both), kWave - 1));
      int32_t const unions     = count1 + count2 - intersects;  // jaccard.cu:414-425
      if (lane == 0) out[base + b] = unions ? static_cast<float>(intersects) / static_cast<float>(unions) : 0.f;
      wave_sync();
    }
  }
}

// The pairs of list FROM whose set fits SLOTS slots, one workgroup of WAVES wavefronts per pair; the others are put on
// list TO.  Three instances: 8192 slots (32 KiB, four workgroups per CU), 16384 (64 KiB, two per CU), 32768 (128 KiB, one).
template <uint32_t SLOTS, int WAVES, int FROM, int TO>
__global__ void __launch_bounds__(WAVES* kWave) jaccard_listed_kernel(ColView c1, ColView c2, int32_t width, float* __restrict__ out,
                                                                       uint32_t* __restrict__ lists)
{
  __shared__ alignas(16) uint32_t slots[SLOTS];
  __shared__ uint32_t in1[SLOTS / 32], in2[SLOTS / 32];
  __shared__ PairScratch<WAVES> scratch;
  int64_t const rows   = c1.size;
  uint32_t const count = *list_count(lists, FROM);
  for (uint32_t i = blockIdx.x; i < count; i += gridDim.x) {
    int64_t const r     = list_entries(lists, FROM, rows)[i];
    int64_t const bytes = pair_bytes(c1, c2, r);
    uint64_t const need = slots_for(bytes);
    if (need > SLOTS) {
      if (threadIdx.x == 0) list_pair(lists, TO, rows, r, bytes);
      continue;
    }
    jaccard_pair<WAVES>(c1, c2, r, width, slots, in1, in2, min(SLOTS, 2u * static_cast<uint32_t>(need)), scratch, out);
  }
}

// The listed pairs, each workgroup with its own set in global memory (`table_slots` slots, then the two bit arrays).
__global__ void __launch_bounds__(kThreads) jaccard_global_kernel(ColView c1, ColView c2, int32_t width, float* __restrict__ out,
                                                                  const uint32_t* __restrict__ big, uint32_t* __restrict__ tables,
                                                                  uint64_t table_slots)
{
  __shared__ PairScratch<kWaves> scratch;
  uint32_t const count = big[0];
  uint32_t* const mine = tables + static_cast<uint64_t>(blockIdx.x) * (table_slots + 2 * (table_slots / 32));
  for (uint32_t i = blockIdx.x; i < count; i += gridDim.x) {
    int64_t const r     = big[kListHeader + i];
    uint32_t const need = static_cast<uint32_t>(slots_for(pair_bytes(c1, c2, r)));
    jaccard_pair<kWaves>(c1, c2, r, width, mine, mine + table_slots, mine + table_slots + table_slots / 32, need, scratch, out);
  }
}

// out[w] = validity word w of column 1 AND of column 2 (bits past `bits` are 0); *nulls += zero bits.
__global__ void and_bitmask_kernel(uint32_t* __restrict__ out, const uint32_t* __restrict__ m1, int32_t begin1, const uint32_t* __restrict__ m2,
                                   int32_t begin2, int32_t bits, int32_t words, uint32_t* __restrict__ nulls)
{
  int32_t const w = blockIdx.x * blockDim.x + threadIdx.x;
  if (w >= words) return;
  auto word_of = [&](const uint32_t* m, int32_t begin) -> uint32_t {
    if (!m) return 0xFFFFFFFFu;
    int64_t const first = static_cast<int64_t>(begin) + static_cast<int64_t>(w) * 32;
    int64_t const sw    = first >> 5;
    int const sh        = static_cast<int>(first & 31);
    int64_t const last  = (static_cast<int64_t>(begin) + bits - 1) >> 5;
    uint32_t v          = m[sw] >> sh;
    if (sh != 0 && sw + 1 <= last) v |= m[sw + 1] << (32 - sh);
    return v;
  };
  uint32_t v              = word_of(m1, begin1) & word_of(m2, begin2);
  int32_t const remaining = bits - w * 32;
  uint32_t const live     = remaining < 32 ? (1u << remaining) - 1u : 0xFFFFFFFFu;
  v &= live;
  out[w] = v;
  uint32_t const zeros = __builtin_popcount(~v & live);
  if (zeros) atomicAdd(nulls, zeros);
}

}  // namespace
}  // namespace nvtext_amd

extern "C" {

nvtext_amd_status nvtext_amd_jaccard_index(const nvtext_amd_strings_column* input1, const nvtext_amd_strings_column* input2, int32_t width,
                                           void* stream_, const nvtext_amd_allocator* mr_, nvtext_amd_fixed_column* out)
{
  using namespace nvtext_amd;
  EntryScope const entry("nvtext_amd_jaccard_index");
  if (!input1 || !input2 || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nvtext_amd_fixed_column{};
  // cpp/src/text/jaccard.cu:441-446, same order and messages
  if (input1->size != input2->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "input columns must be the same size");
  if (width < 2) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameter width should be an integer value of 2 or greater");
  for (const nvtext_amd_strings_column* c : {input1, input2}) {
    if (c->size < 0 || c->null_count < 0 || c->null_count > c->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "invalid column sizes");
    if (c->null_count > 0 && !c->null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");
  }
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Mr mr{mr_, stream};
  int32_t const rows = input1->size;
  out->type          = NVTEXT_AMD_TYPE_FLOAT32;
  out->size          = rows;
  if (rows == 0) return NVTEXT_AMD_SUCCESS;  // jaccard.cu:449: an empty FLOAT32 column

  out->data_bytes = static_cast<size_t>(rows) * sizeof(float);
  out->data       = mr.allocate(out->data_bytes);
  if (!out->data) return fail(NVTEXT_AMD_ALLOC_FAILED, "result allocation failed");
  bool const with_mask = input1->null_count > 0 || input2->null_count > 0;  // 471-476
  if (with_mask) {
    out->null_mask_bytes = mask_alloc_bytes(rows);
    out->null_mask       = static_cast<uint32_t*>(mr.allocate(out->null_mask_bytes));
    if (!out->null_mask) {
      nvtext_amd_fixed_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "mask allocation failed");
    }
  }
  // the four work lists (see list_pair) and the null counter behind them
  Temp big(mr, (4 * static_cast<size_t>(rows) + kListHeader + 4) * sizeof(uint32_t));
  if (!big.ok()) {
    nvtext_amd_fixed_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
  }
  launch_fill_u32(big.as<uint32_t>(), 0u, kListHeader, stream);
  uint32_t* const null_counter = big.as<uint32_t>() + kListHeader + 4 * static_cast<size_t>(rows);
  launch_fill_u32(null_counter, 0u, 1, stream);

  ColView const v1 = make_view(*input1);
  ColView const v2 = make_view(*input2);
  float* const values = static_cast<float*>(out->data);
  int device = 0, cus = 256;
  (void)hipGetDevice(&device);
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
  {
    ProfileScope ps("jaccard_tiny_kernel", stream);
    int64_t const batches = (static_cast<int64_t>(rows) + kWave * kWaves - 1) / (kWave * kWaves);
    unsigned const grid   = static_cast<unsigned>(std::min<int64_t>(batches, static_cast<int64_t>(cus) * 8));
    hipLaunchKernelGGL(jaccard_tiny_kernel, dim3(grid), dim3(kThreads), 0, stream, v1, v2, width, values, big.as<uint32_t>());
  }
  {
    ProfileScope ps("jaccard_small_kernel", stream);
    unsigned const grid = static_cast<unsigned>(std::min<int64_t>(rows, static_cast<int64_t>(cus) * 16));
    hipLaunchKernelGGL(HIP_KERNEL_NAME(jaccard_listed_kernel<kSmallSlots, kWaves, 2, 3>), dim3(grid), dim3(kThreads), 0, stream, v1, v2, width, values,
                       big.as<uint32_t>());
  }
  {
    ProfileScope ps("jaccard_mid_kernel", stream);
    unsigned const grid = static_cast<unsigned>(std::min<int64_t>(rows, static_cast<int64_t>(cus) * 4));
    hipLaunchKernelGGL(HIP_KERNEL_NAME(jaccard_listed_kernel<kMidSlots, kMediumWaves, 3, 1>), dim3(grid), dim3(kMediumWaves * kWave), 0, stream, v1, v2,
                       width, values, big.as<uint32_t>());
  }
  {
    ProfileScope ps("jaccard_medium_kernel", stream);
    unsigned const grid = static_cast<unsigned>(std::min<int64_t>(rows, static_cast<int64_t>(cus) * 2));
    hipLaunchKernelGGL(HIP_KERNEL_NAME(jaccard_listed_kernel<kMediumSlots, kMediumWaves, 1, 0>), dim3(grid), dim3(kMediumWaves * kWave), 0, stream, v1, v2,
                       width, values, big.as<uint32_t>());
  }
  if (with_mask) {
    int32_t const words = (rows + 31) / 32;
    hipLaunchKernelGGL(and_bitmask_kernel, dim3((words + 255) / 256), dim3(256), 0, stream, out->null_mask,
                       input1->null_count > 0 ? input1->null_mask : nullptr, input1->offset,
                       input2->null_count > 0 ? input2->null_mask : nullptr, input2->offset, rows, words, null_counter);
  }
  uint32_t head[4] = {0, 0, 0, 0};
  uint32_t nulls   = 0;
  hipError_t e     = hipMemcpyAsync(head, big.as<uint32_t>(), sizeof(head), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipMemcpyAsync(&nulls, null_counter, sizeof(nulls), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    nvtext_amd_fixed_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
  }
  out->null_count = static_cast<int32_t>(nulls);
  if (head[0] > 0) {
    uint64_t const most = (static_cast<uint64_t>(head[3]) << 32) | head[2];
    uint64_t const slots = slots_for(static_cast<int64_t>(most));
    if (slots > (uint64_t{1} << 31)) {
      nvtext_amd_fixed_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_OVERFLOW, "a row pair is too long");
    }
    unsigned const grid = static_cast<unsigned>(std::min<uint64_t>(head[0], static_cast<uint64_t>(cus)));
    Temp tables(mr, static_cast<size_t>(grid) * (slots + 2 * (slots / 32)) * sizeof(uint32_t));
    if (!tables.ok()) {
      nvtext_amd_fixed_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    }
    ProfileScope ps("jaccard_global_kernel", stream);
    hipLaunchKernelGGL(jaccard_global_kernel, dim3(grid), dim3(kThreads), 0, stream, v1, v2, width, values, big.as<uint32_t>(),
                       tables.as<uint32_t>(), slots);
    NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_fixed_column_free(out, stream_, mr_));
    // the tables are released in stream order when `tables` goes out of scope
  }
  NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_fixed_column_free(out, stream_, mr_));
  return NVTEXT_AMD_SUCCESS;
}

void nvtext_amd_fixed_column_free(nvtext_amd_fixed_column* col, void* stream, const nvtext_amd_allocator* mr)
{
  if (!col) return;
  nvtext_amd::Mr m{mr, static_cast<hipStream_t>(stream)};
  m.deallocate(col->data, col->data_bytes);
  m.deallocate(col->null_mask, col->null_mask_bytes);
  *col = nvtext_amd_fixed_column{};
}

}  // extern "C"

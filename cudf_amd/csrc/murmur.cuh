// MurmurHash3_x86_32 and MurmurHash3_x64_128 (word 0) over a byte range that sits in a
// dword array (LDS tile or global memory), read as unaligned little-endian dwords.
// The arithmetic is the published MurmurHash3 the reference reaches through
// cuco::murmurhash3_32 / cuco::murmurhash3_x64_128
// (cpp/include/cudf/hashing/detail/murmurhash3_x86_32.cuh:21-46,
//  cpp/include/cudf/hashing/detail/murmurhash3_x64_128.cuh:18-43).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nvtext_amd {

__device__ __forceinline__ uint32_t rotl32(uint32_t x, int r) { return __builtin_amdgcn_alignbit(x, x, 32 - r); }
__device__ __forceinline__ uint64_t rotl64(uint64_t x, int r) { return (x << r) | (x >> (64 - r)); }

// Dword starting at byte offset `o` of the dword array `w` (reads w[o/4] and w[o/4+1]).
__device__ __forceinline__ uint32_t load_u32_at(const uint32_t* w, uint32_t o)
{
  uint32_t const i  = o >> 2;
  uint32_t const lo = w[i];
  uint32_t const hi = w[i + 1];
  return __builtin_amdgcn_alignbit(hi, lo, (o & 3u) * 8u);
}

__device__ __forceinline__ uint32_t keep_low_bytes(uint32_t v, int nbytes)
{
  // nbytes in [0, 4]
  return nbytes >= 4 ? v : (v & ((1u << (8 * nbytes)) - 1u));
}

// Byte source over a dword array (an LDS tile): window byte i lives at byte offset base+i.
// u32(i) may read up to 7 bytes past the window (callers mask what they do not need).
struct WordSrc {
  const uint32_t* w;
  uint32_t base;
  __device__ __forceinline__ uint32_t byte(uint32_t i) const { return reinterpret_cast<const uint8_t*>(w)[base + i]; }
  __device__ __forceinline__ uint32_t u32(uint32_t i) const { return load_u32_at(w, base + i); }
};

// Byte source over global memory that never touches a byte at or past `avail`
// (slow; used only for windows too wide for the LDS tile).
struct BoundedSrc {
  const uint8_t* p;
  int64_t avail;
  __device__ __forceinline__ uint32_t byte(uint32_t i) const { return p[i]; }
  __device__ __forceinline__ uint32_t u32(uint32_t i) const
  {
    uint32_t v = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (static_cast<int64_t>(i) + k < avail) v |= static_cast<uint32_t>(p[i + k]) << (8 * k);
    return v;
  }
};

// Hash of window bytes [0, len) of `src`.
template <typename Src>
__device__ __forceinline__ uint32_t murmur3_x86_32(Src const& src, uint32_t len, uint32_t seed)
{
  uint32_t const c1 = 0xcc9e2d51u, c2 = 0x1b873593u;
  uint32_t h1           = seed;
  uint32_t const blocks = len >> 2;
  for (uint32_t i = 0; i < blocks; ++i) {
    uint32_t k1 = src.u32(4 * i);
    k1 *= c1;
    k1 = rotl32(k1, 15);
    k1 *= c2;
    h1 ^= k1;
    h1 = rotl32(h1, 13);
    h1 = h1 * 5u + 0xe6546b64u;
  }
  uint32_t const rem = len & 3u;
  if (rem) {
    uint32_t k1 = keep_low_bytes(src.u32(4 * blocks), static_cast<int>(rem));
    k1 *= c1;
    k1 = rotl32(k1, 15);
    k1 *= c2;
    h1 ^= k1;
  }
  h1 ^= len;
  h1 ^= h1 >> 16;
  h1 *= 0x85ebca6bu;
  h1 ^= h1 >> 13;
  h1 *= 0xc2b2ae35u;
  h1 ^= h1 >> 16;
  return h1;
}

__device__ __forceinline__ uint64_t fmix64(uint64_t k)
{
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ull;
  k ^= k >> 33;
  return k;
}

template <typename Src>
__device__ __forceinline__ uint64_t load_u64(Src const& src, uint32_t i)
{
  return (static_cast<uint64_t>(src.u32(i + 4)) << 32) | src.u32(i);
}

// First 64-bit word of MurmurHash3_x64_128 with h1 = h2 = seed over window bytes [0, len).
template <typename Src>
__device__ __forceinline__ uint64_t murmur3_x64_128_lo(Src const& src, uint32_t len, uint64_t seed)
{
  uint64_t const c1 = 0x87c37b91114253d5ull, c2 = 0x4cf5ad432745937full;
  uint64_t h1 = seed, h2 = seed;
  uint32_t const blocks = len >> 4;
  for (uint32_t i = 0; i < blocks; ++i) {
    uint64_t k1 = load_u64(src, 16 * i);
    uint64_t k2 = load_u64(src, 16 * i + 8);
    k1 *= c1;
    k1 = rotl64(k1, 31);
    k1 *= c2;
    h1 ^= k1;
    h1 = rotl64(h1, 27);
    h1 += h2;
    h1 = h1 * 5 + 0x52dce729;
    k2 *= c2;
    k2 = rotl64(k2, 33);
    k2 *= c1;
    h2 ^= k2;
    h2 = rotl64(h2, 31);
    h2 += h1;
    h2 = h2 * 5 + 0x38495ab5;
  }
  int const rem = static_cast<int>(len & 15u);
  if (rem) {
    uint32_t const t = 16 * blocks;
    if (rem > 8) {
      uint32_t const lo = keep_low_bytes(src.u32(t + 8), rem - 8);
      uint32_t const hi = rem > 12 ? keep_low_bytes(src.u32(t + 12), rem - 12) : 0u;
      uint64_t k2       = (static_cast<uint64_t>(hi) << 32) | lo;
      k2 *= c2;
      k2 = rotl64(k2, 33);
      k2 *= c1;
      h2 ^= k2;
    }
    uint32_t const lo = keep_low_bytes(src.u32(t), rem);
    uint32_t const hi = rem > 4 ? keep_low_bytes(src.u32(t + 4), rem - 4) : 0u;
    uint64_t k1       = (static_cast<uint64_t>(hi) << 32) | lo;
    k1 *= c1;
    k1 = rotl64(k1, 31);
    k1 *= c2;
    h1 ^= k1;
  }
  h1 ^= len;
  h2 ^= len;
  h1 += h2;
  h2 += h1;
  h1 = fmix64(h1);
  h2 = fmix64(h2);
  h1 += h2;
  return h1;
}

}  // namespace nvtext_amd

// Character windows of a row, shared by minhash and jaccard_index: a wavefront stages a tile of row bytes
// in LDS with aligned dword loads and decides, per byte position, whether a `width`-character window
// starts there and how many bytes it spans
// (cpp/src/text/minhash.cu:120-133, cpp/src/text/jaccard.cu:268-277, cpp/include/cudf/strings/string_view.cuh:67-80).
#pragma once

#include "common.cuh"
#include "murmur.cuh"

namespace nvtext_amd {

constexpr int kWaves     = 4;                  // wavefronts per workgroup
constexpr int kThreads   = kWaves * kWave;     // 256
constexpr int kTile      = 256;                // window starts per wavefront tile
constexpr int kHalo      = 128;                // bytes staged past the tile (windows up to 32 4-byte chars)
constexpr int kTileWords = (kTile + kHalo + 4 + 24) / 4;  // +4 misalignment, +24 over-read of the hash tail
constexpr int kSpan      = 16384;              // bytes of a row handled by one workgroup

template <typename T>
struct WaveLds {
  uint32_t bytes[kTileWords];
  alignas(16) T hashes[kTile + 4];
};

// Stage row bytes [base, base+len) into dst; returns the byte offset of `base` inside it.
// Only aligned dwords that overlap the range are read.  *all_ascii: no byte of the range
// has its top bit set (wave-uniform).
__device__ __forceinline__ uint32_t stage_bytes(const uint8_t* row, int64_t base, uint32_t len, uint32_t* dst, int lane, bool* all_ascii)
{
  const uint8_t* g   = row + base;
  uint32_t const mis = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(g) & 3u);
  const uint32_t* ap = reinterpret_cast<const uint32_t*>(g - mis);
  uint32_t const end = mis + len;  // exclusive byte offset inside dst
  uint32_t const nw  = (end + 3u) >> 2;
  uint32_t hibits    = 0;
  for (uint32_t i = lane; i < nw; i += kWave) {
    uint32_t const v = ap[i];
    dst[i]           = v;
    uint32_t keep    = 0xffffffffu;
    if (i == 0) keep <<= 8 * mis;                                    // bytes before the range
    if (4 * i + 4 > end) keep &= (1u << (8 * (end - 4 * i))) - 1u;    // bytes after the range
    hibits |= v & keep & 0x80808080u;
  }
  *all_ascii = ballot64(hibits != 0) == 0;
  return mis;
}

// Decides whether a window starts at this position and how many bytes it hashes
// (cpp/src/text/minhash.cu:120-133 with cpp/include/cudf/strings/string_view.cuh:67-80).
// `remaining` = row bytes from this position on; `readable` = bytes of them reachable through src
// (the whole rest of the row, or at least 4 * width bytes); `g` = this position in the row itself.
template <typename Src>
__device__ __forceinline__ bool window_at(Src const& src, const uint8_t* g, int64_t remaining, uint32_t readable, bool first, bool all_ascii,
                                          int32_t width, uint32_t* hlen)
{
  if (all_ascii) {
    if (remaining >= width) {
      *hlen = static_cast<uint32_t>(width);
      return true;
    }
    *hlen = static_cast<uint32_t>(remaining);
    return first;
  }
  if (is_utf8_continuation(src.byte(0))) return false;
  uint32_t bytes = 0, j = 0;
  int32_t left = width;
  while (left > 0 && j < readable) {  // byte-wise, as the reference walks
    int const w = bytes_in_utf8_byte(src.byte(j));
    left -= (w != 0);
    bytes += w;
    ++j;
  }
  // Well-formed text has `width` characters within 4 * width bytes.  Bytes that continue no character count for
  // nothing, so a run of them can leave characters to find beyond what src reaches: the walk goes on in the row.
  if (left > 0 && j < remaining) {
    int64_t k = j;
    while (left > 0 && k < remaining) {
      int const w = bytes_in_utf8_byte(g[k]);
      left -= (w != 0);
      bytes += w;
      ++k;
    }
  }
  // a malformed trailing lead byte may declare more bytes than the row holds: clamp to the row
  *hlen = static_cast<uint32_t>(min(static_cast<int64_t>(bytes), remaining));
  return first || left <= 0;
}

}  // namespace nvtext_amd

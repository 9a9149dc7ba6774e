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

// Windows repeat (text repeats its words: a tenth of the windows of a tile, a third within 4 KB of ordinary text), and a
// hash that has been folded once changes no minimum when it is folded again.  Every wavefront keeps the hashes it
// saw last in a small direct-mapped table and drops a hash that it finds there; what the table has forgotten is folded
// again, which costs time and nothing else.  Cleared (hashes are never 0) whenever the wavefront begins a row.
template <typename T>
constexpr int recent_entries() { return 256; }  // (512 costs the kernels a workgroup per CU: slower but for the longest rows)

template <typename T>
struct WaveLds {
  uint32_t bytes[kTileWords];
  alignas(16) T hashes[kTile + 4];
  alignas(16) T recent[recent_entries<T>()];
  uint32_t chars[kTile + kHalo];  // the characters that start in the staged bytes, in order: start | end << 16 (see CharMap)
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

// The characters of the staged bytes of a tile, found by the whole wavefront at once, for tiles that hold bytes beyond
// ASCII.  The reference walks from every window start byte by byte, adding up what each first byte of a character
// says of its length until `width` characters are counted (cpp/include/cudf/strings/string_view.cuh:67-80).  Where
// every character of the staged bytes ends exactly where the next one starts, that sum is the distance from the start
// of character k to the end of character k + width - 1: the characters are listed in LDS (start | end << 16, in
// order), a lane takes a character instead of a byte position, and a window costs two reads of the list.  Other tiles
// (stray continuation bytes, first bytes that promise more than follows) keep the walk.
struct CharMap {
  uint32_t count;    // characters that start in the staged bytes
  uint32_t windows;  // of them, in the tile's window starts (the first `cnt` staged bytes)
  bool exact;        // the list gives every window of the tile its length
  bool at_row_end;   // the staged bytes reach the end of the row

  // staged: the tile's bytes in LDS, its first byte at byte offset `mis`; len of them are the row's, the first cnt are
  // window starts; chars: the list (room for a character per staged byte).
  __device__ __forceinline__ void build(const uint32_t* staged, uint32_t mis, uint32_t len, uint32_t cnt, bool reaches_row_end, uint32_t* chars,
                                        int lane)
  {
    const uint8_t* const sb = reinterpret_cast<const uint8_t*>(staged) + mis;
    at_row_end              = reaches_row_end;
    count                   = 0;
    windows                 = 0;
    for (uint32_t base = 0; base < len; base += kWave) {
      uint32_t const pos   = base + static_cast<uint32_t>(lane);
      uint32_t const b     = pos < len ? sb[pos] : 0x80u;
      bool const start     = !is_utf8_continuation(b);
      uint64_t const found = ballot64(start);
      if (start) chars[count + lanes_below(found)] = pos | ((pos + static_cast<uint32_t>(bytes_in_utf8_byte(b))) << 16);
      count += static_cast<uint32_t>(__builtin_popcountll(found));
      if (base < cnt) windows += static_cast<uint32_t>(__builtin_popcountll(ballot64(start && pos < cnt)));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // every character but the first begins where the one before it ends
    bool broken = false;
    for (uint32_t k0 = 0; k0 < count; k0 += kWave) {
      uint32_t const k = k0 + static_cast<uint32_t>(lane);
      if (k >= 1 && k < count) broken = broken || (chars[k - 1] >> 16) != (chars[k] & 0xFFFFu);
    }
    // the last one: ends with the row, or, when the row goes on, begins in the last four staged bytes (then every window
    // start of the tile, at least 4 * width bytes before the end of the staged bytes, has its `width` characters listed)
    bool tail = false;
    if (count > 0) {
      uint32_t const last = chars[count - 1];
      tail                = reaches_row_end ? (last >> 16) == len : len - (last & 0xFFFFu) <= 4u;
    }
    exact = tail && ballot64(broken) == 0;
  }

  // The window that begins with character k (k < windows): whether it counts, where it starts and its bytes.
  // row_start: staged byte 0 is the row's first byte.
  __device__ __forceinline__ bool window(uint32_t k, uint32_t len, bool row_start, int32_t width, const uint32_t* chars, uint32_t* pos,
                                         uint32_t* hlen) const
  {
    uint32_t const first = chars[k] & 0xFFFFu;
    *pos                 = first;
    if (k + static_cast<uint32_t>(width) <= count) {
      *hlen = (chars[k + static_cast<uint32_t>(width) - 1u] >> 16) - first;
      return true;
    }
    // fewer than `width` characters are left (the staged bytes reach the end of the row): only the row's first position counts
    *hlen = len - first;
    return row_start && first == 0;
  }
};

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

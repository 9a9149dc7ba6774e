// nvtext::normalize_characters for gfx950: the BERT basic-tokenizer clean-up of a strings column
// (cpp/src/text/normalize.cu:219-573).
//
// The reference expands every input byte into three uint32 slots in global memory, fixes the special tokens up
// in a second kernel, reduces the slots to row sizes and compacts them.  Here a workgroup takes a tile of
// 2048 input bytes (plus a few either side), each lane keeps the slots of eight consecutive bytes in registers,
// and the column is walked twice: once to learn how many bytes each tile produces, once to write them,
// coalesced, at the offsets a scan of those counts gives.  HBM sees the input twice and the output once; the
// slots never leave the CU.
#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "common.cuh"

struct nvtext_amd_character_normalizer {
  int device            = 0;
  int32_t do_lower      = 0;
  uint32_t* ascii       = nullptr;  // device, 128: slot 0 | slot 1 << 8 | slot 2 << 16 | bytes << 24 of the code points below 0x80
  uint4* bmp            = nullptr;  // device, 65536: {slot 0, slot 1, slot 2, bytes} of the code points below 0x10000
  uint32_t* entries     = nullptr;  // device, kCodepoints: category << 24 | multi << 23 | replacement
  uint64_t* second      = nullptr;  // device, kCodepoints: second << 32 | third replacement code point
  uint8_t* token_chars  = nullptr;  // device: the special tokens, sorted then lower-cased
  int32_t* token_offset = nullptr;  // device, tokens + 1
  int32_t tokens        = 0;
  nvtext_amd::DeviceStore store;    // all of the above, from the allocator given at creation
};

namespace nvtext_amd {
namespace {

#include "codepoint_tables.inc"

constexpr uint32_t kCodepoints   = 0x110000;
constexpr uint32_t kDefaultEntry = 5u << 24;

// categories of an entry (cpp/src/text/detail/cp_data.h, read through the accessors of normalize.cu:44-98)
constexpr uint32_t kPad = 0, kPadIfLower = 1, kRemove = 2, kRemoveIfLower = 3, kReplace = 4;

constexpr int kNormThreads = 256;
constexpr int kNormItems   = 8;     // consecutive input bytes per lane
constexpr int kNormTile    = kNormThreads * kNormItems;  // input bytes per workgroup
constexpr int kBefore      = 5;   // a '[' this many bytes before the tile can still change the tile's slots
constexpr int kAfter       = 6;   // a '[' of the tile reads slots this many bytes past it
constexpr int kSlotBase    = 8;   // index of the tile's first position in the slot arrays (>= kBefore; 8 keeps a lane's bytes aligned)
constexpr int kSlots       = kSlotBase + kNormTile + 8;
constexpr int kRawBefore   = 8;   // bytes staged before the tile (>= kBefore)
constexpr int kRawAfter    = 12;  // bytes staged after it (>= kAfter + 3 for the longest character)
constexpr int kRawWords    = (kNormTile + kRawBefore + kRawAfter + 15 + 15) / 16 * 4;  // whole 16-byte blocks, any alignment
constexpr int kStageBytes  = 4 * kNormTile;  // output bytes of a tile that are assembled in LDS; a tile with more writes them one by one

struct NormTables {
  const uint32_t* ascii;  // 128 entries: the slots of the code points below 0x80
  const uint4* bmp;       // 65536 entries: the three slots and their bytes together, of the code points below 0x10000
  const uint32_t* entries;
  const uint64_t* second;
  const uint8_t* token_chars;
  const int32_t* token_offset;
  int32_t tokens;
  int32_t do_lower;
};

// cudf::strings::detail::codepoint_to_utf8 then from_char_utf8 (cpp/include/cudf/strings/detail/utf8.hpp:170-197,
// 143-168): the bytes of the character, first byte in the low bits, as the reference leaves them in a slot.
__host__ __device__ __forceinline__ uint32_t utf8_le(uint32_t cp)
{
  if (cp < 0x80u) return cp;
  uint32_t const t0 = 0x80u | (cp & 0x3Fu);
  uint32_t const t1 = 0x80u | ((cp >> 6) & 0x3Fu);
  if (cp < 0x800u) return (0xC0u | (cp >> 6)) | (t0 << 8);
  uint32_t const t2 = 0x80u | ((cp >> 12) & 0x3Fu);
  if (cp < 0x10000u) return (0xE0u | (cp >> 12)) | (t1 << 8) | (t0 << 16);
  return (0xF0u | ((cp >> 18) & 0x07u)) | (t2 << 8) | (t1 << 16) | (t0 << 24);
}

__host__ __device__ __forceinline__ uint32_t bytes_of(uint32_t slot)
{
#ifdef __HIP_DEVICE_COMPILE__
  return (39u - static_cast<uint32_t>(__clz(slot))) >> 3;
#else
  return (slot != 0) + (slot > 0xFFu) + (slot > 0xFFFFu) + (slot > 0xFFFFFFu);
#endif
}

// The code point of the character that starts with b0, the next bytes being b1..b3
// (to_char_utf8 and utf8_to_codepoint, cpp/include/cudf/strings/detail/utf8.hpp:68-97,118-140: the first byte
// alone says how many bytes belong to the character).
__device__ __forceinline__ uint32_t decode(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3)
{
  if (b0 < 0x80u) return b0;
  if (b0 < 0xE0u) return ((b0 & 0x1Fu) << 6) | (b1 & 0x3Fu);
  if (b0 < 0xF0u) return ((b0 & 0x0Fu) << 12) | ((b1 & 0x3Fu) << 6) | (b2 & 0x3Fu);
  // packed value above 0xF8000000 decodes to 0
  uint32_t const packed = (b0 << 24) | (b1 << 16) | (b2 << 8) | b3;
  if (packed > 0xF8000000u) return 0u;
  return ((b0 & 0x07u) << 18) | ((b1 & 0x3Fu) << 12) | ((b2 & 0x3Fu) << 6) | (b3 & 0x3Fu);
}

// The slots of one code point (data_normalizer_kernel, cpp/src/text/normalize.cu:331-378).
__host__ __device__ __forceinline__ void slots_of(uint32_t cp, NormTables const& t, uint32_t& s0, uint32_t& s1, uint32_t& s2)
{
  s0 = s1 = s2       = 0;
  uint32_t const e   = cp < kCodepoints ? t.entries[cp] : kDefaultEntry;
  uint32_t const cat = (e >> 24) & 7u;
  bool const lower   = t.do_lower != 0;
  if (cat == kRemove || (lower && cat == kRemoveIfLower)) return;
  uint32_t const repl = (lower || cat == kReplace) ? (e & 0x1FFFFFu) : cp;
  uint32_t const r0   = repl ? repl : cp;
  if (lower && ((e >> 23) & 1u)) {  // two or three code points, never padded
    uint64_t const next = t.second[cp];
    uint32_t const r1 = static_cast<uint32_t>(next >> 32), r2 = static_cast<uint32_t>(next);
    s0 = utf8_le(r0);
    s1 = r1 ? utf8_le(r1) : 0u;
    s2 = r2 ? utf8_le(r2) : 0u;
    return;
  }
  uint32_t const one = utf8_le(r0);
  if (cat == kPad || (lower && cat == kPadIfLower)) {
    s0 = s2 = 0x20u;
    s1      = one;
  } else {
    s0 = one;
  }
}

constexpr int kWaveLeads = 256;  // first bytes of longer characters per wavefront (512 input bytes) that the counting pass lists

template <bool SLOTS>
struct NormLds {
  alignas(16) uint32_t raw[kRawWords];  // the input bytes of the tile and its surroundings, zero outside the column
  uint32_t ascii[128];                 // code points below 0x80: slot 0 | slot 1 << 8 | slot 2 << 16 | bytes << 24
  union {
    // first byte of slot k of tile position i - kSlotBase; only filled where special tokens can be.  A first byte
    // tells '[', ']', a space and a-z from everything else, which is all the special tokens look at or change.
    alignas(8) uint8_t slot[3][kSlots];
    uint32_t staged[(kStageBytes + 8) / 4 + 4];  // afterwards: the tile's output bytes (and room for the dwords of a string that starts at the last one)
  };
  union {
    alignas(16) uint16_t prefix[kNormTile + 8];  // bytes the tile writes before each position; [tile] = all of them
    uint16_t lead_pos[kNormThreads / kWave][kWaveLeads];  // (before that: the tile positions of the first bytes of a wavefront's longer characters)
  };
  uint32_t scan[kNormThreads / kWave + 1];
  uint32_t bracket;  // some lane of the tile saw what can open a special token
};

// The slots of the tile positions a lane owns (kNormItems * lane ..): consecutive bytes in, consecutive bytes out.
struct Owned {
  uint32_t s[kNormItems][3];
};

// Slot `at` of the flat slot sequence (three per position).
template <bool S>
__device__ __forceinline__ uint8_t& flat_slot(NormLds<S>& lds, int at) { return lds.slot[at % 3][at / 3]; }

// Compares the candidate in flat slots [from, to] (spaces and empty slots skipped, one byte per character) with
// special token `i`: < 0, 0, > 0 as the candidate sorts before, equal to or after it.
template <bool S>
__device__ int compare_candidate(NormLds<S>& lds, int from, int to, NormTables const& t, int32_t i)
{
  const uint8_t* tok = t.token_chars + t.token_offset[i];
  int32_t const tl   = t.token_offset[i + 1] - t.token_offset[i];
  int32_t j          = 0;
  for (int at = from; at <= to; ++at) {
    uint32_t const c = flat_slot(lds, at);
    if (c == 0u || c == 0x20u) continue;
    if (j >= tl) return 1;
    uint32_t const b = tok[j++];
    if (c != b) return c < b ? -1 : 1;
  }
  return j < tl ? -1 : 0;
}

__device__ __forceinline__ bool has_byte(uint32_t v, uint32_t byte)
{
  uint32_t const x = v ^ (byte * 0x01010101u);
  return ((x - 0x01010101u) & ~x & 0x80808080u) != 0u;
}

// Whether a special token opens at slot index i (its slot 1 holds '['): the flat slot of its ']' if so, else -1.
// special_tokens_kernel, cpp/src/text/normalize.cu:283-301.
template <bool S>
__device__ int token_opens_at(NormLds<S>& lds, NormTables const& t, int i)
{
  if (lds.slot[1][i] != '[') return -1;
  int const from = 3 * i + 1;
  int to         = -1;
  for (int at = from + 1; at < from + 18; ++at) {
    if (flat_slot(lds, at) == ']') {
      to = at;
      break;
    }
  }
  if (to < 0) return -1;
  int32_t first = 0, count = t.tokens;  // thrust::binary_search: lower_bound by halving, then !(value < *it)
  while (count > 0) {
    int32_t const half = count >> 1;
    if (compare_candidate(lds, from, to, t, first + half) > 0) {
      first += half + 1;
      count -= half + 1;
    } else {
      count = half;
    }
  }
  if (first >= t.tokens || compare_candidate(lds, from, to, t, first) < 0) return -1;
  return to;
}

// special_tokens_kernel (normalize.cu:270-316) over lds.slot, in two steps so that every decision reads unchanged
// slots.  A lane looks at its own positions; the first kBefore lanes also at the positions before the tile (a '['
// in the positions after the tile belongs to the next tile).
template <bool S>
__device__ void apply_special_tokens(NormLds<S>& lds, NormTables const& t)
{
  int const tid = threadIdx.x;
  int found_to[kNormItems + 1];
#pragma unroll
  for (int k = 0; k <= kNormItems; ++k) {
    int const i = k < kNormItems ? kSlotBase + kNormItems * tid + k : kSlotBase - kBefore + tid;
    found_to[k] = (k < kNormItems || tid < kBefore) ? token_opens_at(lds, t, i) : -1;
  }
  lds_barrier();
#pragma unroll
  for (int k = 0; k <= kNormItems; ++k) {
    if (found_to[k] < 0) continue;
    int const i    = k < kNormItems ? kSlotBase + kNormItems * tid + k : kSlotBase - kBefore + tid;
    int const from = 3 * i + 1;
    flat_slot(lds, from + 1)        = 0u;  // the space after '['
    flat_slot(lds, found_to[k] - 1) = 0u;  // the space before ']'
    if (t.do_lower) {
      for (int at = from + 2; at < found_to[k] - 2; ++at) {
        uint32_t const c = flat_slot(lds, at);
        if (c >= 'a' && c <= 'z') flat_slot(lds, at) = static_cast<uint8_t>(c - 'a' + 'A');
      }
    }
  }
  lds_barrier();
}

// Code point of a character of two or three bytes whose bytes start `w` (first byte below 0xF0): decode() without
// its branches.
__device__ __forceinline__ uint32_t decode_short(uint32_t w)
{
  uint32_t const b1    = (w >> 8) & 0x3Fu;
  uint32_t const two   = ((w & 0x1Fu) << 6) | b1;
  uint32_t const three = ((w & 0x0Fu) << 12) | (b1 << 6) | ((w >> 16) & 0x3Fu);
  return (w & 0xFFu) < 0xE0u ? two : three;
}

// Slots of the character whose bytes start `w` (first byte in the low bits) and the bytes they hold together.  The
// Basic Multilingual Plane has them ready in one 16-byte table entry; the rest goes through the code point tables.
__device__ __forceinline__ uint32_t wide_slots(uint32_t w, NormTables const& t, uint32_t& s0, uint32_t& s1, uint32_t& s2)
{
  uint32_t cp = decode_short(w);
  if ((w & 0xFFu) >= 0xF0u) {  // four bytes (seldom)
    cp = decode(w & 0xFFu, (w >> 8) & 0xFFu, (w >> 16) & 0xFFu, w >> 24);
    if (cp >= 0x10000u) {
      slots_of(cp, t, s0, s1, s2);
      return bytes_of(s0) + bytes_of(s1) + bytes_of(s2);
    }
  }
  uint4 const e = t.bmp[cp];
  s0            = e.x;
  s1            = e.y;
  s2            = e.z;
  return e.w;
}

// Bytes that the character whose bytes start `w` produces, without its slots.
__device__ __forceinline__ uint32_t wide_size(uint32_t w, NormTables const& t)
{
  uint32_t cp = decode_short(w);
  if ((w & 0xFFu) >= 0xF0u) {
    cp = decode(w & 0xFFu, (w >> 8) & 0xFFu, (w >> 16) & 0xFFu, w >> 24);
    if (cp >= 0x10000u) {
      uint32_t s0, s1, s2;
      slots_of(cp, t, s0, s1, s2);
      return bytes_of(s0) + bytes_of(s1) + bytes_of(s2);
    }
  }
  return t.bmp[cp].w;
}

// The slots (and sizes) of the eight positions whose bytes are lo64; hi64 = bytes 4..11.  Returns the bytes they produce.
template <bool S>
__device__ __forceinline__ uint32_t owned_slots(NormLds<S> const& lds, uint64_t lo64, uint64_t hi64, NormTables const& t, Owned& mine,
                                                uint32_t (&size)[kNormItems])
{
  uint32_t sum = 0;
  // one-byte characters through the table; continuation bytes give nothing
#pragma unroll
  for (int j = 0; j < kNormItems; ++j) {
    uint32_t const b = static_cast<uint32_t>(lo64 >> (8 * j)) & 0xFFu;
    uint32_t const e = lds.ascii[b & 0x7Fu];  // read in any case: no branch
    uint32_t const d = b < 0x80u ? e : 0u;
    mine.s[j][0]     = d & 0xFFu;
    mine.s[j][1]     = (d >> 8) & 0xFFu;
    mine.s[j][2]     = (d >> 16) & 0xFFu;
    size[j]          = d >> 24;
    sum += size[j];
  }
  // each first byte of a longer character (seldom more than four in eight bytes) goes through the code point tables
  uint64_t leads = lo64 & (lo64 << 1) & 0x8080808080808080ull;  // bit 7 of the bytes >= 0xC0
  while (leads) {
    int const at = (__ffsll(static_cast<long long>(leads)) - 1) >> 3;
    leads &= leads - 1ull;
    uint32_t const w = static_cast<uint32_t>((at < 4 ? lo64 : hi64) >> (8 * (at & 3)));
    uint32_t s0, s1, s2;
    uint32_t const bytes = wide_slots(w, t, s0, s1, s2);
    sum += bytes;
    // (as bit masks: written as "if (j == at)", the eight cases become a tree of branches, which lanes with
    // different `at` walk one leaf after the other)
#pragma unroll
    for (int j = 0; j < kNormItems; ++j) {
      uint32_t const here = static_cast<uint32_t>((static_cast<int32_t>(j ^ at) - 1) >> 31);  // all ones where j == at
      mine.s[j][0] = (mine.s[j][0] & ~here) | (s0 & here);
      mine.s[j][1] = (mine.s[j][1] & ~here) | (s1 & here);
      mine.s[j][2] = (mine.s[j][2] & ~here) | (s2 & here);
      size[j]      = (size[j] & ~here) | (bytes & here);
    }
  }
  return sum;
}

// The bytes of up to three slots side by side, first slot first: (lo, hi) = bytes 0..7 and 8..11.
__device__ __forceinline__ void slots_to_string(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t& d0, uint32_t& d1, uint32_t& d2)
{
  uint32_t const b0  = bytes_of(s0);
  uint32_t const b01 = b0 + bytes_of(s1);  // <= 8
  uint64_t lo        = s0 | (static_cast<uint64_t>(s1) << (8u * b0));
  uint64_t const t   = s2;
  uint32_t const sh  = 8u * b01;
  lo |= b01 < 8u ? t << (sh & 63u) : 0ull;
  d2 = b01 >= 8u ? s2 : b01 > 4u ? static_cast<uint32_t>(t >> ((64u - sh) & 63u)) : 0u;
  d0 = static_cast<uint32_t>(lo);
  d1 = static_cast<uint32_t>(lo >> 32);
}

// owned_slots for the pass that writes: what each position turns into as a string of bytes (mine.s[j][0..2] = bytes
// 0..11, zero padded) instead of slots, ready to be placed.
template <bool S>
__device__ __forceinline__ uint32_t owned_strings(NormLds<S> const& lds, uint64_t lo64, uint64_t hi64, NormTables const& t, Owned& mine,
                                                  uint32_t (&size)[kNormItems])
{
  uint32_t sum = 0;
#pragma unroll
  for (int j = 0; j < kNormItems; ++j) {
    uint32_t const b = static_cast<uint32_t>(lo64 >> (8 * j)) & 0xFFu;
    uint32_t const e = lds.ascii[b & 0x7Fu];  // read in any case: no branch
    uint32_t const d = b < 0x80u ? e : 0u;
    mine.s[j][0]     = d & 0xFFFFFFu;  // one byte per slot, empty slots last: the slots side by side are the string
    mine.s[j][1]     = 0u;
    mine.s[j][2]     = 0u;
    size[j]          = d >> 24;
    sum += size[j];
  }
  uint64_t leads = lo64 & (lo64 << 1) & 0x8080808080808080ull;  // bit 7 of the bytes >= 0xC0
  while (leads) {
    int const at = (__ffsll(static_cast<long long>(leads)) - 1) >> 3;
    leads &= leads - 1ull;
    uint32_t const w = static_cast<uint32_t>((at < 4 ? lo64 : hi64) >> (8 * (at & 3)));
    uint32_t s0, s1, s2, d0, d1, d2;
    uint32_t const bytes = wide_slots(w, t, s0, s1, s2);
    slots_to_string(s0, s1, s2, d0, d1, d2);
    sum += bytes;
#pragma unroll
    for (int j = 0; j < kNormItems; ++j) {
      uint32_t const here = static_cast<uint32_t>((static_cast<int32_t>(j ^ at) - 1) >> 31);  // all ones where j == at
      mine.s[j][0] = (mine.s[j][0] & ~here) | (d0 & here);
      mine.s[j][1] = (mine.s[j][1] & ~here) | (d1 & here);
      mine.s[j][2] = (mine.s[j][2] & ~here) | (d2 & here);
      size[j]      = (size[j] & ~here) | (bytes & here);
    }
  }
  return sum;
}

__device__ __forceinline__ void wave_lds_sync()
{
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The bytes that the wavefront's 512 positions produce, for the pass that only sizes the output (a lane's return value
// holds the sizes of characters that are not its own: only the sum over the wavefront means something).
// One-byte characters go through the table in LDS, lanes <-> bytes.  The first bytes of longer characters are few
// and unevenly spread (none in English text, every other byte in Cyrillic or Greek), and each needs a read of the
// code point tables: the wavefront lists them and goes through the list lanes <-> characters, every lane at work.
// `byte0` = the byte offset in lds.raw of the tile's first byte.
template <bool SLOTS>
__device__ __forceinline__ uint32_t owned_dense(NormLds<SLOTS>& lds, uint64_t lo64, uint64_t hi64, uint32_t byte0, NormTables const& t)
{
  uint32_t sum = 0;
#pragma unroll
  for (int j = 0; j < kNormItems; ++j) {
    uint32_t const b = static_cast<uint32_t>(lo64 >> (8 * j)) & 0xFFu;
    uint32_t const e = lds.ascii[b & 0x7Fu];  // read in any case: no branch
    sum += b < 0x80u ? e >> 24 : 0u;
  }
  uint64_t const leads  = lo64 & (lo64 << 1) & 0x8080808080808080ull;  // bit 7 of the bytes >= 0xC0
  uint32_t const mine_n = static_cast<uint32_t>(__builtin_popcountll(leads));
  uint32_t const incl   = wave_inclusive_scan(mine_n);
  uint32_t const first  = incl - mine_n;
  uint32_t const all    = wave_bcast(incl, kWave - 1);
  if (all == 0) return sum;
  if (all > static_cast<uint32_t>(kWaveLeads)) {
    // more than every other byte begins a character: not text; every lane walks its own
    uint64_t l = leads;
    while (l) {
      int const at = (__ffsll(static_cast<long long>(l)) - 1) >> 3;
      l &= l - 1ull;
      sum += wide_size(static_cast<uint32_t>((at < 4 ? lo64 : hi64) >> (8 * (at & 3))), t);
    }
    return sum;
  }
  int const lane       = lane_id();
  uint16_t* const list = lds.lead_pos[threadIdx.x / kWave];
  {
    uint32_t i = first;
#pragma unroll
    for (int j = 0; j < kNormItems; ++j) {
      bool const is = ((leads >> (8 * j + 7)) & 1ull) != 0;
      if (is) list[i] = static_cast<uint16_t>(kNormItems * threadIdx.x + j);
      i += is ? 1u : 0u;
    }
  }
  wave_lds_sync();
  for (uint32_t r = lane; r < all; r += kWave) {
    uint32_t const off = byte0 + list[r];
    uint32_t const w   = __builtin_amdgcn_alignbit(lds.raw[(off >> 2) + 1], lds.raw[off >> 2], 8u * (off & 3u));
    sum += wide_size(w, t);
  }
  return sum;
}

// One tile: the slots of the lane's positions, special tokens applied.  Returns the bytes they produce.  Without
// SLOTS only that number is wanted: the slots are then built only in tiles that may hold a special token.
template <bool SLOTS>
__device__ __forceinline__ uint32_t tile_slots(NormLds<SLOTS>& lds, const uint8_t* chars, int64_t t0, int64_t n, NormTables const& t, Owned& mine,
                                               uint32_t (&size)[kNormItems])
{
  int const tid = threadIdx.x;
  // stage [t0 - kRawBefore, t0 + kNormTile + kRawAfter) with one aligned 16-byte load per lane (the first 131 lanes);
  // bytes outside [0, n) read as 0.  Everything is requested before anything is waited for.
  uint32_t const table_entry = tid < 128 ? t.ascii[tid] : 0u;
  const uint8_t* const wb    = chars + t0 - kRawBefore;
  uint32_t const mis         = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(wb) & 15u);
  if (tid < kRawWords / 4) {
    int64_t const p = t0 - kRawBefore - mis + 16 * static_cast<int64_t>(tid);  // column position of the block's first byte
    uint4 v         = make_uint4(0u, 0u, 0u, 0u);
    if (p + 15 >= 0 && p < n) {
      v = load_stream(reinterpret_cast<const uint4*>(wb - mis) + tid);
      if (p < 0 || p + 16 > n) {  // the first or the last block of the column: clear what lies outside
        uint32_t* const part = &v.x;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          int64_t const q = p + 4 * k;
          uint32_t keep   = 0xFFFFFFFFu;
          if (q < 0) keep = q <= -4 ? 0u : keep << (8 * static_cast<uint32_t>(-q));
          if (q + 4 > n) keep = q >= n ? 0u : keep & (0xFFFFFFFFu >> (8 * static_cast<uint32_t>(q + 4 - n)));
          part[k] &= keep;
        }
      }
    }
    *reinterpret_cast<uint4*>(&lds.raw[4 * tid]) = v;
  }
  if (tid < 128) lds.ascii[tid] = table_entry;
  if (tid == 0) lds.bracket = 0u;
  lds_barrier();

  // the lane's eight bytes and the four after them, whatever the alignment of the tile in memory
  uint32_t const shift = 8u * (mis & 3u);
  int const word       = static_cast<int>((mis + kRawBefore) >> 2) + 2 * tid;
  uint32_t const r0 = lds.raw[word], r1 = lds.raw[word + 1], r2 = lds.raw[word + 2], r3 = lds.raw[word + 3];
  uint32_t const own0 = __builtin_amdgcn_alignbit(r1, r0, shift);
  uint32_t const own1 = __builtin_amdgcn_alignbit(r2, r1, shift);
  uint32_t const next = __builtin_amdgcn_alignbit(r3, r2, shift);
  uint64_t const lo64 = (static_cast<uint64_t>(own1) << 32) | own0;
  uint64_t const hi64 = (static_cast<uint64_t>(next) << 32) | own1;
  // (the pass that wants the slots keeps them in registers all the way: listing the longer characters for it as well
  // saves it 4 % of its instructions and costs it two of its seven wavefronts per SIMD, 8.6 -> 10.7 ms on the
  // multilingual workload; the pass that only counts gains 13 % from the list)
  uint32_t sum;
  if constexpr (SLOTS) sum = owned_strings(lds, lo64, hi64, t, mine, size);
  else sum = owned_dense(lds, lo64, hi64, mis + kRawBefore, t);

  if (t.tokens > 0) {
    // A special token starts at a position whose slot 1 is '['.  Tiles without one skip the exchange through LDS.
    // No code point's replacement is a '[', so it takes a '[' byte or an over-long encoding of it, which starts
    // with 0xC1, 0xE0 or 0xF0: that is what decides for the positions before the tile (eight looked at, five
    // needed) and, when the slots have not been built, for the lane's own bytes (a superset, which is harmless).
    bool bracket = false;
    if (SLOTS) {
      // (strings: a '[' is padded like all punctuation, so it is the middle byte of " [ ")
#pragma unroll
      for (int j = 0; j < kNormItems; ++j) bracket |= ((mine.s[j][0] >> 8) & 0xFFu) == '[';
    } else {
      bracket = has_byte(own0, '[') || has_byte(own1, '[');
      if ((lo64 & (lo64 << 1) & 0x8080808080808080ull) != 0)
        bracket = bracket || has_byte(own0, 0xC1u) || has_byte(own0, 0xE0u) || has_byte(own0, 0xF0u) || has_byte(own1, 0xC1u) ||
                  has_byte(own1, 0xE0u) || has_byte(own1, 0xF0u);
    }
    if (tid < 2) {
      int const at     = static_cast<int>(mis >> 2) + tid;
      uint32_t const v = __builtin_amdgcn_alignbit(lds.raw[at + 1], lds.raw[at], shift);
      bracket          = bracket || has_byte(v, '[') || has_byte(v, 0xC1u) || has_byte(v, 0xE0u) || has_byte(v, 0xF0u);
    }
    if (ballot64(bracket) != 0 && lane_id() == 0) lds.bracket = 1u;
    lds_barrier();
    if (lds.bracket != 0u) {
      owned_slots(lds, lo64, hi64, t, mine, size);  // (the slots themselves, whatever mine held)
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        uint32_t a = 0, b = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          a |= (mine.s[j][k] & 0xFFu) << (8 * j);
          b |= (mine.s[j + 4][k] & 0xFFu) << (8 * j);
        }
        *reinterpret_cast<uint2*>(&lds.slot[k][kSlotBase + kNormItems * tid]) = make_uint2(a, b);
      }
      if (tid < kBefore + kAfter) {  // the positions either side of the tile
        int const pos             = tid < kBefore ? tid - kBefore : kNormTile + tid - kBefore;
        const uint8_t* const rawb = reinterpret_cast<const uint8_t*>(lds.raw) + mis + kRawBefore + pos;
        uint32_t const b0         = rawb[0];
        uint32_t s0 = 0, s1 = 0, s2 = 0;
        if (b0 < 0x80u) {
          uint32_t const d = lds.ascii[b0];
          s0               = d & 0xFFu;
          s1               = (d >> 8) & 0xFFu;
          s2               = (d >> 16) & 0xFFu;
        } else if (b0 >= 0xC0u) {
          wide_slots(b0 | (static_cast<uint32_t>(rawb[1]) << 8) | (static_cast<uint32_t>(rawb[2]) << 16) | (static_cast<uint32_t>(rawb[3]) << 24),
                     t, s0, s1, s2);
        }
        lds.slot[0][kSlotBase + pos] = static_cast<uint8_t>(s0);
        lds.slot[1][kSlotBase + pos] = static_cast<uint8_t>(s1);
        lds.slot[2][kSlotBase + pos] = static_cast<uint8_t>(s2);
      }
      lds_barrier();
      apply_special_tokens(lds, t);
      // the tokens only ever empty a slot or turn its letter into upper case: take over the first bytes that changed
      sum = 0;
#pragma unroll
      for (int j = 0; j < kNormItems; ++j) {
#pragma unroll
        for (int k = 0; k < 3; ++k) {
          uint32_t const now = lds.slot[k][kSlotBase + kNormItems * tid + j];
          if (now != (mine.s[j][k] & 0xFFu)) mine.s[j][k] = now;
        }
        // keep the filled slots of a position in front (the output is the same): the writer relies on it
#pragma unroll
        for (int again = 0; again < 2; ++again) {
          if (mine.s[j][0] == 0u) {
            mine.s[j][0] = mine.s[j][1];
            mine.s[j][1] = mine.s[j][2];
            mine.s[j][2] = 0u;
          }
        }
        if (mine.s[j][1] == 0u) {
          mine.s[j][1] = mine.s[j][2];
          mine.s[j][2] = 0u;
        }
        size[j] = bytes_of(mine.s[j][0]) + bytes_of(mine.s[j][1]) + bytes_of(mine.s[j][2]);
        sum += size[j];
        if (SLOTS) slots_to_string(mine.s[j][0], mine.s[j][1], mine.s[j][2], mine.s[j][0], mine.s[j][1], mine.s[j][2]);
      }
    }
  }
  return sum;
}

// tile_bytes[tile] = bytes the tile's input positions produce
__global__ void __launch_bounds__(kNormThreads, 8) normalize_count_kernel(const uint8_t* __restrict__ chars, int64_t n, NormTables t,
                                                                       uint32_t* __restrict__ tile_bytes)
{
  __shared__ NormLds<false> lds;
  int64_t const t0 = static_cast<int64_t>(blockIdx.x) * kNormTile;
  Owned mine;
  uint32_t size[kNormItems];
  uint32_t const sum = tile_slots<false>(lds, chars, t0, n, t, mine, size);
  uint32_t total;
  block_exclusive_scan_lds<kNormThreads>(sum, lds.scan, &total);
  if (threadIdx.x == 0) tile_bytes[blockIdx.x] = total;
}

// tile_row[tile] = the first row (of rows + 1: the end counts as one) whose first byte lies at or after the tile's
// first byte.  One thread per tile: the searches of a launch hide each other's latency.
__global__ void __launch_bounds__(256) normalize_tile_rows_kernel(ColView col, int64_t first, int64_t tiles, int32_t* __restrict__ tile_row)
{
  int64_t const tile = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tile >= tiles) return;
  int64_t const t0 = tile * kNormTile;
  int64_t lo = 0, hi = static_cast<int64_t>(col.size) + 1;
  while (lo < hi) {
    int64_t const mid = (lo + hi) >> 1;
    if (col.off(mid) - first < t0) lo = mid + 1;
    else hi = mid;
  }
  tile_row[tile] = static_cast<int32_t>(lo);
}

// Writes the tile's bytes at tile_offset[tile] and the output offset of every row that starts in the tile.
__global__ void __launch_bounds__(kNormThreads) normalize_write_kernel(ColView col, int64_t first, int64_t n, NormTables t,
                                                                       const uint64_t* __restrict__ tile_offset,
                                                                       const int32_t* __restrict__ tile_row, uint8_t* __restrict__ out_chars,
                                                                       void* __restrict__ out_offsets, int offsets_are_int64)
{
  __shared__ NormLds<true> lds;
  int const tid        = threadIdx.x;
  int64_t const t0     = static_cast<int64_t>(blockIdx.x) * kNormTile;
  uint64_t const base  = tile_offset[blockIdx.x];
  // the rows that start in this tile are looked up now; the barriers below do not wait for global loads, so this
  // one is back when the tile is done
  int64_t const rows     = col.size;
  int64_t const my_row   = static_cast<int64_t>(tile_row[blockIdx.x]) + tid;
  // the rows that start in this tile end where the next tile's begin (the last tile also takes the end of the last row)
  int64_t const row_end  = blockIdx.x + 1 == gridDim.x ? rows + 1 : static_cast<int64_t>(tile_row[blockIdx.x + 1]);
  uint32_t start_lo = 0, start_hi = 0;  // the raw offset entry; not touched before the end
  if (my_row <= rows) {
    if (col.is64) {
      uint2 const v = static_cast<const uint2*>(col.offsets)[my_row + col.offset];
      start_lo      = v.x;
      start_hi      = v.y;
    } else {
      start_lo = static_cast<const uint32_t*>(col.offsets)[my_row + col.offset];
    }
  }
  Owned mine;
  uint32_t size[kNormItems];
  uint32_t const sum = tile_slots<true>(lds, col.chars + first, t0, n, t, mine, size);
  // the buffer that the output bytes are assembled in starts out as zeros (the scan's barriers stand between this
  // and the first byte placed); in a tile that went through the special tokens it lies where the slots' first bytes
  // were, which the other wavefronts may still be reading
  if (t.tokens > 0 && lds.bracket != 0u) lds_barrier();
  for (int i = tid; i < static_cast<int>(sizeof(lds.staged) / 16); i += kNormThreads) reinterpret_cast<uint4*>(lds.staged)[i] = make_uint4(0u, 0u, 0u, 0u);
  if (tid < static_cast<int>(sizeof(lds.staged) % 16) / 4) lds.staged[sizeof(lds.staged) / 16 * 4 + tid] = 0u;
  uint32_t total;
  uint32_t const before = block_exclusive_scan_lds<kNormThreads>(sum, lds.scan, &total);
  {
    uint32_t run = before;
    uint32_t packed[kNormItems / 2];
#pragma unroll
    for (int j = 0; j < kNormItems; ++j) {
      if (j & 1) packed[j >> 1] |= run << 16;
      else packed[j >> 1] = run;
      run += size[j];
    }
    *reinterpret_cast<uint4*>(&lds.prefix[kNormItems * tid]) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    if (tid == kNormThreads - 1) lds.prefix[kNormTile] = static_cast<uint16_t>(run);
  }

  uint8_t* const dst = out_chars + base;
  if (total <= static_cast<uint32_t>(kStageBytes)) {
    // the output bytes, laid out in LDS as they will lie in memory relative to an aligned dword.  A slot is stored
    // as one (unaligned) dword wherever the three bytes that may follow it still belong to this lane: later slots
    // overwrite them.  The last slots of the lane go byte by byte.
    uint32_t const lead = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dst) & 3u);
    uint8_t* const sb   = reinterpret_cast<uint8_t*>(lds.staged);
    uint32_t o          = lead + before;
    uint32_t const mine_end = o + sum;
    uint32_t big = 0;
#pragma unroll
    for (int j = 0; j < kNormItems; ++j) big |= (mine.s[j][0] >> 24) | mine.s[j][1] | mine.s[j][2];
    if (ballot64(big != 0u) == 0) {
      // no position of the wavefront turns into more than three bytes: a position's bytes travel together, as one
      // (unaligned) dword whose spare bytes the next positions overwrite.  A position that starts in the lane's last
      // three bytes is skipped; those bytes are kept in `last` (the four bytes written last, newest on top) and
      // stored one by one at the end.
      uint32_t last = 0;
#pragma unroll
      for (int j = 0; j < kNormItems; ++j) {
        uint32_t const three = mine.s[j][0];
        if (size[j] != 0u && o + 4u <= mine_end) __builtin_memcpy(sb + o, &three, 4);
        last = __builtin_amdgcn_alignbit(three, last, 8u * size[j]);
        o += size[j];
      }
      if (sum >= 1u) sb[mine_end - 1u] = static_cast<uint8_t>(last >> 24);
      if (sum >= 2u) sb[mine_end - 2u] = static_cast<uint8_t>(last >> 16);
      if (sum >= 3u) sb[mine_end - 3u] = static_cast<uint8_t>(last >> 8);
    } else {
      // longer strings: every position's bytes (zero padded) are or-ed into the aligned dwords they fall into;
      // the buffer was cleared, and what the neighbours put into a shared dword is theirs
      bool const past8 = ballot64(mine.s[0][2] | mine.s[1][2] | mine.s[2][2] | mine.s[3][2] | mine.s[4][2] | mine.s[5][2] | mine.s[6][2] |
                                  mine.s[7][2]) != 0;
#pragma unroll
      for (int j = 0; j < kNormItems; ++j) {
        uint32_t const sh   = 8u * (o & 3u);
        uint32_t* const at  = lds.staged + (o >> 2);
        uint64_t const a    = static_cast<uint64_t>(mine.s[j][0]) << sh;
        uint64_t const b    = static_cast<uint64_t>(mine.s[j][1]) << sh;
        atomicOr(at, static_cast<uint32_t>(a));
        atomicOr(at + 1, static_cast<uint32_t>(a >> 32) | static_cast<uint32_t>(b));
        atomicOr(at + 2, static_cast<uint32_t>(b >> 32));
        if (past8) {  // (a character that turns into three characters of three bytes, or into characters beyond U+FFFF)
          uint64_t const c = static_cast<uint64_t>(mine.s[j][2]) << sh;
          atomicOr(at + 2, static_cast<uint32_t>(c));
          atomicOr(at + 3, static_cast<uint32_t>(c >> 32));
        }
        o += size[j];
      }
    }
    lds_barrier();
    uint32_t const end  = lead + total;
    uint32_t const w_lo = (lead + 3u) >> 2;
    uint32_t const w_hi = end >> 2;
    uint32_t* const dw  = reinterpret_cast<uint32_t*>(dst - lead);
    for (uint32_t w = w_lo + tid; w < w_hi; w += kNormThreads) store_stream(dw + w, lds.staged[w]);
    uint32_t const head_end   = min(4u * w_lo, end);
    uint32_t const tail_begin = max(4u * w_hi, head_end);
    if (tid < 4) {
      uint32_t const at = lead + tid;
      if (at < head_end) (dst - lead)[at] = sb[at];
    } else if (tid < 8) {
      uint32_t const at = tail_begin + (tid - 4);
      if (at < end) (dst - lead)[at] = sb[at];
    }
  } else {
    // more than four output bytes per input byte (only input that is not UTF-8 gets there): byte by byte
    uint8_t* o = dst + before;
#pragma unroll
    for (int j = 0; j < kNormItems; ++j)
      for (uint32_t k = 0; k < size[j]; ++k) *o++ = static_cast<uint8_t>((k < 4 ? mine.s[j][0] : k < 8 ? mine.s[j][1] : mine.s[j][2]) >> (8u * (k & 3u)));
    lds_barrier();  // lds.prefix is complete for the rows below
  }

  // rows whose first byte lies in [t0, t1) -- in [t0, n] for the last tile -- start at base + prefix
  int64_t const my_start = (col.is64 ? static_cast<int64_t>((static_cast<uint64_t>(start_hi) << 32) | start_lo)
                                     : static_cast<int64_t>(static_cast<int32_t>(start_lo))) - first;
  for (int64_t r = my_row; r < row_end; r += kNormThreads) {  // (more than one trip only in a tile of very short rows)
    int64_t const p = r == my_row ? my_start : col.off(r) - first;
    uint64_t const at = base + lds.prefix[p - t0];
    if (offsets_are_int64) static_cast<int64_t*>(out_offsets)[r] = static_cast<int64_t>(at);
    else static_cast<int32_t*>(out_offsets)[r] = static_cast<int32_t>(at);
  }
}

struct TileBytes {
  const uint32_t* counts;
  __device__ uint64_t operator()(int64_t i) const { return counts[i]; }
};

// ------------------------------------------------------------------ host: tables and tokens
void append_utf8(std::string& s, uint32_t cp)
{
  if (cp < 0x80u) {
    s.push_back(static_cast<char>(cp));
  } else if (cp < 0x800u) {
    s.push_back(static_cast<char>(0xC0u | (cp >> 6)));
    s.push_back(static_cast<char>(0x80u | (cp & 0x3Fu)));
  } else if (cp < 0x10000u) {
    s.push_back(static_cast<char>(0xE0u | (cp >> 12)));
    s.push_back(static_cast<char>(0x80u | ((cp >> 6) & 0x3Fu)));
    s.push_back(static_cast<char>(0x80u | (cp & 0x3Fu)));
  } else {
    s.push_back(static_cast<char>(0xF0u | ((cp >> 18) & 0x07u)));
    s.push_back(static_cast<char>(0x80u | ((cp >> 12) & 0x3Fu)));
    s.push_back(static_cast<char>(0x80u | ((cp >> 6) & 0x3Fu)));
    s.push_back(static_cast<char>(0x80u | (cp & 0x3Fu)));
  }
}

// cudf::strings::to_lower of one string (cpp/src/strings/case.cu:142-148: code points above U+FFFF stay).
// Bytes that are not well-formed UTF-8 are copied as they are.
std::string to_lower_bmp(std::string const& in)
{
  std::string out;
  size_t i = 0;
  auto cont = [&](size_t k) { return k < in.size() && (static_cast<uint8_t>(in[k]) & 0xC0u) == 0x80u; };
  while (i < in.size()) {
    uint32_t const b0 = static_cast<uint8_t>(in[i]);
    uint32_t cp       = b0;
    size_t len        = 1;
    if (b0 >= 0xC2u && b0 < 0xE0u && cont(i + 1)) {
      cp  = ((b0 & 0x1Fu) << 6) | (static_cast<uint8_t>(in[i + 1]) & 0x3Fu);
      len = 2;
    } else if (b0 >= 0xE0u && b0 < 0xF0u && cont(i + 1) && cont(i + 2)) {
      cp  = ((b0 & 0x0Fu) << 12) | ((static_cast<uint8_t>(in[i + 1]) & 0x3Fu) << 6) | (static_cast<uint8_t>(in[i + 2]) & 0x3Fu);
      len = 3;
    } else if (b0 >= 0x80u) {
      len = 1;
      cp  = 0xFFFFFFFFu;  // not a BMP character: copied
      if (b0 >= 0xF0u && cont(i + 1) && cont(i + 2) && cont(i + 3)) len = 4;
    }
    const uint32_t(*row)[4] = nullptr;
    if (cp <= 0xFFFFu) {
      auto const* end = kLowerCase + sizeof(kLowerCase) / sizeof(kLowerCase[0]);
      auto const* it  = std::lower_bound(kLowerCase, end, cp, [](const uint32_t(&r)[4], uint32_t v) { return r[0] < v; });
      if (it != end && (*it)[0] == cp) row = it;
    }
    if (row) {
      for (int k = 1; k < 4; ++k)
        if ((*row)[k]) append_utf8(out, (*row)[k]);
    } else {
      out.append(in, i, len);
    }
    i += len;
  }
  return out;
}

}  // namespace
}  // namespace nvtext_amd

extern "C" {

nvtext_amd_status nvtext_amd_character_normalizer_create(int32_t do_lower_case, const nvtext_amd_strings_column* special_tokens, void* stream_,
                                                         const nvtext_amd_allocator* mr, nvtext_amd_character_normalizer** out)
{
  using namespace nvtext_amd;
  EntryScope const entry("nvtext_amd_character_normalizer_create");
  if (!out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out               = nullptr;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  std::vector<std::string> tokens;
  if (special_tokens && special_tokens->size > 0) {
    // cpp/src/text/normalize.cu:227-228
    if (special_tokens->null_count > 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "special tokens should not have nulls");
    int32_t const count = special_tokens->size;
    size_t const ow     = special_tokens->offsets_is_int64 ? 8 : 4;
    std::vector<uint8_t> h_off((static_cast<size_t>(count) + 1) * ow);
    const uint8_t* d_off = static_cast<const uint8_t*>(special_tokens->offsets) + static_cast<size_t>(special_tokens->offset) * ow;
    NVTEXT_HIP_TRY(hipMemcpyAsync(h_off.data(), d_off, h_off.size(), hipMemcpyDeviceToHost, stream));
    NVTEXT_HIP_TRY(hipStreamSynchronize(stream));
    auto off_at = [&](int32_t i) -> int64_t {
      if (ow == 8) {
        int64_t v;
        std::memcpy(&v, h_off.data() + static_cast<size_t>(i) * 8, 8);
        return v;
      }
      int32_t v;
      std::memcpy(&v, h_off.data() + static_cast<size_t>(i) * 4, 4);
      return v;
    };
    int64_t const first = off_at(0), last = off_at(count);
    if (last < first) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "special token offsets are not monotone");
    std::string pool(static_cast<size_t>(last - first), '\0');
    if (!pool.empty()) {
      NVTEXT_HIP_TRY(hipMemcpyAsync(&pool[0], special_tokens->chars + first, pool.size(), hipMemcpyDeviceToHost, stream));
      NVTEXT_HIP_TRY(hipStreamSynchronize(stream));
    }
    for (int32_t i = 0; i < count; ++i) tokens.emplace_back(pool, static_cast<size_t>(off_at(i) - first), static_cast<size_t>(off_at(i + 1) - off_at(i)));
    // cpp/src/text/normalize.cu:230-235: sorted by bytes first, lower-cased afterwards
    std::sort(tokens.begin(), tokens.end(), [](std::string const& a, std::string const& b) {
      int const c = std::memcmp(a.data(), b.data(), std::min(a.size(), b.size()));
      return c != 0 ? c < 0 : a.size() < b.size();
    });
    if (do_lower_case)
      for (auto& tk : tokens) tk = to_lower_bmp(tk);
  }

  // dense tables from the generated runs; the Hangul syllables decompose by arithmetic (The Unicode Standard, 3.12)
  std::vector<uint32_t> entries(kCodepoints, kDefaultEntry);
  std::vector<uint64_t> second(kCodepoints, 0);
  for (auto const& run : kCodepointRuns) std::fill(entries.begin() + run[0], entries.begin() + run[0] + run[1], run[2]);
  for (auto const& pair : kCodepointSecond) second[static_cast<size_t>(pair[0])] = pair[1];
  for (uint32_t s = 0; s < 11172u; ++s) {
    uint32_t const lead = 0x1100u + s / 588u, vowel = 0x1161u + (s % 588u) / 28u, trail = s % 28u;
    entries[0xAC00u + s] = (5u << 24) | (1u << 23) | lead;
    second[0xAC00u + s]  = (static_cast<uint64_t>(vowel) << 32) | (trail ? 0x11A7u + trail : 0u);
  }

  // the slots of the one-byte code points, decided here once (the rules of slots_of)
  uint32_t ascii[128];
  for (uint32_t cp = 0; cp < 128u; ++cp) {
    uint32_t const e = entries[cp], cat = (e >> 24) & 7u;
    uint32_t d       = 0;
    if (!(cat == kRemove || (do_lower_case && cat == kRemoveIfLower))) {
      uint32_t const repl = (do_lower_case || cat == kReplace) ? (e & 0x1FFFFFu) : cp;
      uint32_t const r0   = repl ? repl : cp;
      d                   = (cat == kPad || (do_lower_case && cat == kPadIfLower)) ? (0x20u | (r0 << 8) | (0x20u << 16) | (3u << 24)) : (r0 | (1u << 24));
    }
    ascii[cp] = d;
  }

  // the finished slots of the Basic Multilingual Plane (the rules of slots_of, run here once per code point)
  std::vector<uint4> bmp(0x10000);
  {
    NormTables const host_tables{nullptr, nullptr, entries.data(), second.data(), nullptr, nullptr, 0, do_lower_case ? 1 : 0};
    for (uint32_t cp = 0; cp < 0x10000u; ++cp) {
      uint32_t s0, s1, s2;
      slots_of(cp, host_tables, s0, s1, s2);
      bmp[cp] = make_uint4(s0, s1, s2, bytes_of(s0) + bytes_of(s1) + bytes_of(s2));
    }
  }

  auto* obj      = new nvtext_amd_character_normalizer();
  obj->do_lower  = do_lower_case ? 1 : 0;
  obj->tokens    = static_cast<int32_t>(tokens.size());
  auto fail_with = [&](hipError_t e) {
    nvtext_amd_character_normalizer_destroy(obj);
    return fail(e == hipErrorOutOfMemory ? NVTEXT_AMD_ALLOC_FAILED : NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
  };
  obj->store.bind(mr, stream);
  std::vector<int32_t> token_offsets(tokens.size() + 1, 0);
  std::string token_chars;
  for (size_t i = 0; i < tokens.size(); ++i) {
    token_chars += tokens[i];
    if (token_chars.size() > 0x7FFFFFFFull) {
      nvtext_amd_character_normalizer_destroy(obj);
      return fail(NVTEXT_AMD_OVERFLOW, "special tokens too large");
    }
    token_offsets[i + 1] = static_cast<int32_t>(token_chars.size());
  }
  hipError_t e = hipGetDevice(&obj->device);
  if (e != hipSuccess) return fail_with(e);
  bool ok = obj->store.allocate(&obj->ascii, 128) && obj->store.allocate(&obj->bmp, bmp.size()) &&
            obj->store.allocate(&obj->entries, entries.size()) && obj->store.allocate(&obj->second, second.size());
  if (ok && !tokens.empty())
    ok = obj->store.allocate(&obj->token_offset, token_offsets.size()) && obj->store.allocate(&obj->token_chars, std::max<size_t>(token_chars.size(), 1));
  if (!ok) return fail_with(hipErrorOutOfMemory);
  e = hipMemcpyAsync(obj->ascii, ascii, sizeof(ascii), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess) e = hipMemcpyAsync(obj->bmp, bmp.data(), bmp.size() * sizeof(uint4), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess) e = hipMemcpyAsync(obj->entries, entries.data(), entries.size() * sizeof(uint32_t), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess) e = hipMemcpyAsync(obj->second, second.data(), second.size() * sizeof(uint64_t), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess && !tokens.empty())
    e = hipMemcpyAsync(obj->token_offset, token_offsets.data(), token_offsets.size() * sizeof(int32_t), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess && !token_chars.empty()) e = hipMemcpyAsync(obj->token_chars, token_chars.data(), token_chars.size(), hipMemcpyHostToDevice, stream);
  hipError_t const synced = hipStreamSynchronize(stream);  // the host copies die at return
  if (e == hipSuccess) e = synced;
  if (e != hipSuccess) return fail_with(e);
  *out = obj;
  return NVTEXT_AMD_SUCCESS;
}

void nvtext_amd_character_normalizer_destroy(nvtext_amd_character_normalizer* normalizer)
{
  delete normalizer;  // the store hands the tables back
}

nvtext_amd_status nvtext_amd_normalize_characters(const nvtext_amd_strings_column* input, const nvtext_amd_character_normalizer* normalizer,
                                                  void* stream_, const nvtext_amd_allocator* mr_, nvtext_amd_strings_result* out)
{
  using namespace nvtext_amd;
  EntryScope const entry("nvtext_amd_normalize_characters");
  if (!input || !normalizer || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nvtext_amd_strings_result{};
  if (input->size < 0 || input->null_count < 0 || input->null_count > input->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "invalid column sizes");
  if (input->null_count > 0 && !input->null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");
  int device = 0;
  NVTEXT_HIP_TRY(hipGetDevice(&device));
  if (device != normalizer->device) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "the normalizer belongs to another device");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Mr mr{mr_, stream};
  int32_t const rows = input->size;
  if (rows == 0) return NVTEXT_AMD_SUCCESS;  // normalize.cu:497: the empty strings column
  if (!input->offsets) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "offsets missing");

  // normalize.cu:499-501: the byte range of the view
  size_t const ow      = input->offsets_is_int64 ? 8 : 4;
  const uint8_t* d_off = static_cast<const uint8_t*>(input->offsets) + static_cast<size_t>(input->offset) * ow;
  int64_t ends[2]      = {0, 0};
  int32_t ends32[2]    = {0, 0};
  for (int k = 0; k < 2; ++k) {
    void* host = ow == 8 ? static_cast<void*>(&ends[k]) : static_cast<void*>(&ends32[k]);
    NVTEXT_HIP_TRY(hipMemcpyAsync(host, d_off + (k ? static_cast<size_t>(rows) * ow : 0), ow, hipMemcpyDeviceToHost, stream));
  }
  NVTEXT_HIP_TRY(hipStreamSynchronize(stream));
  int64_t const first = ow == 8 ? ends[0] : ends32[0];
  int64_t const last  = ow == 8 ? ends[1] : ends32[1];
  if (last < first) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "offsets are not monotone");
  int64_t const n = last - first;
  if (n > 0 && !input->chars) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "chars missing");

  auto release = [&](nvtext_amd_status st, const char* msg) {
    nvtext_amd_strings_result_free(out, stream_, mr_);
    return fail(st, msg);
  };
  out->size         = rows;
  out->null_count   = input->null_count;
  out->offsets_size = rows + 1;
  auto allocate_offsets = [&](bool wide) {
    out->offsets_is_int64 = wide ? 1 : 0;
    out->offsets_bytes    = (static_cast<size_t>(rows) + 1) * (wide ? sizeof(int64_t) : sizeof(int32_t));
    out->offsets          = mr.allocate(out->offsets_bytes);
    return out->offsets != nullptr;
  };
  if (input->null_mask) {  // copy_bitmask(input): cpp/src/bitmask/null_mask.cu:381-391
    out->null_mask_bytes = mask_alloc_bytes(rows);
    out->null_mask       = static_cast<uint32_t*>(mr.allocate(out->null_mask_bytes));
    if (!out->null_mask) return release(NVTEXT_AMD_ALLOC_FAILED, "mask allocation failed");
    launch_copy_bitmask(out->null_mask, input->null_mask, input->offset, rows, stream);
  }
  if (n == 0) {  // normalize.cu:504: nothing to normalize, every row is empty
    if (!allocate_offsets(false)) return release(NVTEXT_AMD_ALLOC_FAILED, "result allocation failed");
    launch_fill_u32(static_cast<uint32_t*>(out->offsets), 0u, static_cast<int64_t>(rows) + 1, stream);
    NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_strings_result_free(out, stream_, mr_));
    return NVTEXT_AMD_SUCCESS;
  }

  int64_t const tiles = (n + kNormTile - 1) / kNormTile;
  if (tiles > 0x7FFFFFFFll) return release(NVTEXT_AMD_OVERFLOW, "input too large");
  size_t const temp_bytes[4] = {static_cast<size_t>(tiles) * sizeof(uint32_t), (static_cast<size_t>(tiles) + 1) * sizeof(uint64_t),
                                scan_temp_bytes(tiles), static_cast<size_t>(tiles) * sizeof(int32_t)};
  TempParts<4> const temps(mr, temp_bytes);
  uint32_t* const tile_bytes  = temps.part<uint32_t>(0);
  uint64_t* const tile_offset = temps.part<uint64_t>(1);
  uint64_t* const scan_temp   = temps.part<uint64_t>(2);
  int32_t* const tile_row     = temps.part<int32_t>(3);
  if (!temps.ok()) return release(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
  NormTables const tables{normalizer->ascii, normalizer->bmp, normalizer->entries, normalizer->second, normalizer->token_chars, normalizer->token_offset, normalizer->tokens,
                          normalizer->do_lower};
  ColView const view = make_view(*input);
  {
    ProfileScope ps("normalize_count_kernel", stream);
    hipLaunchKernelGGL(normalize_count_kernel, dim3(static_cast<unsigned>(tiles)), dim3(kNormThreads), 0, stream, view.chars + first, n, tables,
                       tile_bytes);
  }
  hipLaunchKernelGGL(normalize_tile_rows_kernel, dim3(static_cast<unsigned>((tiles + 255) / 256)), dim3(256), 0, stream, view, first, tiles,
                     tile_row);
  device_exclusive_scan(TileBytes{tile_bytes}, tiles, tile_offset, scan_temp, stream);
  uint64_t total = 0;
  hipError_t e   = hipMemcpyAsync(&total, tile_offset + tiles, sizeof(total), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) return release(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
  // int64 offsets from the large-strings threshold on (cpp/include/cudf/strings/detail/strings_children.cuh:164-175)
  if (!allocate_offsets(total >= 0x7FFFFFFFull)) return release(NVTEXT_AMD_ALLOC_FAILED, "result allocation failed");
  out->chars_size = static_cast<int64_t>(total);
  if (total > 0) {
    out->chars_bytes = static_cast<size_t>(total);
    out->chars       = static_cast<char*>(mr.allocate(out->chars_bytes));
    if (!out->chars) return release(NVTEXT_AMD_ALLOC_FAILED, "result allocation failed");
  }
  {
    ProfileScope ps("normalize_write_kernel", stream);
    hipLaunchKernelGGL(normalize_write_kernel, dim3(static_cast<unsigned>(tiles)), dim3(kNormThreads), 0, stream, view, first, n, tables,
                       tile_offset, tile_row, reinterpret_cast<uint8_t*>(out->chars), out->offsets,
                       out->offsets_is_int64);
  }
  e = hipGetLastError();
  if (e != hipSuccess) return release(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
  return NVTEXT_AMD_SUCCESS;
}

void nvtext_amd_strings_result_free(nvtext_amd_strings_result* col, void* stream, const nvtext_amd_allocator* mr)
{
  if (!col) return;
  nvtext_amd::Mr m{mr, static_cast<hipStream_t>(stream)};
  m.deallocate(col->offsets, col->offsets_bytes);
  m.deallocate(col->chars, col->chars_bytes);
  m.deallocate(col->null_mask, col->null_mask_bytes);
  *col = nvtext_amd_strings_result{};
}

}  // extern "C"

// wordpiece_vocabulary + wordpiece_tokenize for gfx950.
//
// The reference (cpp/src/text/wordpiece_tokenize.cu) keeps two cuco hash maps keyed by
// MurmurHash3 of the candidate substring, marks word starts with a copy_if over all bytes,
// merges them with the row offsets and writes tokens into a 4-byte-per-input-byte temporary
// that is then counted and compacted (503-568, 462-491, 877-881).
//
// Here:
//   * one open-addressing table of 2-slot buckets (16-byte slots, load <= 0.5) holds both key
//     spaces: whole entries (kind 0) and "##" entries without their prefix (kind 1).  Keys of
//     up to 8 bytes sit inside the slot, so a probe is one 32-byte read and the key's two dwords
//     are also what gets hashed; the table for a 30k-entry vocabulary is 2 MiB and stays in L2.
//     A hashed length filter (which key lengths exist for a given first three bytes) lets the
//     longest-match search skip the lengths that cannot match.
//   * probe pass: a wavefront is four groups of 16 lanes; a group owns a run of consecutive rows holding an
//     equal share of the column's work and walks one row at a time in 256-byte chunks, 16 bytes per lane.
//     Spaces become a 16-bit mask per lane with four SWAR operations per dword; word starts and ends are bit
//     operations on that mask; DPP scans place the words of the chunk in an LDS list.  Then lanes <-> words,
//     the four groups pooled: ONE probe per word.  A hit stores the token in the row's word arena (one slot
//     per word, floor(bytes/2)+1 slots per row); a miss stores a marker and queues the word with its first
//     16 bytes.
//   * out-of-vocabulary pass: one lane per queued word, all lanes busy.  Words of up to 16 bytes are tokenized
//     in registers, the greedy longest-match rule reduced to bit operations on a mask of candidate lengths,
//     one table probe per trip; longer words go through a general state machine in a second kernel.  (Inside
//     the probe pass this chain of dependent probes would idle 90 % of the lanes.)
//   * a device-wide scan of the per-row token counts makes the int32 list offsets; the emit pass expands the
//     word arena into the tokens, a block of rows with an even number of tokens per wavefront; the few words
//     with more pieces than a result record keeps are tokenized again, into place, by a kernel of their own.
//     No chars-sized temporary is written.
//   * without a word limit, rows beyond 32 KiB are cut at spaces into pieces that go through all of this as
//     rows of their own (a row is walked by 16 lanes: a row of megabytes would keep the device waiting).
#include "common.cuh"

#include <algorithm>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

namespace nvtext_amd {
namespace {

constexpr uint32_t kMaxWord = 200;  // wordpiece_tokenize.cu:300: words this long become one [UNK]

__host__ __device__ __forceinline__ uint32_t mix32(uint32_t h)
{
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}

// Key hash: the key is consumed in 8-byte blocks (two little-endian dwords, zero padded).
__host__ __device__ __forceinline__ uint32_t key_hash_init(uint32_t len) { return len * 0xC2B2AE3Du; }
__host__ __device__ __forceinline__ uint32_t key_hash_block(uint32_t h, uint32_t lo, uint32_t hi)
{
  h = (h ^ lo) * 0x9E3779B1u;
  h = (h ^ hi) * 0x85EBCA77u;
  return h ^ (h >> 15);
}

// slot.x = (tag23 << 9) | (kind << 8) | len   (0 = empty; len in 1..199)
// slot.y = token id; in slot 0 of a bucket, bit 31 says that some key has been carried past this bucket
//          (kSearchOn: a key that is not in a bucket without the bit is not in the table)
// slot.z, slot.w = the key itself when len <= 8 (zero padded), else (byte offset of the key in the pool, 0);
// the pool holds the keys of more than 8 bytes, each zero padded to a multiple of 8 at an 8-byte aligned offset
// Bucket b = slots[2b], slots[2b+1]; a bucket fills slot 0 first, overflow goes to the next bucket.
constexpr uint32_t kSearchOn = 0x80000000u;
struct VocabTable {
  const uint4* slots;
  const uint8_t* pool;
  uint32_t bucket_mask;  // buckets - 1
  int32_t unk_id;
  uint32_t max_len[2];   // longest key of each key space (longer candidates cannot match)
  // Length filter: lens[length_filter_index(kind, first three key bytes) & lens_mask] has bit i (i < 31) set
  // when some key of that key space with those first bytes is i + 3 bytes long, bit 31 for 34 bytes and more.
  // Entries are shared by hashing, so a set bit promises nothing, a clear bit rules the length out.
  const uint32_t* lens;
  uint32_t lens_mask;
  // Direct tables for keys of one and two bytes: short_ids[kind * 65536 + (byte0 | byte1 << 8)] for two bytes,
  // short_ids[131072 + kind * 256 + byte0] for one; the token id, or INT32_MIN when there is no such key.
  const int32_t* short_ids;
};
constexpr uint32_t kShortIds = 2 * 65536 + 2 * 256;

__host__ __device__ __forceinline__ uint32_t length_filter_index(uint32_t kind, uint32_t first3)
{
  uint32_t x = (first3 | (kind << 24)) * 0x9E3779B1u;
  x ^= x >> 15;
  x *= 0x85EBCA77u;
  return x ^ (x >> 13);
}
__host__ __device__ __forceinline__ uint32_t length_filter_bit(uint32_t len) { return len >= 34 ? 31u : len - 3u; }

__host__ __device__ __forceinline__ uint32_t slot_word0(uint32_t h, uint32_t kind, uint32_t len, uint32_t* bucket)
{
  uint32_t const x = mix32(h + kind * 0x7F4A7C15u);
  *bucket          = x;
  return (x & 0xFFFFFE00u) | (kind << 8) | len;
}

}  // namespace
}  // namespace nvtext_amd

struct nvtext_amd_wordpiece_vocabulary {
  nvtext_amd::VocabTable table{};
  void* d_slots     = nullptr;
  void* d_pool      = nullptr;
  void* d_lens      = nullptr;
  void* d_short     = nullptr;
  size_t slot_bytes = 0;
  size_t pool_bytes = 0;
  int32_t entries   = 0;
};

namespace nvtext_amd {
namespace {

constexpr int kTokWaves     = 4;
constexpr int kTokThreads   = kTokWaves * kWave;
constexpr int kGroups       = 4;     // rows a wavefront walks at the same time, 16 lanes each
constexpr int kGroupLanes   = kWave / kGroups;
constexpr int kChunk        = 16 * kGroupLanes;  // bytes per group step (16 per lane) = 256
constexpr int kRing         = 2 * kChunk;        // per group: the current chunk and the one before it
constexpr int32_t kNone     = std::numeric_limits<int32_t>::min();
constexpr int kOovKeep      = 7;     // tokens stored per queued word; longer results are redone at emit time
constexpr uint32_t kOovMark = 0x80000000u;  // word-arena value 0x80000000 | queue index (never 0xFFFFFFFF = id -1)

struct OovEntry {
  int32_t row;     // -1: unused entry
  uint32_t delta;  // byte offset of the word inside its row
  uint32_t widx;   // index of the word inside its row (its word-arena slot)
  uint32_t len;    // bytes in the word (1..199)
  uint32_t head[4];  // the word's first 16 bytes, zero padded: most words are tokenized without reading the chars again
};
struct OovResult {
  int32_t tok[kOovKeep];
  uint32_t count;  // tokens of the word (may exceed kOovKeep)
};
static_assert(sizeof(OovEntry) == 32 && sizeof(OovResult) == 32, "queue records are two 16-byte stores");

// ------------------------------------------------------------------ where candidate keys live
// Each source offers byte(k) and key8(p, len, &k0, &k1): bytes [p, p+8) as two dwords, zero padded past len.
__device__ __forceinline__ void trim_key8(uint32_t len, uint32_t& lo, uint32_t& hi)
{
  // keep bytes [0, len) of the eight (selects, no branches)
  uint32_t const nlo = min(len, 4u), nhi = max(min(len, 8u), 4u) - 4u;
  lo &= nlo >= 4 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << (8 * nlo));
  hi &= nhi >= 4 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << (8 * nhi));
}

// A word inside a group's 512-byte LDS ring of the probe pass: byte k of the word is ring byte (start + k) & 511.
struct RingWord {
  const uint32_t* ring;
  uint32_t start;
  __device__ __forceinline__ uint32_t byte(uint32_t k) const { return reinterpret_cast<const uint8_t*>(ring)[(start + k) & (kRing - 1)]; }
  __device__ __forceinline__ void key8(uint32_t p, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    uint32_t const o  = (start + p) & (kRing - 1);
    uint32_t const i  = o >> 2;
    uint32_t const sh = (o & 3u) * 8u;
    uint32_t const d0 = ring[i], d1 = ring[(i + 1) & (kRing / 4 - 1)], d2 = ring[(i + 2) & (kRing / 4 - 1)];
    uint32_t lo       = __builtin_amdgcn_alignbit(d1, d0, sh);
    uint32_t hi       = __builtin_amdgcn_alignbit(d2, d1, sh);
    trim_key8(len, lo, hi);
    *k0 = lo;
    *k1 = hi;
  }
  // bytes [0, 16) of the word, untrimmed
  __device__ __forceinline__ void head16(uint32_t (&k)[4]) const
  {
    uint32_t const i  = start >> 2;
    uint32_t const sh = (start & 3u) * 8u;
    uint32_t d[5];
#pragma unroll
    for (uint32_t j = 0; j < 5; ++j) d[j] = ring[(i + j) & (kRing / 4 - 1)];
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) k[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
  }
};

// A word in global memory (emit pass, rare path).  key8 reads only aligned dwords that overlap the key.
struct GlobalWord {
  const uint8_t* p;
  __device__ __forceinline__ uint32_t byte(uint32_t k) const { return p[k]; }
  __device__ __forceinline__ void key8(uint32_t off, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    const uint8_t* q    = p + off;
    uint32_t const mis  = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(q) & 3u);
    const uint32_t* a   = reinterpret_cast<const uint32_t*>(q - mis);
    uint32_t const need = mis + (len < 8 ? len : 8);  // bytes from the aligned base
    uint32_t const d0   = a[0];
    uint32_t const d1   = need > 4 ? a[1] : 0u;
    uint32_t const d2   = need > 8 ? a[2] : 0u;
    uint32_t lo         = __builtin_amdgcn_alignbit(d1, d0, mis * 8u);
    uint32_t hi         = __builtin_amdgcn_alignbit(d2, d1, mis * 8u);
    trim_key8(len, lo, hi);
    *k0 = lo;
    *k1 = hi;
  }
};

constexpr uint32_t kStage      = 64;   // bytes of each queued word kept in LDS (from a 16-byte aligned base)
constexpr uint32_t kOovThreads = 256;

// A queued word whose first kStage - mis bytes sit in LDS; later bytes come from memory.  The windows of
// the workgroup are interleaved dword by dword (dword j of thread t at [j][t]), so that the lanes of a
// wavefront reading "their" dword j hit 64 different banks instead of one.
struct StagedWord {
  const uint32_t* win;  // dword 0 of this lane's window; dword j is win[j * kOovThreads]
  const uint8_t* p;     // the word in global memory
  uint32_t mis;         // offset of the word inside the window
  __device__ __forceinline__ uint32_t dword(uint32_t j) const { return win[j * kOovThreads]; }
  __device__ __forceinline__ uint32_t byte(uint32_t k) const
  {
    uint32_t const o = mis + k;
    return o < kStage ? (dword(o >> 2) >> (8 * (o & 3u))) & 0xffu : p[k];
  }
  __device__ __forceinline__ void key8(uint32_t off, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    uint32_t const o = mis + off;
    uint32_t lo, hi;
    if (o + 12 <= kStage) {
      uint32_t const i  = o >> 2;
      uint32_t const sh = (o & 3u) * 8u;
      uint32_t const d0 = dword(i), d1 = dword(i + 1), d2 = dword(i + 2);
      lo                = __builtin_amdgcn_alignbit(d1, d0, sh);
      hi                = __builtin_amdgcn_alignbit(d2, d1, sh);
    } else {
      lo = hi = 0;
      for (uint32_t k = 0; k < 8 && k < len; ++k) {
        uint32_t const b = byte(off + k);
        if (k < 4) lo |= b << (8 * k); else hi |= b << (8 * (k - 4));
      }
    }
    trim_key8(len, lo, hi);
    *k0 = lo;
    *k1 = hi;
  }
};

// A candidate key, ready to be probed: its first block (trimmed), tag word and home bucket.
struct Probe {
  uint32_t k0, k1;  // key bytes [0, 8), zero padded
  uint32_t want;    // slot.x of a matching slot
  uint32_t bucket;  // home bucket (already masked)
};

// Hash contribution of key bytes [8, len) (keys that do not fit the slot; kept out of line).
template <typename W>
__device__ __forceinline__ uint32_t hash_long_key(W const& w, uint32_t p, uint32_t len, uint32_t h)
{
  for (uint32_t done = 8; done < len; done += 8) {
    uint32_t b0, b1;
    w.key8(p + done, len - done, &b0, &b1);
    h = key_hash_block(h, b0, b1);
  }
  return h;
}

// (raw0, raw1) = bytes [p, p+8) of `w`; whatever lies past the key is trimmed here.  1 <= len < 200.
template <typename W>
__device__ __forceinline__ Probe make_probe(VocabTable const& t, uint32_t kind, W const& w, uint32_t p, uint32_t len, uint32_t raw0, uint32_t raw1)
{
  Probe pr;
  pr.k0 = raw0;
  pr.k1 = raw1;
  trim_key8(len, pr.k0, pr.k1);
  uint32_t h = key_hash_block(key_hash_init(len), pr.k0, pr.k1);
  if (len > 8) h = hash_long_key(w, p, len, h);
  uint32_t b;
  pr.want   = slot_word0(h, kind, len, &b);
  pr.bucket = b & t.bucket_mask;
  return pr;
}

template <typename W>
__device__ __forceinline__ bool pool_key_equal(VocabTable const& t, uint32_t pool_off, W const& w, uint32_t p, uint32_t len)
{
  const uint2* e = reinterpret_cast<const uint2*>(t.pool + pool_off);
  for (uint32_t done = 0; done < len; done += 8) {
    uint32_t k0, k1;
    w.key8(p + done, len - done, &k0, &k1);
    uint2 const v = e[done >> 3];
    if (v.x != k0 || v.y != k1) return false;
  }
  return true;
}

// Examines one slot: 1 = it holds the key (id set), 0 = it is empty (the key is absent), -1 = look further.
template <typename W>
__device__ __forceinline__ int check_slot(VocabTable const& t, uint4 const& s, Probe const& pr, W const& w, uint32_t p, uint32_t len, int32_t* id)
{
  if (s.x == pr.want) {
    bool const same = len <= 8 ? (s.z == pr.k0 && s.w == pr.k1) : pool_key_equal(t, s.z, w, p, len);
    if (same) {
      *id = static_cast<int32_t>(s.y & ~kSearchOn);
      return 1;
    }
  }
  return s.x == 0 ? 0 : -1;
}

// Continues a lookup past a full home bucket without a match (rare at load <= 0.5).
template <typename W>
__device__ __forceinline__ int32_t lookup_further(VocabTable const& t, Probe const& pr, W const& w, uint32_t p, uint32_t len)
{
  uint32_t b = pr.bucket;
  for (;;) {
    b = (b + 1) & t.bucket_mask;
    int32_t id;
    int r = check_slot(t, t.slots[2 * b], pr, w, p, len, &id);
    if (r > 0) return id;
    if (r == 0) return kNone;
    r = check_slot(t, t.slots[2 * b + 1], pr, w, p, len, &id);
    if (r > 0) return id;
    if (r == 0) return kNone;
  }
}

// Outcome of a probe whose two home slots s0, s1 have been loaded.
template <typename W>
__device__ __forceinline__ int32_t finish_probe(VocabTable const& t, Probe const& pr, uint4 const& s0, uint4 const& s1, W const& w, uint32_t p,
                                                uint32_t len)
{
  int32_t id;
  int r = check_slot(t, s0, pr, w, p, len, &id);
  if (r > 0) return id;
  if (r == 0) return kNone;
  r = check_slot(t, s1, pr, w, p, len, &id);
  if (r > 0) return id;
  if (r == 0 || (s0.y & kSearchOn) == 0) return kNone;
  return lookup_further(t, pr, w, p, len);
}

// Token id of key bytes [p, p+len) of `w` in key space `kind`, or kNone.
template <typename W>
__device__ __forceinline__ int32_t lookup(VocabTable const& t, uint32_t kind, W const& w, uint32_t p, uint32_t len, uint32_t raw0, uint32_t raw1)
{
  Probe const pr = make_probe(t, kind, w, p, len, raw0, raw1);
  uint4 const s0 = t.slots[2 * pr.bucket];
  uint4 const s1 = t.slots[2 * pr.bucket + 1];
  return finish_probe(t, pr, s0, s1, w, p, len);
}

// What the two home slots say about a key of l bytes without any further memory access:
// 1 = found (*id set), 0 = absent, 2 = undecided (a key of more than 8 bytes has the right tag, or keys have been
// carried past this bucket and the search goes on in the next one).  Straight-line code.
__device__ __forceinline__ uint32_t verdict(Probe const& pr, uint4 const& s0, uint4 const& s1, uint32_t l, int32_t* id)
{
  bool const tag0  = s0.x == pr.want, tag1 = s1.x == pr.want;
  bool const is0   = tag0 && s0.z == pr.k0 && s0.w == pr.k1;
  bool const is1   = tag1 && s1.z == pr.k0 && s1.w == pr.k1;
  bool const small = l <= 8;
  bool const found = small && (is0 || is1);
  bool const more  = (!small && (tag0 || tag1)) || (!found && (s0.y & kSearchOn) != 0);
  *id              = static_cast<int32_t>((is0 ? s0.y : s1.y) & ~kSearchOn);
  return found ? 1u : more ? 2u : 0u;
}

// The same for a key of 9 to 16 bytes whose bytes are k[0..3] (zero padded): a home slot with the right tag
// names the key's place in the pool, and one 16-byte read there decides.  Still undecided (2) only when both home
// slots carry the tag or the search goes on in the next bucket.
__device__ __forceinline__ uint32_t verdict_16(VocabTable const& t, Probe const& pr, uint4 const& s0, uint4 const& s1, const uint32_t (&k)[4],
                                               int32_t* id)
{
  bool const tag0 = s0.x == pr.want, tag1 = s1.x == pr.want;
  bool const on   = (s0.y & kSearchOn) != 0;
  if (tag0 && tag1) return 2u;
  if (!tag0 && !tag1) return on ? 2u : 0u;
  const uint2* const e = reinterpret_cast<const uint2*>(t.pool + (tag0 ? s0.z : s1.z));
  uint2 const a = e[0], b = e[1];
  if (a.x == k[0] && a.y == k[1] && b.x == k[2] && b.y == k[3]) {
    *id = static_cast<int32_t>((tag0 ? s0.y : s1.y) & ~kSearchOn);
    return 1u;
  }
  return on ? 2u : 0u;
}

// ------------------------------------------------------------------ wavefront helpers of the probe pass
template <int CTRL, int ROW_MASK, int OLD>
__device__ __forceinline__ uint32_t dpp_old(uint32_t v)
{
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(OLD, static_cast<int>(v), CTRL, ROW_MASK, 0xf, false));
}

__device__ __forceinline__ uint32_t wave_scan_max(uint32_t v)
{
  v = max(v, dpp_zero<0x111, 0xf>(v));
  v = max(v, dpp_zero<0x112, 0xf>(v));
  v = max(v, dpp_zero<0x114, 0xf>(v));
  v = max(v, dpp_zero<0x118, 0xf>(v));
  v = max(v, dpp_zero<0x142, 0xa>(v));
  v = max(v, dpp_zero<0x143, 0xc>(v));
  return v;
}

// value of the lane below (lane 0 gets FIRST)
template <int FIRST>
__device__ __forceinline__ uint32_t from_lane_below(uint32_t v)
{
  return dpp_old<0x138, 0xf, FIRST>(v);  // wave_shr:1
}

// Bit 7 of every byte of x that equals ' ' (exact: no carries cross bytes).
__device__ __forceinline__ uint32_t space_bytes(uint32_t x)
{
  uint32_t const t = x ^ 0x20202020u;
  return ~(((t & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | t) & 0x80808080u;
}
// Gathers bits 7, 15, 23, 31 into bits 0..3.
__device__ __forceinline__ uint32_t gather_byte_flags(uint32_t z) { return (((z >> 7) * 0x00204081u) >> 21) & 0xFu; }

// Row r owns the word-arena slots [arena_pos(r), arena_pos(r+1)): at least floor(bytes/2) + 1, and a
// row cannot hold more words than that.
__device__ __forceinline__ int64_t arena_pos(ColView const& col, int64_t first_offset, int64_t r) { return ((col.off(r) - first_offset) >> 1) + r; }

struct ProbeLds {
  alignas(16) uint32_t bytes[kGroups][kRing / 4];  // per group: the bytes of the current chunk and the one before it, as in memory
  uint32_t word[kGroups * kChunk / 2 + 2];         // per word ending in this step: (length, clamped to kMaxWord) << 16 | offset of its last byte in the chunk
  alignas(16) uint32_t group[kGroups][8];          // per group: first word slot, words that count, chunk base, words so far, row start in its block, row, arena slot of the row
};

// Where a row sits relative to 16-byte aligned memory.  Coordinates count bytes from `base` and fit 32 bits
// (a row is below 2 GiB).
struct RowCtx {
  const uint4* base;  // aligned address at or below the row's first byte
  uint32_t mis;       // row start inside that block
  uint32_t aend;      // row end (mis + row bytes)
  // the 16 bytes at coordinate a0 (a multiple of 16) as they are in memory, if any of them belongs to the row
  __device__ __forceinline__ uint4 load_raw(uint32_t a0) const
  {
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (a0 < aend && a0 + 16 > mis) v = load_stream(base + (a0 >> 4));
    return v;
  }
  // which of the 16 bytes at coordinate a0 belong to the row (bit k = byte a0 + k)
  __device__ __forceinline__ uint32_t inside(uint32_t a0) const
  {
    uint32_t const lo = mis > a0 ? min(mis - a0, 16u) : 0u;
    uint32_t const hi = aend > a0 ? min(aend - a0, 16u) : 0u;
    return ((1u << hi) - 1u) & ~((1u << lo) - 1u);
  }
  // the byte at coordinate a (any alignment); ' ' outside the row
  __device__ __forceinline__ uint32_t byte_at(uint32_t a) const
  {
    if (a < mis || a >= aend) return 0x20u;
    return reinterpret_cast<const uint8_t*>(base)[a];
  }
};

__device__ __forceinline__ RowCtx make_row_ctx(ColView const& col, int64_t o, int64_t n)
{
  const uint8_t* row = col.chars + o;
  RowCtx c;
  c.mis  = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row) & 15u);
  c.base = reinterpret_cast<const uint4*>(row - c.mis);
  c.aend = c.mis + static_cast<uint32_t>(n);
  return c;
}

// ------------------------------------------------------------------ probe pass
// DPP moves inside a row of 16 lanes; lanes without a source keep `old`.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_row(uint32_t old, uint32_t v)
{
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(old), static_cast<int>(v), CTRL, 0xf, 0xf, false));
}
// inclusive max-scan inside each group of 16 lanes
__device__ __forceinline__ uint32_t group_scan_max(uint32_t v)
{
  v = max(v, dpp_row<0x111>(0u, v));  // row_shr:1
  v = max(v, dpp_row<0x112>(0u, v));  // row_shr:2
  v = max(v, dpp_row<0x114>(0u, v));  // row_shr:4
  v = max(v, dpp_row<0x118>(0u, v));  // row_shr:8
  return v;
}
__device__ __forceinline__ uint32_t shfl_u32(uint32_t v, int src_lane) { return static_cast<uint32_t>(__shfl(static_cast<int>(v), src_lane)); }

// Persistent wavefronts.  Each group of 16 lanes walks its own row in 256-byte chunks (16 bytes per lane),
// so a wavefront has four rows in flight; the words the four groups find in a step are pooled and probed
// with lanes <-> words.  The next chunk of every group (the rest of its row, else the start of its next
// row, whose offsets were fetched a row earlier) is requested before the probes of the current step.
// For row r and its word k (slot = arena_pos(r) + k): arena[slot] = the token, or an out-of-vocabulary
// marker carrying the queue index; nwords[r] = counts[r] = words kept.
__global__ void __launch_bounds__(kTokThreads, 7) wordpiece_probe_kernel(ColView col, VocabTable table, int32_t max_words, int64_t first_offset,
                                                                      int64_t last_offset, uint32_t* __restrict__ arena,
                                                                      int32_t* __restrict__ nwords, int32_t* __restrict__ counts,
                                                                      OovEntry* __restrict__ queue, uint32_t queue_capacity, uint32_t queue_block,
                                                                      uint32_t* __restrict__ queue_size)
{
  __shared__ ProbeLds lds_all[kTokWaves];
  int const lane       = lane_id();
  int const wave       = threadIdx.x / kWave;
  int const g          = lane / kGroupLanes;  // my group
  int const gl         = lane % kGroupLanes;  // my lane inside it
  int const g_first    = g * kGroupLanes;
  int const g_last     = g_first + kGroupLanes - 1;
  ProbeLds& lds        = lds_all[wave];
  int64_t const rows   = col.size;
  uint32_t q_pos = 0, q_lim = 0;  // this wavefront's reserved queue range
  uint32_t my_block       = min(queue_block, 128u);  // entries reserved at a time: doubled up to queue_block when ranges fill fast
  uint32_t steps_in_range = 0;                       // steps of the loop below since the range was reserved

  // wordpiece_tokenize.cu:776-781: with a word limit, null rows have no words and the limit is
  // min(max_words, size_bytes / 2); without one, validity is not consulted (503-568).
  auto word_cap = [&](int64_t row, int64_t bytes) -> uint32_t {
    if (max_words <= 0) return static_cast<uint32_t>(std::numeric_limits<int32_t>::max());
    return col.valid(row) ? static_cast<uint32_t>(min(static_cast<int64_t>(max_words), bytes / 2)) : 0u;
  };

  // ---- the rows of a group: consecutive ones, [r, r_end), that hold its share of the column's WORK, a row counting
  // as its bytes plus one chunk (which is about what walking it costs; rows without bytes must count, or a long run
  // of them would fall to one group).  Group k of G begins with the first row at or after k/G of the total.  With a
  // share of the rows instead (every G-th row) the groups with the longest rows walked a seventh more chunks than the
  // average group, and the pass waited for them.  r_end is found together with r: two searches over the offsets in
  // step, 22 dependent reads for 4M rows.
  uint32_t r = 0, r_end = 0;
  {
    uint32_t const groups = gridDim.x * kTokWaves * kGroups;
    uint32_t const k      = (blockIdx.x * kTokWaves + wave) * kGroups + g;
    auto work_before = [&](int64_t row) -> int64_t { return col.off(row) - first_offset + row * static_cast<int64_t>(kChunk); };
    // (work < 2^48 and groups < 2^16: the products fit)
    int64_t const work = last_offset - first_offset + rows * static_cast<int64_t>(kChunk);
    int64_t const t0   = work / groups * k + work % groups * k / groups;
    int64_t const t1   = work / groups * (k + 1) + work % groups * (k + 1) / groups;
    // number of rows 0..rows with less work before them than t, which is the first row at or after t
    uint32_t below0 = 0, below1 = 0;
    uint32_t step   = 1;
    while (step <= static_cast<uint32_t>(rows)) step <<= 1;  // rows + 1 entries; rows < 2^31
    for (; step > 0; step >>= 1) {
      uint32_t const p0 = below0 + step, p1 = below1 + step;
      int64_t const v0  = p0 <= static_cast<uint32_t>(rows) + 1u ? work_before(static_cast<int64_t>(p0) - 1) : std::numeric_limits<int64_t>::max();
      int64_t const v1  = p1 <= static_cast<uint32_t>(rows) + 1u ? work_before(static_cast<int64_t>(p1) - 1) : std::numeric_limits<int64_t>::max();
      if (v0 < t0) below0 = p0;
      if (v1 < t1) below1 = p1;
    }
    r     = min(below0, static_cast<uint32_t>(rows));
    r_end = k + 1 == groups ? static_cast<uint32_t>(rows) : min(below1, static_cast<uint32_t>(rows));
    if (k == 0) r = 0;
  }
  // ---- per-group state (the same value in all 16 lanes of a group).  Kept small: the row being walked is known by its
  // RowCtx alone (its first byte's address gives back its offset; the next row begins where it ends), the row after
  // it by its end.
  int64_t e_nxt = 0;
  uint32_t cap  = 0;
  RowCtx ctx;
  {
    int64_t o = 0, n = 0;
    if (r < r_end) {
      o   = col.off(r);
      n   = col.off(r + 1) - o;
      cap = word_cap(r, n);
    }
    ctx = make_row_ctx(col, o, n);
  }
  if (r + 1 < r_end) e_nxt = col.off(static_cast<int64_t>(r) + 2);
  uint32_t cbase   = 0;
  uint32_t wdone   = 0;     // words kept so far in this row
  uint32_t carry_start = 0; // 1-based coordinate of the start of the word running into the chunk
  uint32_t prev_space  = 1; // the byte before the chunk is a space (or the row starts here)
  // the chunk about to be processed: my sixteen bytes and (last lane of the group) the byte after the chunk
  uint4 mine_cur    = make_uint4(0u, 0u, 0u, 0u);
  uint32_t tail_cur = 0x20u;
  if (r < r_end) {
    mine_cur = ctx.load_raw(16 * gl);
    if (gl == kGroupLanes - 1) tail_cur = ctx.byte_at(kChunk);
  }

  while (ballot64(r < r_end) != 0) {
    ++steps_in_range;
    bool const has_row  = r < r_end;
    bool const chunk_ok = has_row && cbase < ctx.aend && wdone < cap;

    // ---- bytes -> word ends (lanes <-> bytes, per group)
    uint32_t ends = 0, starts = 0, xs = 0;
    uint32_t const a0 = cbase + 16u * gl;
    if (chunk_ok) *reinterpret_cast<uint4*>(&lds.bytes[g][(a0 & (kRing - 1)) >> 2]) = mine_cur;
    {
      uint4 const mine  = mine_cur;
      // spaces, and everything outside the row counts as one
      uint32_t const sp = (gather_byte_flags(space_bytes(mine.x)) | (gather_byte_flags(space_bytes(mine.y)) << 4) |
                           (gather_byte_flags(space_bytes(mine.z)) << 8) | (gather_byte_flags(space_bytes(mine.w)) << 12) | ~ctx.inside(a0)) &
                          0xFFFFu;
      // is the byte before my sixteen a space, and the byte after them
      uint32_t const before = dpp_row<0x111>(prev_space, sp >> 15);                       // row_shr:1
      uint32_t const after  = dpp_row<0x101>(tail_cur == 0x20u ? 1u : 0u, sp & 1u);        // row_shl:1
      uint32_t const word   = ~sp & 0xFFFFu;
      starts                = word & ((sp << 1) | before);         // a word byte after a space
      ends                  = word & ((sp >> 1) | (after << 15));  // a word byte before a space
      if (!chunk_ok) ends = starts = 0;
      // start of the word that runs into my bytes: the last start in the lanes below, else the carry
      uint32_t const my_last = starts ? a0 + (32u - __builtin_clz(starts)) : 0u;
      uint32_t const is      = group_scan_max(my_last);
      xs                     = max(dpp_row<0x111>(0u, is), carry_start);
      if (chunk_ok) {
        carry_start = max(carry_start, shfl_u32(is, g_last));
        prev_space  = shfl_u32(sp >> 15, g_last);
      }
    }
    uint32_t const ne   = __builtin_popcount(ends);
    uint32_t const incl = wave_inclusive_scan(ne);
    // first word slot of every group and the total
    uint32_t const gb1 = wave_bcast(incl, 15), gb2 = wave_bcast(incl, 31), gb3 = wave_bcast(incl, 47), total = wave_bcast(incl, 63);
    uint32_t const my_gbase  = g == 0 ? 0u : g == 1 ? gb1 : g == 2 ? gb2 : gb3;
    uint32_t const my_gtotal = (g == 0 ? gb1 : g == 1 ? gb2 : g == 2 ? gb3 : total) - my_gbase;
    uint32_t slot            = incl - ne;
    for (uint32_t em = ends; em; em &= em - 1) {
      uint32_t const p  = __builtin_ctz(em);
      uint32_t const sb = starts & ((2u << p) - 1u);
      uint32_t const st = sb ? a0 + (32u - __builtin_clz(sb)) : xs;  // 1-based
      uint32_t const wl = a0 + p + 1u - st + 1u;
      lds.word[slot]    = (min(wl, kMaxWord) << 16) | (16u * gl + p);
      ++slot;
    }
    // words of this chunk that count (the row's word limit may cut them short)
    uint32_t const allowed = chunk_ok ? min(my_gtotal, cap - wdone) : 0u;
    uint32_t const wd_after = wdone + allowed;
    uint32_t const r_now    = r;
    if (gl == 0) {
      int64_t const o_cur    = reinterpret_cast<const uint8_t*>(ctx.base) + ctx.mis - col.chars;
      int64_t const row_slot = ((o_cur - first_offset) >> 1) + r;
      *reinterpret_cast<uint4*>(&lds.group[g][0]) = make_uint4(my_gbase, allowed, cbase, wdone);
      *reinterpret_cast<uint4*>(&lds.group[g][4]) =
        make_uint4(ctx.mis, static_cast<uint32_t>(r), static_cast<uint32_t>(row_slot), static_cast<uint32_t>(static_cast<uint64_t>(row_slot) >> 32));
    }

    // ---- what this group looks at next; request it now so it arrives while the probes run
    bool const row_done = has_row && !(chunk_ok && cbase + kChunk < ctx.aend && wd_after < cap);
    if (has_row) {
      if (!row_done) {
        cbase += kChunk;
        wdone = wd_after;
      } else {
        // the next row begins where this one ends
        int64_t const o_new = reinterpret_cast<const uint8_t*>(ctx.base) + ctx.aend - col.chars;
        int64_t const n_new = r + 1 < r_end ? e_nxt - o_new : 0;
        ++r;
        ctx   = make_row_ctx(col, o_new, n_new);
        cbase = 0;
        wdone = 0;
        carry_start = 0;
        prev_space  = 1;
        if (r < r_end) cap = word_cap(r, n_new);
        if (r + 1 < r_end) e_nxt = col.off(static_cast<int64_t>(r) + 2);
      }
      if (r < r_end) {
        mine_cur = ctx.load_raw(cbase + 16 * gl);
        tail_cur = gl == kGroupLanes - 1 ? ctx.byte_at(cbase + kChunk) : 0x20u;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- probes (lanes <-> words, all groups pooled)
    for (uint32_t w0 = 0; w0 < total; w0 += kWave) {
      uint32_t const ws = w0 + lane;  // word slot
      int const gw      = (ws >= gb1) + (ws >= gb2) + (ws >= gb3);
      uint4 const ga    = *reinterpret_cast<const uint4*>(&lds.group[gw][0]);  // first slot, allowed, chunk base, words so far
      uint4 const gb    = *reinterpret_cast<const uint4*>(&lds.group[gw][4]);  // row start in its block, row, arena slot of the row
      uint32_t const idx = ws - ga.x;
      bool const active  = ws < total && idx < ga.y;
      bool miss       = false;
      uint32_t value  = 0, wl = 0, wstart = 0;
      uint32_t head[4] = {0u, 0u, 0u, 0u};
      if (active) {
        uint32_t const rec = lds.word[ws];
        wl     = rec >> 16;
        wstart = ga.z + (rec & 0xFFFFu) + 1u - wl;  // coordinate of the word's first byte
        if (wl >= kMaxWord) {
          value = static_cast<uint32_t>(table.unk_id);  // wordpiece_tokenize.cu:442-445, 738-741
        } else {
          int32_t id = kNone;
          RingWord const rw_{lds.bytes[gw], wstart & (kRing - 1)};
          rw_.head16(head);
          trim_key8(wl, head[0], head[1]);
          trim_key8(wl > 8 ? wl - 8u : 0u, head[2], head[3]);
          if (wl <= table.max_len[0]) {
            // hash of the first two blocks without a loop; longer words go on from there
            Probe pr;
            pr.k0 = head[0];
            pr.k1 = head[1];
            uint32_t h        = key_hash_block(key_hash_init(wl), pr.k0, pr.k1);
            uint32_t const h2 = key_hash_block(h, head[2], head[3]);
            h                 = wl > 8 ? h2 : h;
            if (wl > 16) {
              for (uint32_t done = 16; done < wl; done += 8) {
                uint32_t b0, b1;
                rw_.key8(done, wl - done, &b0, &b1);
                h = key_hash_block(h, b0, b1);
              }
            }
            uint32_t b;
            pr.want   = slot_word0(h, 0, wl, &b);
            pr.bucket = b & table.bucket_mask;
            uint4 const s0 = table.slots[2 * pr.bucket];
            uint4 const s1 = table.slots[2 * pr.bucket + 1];
            uint32_t v = verdict(pr, s0, s1, wl, &id);
            if (v == 2u && wl > 8 && wl <= 16) v = verdict_16(table, pr, s0, s1, head, &id);
            if (v == 2u) id = finish_probe(table, pr, s0, s1, rw_, 0u, wl);
            else if (v == 0u) id = kNone;
          }
          miss  = id == kNone;
          value = static_cast<uint32_t>(id);
        }
      }
      uint64_t const mm = ballot64(miss);
      if (mm) {
        uint32_t const nm   = static_cast<uint32_t>(__builtin_popcountll(mm));
        uint32_t const room = q_lim - q_pos;  // left of the reserved range: filled up before the next one is begun,
        uint32_t fresh      = 0;              // so that unused entries only ever follow a wavefront's last word
        if (nm > room) {                      // my_block >= 64 >= nm
          // a range that lasted only a few steps is followed by one twice as long: atomics on the one counter
          // run at about 150 M/s for the whole device, and unused entries cost the next pass time
          if (steps_in_range < 8u && my_block < queue_block) my_block <<= 1;
          steps_in_range = 0;
          if (lane == 0) fresh = atomicAdd(queue_size, my_block);
          fresh = wave_bcast(fresh, 0);
        }
        if (miss) {
          uint32_t const rank = lanes_below(mm);
          uint32_t const q    = rank < room ? q_pos + rank : fresh + (rank - room);
          if (q < queue_capacity) {
            uint4* const dst = reinterpret_cast<uint4*>(queue + q);
            store_stream(dst, make_uint4(gb.y, wstart - gb.x, ga.w + idx, wl));
            store_stream(dst + 1, make_uint4(head[0], head[1], head[2], head[3]));
          }
          value = kOovMark | q;
        }
        if (nm > room) {
          q_pos = fresh + (nm - room);
          q_lim = fresh + my_block;
        } else {
          q_pos += nm;
        }
      }
      if (active) {
        int64_t const s = static_cast<int64_t>((static_cast<uint64_t>(gb.w) << 32) | gb.z) + ga.w + idx;
        store_stream(arena + s, value);
      }
    }
    if (row_done && gl == 0) {
      // one token per word; the out-of-vocabulary pass adds what its words give beyond that
      nwords[r_now] = static_cast<int32_t>(wd_after);
      counts[r_now] = static_cast<int32_t>(wd_after);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  for (uint32_t q = q_pos + lane; q < q_lim; q += kWave)
    if (q < queue_capacity) queue[q] = OovEntry{-1, 0u, 0u, 0u, {0u, 0u, 0u, 0u}};
}

// ------------------------------------------------------------------ out-of-vocabulary pass
// Greedy longest-match-first tokenization (cpp/src/text/wordpiece_tokenize.cu:349-407) of a word whose
// whole-word lookup has already failed, as a resumable state machine: every step() examines up to two
// candidates (their table reads are in flight together) and the lanes of a wavefront, each somewhere
// inside its own word, share the trips.  The state is the piece being searched, bytes [start, e): the
// first piece (start 0) lives in the full key space, later ones in the "##" space.
template <typename W>
struct OovStepper {
  uint32_t len, start, e, count;
  uint32_t raw0, raw1;  // bytes [start, start+8) of the word
  uint32_t lens;        // length filter word of the piece that starts at `start` (all ones when it is shorter than 3 bytes)
  bool ascii;           // no byte of the word has bit 7 set: every position is a character boundary
  bool fresh;           // [start, e) itself is still untried
  bool done;

  __device__ __forceinline__ bool inside_character(W const& w, uint32_t x) const { return !ascii && is_utf8_continuation(w.byte(x)); }

  // wordpiece_tokenize.cu:307-317: the end after dropping the last UTF-8 character of [start, x); start if none is left
  __device__ __forceinline__ uint32_t drop(W const& w, uint32_t x) const
  {
    if (x - start < 2) return start;
    --x;
    while (x > start && inside_character(w, x)) --x;
    return x;
  }

  // The longest candidate end <= x (x on a character boundary, start < x < len or x == len) that the length
  // filter does not rule out and that ends on a character boundary; start if there is none.  Only lengths
  // without a key are skipped, so the candidates that can match are visited in the reference's order.
  __device__ __forceinline__ uint32_t allowed_end(W const& w, uint32_t x) const
  {
    uint32_t l = x - start;
    bool boundary = true;  // start + l is known to be a character boundary
    while (l >= 3) {
      if (l >= 34 && (lens >> 31)) break;
      uint32_t const top = min(l - 3u, 30u);
      uint32_t const m   = lens & (0xFFFFFFFFu >> (31u - top));
      if (m == 0) {
        l        = 2;
        boundary = false;
        break;
      }
      uint32_t const best = 34u - static_cast<uint32_t>(__builtin_clz(m));  // 3 + index of the highest set bit
      boundary            = boundary && best == l;
      l                   = best;
      if (boundary || !inside_character(w, start + l)) {
        boundary = true;
        break;
      }
      --l;
    }
    if (!boundary)
      while (l > 0 && inside_character(w, start + l)) --l;
    return start + l;
  }

  __device__ __forceinline__ void load_filter(VocabTable const& t, uint32_t kind)
  {
    lens = len - start >= 3 ? t.lens[length_filter_index(kind, raw0 & 0x00FFFFFFu) & t.lens_mask] : 0xFFFFFFFFu;
  }

  __device__ __forceinline__ void begin(VocabTable const& t, W const& w, uint32_t len_, bool ascii_)
  {
    len = len_; start = 0; e = len_; count = 0;
    ascii = ascii_;
    fresh = false;  // the whole word is known to be absent: begin by shortening it
    done  = false;
    w.key8(0, min(len, 8u), &raw0, &raw1);
    load_filter(t, 0);
  }

  template <typename Emit>
  __device__ __forceinline__ void step(VocabTable const& t, W const& w, Emit&& emit)
  {
    uint32_t const kind = count ? 1u : 0u;
    uint32_t const maxl = t.max_len[kind];
    uint32_t ea         = fresh ? e : drop(w, e);
    if (ea - start > maxl) {
      // no key is this long: go straight to the longest candidate that can exist (on a character boundary)
      ea = start + maxl;
      while (ea > start && inside_character(w, ea)) --ea;
    }
    ea = allowed_end(w, ea);
    if (ea == start) {
      // no prefix of the word matched (375-379), or a later piece has no match and the word collapses
      // (396-404): either way a single unknown token
      emit(0u, t.unk_id);
      count = 1;
      done  = true;
      return;
    }
    uint32_t const eb = allowed_end(w, drop(w, ea));
    bool const has_b  = eb > start;
    Probe const pa    = make_probe(t, kind, w, start, ea - start, raw0, raw1);
    Probe const pb    = make_probe(t, kind, w, start, has_b ? eb - start : 1u, raw0, raw1);
    uint4 const a0 = t.slots[2 * pa.bucket], a1 = t.slots[2 * pa.bucket + 1];
    uint4 b0 = make_uint4(0, 0, 0, 0), b1 = b0;
    if (has_b) {
      b0 = t.slots[2 * pb.bucket];
      b1 = t.slots[2 * pb.bucket + 1];
    }
    uint32_t hit_end = ea;
    int32_t id       = finish_probe(t, pa, a0, a1, w, start, ea - start);
    if (id == kNone && has_b) {
      hit_end = eb;
      id      = finish_probe(t, pb, b0, b1, w, start, eb - start);
    }
    if (id == kNone) {
      e     = has_b ? eb : ea;
      fresh = false;
      return;
    }
    emit(count++, id);
    if (hit_end == len) {
      done = true;
      return;
    }
    // next piece: the rest of the word (381-395)
    start = hit_end;
    e     = len;
    fresh = true;
    w.key8(start, min(len - start, 8u), &raw0, &raw1);
    load_filter(t, 1);
  }
};

// Runs one word to completion (used where out-of-vocabulary words are rare).  Returns the token count.
template <typename W, typename Emit>
__device__ __forceinline__ uint32_t tokenize_oov_word(VocabTable const& t, W const& w, uint32_t len, Emit emit)
{
  OovStepper<W> st;
  st.begin(t, w, len, false);
  while (!st.done) st.step(t, w, emit);
  return st.count;
}

// Brings the first bytes of the `len`-byte word at p into this lane's LDS window with 16-byte aligned
// loads (only blocks that overlap the word).  *ascii = no byte of the word has bit 7 set (judged on the
// whole blocks, so it may be false for a plain word next to other text; never true wrongly).
__device__ __forceinline__ uint32_t stage_word(const uint8_t* p, uint32_t len, uint32_t* win, bool* ascii)
{
  uint32_t const mis    = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p) & 15u);
  const uint4* a        = reinterpret_cast<const uint4*>(p - mis);
  uint32_t const need   = (mis + len + 15u) >> 4;
  uint32_t const blocks = min(kStage / 16, need);
  uint32_t seen         = 0;
  for (uint32_t i = 0; i < blocks; ++i) {
    uint4 const v = a[i];
    seen |= v.x | v.y | v.z | v.w;
    win[(4 * i + 0) * kOovThreads] = v.x;
    win[(4 * i + 1) * kOovThreads] = v.y;
    win[(4 * i + 2) * kOovThreads] = v.z;
    win[(4 * i + 3) * kOovThreads] = v.w;
  }
  *ascii = (seen & 0x80808080u) == 0 && need <= kStage / 16;
  return mis;
}

// Bit 7 of every byte of x that is a UTF-8 continuation byte (10xxxxxx); exact, no carries cross bytes.
__device__ __forceinline__ uint32_t continuation_bytes(uint32_t x)
{
  uint32_t const t = (x & 0xC0C0C0C0u) ^ 0x80808080u;
  return ~(((t & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | t) & 0x80808080u;
}

// The rest of a word of at most 16 bytes, held in registers from the piece being searched on: the whole
// greedy longest-match-first rule (cpp/src/text/wordpiece_tokenize.cu:349-407) becomes bit operations
// on a mask of candidate lengths, with no loop over bytes and no memory but the table reads.
struct ShortWord {
  uint32_t r[4];   // bytes [start, start + 16) of the word, zero padded
  uint32_t rem;    // bytes from start to the end of the word
  uint32_t bnd;    // bit i: start + i is a character boundary (bit rem is set)
  uint32_t cand;   // lengths still to try for the piece at start (bit l - 1), longest first
  uint32_t count;  // tokens so far
  int32_t id1, id2;  // ids of the piece's first byte and first two bytes as keys (kNone: no such key)
  bool done;

  __device__ __forceinline__ uint32_t byte(uint32_t k) const
  {
    uint32_t const d = k >> 2;
    uint32_t const v = d == 0 ? r[0] : d == 1 ? r[1] : d == 2 ? r[2] : r[3];
    return (v >> (8 * (k & 3u))) & 0xffu;
  }
  __device__ __forceinline__ void key8(uint32_t p, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    // only called with p = 8 by the generic probe code (keys of 9 to 16 bytes)
    uint32_t lo = p == 0 ? r[0] : r[2], hi = p == 0 ? r[1] : r[3];
    trim_key8(len, lo, hi);
    *k0 = lo;
    *k1 = hi;
  }

  // Candidate lengths of the piece at start: on a character boundary, no longer than the rest of the word
  // or the longest key, and not ruled out by the length filter of the piece's first three bytes.
  __device__ __forceinline__ void open_piece(VocabTable const& t, uint32_t kind)
  {
    uint32_t const lens = rem >= 3 ? t.lens[length_filter_index(kind, r[0] & 0x00FFFFFFu) & t.lens_mask] : 0xFFFFFFFFu;
    uint32_t const lim  = min(min(rem, t.max_len[kind]), 16u);
    cand                = (bnd >> 1) & ((1u << lim) - 1u) & ((lens << 2) | 3u);
    id1                 = t.short_ids[2 * 65536 + kind * 256 + (r[0] & 0xFFu)];
    id2                 = rem >= 2 ? t.short_ids[kind * 65536 + (r[0] & 0xFFFFu)] : kNone;
  }

  __device__ __forceinline__ void begin(VocabTable const& t, const uint32_t (&head)[4], uint32_t len)
  {
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = head[k];
    rem   = len;
    count = 0;
    done  = false;
    uint32_t const cont = gather_byte_flags(continuation_bytes(r[0])) | (gather_byte_flags(continuation_bytes(r[1])) << 4) |
                          (gather_byte_flags(continuation_bytes(r[2])) << 8) | (gather_byte_flags(continuation_bytes(r[3])) << 12);
    bnd = (~cont & ((1u << len) - 1u)) | (1u << len);
    open_piece(t, 0);
    cand &= ~(1u << (len - 1));  // the whole word is known to be absent
  }

  __device__ __forceinline__ Probe probe_of(VocabTable const& t, uint32_t kind, uint32_t l) const
  {
    Probe pr;
    pr.k0 = r[0];
    pr.k1 = r[1];
    trim_key8(min(l, 8u), pr.k0, pr.k1);
    uint32_t h  = key_hash_block(key_hash_init(l), pr.k0, pr.k1);
    uint32_t k2 = r[2], k3 = r[3];
    trim_key8(l > 8 ? l - 8u : 0u, k2, k3);
    uint32_t const h2 = key_hash_block(h, k2, k3);
    h                 = l > 8 ? h2 : h;
    uint32_t b;
    pr.want   = slot_word0(h, kind, l, &b);
    pr.bucket = b & t.bucket_mask;
    return pr;
  }

  // Drops the first l bytes (a matched piece).
  __device__ __forceinline__ void advance(uint32_t l)
  {
    uint32_t const d  = l >> 2;
    uint32_t const sh = (l & 3u) * 8u;
    uint32_t const t0 = d == 0 ? r[0] : d == 1 ? r[1] : d == 2 ? r[2] : r[3];
    uint32_t const t1 = d == 0 ? r[1] : d == 1 ? r[2] : d == 2 ? r[3] : 0u;
    uint32_t const t2 = d == 0 ? r[2] : d == 1 ? r[3] : 0u;
    uint32_t const t3 = d == 0 ? r[3] : 0u;
    r[0] = __builtin_amdgcn_alignbit(t1, t0, sh);
    r[1] = __builtin_amdgcn_alignbit(t2, t1, sh);
    r[2] = __builtin_amdgcn_alignbit(t3, t2, sh);
    r[3] = t3 >> sh;
    rem -= l;
    bnd >>= l;
  }

  // One trip: probes the longest remaining candidate of three bytes and more; when none of those is left, the
  // candidates of two bytes and of one byte are settled from the ids fetched when the piece was opened, without
  // hashing or further reads.  (The length filter leaves few candidates: a piece that has any has 1.4 on average,
  // so a second probe in the same trip would mostly be wasted work.)
  template <typename Emit>
  __device__ __forceinline__ void step(VocabTable const& t, Emit&& emit)
  {
    uint32_t const kind   = count ? 1u : 0u;
    uint32_t const longer = cand & ~3u;
    bool const has_a      = longer != 0;
    uint32_t const la     = 32u - static_cast<uint32_t>(__builtin_clz(has_a ? longer : 4u));
    bool hit_a            = false;
    int32_t ida           = kNone;
    if (has_a) {
      Probe const pa = probe_of(t, kind, la);
      uint4 const a0 = t.slots[2 * pa.bucket], a1 = t.slots[2 * pa.bucket + 1];
      uint32_t va    = verdict(pa, a0, a1, la, &ida);
      if (va == 2u) {  // the general lookup (keys in the pool, overflowing buckets)
        ida = finish_probe(t, pa, a0, a1, *this, 0u, la);
        va  = ida == kNone ? 0u : 1u;
      }
      hit_a = va == 1u;
    }
    uint32_t const longer_left = has_a ? longer ^ (1u << (la - 1)) : 0u;  // after a miss
    bool hit     = hit_a;
    uint32_t len = la;
    int32_t id   = ida;
    bool unknown = false;
    if (!hit && longer_left == 0) {
      // two bytes, then one byte; else no prefix of the word matched (375-379), or a later piece has no match and
      // the word collapses (396-404): either way a single unknown token
      bool const two = (cand & 2u) != 0 && id2 != kNone;
      bool const one = (cand & 1u) != 0 && id1 != kNone;
      hit            = two || one;
      len            = two ? 2u : 1u;
      id             = two ? id2 : id1;
      unknown        = !hit;
    }
    if (hit || unknown) emit(unknown ? 0u : count, unknown ? t.unk_id : id);
    count = unknown ? 1u : count + (hit ? 1u : 0u);
    done  = unknown || (hit && len == rem);
    cand  = longer_left | (cand & 3u);
    if (hit && !done) {
      advance(len);  // next piece: the rest of the word (381-395)
      open_piece(t, 1);
    }
  }
};

// One lane per queued word, and a lane that finishes its word takes the next one: every wavefront owns a
// contiguous part of the queue and, every eighth trip, lets its idle lanes store their result and pick up
// new entries, so lanes with short words do not wait for the longest word of a batch.  Words of up to 16
// bytes (whole in their queue record) run in registers; the few longer ones are set aside for the kernel
// below: their queue indices go to longer[first entry of the part ...], their number to
// longer[queue_capacity + wavefront].
// results[q] = the word's first kOovKeep tokens and its token count; counts[row] += count - 1.
__global__ void __launch_bounds__(kOovThreads, 8) wordpiece_oov_kernel(ColView col, VocabTable table, const OovEntry* __restrict__ queue,
                                                                    const uint32_t* __restrict__ queue_size, uint32_t queue_capacity,
                                                                    OovResult* __restrict__ results, int32_t* __restrict__ counts,
                                                                    uint32_t* __restrict__ longer)
{
  if (*queue_size > queue_capacity) return;  // the queue was too small: the host repeats the passes with a larger one
  uint32_t const total  = min(*queue_size, queue_capacity);
  uint32_t const nwave  = gridDim.x * (kOovThreads / kWave);
  uint32_t const wave   = blockIdx.x * (kOovThreads / kWave) + threadIdx.x / kWave;
  uint32_t const chunk  = (total + nwave - 1) / nwave;
  uint32_t const q_begin = min(total, wave * chunk);
  uint32_t next          = q_begin;                          // wave-uniform cursor into this wavefront's part
  uint32_t const q_end   = min(total, next + chunk);
  uint32_t n_longer      = 0;                                // entries of this part set aside (wave-uniform)
  int const lane         = lane_id();

  int32_t tok[kOovKeep];
  auto keep_token = [&](uint32_t j, int32_t id) {
#pragma unroll
    for (int k = 0; k < kOovKeep; ++k)
      if (j == static_cast<uint32_t>(k)) tok[k] = id;
  };
  auto deliver = [&](uint32_t q, int32_t row, uint32_t count) {
    uint4* const dst = reinterpret_cast<uint4*>(results + q);
    store_stream(dst, make_uint4(static_cast<uint32_t>(tok[0]), static_cast<uint32_t>(tok[1]), static_cast<uint32_t>(tok[2]), static_cast<uint32_t>(tok[3])));
    store_stream(dst + 1, make_uint4(static_cast<uint32_t>(tok[4]), static_cast<uint32_t>(tok[5]), static_cast<uint32_t>(tok[6]), count));
    if (count > 1) atomicAdd(&counts[row], static_cast<int32_t>(count - 1));  // the probe pass has counted one token per word
  };

  {
    ShortWord sw;
    sw.done    = true;
    bool busy  = false;  // this lane holds a word (finished or not)
    uint32_t q = 0;
    int32_t row = -1;
    for (uint32_t trip = 0;; ++trip) {
      if ((trip & 7u) == 0) {
        if (busy && sw.done) {
          deliver(q, row, sw.count);
          busy = false;
        }
        uint64_t const idle = ballot64(!busy);
        if (idle != 0 && next < q_end) {  // refill
          uint32_t const mine = next + lanes_below(idle);
          next += static_cast<uint32_t>(__builtin_popcountll(idle));
          bool is_longer = false;
          if (!busy && mine < q_end) {
            const uint4* const src = reinterpret_cast<const uint4*>(queue + mine);
            uint4 const a = load_stream(src), b = load_stream(src + 1);
            if (static_cast<int32_t>(a.x) >= 0) {  // (-1 marks the unused tail of a reserved queue range)
              if (a.w <= 16) {
                q   = mine;
                row = static_cast<int32_t>(a.x);
                uint32_t const head[4] = {b.x, b.y, b.z, b.w};
                sw.begin(table, head, a.w);
                busy = true;
              } else {
                is_longer = true;
              }
            }
          }
          uint64_t const lm = ballot64(is_longer);
          if (lm != 0) {
            if (is_longer) longer[q_begin + n_longer + lanes_below(lm)] = mine;
            n_longer += static_cast<uint32_t>(__builtin_popcountll(lm));
          }
        }
        if (ballot64(busy) == 0 && next >= q_end) break;
      }
      if (busy && !sw.done) sw.step(table, keep_token);
    }
  }

  if (lane == 0) longer[queue_capacity + wave] = n_longer;
}

// The queued words of more than 16 bytes, which the kernel above has set aside (same grid, same parts):
// one lane per word, bytes staged from the chars into the lane's LDS window, the general state machine.
__global__ void __launch_bounds__(kOovThreads) wordpiece_oov_long_kernel(ColView col, VocabTable table, const OovEntry* __restrict__ queue,
                                                                         const uint32_t* __restrict__ queue_size, uint32_t queue_capacity,
                                                                         OovResult* __restrict__ results, int32_t* __restrict__ counts,
                                                                         const uint32_t* __restrict__ longer)
{
  __shared__ uint32_t windows[kStage / 4][kOovThreads];
  uint32_t* const win    = &windows[0][threadIdx.x];
  if (*queue_size > queue_capacity) return;  // (see wordpiece_oov_kernel)
  uint32_t const total   = min(*queue_size, queue_capacity);
  uint32_t const nwave   = gridDim.x * (kOovThreads / kWave);
  uint32_t const wave    = blockIdx.x * (kOovThreads / kWave) + threadIdx.x / kWave;
  uint32_t const chunk   = (total + nwave - 1) / nwave;
  uint32_t const q_begin = min(total, wave * chunk);
  uint32_t const n_longer = longer[queue_capacity + wave];
  uint32_t const lane    = static_cast<uint32_t>(lane_id());
  for (uint32_t base = 0; base < n_longer; base += kWave) {
    if (base + lane < n_longer) {
      uint32_t const q = longer[q_begin + base + lane];
      OovEntry const e = queue[q];
      const uint8_t* p = col.chars + col.off(e.row) + e.delta;
      bool ascii;
      StagedWord w{win, p, 0};
      w.mis = stage_word(p, e.len, win, &ascii);
      OovResult res;
      OovStepper<StagedWord> st;
      st.begin(table, w, e.len, ascii);
      while (!st.done) {
        st.step(table, w, [&](uint32_t j, int32_t id) {
#pragma unroll
          for (int k = 0; k < kOovKeep; ++k)
            if (j == static_cast<uint32_t>(k)) res.tok[k] = id;
        });
      }
      res.count  = st.count;
      results[q] = res;
      if (st.count > 1) atomicAdd(&counts[e.row], static_cast<int32_t>(st.count - 1));
    }
  }
}

// ------------------------------------------------------------------ emit pass
// Expands the word arena into the child column.  A wavefront takes a block of consecutive rows at a time (at most
// 64, fewer where rows have many tokens: emit_blocks_kernel; lanes <-> rows for the descriptors), then walks ALL
// their words flat, lanes <-> words: because the
// list offsets are a prefix sum in row order, the tokens of consecutive words are consecutive in the
// child even across row boundaries, so only the block's first offset is needed.  Each word finds its
// row by binary search in the block's word-count prefix (LDS); its lane then writes its tokens (one, or the up to
// kOovKeep that the out-of-vocabulary pass left in its result record) behind those of the lanes below it.
struct EmitLds {
  uint32_t word_prefix[kWave + 1];  // words before row k of the block
  int64_t slot0[kWave];             // arena slot of word 0 of row k
};

__global__ void __launch_bounds__(kTokThreads) wordpiece_emit_kernel(ColView col, VocabTable table, int64_t first_offset,
                                                                     const uint32_t* __restrict__ arena,
                                                                     const int32_t* __restrict__ nwords, OovResult* __restrict__ results,
                                                                     const int32_t* __restrict__ offsets, int32_t* __restrict__ out,
                                                                     const int32_t* __restrict__ block_first, int64_t nblocks,
                                                                     uint32_t* __restrict__ again, uint32_t* __restrict__ again_count)
{
  // block_rows (1..64) rows per wavefront at a time: fewer when rows are long, so that the walks stay
  // short and there are enough of them to fill the device
  __shared__ EmitLds lds_all[kTokWaves];
  int const lane        = lane_id();
  int const wave        = threadIdx.x / kWave;
  EmitLds& lds          = lds_all[wave];
  int64_t const nwave   = static_cast<int64_t>(gridDim.x) * kTokWaves;
  auto lds_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  for (int64_t blk = static_cast<int64_t>(blockIdx.x) * kTokWaves + wave; blk < nblocks; blk += nwave) {
    // rows [first, next) of the block: at most kWave
    int32_t const first = block_first[blk], next = block_first[blk + 1];
    int64_t const r     = static_cast<int64_t>(first) + lane;
    uint32_t W          = 0;
    int64_t slot0       = 0;
    if (lane < next - first) {
      W     = static_cast<uint32_t>(nwords[r]);
      slot0 = arena_pos(col, first_offset, r);
    }
    int32_t const base   = offsets[first];
    uint32_t const incl  = wave_inclusive_scan(W);
    uint32_t const total = wave_bcast(incl, kWave - 1);
    lds.word_prefix[lane] = incl - W;
    if (lane == kWave - 1) lds.word_prefix[kWave] = total;
    lds.slot0[lane] = slot0;
    lds_sync();

    // the arena entry of flat word j: row k = last row with word_prefix[k] <= j (rows without words are skipped
    // because their prefix equals the next row's)
    auto load_value = [&](uint32_t j) -> uint32_t {
      if (j >= total) return 0u;
      uint32_t lo = 0;
#pragma unroll
      for (uint32_t step = kWave / 2; step > 0; step >>= 1)
        if (lds.word_prefix[lo + step] <= j) lo += step;
      return arena[lds.slot0[lo] + (j - lds.word_prefix[lo])];
    };
    // tokens of flat word j whose arena value is v: one, or what the out-of-vocabulary pass found (its whole
    // result record is fetched here, once)
    auto count_of = [&](uint32_t j, uint32_t v, uint4& ra, uint4& rb) -> uint32_t {
      if (j >= total) return 0u;
      if ((v & kOovMark) == 0 || v == 0xFFFFFFFFu) return 1u;
      const uint4* const src = reinterpret_cast<const uint4*>(results + (v & ~kOovMark));
      ra = src[0];
      rb = src[1];
      return rb.w;  // OovResult: seven tokens, then the count
    };

    int32_t* const dst = out + base;
    uint32_t done      = 0;  // tokens written so far in this block
    // three stages in flight: arena value two rounds ahead, token count one round ahead, the round being written
    uint32_t v_nxt = load_value(lane);
    uint32_t v_far = load_value(kWave + lane);
    uint4 a_nxt = make_uint4(0u, 0u, 0u, 0u), b_nxt = a_nxt;
    uint32_t c_nxt = count_of(lane, v_nxt, a_nxt, b_nxt);
    for (uint32_t j0 = 0; j0 < total; j0 += kWave) {
      uint32_t const value = v_nxt, cnt = c_nxt;
      uint4 const ra = a_nxt, rb = b_nxt;
      v_nxt = v_far;
      c_nxt = count_of(j0 + kWave + lane, v_nxt, a_nxt, b_nxt);
      v_far = load_value(j0 + 2 * kWave + lane);
      uint32_t const here   = min(total - j0, static_cast<uint32_t>(kWave));  // words of this round (every word has >= 1 token)
      uint32_t const incl2  = wave_inclusive_scan(cnt);
      uint32_t const tokens = wave_bcast(incl2, kWave - 1);
      bool const marked     = static_cast<uint32_t>(lane) < here && (value & kOovMark) != 0 && value != 0xFFFFFFFFu;
      // lanes <-> words: every lane writes its word's tokens behind those of the words below it, token k of all
      // words at a time (a word from the queue has up to kOovKeep of them in its record)
      int32_t* const mine = dst + done + (incl2 - cnt);
      if (marked && cnt > kOovKeep) {
        // more pieces than a result record keeps (seldom): noted for wordpiece_retokenize_kernel, with the
        // place of the word's first token in the child left where its tokens would have been
        uint32_t const q = value & ~kOovMark;
        again[atomicAdd(again_count, 1u)] = q;
        results[q].tok[0]                 = base + static_cast<int32_t>(done + (incl2 - cnt));
      } else {
        uint32_t const mc = static_cast<uint32_t>(lane) < here ? cnt : 0u;
        if (mc > 0u) mine[0] = static_cast<int32_t>(marked ? ra.x : value);
        if (ballot64(mc > 1u) != 0) {
          if (mc > 1u) mine[1] = static_cast<int32_t>(ra.y);
          if (mc > 2u) mine[2] = static_cast<int32_t>(ra.z);
          if (ballot64(mc > 3u) != 0) {
            if (mc > 3u) mine[3] = static_cast<int32_t>(ra.w);
            if (mc > 4u) mine[4] = static_cast<int32_t>(rb.x);
            if (mc > 5u) mine[5] = static_cast<int32_t>(rb.y);
            if (mc > 6u) mine[6] = static_cast<int32_t>(rb.z);
          }
        }
      }
      done += tokens;
    }
    lds_sync();
  }
}

// The words that have more pieces than a result record keeps (the emit pass has listed them in again[0 .. *again_count)
// and left the index of each one's first token in the child in its result record): tokenized again, straight into
// place.  One lane per word; kept apart from the emit pass so that it is compiled for its common case (a third of
// the registers, all the wavefronts a unit can hold).
__global__ void __launch_bounds__(kOovThreads) wordpiece_retokenize_kernel(ColView col, VocabTable table, const OovEntry* __restrict__ queue,
                                                                           const OovResult* __restrict__ results,
                                                                           const uint32_t* __restrict__ again,
                                                                           const uint32_t* __restrict__ again_count, int32_t* __restrict__ out)
{
  uint32_t const n = *again_count;
  for (uint32_t i = blockIdx.x * kOovThreads + threadIdx.x; i < n; i += gridDim.x * kOovThreads) {
    uint32_t const q = again[i];
    OovEntry const e = queue[q];
    const uint8_t* p = col.chars + col.off(e.row) + e.delta;
    int32_t* const d = out + results[q].tok[0];
    tokenize_oov_word(table, GlobalWord{p}, e.len, [&](uint32_t j, int32_t id) { d[j] = id; });
  }
}

// The blocks of rows of the emit pass: block b begins with the first row r for which offsets[r] + kEmitRowWeight * r
// reaches b * kEmitBlockWork, so a block holds at most kEmitBlockWork / kEmitRowWeight = 64 rows and, unless it is a
// single row, fewer than kEmitBlockWork tokens, however uneven the rows are.  block_first has nblocks + 1 entries.
constexpr int64_t kEmitRowWeight = 128;
constexpr int64_t kEmitBlockWork = kEmitRowWeight * kWave;
__global__ void emit_blocks_kernel(const int32_t* __restrict__ offsets, int64_t rows, int64_t nblocks, int32_t* __restrict__ block_first)
{
  int64_t const b = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (b > nblocks) return;
  int64_t lo = 0, hi = rows;  // the first row in [0, rows] with that much work before it
  if (b == nblocks) lo = rows;
  int64_t const target = b * kEmitBlockWork;
  while (lo < hi) {
    int64_t const mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(offsets[mid]) + kEmitRowWeight * mid < target) lo = mid + 1;
    else hi = mid;
  }
  block_first[b] = static_cast<int32_t>(lo);
}

// ------------------------------------------------------------------ very long rows
// A row is walked by one group of lanes in the probe pass and by one wavefront in the emit pass, so a row of
// megabytes would take milliseconds while the rest of the device is idle.  Without a word limit the tokens of a row
// are simply those of its words in order, so such a row can be cut at spaces into pieces that are tokenized as
// rows of their own; the list offsets of the original rows are then those of their first pieces.
constexpr int64_t kLongRow  = 32 * 1024;  // rows beyond this many bytes are cut
constexpr int64_t kRowPiece = 16 * 1024;  // into pieces of about this many

// pieces[r] = pieces row r is cut into (1 for rows that stay whole); *any_long = 1 when some row is cut
__global__ void long_rows_kernel(ColView col, uint32_t* __restrict__ pieces, uint32_t* __restrict__ any_long)
{
  int64_t const r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r >= col.size) return;
  int64_t const bytes = col.off(r + 1) - col.off(r);
  bool const is_long  = bytes > kLongRow;
  pieces[r]           = is_long ? static_cast<uint32_t>((bytes + kRowPiece - 1) / kRowPiece) : 1u;
  if (is_long) *any_long = 1u;
}

struct PiecesOf {
  const uint32_t* pieces;
  __device__ uint64_t operator()(int64_t i) const { return pieces[i]; }
};

// piece_offset[v] = where piece v begins: piece j > 0 of a row begins at the first space at or after byte
// j * kRowPiece of the row (the row's end if there is none), so no word is cut.  first_piece[r] = index of row r's
// first piece, first_piece[rows] = number of pieces.
__global__ void piece_offsets_kernel(ColView col, const uint32_t* __restrict__ first_piece, int64_t pieces, int64_t* __restrict__ piece_offset)
{
  int64_t const v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (v > pieces) return;
  int64_t const rows = col.size;
  if (v == pieces) {
    piece_offset[v] = col.off(rows);
    return;
  }
  int64_t lo = 0, hi = rows - 1;  // the last row whose first piece is at or before v
  while (lo < hi) {
    int64_t const mid = (lo + hi + 1) >> 1;
    if (static_cast<int64_t>(first_piece[mid]) <= v) lo = mid;
    else hi = mid - 1;
  }
  int64_t const j = v - first_piece[lo];
  int64_t p       = col.off(lo);
  if (j > 0) {
    int64_t const end = col.off(lo + 1);
    p += j * kRowPiece;
    // eight bytes at a time from an aligned address (ordinary text has a space within a few bytes; a stretch
    // without one is read to its end)
    const uint8_t* const chars = col.chars;
    while (p < end && (reinterpret_cast<uintptr_t>(chars + p) & 7u) != 0 && chars[p] != ' ') ++p;
    while (p + 8 <= end && chars[p] != ' ') {
      uint2 const w      = *reinterpret_cast<const uint2*>(chars + p);
      uint32_t const lo  = space_bytes(w.x), hi = space_bytes(w.y);
      if ((lo | hi) != 0) {
        p += lo ? (__builtin_ctz(lo) >> 3) : 4 + (__builtin_ctz(hi) >> 3);
        break;
      }
      p += 8;
    }
    while (p < end && chars[p] != ' ') ++p;
  }
  piece_offset[v] = p;
}

// offsets[r] = piece_token_offsets[first_piece[r]] for r in 0..rows
__global__ void row_offsets_of_pieces_kernel(const int32_t* __restrict__ piece_token_offsets, const uint32_t* __restrict__ first_piece,
                                             int64_t rows, int32_t* __restrict__ offsets)
{
  int64_t const r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r <= rows) offsets[r] = piece_token_offsets[first_piece[r]];
}

struct CountOf {
  const int32_t* counts;
  __device__ uint64_t operator()(int64_t i) const { return static_cast<uint64_t>(counts[i]); }
};

// ------------------------------------------------------------------ vocabulary construction (host)
struct HostSlot {
  uint32_t x, y, z, w;
};

void host_key8(const uint8_t* key, uint32_t len, uint32_t* k0, uint32_t* k1)
{
  uint8_t buf[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  std::memcpy(buf, key, len < 8 ? len : 8);
  std::memcpy(k0, buf, 4);
  std::memcpy(k1, buf + 4, 4);
}

uint32_t host_hash(const uint8_t* key, uint32_t len)
{
  uint32_t h = key_hash_init(len);
  for (uint32_t done = 0; done < len; done += 8) {
    uint32_t lo, hi;
    host_key8(key + done, len - done, &lo, &hi);
    h = key_hash_block(h, lo, hi);
  }
  return h;
}

bool host_same(HostSlot const& s, uint32_t w0, const std::vector<uint8_t>& pool, const uint8_t* key, uint32_t len, uint32_t k0, uint32_t k1)
{
  if (s.x != w0) return false;
  return len <= 8 ? (s.z == k0 && s.w == k1) : (std::memcmp(pool.data() + s.z, key, len) == 0);
}

void host_insert(std::vector<HostSlot>& slots, uint32_t bucket_mask, const std::vector<uint8_t>& pool, uint32_t kind, const uint8_t* key,
                 uint32_t len, uint32_t pool_off, int32_t id)
{
  uint32_t b;
  uint32_t const w0 = slot_word0(host_hash(key, len), kind, len, &b);
  uint32_t k0 = 0, k1 = 0;
  if (len <= 8) host_key8(key, len, &k0, &k1);
  for (;;) {
    b &= bucket_mask;
    for (int j = 0; j < 2; ++j) {
      HostSlot& s = slots[2 * static_cast<size_t>(b) + j];
      if (s.x == 0) {
        s.x = w0;
        s.y = static_cast<uint32_t>(id);
        s.z = len <= 8 ? k0 : pool_off;
        s.w = len <= 8 ? k1 : 0u;
        return;
      }
      // the same key again: the first entry wins (duplicates are undefined in the reference)
      if (host_same(s, w0, pool, key, len, k0, k1)) return;
    }
    slots[2 * static_cast<size_t>(b)].y |= kSearchOn;  // the key is carried past this bucket
    ++b;
  }
}

int32_t host_find(const std::vector<HostSlot>& slots, uint32_t bucket_mask, const std::vector<uint8_t>& pool, const char* text)
{
  uint32_t const len = static_cast<uint32_t>(std::strlen(text));
  const uint8_t* key = reinterpret_cast<const uint8_t*>(text);
  uint32_t b;
  uint32_t const w0 = slot_word0(host_hash(key, len), 0, len, &b);
  uint32_t k0 = 0, k1 = 0;
  host_key8(key, len, &k0, &k1);
  for (;;) {
    b &= bucket_mask;
    for (int j = 0; j < 2; ++j) {
      HostSlot const& s = slots[2 * static_cast<size_t>(b) + j];
      if (s.x == 0) return -1;
      if (host_same(s, w0, pool, key, len, k0, k1)) return static_cast<int32_t>(s.y & ~kSearchOn);
    }
    ++b;
  }
}

}  // namespace
}  // namespace nvtext_amd

extern "C" {

nvtext_amd_status nvtext_amd_wordpiece_vocabulary_create(const nvtext_amd_strings_column* vocabulary, void* stream_, const nvtext_amd_allocator* mr,
                                                         nvtext_amd_wordpiece_vocabulary** out)
{
  using namespace nvtext_amd;
  (void)mr;  // the tables live as long as the object: plain hipMalloc / hipFree
  if (!vocabulary || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  // cpp/src/text/wordpiece_tokenize.cu:217-218
  if (vocabulary->size == 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary must not be empty");
  if (vocabulary->null_count > 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary must not have nulls");
  hipStream_t stream = static_cast<hipStream_t>(stream_);

  // bring the entries to the host (one-time, a few MB at most)
  int32_t const V      = vocabulary->size;
  size_t const ow      = vocabulary->offsets_is_int64 ? 8 : 4;
  std::vector<uint8_t> h_off((static_cast<size_t>(V) + 1) * ow);
  const uint8_t* d_off = static_cast<const uint8_t*>(vocabulary->offsets) + static_cast<size_t>(vocabulary->offset) * ow;
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
  int64_t const first = off_at(0), last = off_at(V);
  if (last < first) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary offsets are not monotone");
  std::vector<uint8_t> pool(static_cast<size_t>(last - first));
  if (!pool.empty()) {
    NVTEXT_HIP_TRY(hipMemcpyAsync(pool.data(), vocabulary->chars + first, pool.size(), hipMemcpyDeviceToHost, stream));
    NVTEXT_HIP_TRY(hipStreamSynchronize(stream));
  }

  // both key spaces share one table (wordpiece_tokenize.cu:224-263 builds two maps of capacity 2x each)
  size_t keys = 0;
  for (int32_t i = 0; i < V; ++i) {
    int64_t const b = off_at(i) - first, e = off_at(i + 1) - first;
    int64_t const len = e - b;
    if (len >= 1 && len < kMaxWord) ++keys;
    if (len >= 3 && len - 2 < kMaxWord && pool[b] == '#' && pool[b + 1] == '#') ++keys;
  }
  size_t capacity = 64;
  while (capacity < 2 * keys) capacity <<= 1;
  if (capacity > (size_t{1} << 31)) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary too large");
  uint32_t const mask = static_cast<uint32_t>(capacity / 2 - 1);  // buckets of two slots
  std::vector<HostSlot> slots(capacity, HostSlot{0, 0, 0, 0});
  uint32_t max_len[2] = {0, 0};
  // keys of more than 8 bytes, zero padded to whole 8-byte blocks
  std::vector<uint8_t> blocks;
  auto add_blocks = [&](const uint8_t* key, uint32_t len) -> uint32_t {
    if (len <= 8) return 0u;
    size_t const at = blocks.size();
    blocks.resize(at + ((static_cast<size_t>(len) + 7) & ~size_t{7}), 0);
    std::memcpy(blocks.data() + at, key, len);
    return static_cast<uint32_t>(at);
  };
  for (int32_t i = 0; i < V; ++i) {
    int64_t const b = off_at(i) - first, e = off_at(i + 1) - first;
    int64_t const len = e - b;
    // entries of 200 bytes or more can never equal a tokenizable word or piece; empty ones are never looked up
    if (len >= 1 && len < kMaxWord) {
      host_insert(slots, mask, blocks, 0, pool.data() + b, static_cast<uint32_t>(len), add_blocks(pool.data() + b, static_cast<uint32_t>(len)), i);
      max_len[0] = std::max(max_len[0], static_cast<uint32_t>(len));
    }
    // wordpiece_tokenize.cu:184-192: "##" entries also live, without the prefix, in the second key space
    if (len >= 3 && len - 2 < kMaxWord && pool[b] == '#' && pool[b + 1] == '#') {
      host_insert(slots, mask, blocks, 1, pool.data() + b + 2, static_cast<uint32_t>(len - 2), add_blocks(pool.data() + b + 2, static_cast<uint32_t>(len - 2)), i);
      max_len[1] = std::max(max_len[1], static_cast<uint32_t>(len - 2));
    }
  }
  if (blocks.size() > 0xFFFFFFF0ull) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary too large");

  // length filter over the first three bytes of every key of three bytes and more
  size_t lens_size = 1024;
  while (lens_size < 4 * keys) lens_size <<= 1;
  std::vector<uint32_t> lens(lens_size, 0u);
  auto note_length = [&](uint32_t kind, const uint8_t* key, uint32_t len) {
    if (len < 3) return;
    uint32_t const first3 = key[0] | (uint32_t{key[1]} << 8) | (uint32_t{key[2]} << 16);
    lens[length_filter_index(kind, first3) & (lens_size - 1)] |= 1u << length_filter_bit(len);
  };
  for (int32_t i = 0; i < V; ++i) {
    int64_t const b = off_at(i) - first, e = off_at(i + 1) - first;
    int64_t const len = e - b;
    if (len >= 1 && len < kMaxWord) note_length(0, pool.data() + b, static_cast<uint32_t>(len));
    if (len >= 3 && len - 2 < kMaxWord && pool[b] == '#' && pool[b + 1] == '#') note_length(1, pool.data() + b + 2, static_cast<uint32_t>(len - 2));
  }

  // direct tables for the keys of one and two bytes (the first entry with a key wins, as in the table)
  std::vector<int32_t> short_ids(kShortIds, kNone);
  auto note_short = [&](uint32_t kind, const uint8_t* key, uint32_t len, int32_t id) {
    if (len > 2) return;
    size_t const at = len == 2 ? kind * 65536u + (key[0] | (uint32_t{key[1]} << 8)) : 2 * 65536u + kind * 256u + key[0];
    if (short_ids[at] == kNone) short_ids[at] = id;
  };
  for (int32_t i = 0; i < V; ++i) {
    int64_t const b = off_at(i) - first, e = off_at(i + 1) - first;
    int64_t const len = e - b;
    if (len >= 1 && len <= 2) note_short(0, pool.data() + b, static_cast<uint32_t>(len), i);
    if (len >= 3 && len <= 4 && pool[b] == '#' && pool[b + 1] == '#') note_short(1, pool.data() + b + 2, static_cast<uint32_t>(len - 2), i);
  }

  auto* v = new nvtext_amd_wordpiece_vocabulary;
  v->entries = V;
  // wordpiece_tokenize.cu:199-209, 273-275
  int32_t unk = host_find(slots, mask, blocks, "[UNK]");
  if (unk < 0) unk = host_find(slots, mask, blocks, "[unk]");
  v->slot_bytes = capacity * sizeof(HostSlot);
  v->pool_bytes = blocks.size() + 16;
  if (hipMalloc(&v->d_slots, v->slot_bytes) != hipSuccess || hipMalloc(&v->d_pool, v->pool_bytes) != hipSuccess ||
      hipMalloc(&v->d_lens, lens.size() * sizeof(uint32_t)) != hipSuccess || hipMalloc(&v->d_short, short_ids.size() * sizeof(int32_t)) != hipSuccess) {
    nvtext_amd_wordpiece_vocabulary_destroy(v);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "vocabulary allocation failed");
  }
  hipError_t e1 = hipMemcpyAsync(v->d_slots, slots.data(), v->slot_bytes, hipMemcpyHostToDevice, stream);
  hipError_t e2 = blocks.empty() ? hipSuccess : hipMemcpyAsync(v->d_pool, blocks.data(), blocks.size(), hipMemcpyHostToDevice, stream);
  hipError_t e4 = hipMemcpyAsync(v->d_lens, lens.data(), lens.size() * sizeof(uint32_t), hipMemcpyHostToDevice, stream);
  hipError_t e5 = hipMemcpyAsync(v->d_short, short_ids.data(), short_ids.size() * sizeof(int32_t), hipMemcpyHostToDevice, stream);
  hipError_t e3 = hipStreamSynchronize(stream);  // host vectors die at return
  if (e1 != hipSuccess || e2 != hipSuccess || e3 != hipSuccess || e4 != hipSuccess || e5 != hipSuccess) {
    nvtext_amd_wordpiece_vocabulary_destroy(v);
    return fail(NVTEXT_AMD_DEVICE_ERROR, "vocabulary upload failed");
  }
  v->table.slots  = static_cast<const uint4*>(v->d_slots);
  v->table.pool   = static_cast<const uint8_t*>(v->d_pool);
  v->table.bucket_mask = mask;
  v->table.unk_id      = unk;
  v->table.max_len[0]  = max_len[0];
  v->table.max_len[1]  = max_len[1];
  v->table.lens        = static_cast<const uint32_t*>(v->d_lens);
  v->table.lens_mask   = static_cast<uint32_t>(lens_size - 1);
  v->table.short_ids   = static_cast<const int32_t*>(v->d_short);
  *out            = v;
  return NVTEXT_AMD_SUCCESS;
}

void nvtext_amd_wordpiece_vocabulary_destroy(nvtext_amd_wordpiece_vocabulary* v)
{
  if (!v) return;
  if (v->d_slots) (void)hipFree(v->d_slots);
  if (v->d_pool) (void)hipFree(v->d_pool);
  if (v->d_lens) (void)hipFree(v->d_lens);
  if (v->d_short) (void)hipFree(v->d_short);
  delete v;
}

int32_t nvtext_amd_wordpiece_vocabulary_unk_id(const nvtext_amd_wordpiece_vocabulary* v) { return v ? v->table.unk_id : -1; }

// may_cut_rows: very long rows may be cut into pieces that are tokenized as rows (false in the call that does the pieces)
static nvtext_amd_status tokenize_rows(const nvtext_amd_strings_column* input, const nvtext_amd_wordpiece_vocabulary* vocabulary,
                                       int32_t max_words_per_row, void* stream_, const nvtext_amd_allocator* mr_, nvtext_amd_list_column* out,
                                       bool may_cut_rows);

nvtext_amd_status nvtext_amd_wordpiece_tokenize(const nvtext_amd_strings_column* input, const nvtext_amd_wordpiece_vocabulary* vocabulary,
                                                int32_t max_words_per_row, void* stream_, const nvtext_amd_allocator* mr_,
                                                nvtext_amd_list_column* out)
{
  return tokenize_rows(input, vocabulary, max_words_per_row, stream_, mr_, out, true);
}

static nvtext_amd_status tokenize_rows(const nvtext_amd_strings_column* input, const nvtext_amd_wordpiece_vocabulary* vocabulary,
                                       int32_t max_words_per_row, void* stream_, const nvtext_amd_allocator* mr_, nvtext_amd_list_column* out,
                                       bool may_cut_rows)
{
  using namespace nvtext_amd;
  if (!input || !vocabulary || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nvtext_amd_list_column{};
  // cpp/src/text/wordpiece_tokenize.cu:845-846
  if (max_words_per_row < 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Invalid value for max_words_per_row argument");
  if (input->size < 0 || input->null_count < 0 || input->null_count > input->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "invalid column sizes");
  if (input->null_count > 0 && !input->null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Mr mr{mr_, stream};
  int32_t const rows = input->size;
  out->child_type    = NVTEXT_AMD_TYPE_INT32;

  if (rows == input->null_count) {  // wordpiece_tokenize.cu:849-853
    if (rows == 0) return NVTEXT_AMD_SUCCESS;  // canonical empty list column: no rows, no offsets
    // every row null: zero offsets, empty child, all-null mask (lists_column_factories.cu:80-93)
    out->size          = rows;
    out->null_count    = rows;
    out->offsets_size  = rows + 1;
    out->offsets_bytes = static_cast<size_t>(rows + 1) * sizeof(int32_t);
    out->offsets       = static_cast<int32_t*>(mr.allocate(out->offsets_bytes));
    out->null_mask_bytes = mask_alloc_bytes(rows);
    out->null_mask       = static_cast<uint32_t*>(mr.allocate(out->null_mask_bytes));
    if (!out->offsets || !out->null_mask) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "allocation failed");
    }
    launch_fill_u32(reinterpret_cast<uint32_t*>(out->offsets), 0u, rows + 1, stream);
    launch_fill_u32(out->null_mask, 0u, static_cast<int64_t>(out->null_mask_bytes / 4), stream);
    NVTEXT_HIP_TRY(hipGetLastError());
    return NVTEXT_AMD_SUCCESS;
  }

  out->size          = rows;
  out->null_count    = input->null_count;
  out->offsets_size  = rows + 1;
  out->offsets_bytes = static_cast<size_t>(rows + 1) * sizeof(int32_t);
  out->offsets       = static_cast<int32_t*>(mr.allocate(out->offsets_bytes));
  if (!out->offsets) return fail(NVTEXT_AMD_ALLOC_FAILED, "offsets allocation failed");
  if (input->null_mask) {
    out->null_mask_bytes = mask_alloc_bytes(rows);
    out->null_mask       = static_cast<uint32_t*>(mr.allocate(out->null_mask_bytes));
    if (!out->null_mask) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "mask allocation failed");
    }
    launch_copy_bitmask(out->null_mask, input->null_mask, input->offset, rows, stream);
  }

  ColView const v = make_view(*input);
  // Without a word limit very long rows are cut into pieces (see long_rows_kernel): are there any?  The answer
  // comes back with the two offsets read below.
  bool const look_for_long_rows = may_cut_rows && max_words_per_row == 0;
  size_t const cut_bytes[3]     = {look_for_long_rows ? static_cast<size_t>(rows) * sizeof(uint32_t) : 0,
                                   look_for_long_rows ? (static_cast<size_t>(rows) + 1) * sizeof(uint32_t) : 0, look_for_long_rows ? 256u : 0u};
  TempParts<3> const cut_temps(mr, cut_bytes);
  uint32_t* const pieces      = cut_temps.part<uint32_t>(0);
  uint32_t* const first_piece = cut_temps.part<uint32_t>(1);
  uint32_t* const any_long    = cut_temps.part<uint32_t>(2);
  uint32_t has_long           = 0;
  if (look_for_long_rows) {
    if (!cut_temps.ok()) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    }
    launch_fill_u32(any_long, 0u, 1, stream);
    hipLaunchKernelGGL(long_rows_kernel, dim3(static_cast<unsigned>((rows + 255) / 256)), dim3(256), 0, stream, v, pieces, any_long);
  }
  // first and last offset of the view (the reference reads the same two scalars,
  // cpp/src/strings/utilities.cu:180-190); they size the token arena
  size_t const ow = input->offsets_is_int64 ? 8 : 4;
  int64_t first_offset = 0, last_offset = 0;
  {
    unsigned char buf[16] = {0};
    const uint8_t* d_off  = static_cast<const uint8_t*>(input->offsets) + static_cast<size_t>(input->offset) * ow;
    hipError_t e          = hipMemcpyAsync(buf, d_off, ow, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipMemcpyAsync(buf + 8, d_off + static_cast<size_t>(rows) * ow, ow, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess && look_for_long_rows) e = hipMemcpyAsync(&has_long, any_long, sizeof(uint32_t), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
    }
    if (ow == 8) {
      std::memcpy(&first_offset, buf, 8);
      std::memcpy(&last_offset, buf + 8, 8);
    } else {
      int32_t a32, b32;
      std::memcpy(&a32, buf, 4);
      std::memcpy(&b32, buf + 8, 4);
      first_offset = a32;
      last_offset  = b32;
    }
  }
  if (last_offset < first_offset) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_INVALID_ARGUMENT, "offsets are not monotone");
  }
  if (has_long != 0) {
    // the pieces as a strings column of their own over the same chars (int64 offsets, no mask: validity is not
    // consulted without a word limit), tokenized by this same function; then the rows' offsets from their first pieces
    auto give_up = [&](nvtext_amd_status st, const char* what) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(st, what);
    };
    Temp scan_tmp(mr, scan_temp_bytes(rows));
    if (!scan_tmp.ok()) return give_up(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    device_exclusive_scan(PiecesOf{pieces}, static_cast<int64_t>(rows), first_piece, scan_tmp.as<uint64_t>(), stream);
    uint64_t n_pieces = 0;
    hipError_t e      = hipMemcpyAsync(&n_pieces, scan_tmp.as<uint64_t>() + scan_tiles(rows), sizeof(uint64_t), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
    if (n_pieces > static_cast<uint64_t>(std::numeric_limits<int32_t>::max()) - 1) return give_up(NVTEXT_AMD_LOGIC_ERROR, "words exceed internal limit");
    Temp piece_offset(mr, (static_cast<size_t>(n_pieces) + 1) * sizeof(int64_t));
    if (!piece_offset.ok()) return give_up(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    hipLaunchKernelGGL(piece_offsets_kernel, dim3(static_cast<unsigned>((n_pieces + 1 + 255) / 256)), dim3(256), 0, stream, v, first_piece,
                       static_cast<int64_t>(n_pieces), piece_offset.as<int64_t>());
    nvtext_amd_strings_column cut{};
    cut.chars            = input->chars;
    cut.offsets          = piece_offset.ptr;
    cut.offsets_is_int64 = 1;
    cut.size             = static_cast<int32_t>(n_pieces);
    nvtext_amd_list_column of_pieces{};
    nvtext_amd_status const st = tokenize_rows(&cut, vocabulary, 0, stream_, mr_, &of_pieces, false);
    if (st != NVTEXT_AMD_SUCCESS) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return st;
    }
    hipLaunchKernelGGL(row_offsets_of_pieces_kernel, dim3(static_cast<unsigned>((rows + 1 + 255) / 256)), dim3(256), 0, stream, of_pieces.offsets,
                       first_piece, static_cast<int64_t>(rows), out->offsets);
    out->child       = of_pieces.child;  // the tokens are the pieces' tokens, in the same order
    out->child_size  = of_pieces.child_size;
    out->child_bytes = of_pieces.child_bytes;
    of_pieces.child  = nullptr;
    of_pieces.child_bytes = 0;
    nvtext_amd_list_column_free(&of_pieces, stream_, mr_);
    NVTEXT_HIP_TRY(hipGetLastError());
    return NVTEXT_AMD_SUCCESS;
  }
  // word arena: one slot per possible word; row r gets floor(bytes/2) + 1 slots
  size_t const arena_slots = static_cast<size_t>((last_offset - first_offset) >> 1) + static_cast<size_t>(rows) + 1;
  // queue of words whose whole-word probe missed.  Sized for a generous share of the input; if a run
  // overflows it the exact size is known afterwards and the passes are repeated once.
  int device = 0, cus = 256;
  (void)hipGetDevice(&device);
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
  // persistent kernels: as many workgroups as can be resident at once
  auto resident = [&](const void* kernel, int threads) -> int64_t {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess || per_cu < 1) per_cu = 4;
    return static_cast<int64_t>(per_cu) * cus;
  };
  unsigned const row_blocks = static_cast<unsigned>(std::min<int64_t>((static_cast<int64_t>(rows) + kTokWaves * kGroups - 1) / (kTokWaves * kGroups),
                                                                      resident(reinterpret_cast<const void*>(wordpiece_probe_kernel), kTokThreads)));
  // Each wavefront reserves queue entries a range at a time (one atomic per range), at most `queue_block` of them:
  // it starts with short ranges and doubles them while they fill within a few steps, because atomics on one
  // address are slow (about 150 M/s) and the unused tail of each wavefront's last range, half a range on
  // average, is time lost in the pass that reads the queue.
  uint64_t const waves = static_cast<uint64_t>(row_blocks) * kTokWaves;
  uint32_t queue_block = 64;
  while (queue_block < 1024 && static_cast<uint64_t>(queue_block) * waves * 64 < static_cast<uint64_t>(last_offset - first_offset)) queue_block <<= 1;
  uint64_t queue_capacity = static_cast<uint64_t>((last_offset - first_offset) >> 4) + waves * queue_block + 4096;
  size_t const temp_bytes[5] = {arena_slots * sizeof(uint32_t), static_cast<size_t>(rows) * sizeof(int32_t),
                                static_cast<size_t>(rows) * sizeof(int32_t), scan_temp_bytes(rows), 256};
  TempParts<5> const temps(mr, temp_bytes);
  uint32_t* const arena    = temps.part<uint32_t>(0);
  int32_t* const nwords    = temps.part<int32_t>(1);
  int32_t* const counts    = temps.part<int32_t>(2);
  uint64_t* const scan_tmp = temps.part<uint64_t>(3);
  uint32_t* const qsize    = temps.part<uint32_t>(4);
  if (!temps.ok()) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
  }
  uint64_t total = 0;
  for (int attempt = 0;; ++attempt) {
    if (queue_capacity > 0x7FFFFFFEull) queue_capacity = 0x7FFFFFFEull;
    uint32_t const qcap = static_cast<uint32_t>(queue_capacity);
    // (third part: queue indices of the words of more than 16 bytes, then one count per wavefront of the out-of-vocabulary pass)
    int64_t const oov_blocks    = resident(reinterpret_cast<const void*>(wordpiece_oov_kernel), kOovThreads);
    size_t const queue_bytes[3] = {static_cast<size_t>(qcap) * sizeof(OovEntry), static_cast<size_t>(qcap) * sizeof(OovResult),
                                   (static_cast<size_t>(qcap) + static_cast<size_t>(oov_blocks) * (kOovThreads / kWave)) * sizeof(uint32_t)};
    TempParts<3> const queue_temps(mr, queue_bytes);
    OovEntry* const queue    = queue_temps.part<OovEntry>(0);
    OovResult* const results = queue_temps.part<OovResult>(1);
    uint32_t* const longer   = queue_temps.part<uint32_t>(2);
    if (!queue_temps.ok()) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    }
    launch_fill_u32(qsize, 0u, 2, stream);  // queue size; words the emit pass hands on
    {
      ProfileScope ps("wordpiece_probe_kernel", stream);
      hipLaunchKernelGGL(wordpiece_probe_kernel, dim3(row_blocks), dim3(kTokThreads), 0, stream, v, vocabulary->table, max_words_per_row,
                         first_offset, last_offset, arena, nwords, counts, queue, qcap,
                         queue_block, qsize);
    }
    {
      ProfileScope ps("wordpiece_oov_kernel", stream);
      hipLaunchKernelGGL(wordpiece_oov_kernel, dim3(static_cast<unsigned>(oov_blocks)), dim3(kOovThreads), 0, stream, v, vocabulary->table,
                         queue, qsize, qcap, results, counts, longer);
    }
    {
      ProfileScope ps("wordpiece_oov_long_kernel", stream);
      hipLaunchKernelGGL(wordpiece_oov_long_kernel, dim3(static_cast<unsigned>(oov_blocks)), dim3(kOovThreads), 0, stream, v, vocabulary->table,
                         queue, qsize, qcap, results, counts, longer);
    }
    // int32 list offsets; the total decides the child size (cpp/include/cudf/detail/sizes_to_offsets_iterator.cuh:302-339)
    device_exclusive_scan(CountOf{counts}, static_cast<int64_t>(rows), out->offsets, scan_tmp, stream);
    uint32_t queued = 0;
    hipError_t e    = hipMemcpyAsync(&total, scan_tmp + scan_tiles(rows), sizeof(uint64_t), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipMemcpyAsync(&queued, qsize, sizeof(uint32_t), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
    }
    if (queued > qcap) {  // the queue was too small: repeat once with the exact size
      if (attempt > 0 || queued > 0x7FFFFFFEu) {
        nvtext_amd_list_column_free(out, stream_, mr_);
        return fail(NVTEXT_AMD_LOGIC_ERROR, "words exceed internal limit");
      }
      queue_capacity = queued;
      continue;
    }
    if (total > static_cast<uint64_t>(std::numeric_limits<int32_t>::max())) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_OVERFLOW, "Size of output exceeds the column size limit");
    }
    out->child_size  = static_cast<int64_t>(total);
    out->child_bytes = static_cast<size_t>(total) * sizeof(int32_t);
    if (total) {
      out->child = mr.allocate(out->child_bytes);
      if (!out->child) {
        nvtext_amd_list_column_free(out, stream_, mr_);
        return fail(NVTEXT_AMD_ALLOC_FAILED, "child allocation failed");
      }
      ProfileScope ps("wordpiece_emit_kernel", stream);
      // the blocks of rows that a wavefront walks at a time: evened out by tokens (see emit_blocks_kernel)
      int64_t const emit_work   = static_cast<int64_t>(total) + kEmitRowWeight * rows;
      int64_t const nblocks     = (emit_work + kEmitBlockWork - 1) / kEmitBlockWork;
      Temp block_first(mr, static_cast<size_t>(nblocks + 1) * sizeof(int32_t));
      if (!block_first.ok()) {
        nvtext_amd_list_column_free(out, stream_, mr_);
        return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
      }
      hipLaunchKernelGGL(emit_blocks_kernel, dim3(static_cast<unsigned>((nblocks + 1 + 255) / 256)), dim3(256), 0, stream, out->offsets,
                         static_cast<int64_t>(rows), nblocks, block_first.as<int32_t>());
      int64_t const emit_blocks = (nblocks + kTokWaves - 1) / kTokWaves;
      unsigned const emit_grid  = static_cast<unsigned>(std::min<int64_t>(emit_blocks, resident(reinterpret_cast<const void*>(wordpiece_emit_kernel), kTokThreads)));
      hipLaunchKernelGGL(wordpiece_emit_kernel, dim3(emit_grid), dim3(kTokThreads), 0, stream, v, vocabulary->table, first_offset,
                         arena, nwords, results, out->offsets,
                         static_cast<int32_t*>(out->child), block_first.as<int32_t>(), nblocks, longer, qsize + 1);
      // (the list of longer words has served its purpose by now: its memory takes the list of words to do again,
      // at most one entry per queued word)
      hipLaunchKernelGGL(wordpiece_retokenize_kernel, dim3(static_cast<unsigned>(cus)), dim3(kOovThreads), 0, stream, v, vocabulary->table,
                         queue, results, longer, qsize + 1,
                         static_cast<int32_t*>(out->child));
    }
    break;
  }
  NVTEXT_HIP_TRY(hipGetLastError());
  return NVTEXT_AMD_SUCCESS;
}

}  // extern "C"

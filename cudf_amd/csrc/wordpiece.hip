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
//     are also what gets hashed; the table for a 30k-entry vocabulary is 1 MiB and stays in L2.
//     A hashed length filter (which key lengths exist for a given first three bytes) lets the
//     longest-match search skip the lengths that cannot match.  The tables are built by kernels: every key bids
//     for its home bucket with its number in the vocabulary, so the keys that come first get the home slots.
//   * a sample of the column (512 windows, each word looked up as the word pass will) sizes the word slots and the
//     queue of the first attempt; what still overflows repeats the passes once with sizes that cannot fail.
//   * the column's bytes are cut into tiles of 2048 bytes from the 16-byte aligned address below its first byte,
//     without regard to rows; up to 8 tiles form a range, and every pass hands out ranges to wavefronts.
//   * word pass: a wavefront takes a range and walks its tiles: bytes staged in LDS (the next tile's loads in
//     flight), row starts marked as extra separators, spaces found with four SWAR operations per dword (16 bytes per
//     lane), word starts and ends paired through scans, the words past a row's limit dropped; then lanes <->
//     words: ONE lookup per word in straight-line code.  Every word gets one 4-byte slot, densely per range: its
//     token, or the index of its 32-byte record (first 16 bytes, length, place) in the queue of words that are
//     not in the vocabulary as they stand.  Rows get the number of words of their range before them.
//   * out-of-vocabulary pass: one lane per queued word, lanes refilled from LDS as words finish.  Words of up to
//     16 bytes are tokenized in registers, the greedy longest-match rule reduced to bit operations on a mask of
//     candidate lengths, one table lookup per trip; the result (up to seven tokens and their number) takes the
//     place of the queue record.  Longer words go through a general state machine in a second kernel.
//   * a device-wide scan of the ranges' token counts gives every range its place in the result; the emit pass
//     (a wavefront per range) expands the word slots into the tokens and turns the rows' word counts into list
//     offsets.  The few words with more pieces than a record keeps are tokenized again, into place, by a kernel
//     of their own.  No chars-sized temporary is written: 2.4 bytes of temporaries per input byte.
#include "common.cuh"

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

namespace nvtext_amd {
namespace {

constexpr uint32_t kMaxWord = 200;  // wordpiece_tokenize.cu:300: words this long become one [UNK]

// Key hash, 64 bits: the key is consumed in 8-byte blocks (two little-endian dwords, zero padded), every dword times an
// odd constant of its own, summed: for a key of up to 16 bytes four multiply-adds of 32 x 32 + 64 bits, the unit the
// vector ALUs have, and nothing that waits for the step before it beyond the running sum.  (A bucket needs the key's
// home and fifteen bits to tell keys apart, not an avalanche: the home comes from the low bits of the sum's upper half,
// which every bit of the key reaches, the tag from the top of its lower half.)  The two key spaces multiply the first
// dword by different constants; the length is not hashed (the slot holds it).  Blocks from the third on (keys of more
// than 16 bytes) rotate the sum first, so that the constants can be used again.
constexpr uint32_t kMulFirst[2] = {0x9E3779B1u, 0xD2B74407u};
constexpr uint32_t kMulSecond = 0x85EBCA77u, kMulThird = 0xC2B2AE3Du, kMulFourth = 0x27D4EB2Fu;
__host__ __device__ __forceinline__ uint64_t key_hash_first(uint32_t kind, uint32_t lo, uint32_t hi)
{
  return static_cast<uint64_t>(lo) * (kind ? kMulFirst[1] : kMulFirst[0]) + static_cast<uint64_t>(hi) * kMulSecond;
}
// block: 1 for key bytes [8, 16), 2 for [16, 24), ..
__host__ __device__ __forceinline__ uint64_t key_hash_next(uint64_t h, uint32_t lo, uint32_t hi, uint32_t block)
{
  if (block > 1) h = (h << 25) | (h >> 39);
  return h + static_cast<uint64_t>(lo) * kMulThird + static_cast<uint64_t>(hi) * kMulFourth;
}

// slot.x = (tag15 << 17) | (carried8 << 9) | (kind << 8) | len   (0 = empty; len in 1..199).  carried8, in slot 0 of a bucket only:
//          one of eight bits per key that has been carried past this bucket (which bit: HashParts::fp of the key)
// slot.y = token id; in slot 0 of a bucket, bit 31 says that some key has been carried past this bucket
//          (kSearchOn: a key that is not in a bucket without the bit is not in the table)
// slot.z, slot.w = the key itself when len <= 8 (zero padded), else (byte offset of the key in the pool, 0);
// the pool holds the keys of more than 8 bytes, each zero padded to a multiple of 8 at an 8-byte aligned offset
// Bucket b = slots[2b], slots[2b+1]; a bucket fills slot 0 first, overflow goes to the next bucket.
constexpr uint32_t kSearchOn = 0x80000000u;
constexpr uint32_t kCarried  = 0x0001FE00u;
struct VocabTable {
  const uint4* slots;
  const uint8_t* pool;
  uint32_t bucket_mask;  // buckets - 1
  uint32_t bucket_bits;  // log2(buckets)
  int32_t unk_id;
  uint32_t max_len[2];   // longest key of each key space (longer candidates cannot match)
  // Length filter: lens[length_filter_index(kind, first three key bytes) & lens_mask] has bit i (i < 31) set
  // when some key of that key space with those first bytes is i + 3 bytes long, bit 31 for 34 bytes and more.
  // Entries are shared by hashing, so a set bit promises nothing, a clear bit rules the length out.
  // (stored in the low half of a 32-bit word: bits 0..14 for 3..17 bytes, bit 15 for 18 bytes and more; filter_word()
  // spreads it out.)  The high half says which fourth bytes the keys of four bytes and more of the entry have, bit
  // 16 + (byte & 15): a piece whose fourth byte finds no bit has no candidate of more than three bytes
  // (piece_filter_word()).
  const uint32_t* lens;
  uint32_t lens_mask;
  // Direct tables for keys of one and two bytes: short_ids[kind * 65536 + (byte0 | byte1 << 8)] for two bytes,
  // short_ids[131072 + kind * 256 + byte0] for one; the token id, or INT32_MIN when there is no such key.
  const int32_t* short_ids;
  // The length filter once more, exact, for the keys of the second key space (the "##" entries) that begin with three
  // lower-case ASCII letters c0 c1 c2: letters3[((c0 - 'a') * 26 + (c1 - 'a')) * 26 + (c2 - 'a')] has bit i (i < 7) set
  // when some such key is i + 3 bytes long (3..9), bit 7 when one is longer; and bit 8 + (c3 & 7) when some such key of
  // four bytes and more has c3 as its fourth byte: a piece whose fourth byte finds no bit has no candidate of more
  // than three bytes, whatever the lengths say (text that the vocabulary does not know is mostly turned away here,
  // before a lookup is spent on it).  Small enough for LDS.
  const uint16_t* letters3;
};
constexpr uint32_t kShortIds = 2 * 65536 + 2 * 256;
constexpr uint32_t kLetters3 = 26 * 26 * 26;
constexpr uint32_t kLetters2 = 26 * 26;

__host__ __device__ __forceinline__ uint32_t length_filter_index(uint32_t kind, uint32_t first3)
{
  uint32_t x = (first3 | (kind << 24)) * 0x9E3779B1u;
  x ^= x >> 15;
  x *= 0x85EBCA77u;
  return x ^ (x >> 13);
}
__host__ __device__ __forceinline__ uint32_t length_filter_bit(uint32_t len) { return len >= 34 ? 31u : len - 3u; }
// The stored form of a filter word and back: the lengths of 18 bytes and more share one bit.
__host__ __device__ __forceinline__ uint16_t packed_filter_word(uint32_t w) { return static_cast<uint16_t>((w & 0x7FFFu) | ((w >> 15) ? 0x8000u : 0u)); }
__host__ __device__ __forceinline__ uint32_t filter_word(uint32_t stored) { return (stored & 0x7FFFu) | ((stored & 0x8000u) ? 0xFFFF8000u : 0u); }
// The candidate lengths (bit i: i + 3 bytes) that a filter entry leaves a piece whose first four bytes are first4
// (bytes past the piece may hold anything: candidates that long do not exist).
__host__ __device__ __forceinline__ uint32_t piece_filter_word(uint32_t stored, uint32_t first4)
{
  uint32_t const w = filter_word(stored & 0xFFFFu);
  return ((stored >> (16u + ((first4 >> 24) & 15u))) & 1u) ? w : (w & 1u);
}

// What a lookup takes from a key's hash: the two halves folded and multiplied once more (the top bits of such a product
// depend on every bit of both halves), the key's home bucket from the top `bucket_bits` bits, the tag and the carried
// bit (see above) from the bits below them.
struct HashParts {
  uint32_t bucket;  // home bucket
  uint32_t tag;     // slot.x of a matching slot without kind and length: bits 17..31
  uint32_t fp;      // the bit that the key sets in the carried8 field of the buckets it is carried past
};
__host__ __device__ __forceinline__ HashParts hash_parts(uint64_t h, uint32_t bucket_bits)
{
  uint32_t const x    = (static_cast<uint32_t>(h) ^ static_cast<uint32_t>(h >> 32)) * 0x9E3779B1u;
  uint32_t const rest = x << bucket_bits;  // (bucket_bits: 5 .. 30)
  HashParts p;
  p.bucket = x >> (32u - bucket_bits);
  p.tag    = rest & 0xFFFE0000u;
  p.fp     = 0x200u << (rest >> 29);
  return p;
}
__host__ __device__ __forceinline__ uint32_t slot_word0(uint32_t tag, uint32_t kind, uint32_t len) { return tag | (kind << 8) | len; }

}  // namespace
}  // namespace nvtext_amd

struct nvtext_amd_wordpiece_vocabulary {
  nvtext_amd::VocabTable table{};
  nvtext_amd::DeviceStore store;  // the tables, from the allocator given at creation
  void* d_slots     = nullptr;
  void* d_pool      = nullptr;
  void* d_lens      = nullptr;
  void* d_short     = nullptr;
  void* d_letters   = nullptr;
  size_t slot_bytes = 0;
  size_t pool_bytes = 0;
  int32_t entries   = 0;
};

namespace nvtext_amd {
namespace {

constexpr int kTokWaves     = 4;
constexpr int kTokThreads   = kTokWaves * kWave;
constexpr int32_t kNone     = std::numeric_limits<int32_t>::min();
constexpr int kOovKeep      = 7;     // tokens of an out-of-vocabulary word that are kept while it is tokenized
// ------------------------------------------------------------------ where candidate keys live
// Each source offers byte(k) and key8(p, len, &k0, &k1): bytes [p, p+8) as two dwords, zero padded past len.
__device__ __forceinline__ void trim_key8(uint32_t len, uint32_t& lo, uint32_t& hi)
{
  // keep bytes [0, len) of the eight (selects, no branches)
  uint32_t const nlo = min(len, 4u), nhi = max(min(len, 8u), 4u) - 4u;
  lo &= nlo >= 4 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << (8 * nlo));
  hi &= nhi >= 4 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << (8 * nhi));
}

// trim[len] (len 0..16): the masks that keep bytes [0, len) of sixteen, as four dwords; what trim_key8 computes, read
// from LDS where a kernel trims a key for every word.
__device__ __forceinline__ void fill_trim_table(uint4* trim)
{
  if (threadIdx.x <= 16) {
    uint32_t m[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      int const n = min(max(static_cast<int>(threadIdx.x) - 4 * d, 0), 4);
      m[d]        = n >= 4 ? 0xFFFFFFFFu : ~(0xFFFFFFFFu << (8 * n));
    }
    trim[threadIdx.x] = make_uint4(m[0], m[1], m[2], m[3]);
  }
}

// A word inside the bytes a wavefront has staged in LDS: `bytes` points at the staged dwords, `start` is the
// byte index of the word's first byte in them.  Everything a word of fewer than kMaxWord bytes can touch is staged.
struct TileWord {
  const uint32_t* bytes;
  uint32_t start;
  __device__ __forceinline__ uint32_t byte(uint32_t k) const { return reinterpret_cast<const uint8_t*>(bytes)[start + k]; }
  __device__ __forceinline__ void key8(uint32_t p, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    uint32_t const o  = start + p;
    uint32_t const i  = o >> 2;
    uint32_t const sh = (o & 3u) * 8u;
    uint32_t const d0 = bytes[i], d1 = bytes[i + 1], d2 = bytes[i + 2];
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
    for (uint32_t j = 0; j < 5; ++j) d[j] = bytes[i + j];
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

// A candidate key, ready to be probed: its first block (trimmed), tag word and home bucket.
struct Probe {
  uint32_t k0, k1;  // key bytes [0, 8), zero padded
  uint32_t want;    // slot.x of a matching slot (without the carried8 field)
  uint32_t fp;      // HashParts::fp of the key
  uint32_t bucket;  // home bucket (already masked)
};

// Hash contribution of key bytes [8, len) (keys that do not fit the slot; kept out of line).
template <typename W>
__device__ __forceinline__ uint64_t hash_long_key(W const& w, uint32_t p, uint32_t len, uint64_t h)
{
  for (uint32_t done = 8; done < len; done += 8) {
    uint32_t b0, b1;
    w.key8(p + done, len - done, &b0, &b1);
    h = key_hash_next(h, b0, b1, done >> 3);
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
  uint64_t h = key_hash_first(kind, pr.k0, pr.k1);
  if (len > 8) h = hash_long_key(w, p, len, h);
  HashParts const hp = hash_parts(h, t.bucket_bits);
  pr.want            = slot_word0(hp.tag, kind, len);
  pr.fp              = hp.fp;
  pr.bucket          = hp.bucket;
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
  if ((s.x & ~kCarried) == pr.want) {
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

// The general lookup, kept out of line: the callers have straight-line code for the common outcomes and come here
// for the rest (keys in the pool, buckets that keys have been carried past).
template <typename W>
__device__ __forceinline__ int32_t lookup_slow(VocabTable const& t, uint32_t kind, W w, uint32_t p, uint32_t len)
{
  uint32_t r0, r1;
  w.key8(p, min(len, 8u), &r0, &r1);
  return lookup(t, kind, w, p, len, r0, r1);
}

// Sixteen bytes held in registers as a key source.
struct RegWord {
  uint32_t r[4];
  __device__ __forceinline__ uint32_t byte(uint32_t k) const
  {
    uint32_t const d = k >> 2;
    uint32_t const v = d == 0 ? r[0] : d == 1 ? r[1] : d == 2 ? r[2] : r[3];
    return (v >> (8 * (k & 3u))) & 0xffu;
  }
  __device__ __forceinline__ void key8(uint32_t p, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    uint32_t lo = p == 0 ? r[0] : r[2], hi = p == 0 ? r[1] : r[3];  // p is 0 or 8
    trim_key8(len, lo, hi);
    *k0 = lo;
    *k1 = hi;
  }
};

// What the two home slots say about a key of l bytes without any further memory access:
// 1 = found (*id set), 0 = absent, 2 = undecided (a key of more than 8 bytes has the right tag, or keys have been
// carried past this bucket and the search goes on in the next one).  Straight-line code.
__device__ __forceinline__ uint32_t verdict(Probe const& pr, uint4 const& s0, uint4 const& s1, uint32_t l, int32_t* id)
{
  bool const tag0  = (s0.x & ~kCarried) == pr.want, tag1 = s1.x == pr.want;
  bool const is0   = tag0 & (s0.z == pr.k0) & (s0.w == pr.k1);  // (no short cuts: the slots are read whole, at once)
  bool const is1   = tag1 & (s1.z == pr.k0) & (s1.w == pr.k1);
  bool const small = l <= 8;
  bool const found = small && (is0 || is1);
  bool const more  = (!small && (tag0 || tag1)) || (!found && (s0.x & pr.fp) != 0);
  *id              = static_cast<int32_t>((is0 ? s0.y : s1.y) & ~kSearchOn);
  return found ? 1u : more ? 2u : 0u;
}

// The same for a key of 9 to 16 bytes whose bytes are k[0..3] (zero padded): a home slot with the right tag
// names the key's place in the pool, and one 16-byte read there decides.  Still undecided (2) only when both home
// slots carry the tag or the search goes on in the next bucket.
__device__ __forceinline__ uint32_t verdict_16(VocabTable const& t, Probe const& pr, uint4 const& s0, uint4 const& s1, const uint32_t (&k)[4],
                                               int32_t* id)
{
  bool const tag0 = (s0.x & ~kCarried) == pr.want, tag1 = s1.x == pr.want;
  bool const on   = (s0.x & pr.fp) != 0;
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


// Bit 7 of every byte of x that equals ' ' (exact: no carries cross bytes).
__device__ __forceinline__ uint32_t space_bytes(uint32_t x)
{
  uint32_t const t = x ^ 0x20202020u;
  return ~(((t & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | t) & 0x80808080u;
}
// Gathers bits 7, 15, 23, 31 into bits 0..3.
__device__ __forceinline__ uint32_t gather_byte_flags(uint32_t z) { return (((z >> 7) * 0x00204081u) >> 21) & 0xFu; }

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
    lens = len - start >= 3 ? piece_filter_word(t.lens[length_filter_index(kind, raw0 & 0x00FFFFFFu) & t.lens_mask], raw0) : 0xFFFFFFFFu;
  }

  // probed: the whole word has been looked up and is known to be absent
  __device__ __forceinline__ void begin(VocabTable const& t, W const& w, uint32_t len_, bool ascii_, bool probed)
  {
    len = len_; start = 0; e = len_; count = 0;
    ascii = ascii_;
    fresh = !probed;  // a word known to be absent begins by being shortened
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

// Runs one word, which has not been looked up whole, to completion (used where such words are rare).  Returns the
// token count.
template <typename W, typename Emit>
__device__ __forceinline__ uint32_t tokenize_oov_word(VocabTable const& t, W const& w, uint32_t len, Emit emit)
{
  OovStepper<W> st;
  st.begin(t, w, len, false, false);
  while (!st.done) st.step(t, w, emit);
  return st.count;
}

// The same, out of line, for the callers' rare cases: the number of tokens of a word staged in LDS, and the tokens
// of a word in memory written to dst[0 .. cnt) (cnt = the number counted before).
__device__ __forceinline__ uint32_t count_oov_tokens(VocabTable const& t, const uint32_t* bytes, uint32_t start, uint32_t len)
{
  return tokenize_oov_word(t, TileWord{bytes, start}, len, [](uint32_t, int32_t) {});
}
__device__ __forceinline__ void write_oov_tokens(VocabTable const& t, const uint8_t* p, uint32_t len, uint32_t* dst, uint32_t cnt)
{
  tokenize_oov_word(t, GlobalWord{p}, len, [&](uint32_t j, int32_t id) {
    if (j < cnt) dst[j] = static_cast<uint32_t>(id);
  });
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
  uint32_t cand;   // lengths still to try for the piece at start (bit l - 1), longest first, once the length filter has been applied
  uint32_t lens;   // the length filter word of the piece's opening (all ones once applied)
  uint32_t count;  // tokens so far
  int32_t id1, id2;  // ids of the piece's first byte and first two bytes as keys (kNone: no such key)
  bool done;

  // What a piece needs to know before any of its candidates is looked up: which lengths of three bytes and more
  // can exist for its first three bytes, and the ids of its first byte and first two bytes as keys.
  struct Opening {
    uint32_t lens;
    int32_t id1, id2;
  };

  __device__ __forceinline__ uint32_t byte(uint32_t k) const
  {
    uint32_t const d = k >> 2;
    uint32_t const v = d == 0 ? r[0] : d == 1 ? r[1] : d == 2 ? r[2] : r[3];
    return (v >> (8 * (k & 3u))) & 0xffu;
  }
  // bytes [p, p + 4) of the rest of the word (p < 16)
  __device__ __forceinline__ uint32_t dword_at(uint32_t p) const
  {
    uint32_t const d  = p >> 2;
    uint32_t const lo = d == 0 ? r[0] : d == 1 ? r[1] : d == 2 ? r[2] : r[3];
    uint32_t const hi = d == 0 ? r[1] : d == 1 ? r[2] : d == 2 ? r[3] : 0u;
    return __builtin_amdgcn_alignbit(hi, lo, (p & 3u) * 8u);
  }

  // Requests the opening of the piece that would start p bytes on (key space `kind`).  The reads are made whatever p
  // is (bytes past the word are zeros, every index is inside its table); what they give only counts for the p
  // that the word goes on from.  first_ids: the ids of the one-byte keys, [kind * 256 + byte], in LDS.
  __device__ __forceinline__ Opening request(VocabTable const& t, const int32_t* first_ids, uint32_t kind, uint32_t p) const
  {
    uint32_t const b    = dword_at(p);
    uint32_t const left = rem - min(p, rem);
    Opening o;
    uint32_t const lens = piece_filter_word(t.lens[length_filter_index(kind, b & 0x00FFFFFFu) & t.lens_mask], b);
    int32_t const two   = t.short_ids[kind * 65536 + (b & 0xFFFFu)];
    o.id1               = first_ids[kind * 256 + (b & 0xFFu)];
    o.lens              = left >= 3 ? lens : 0xFFFFFFFFu;
    o.id2               = left >= 2 ? two : kNone;
    return o;
  }

  // The opening of the next piece of the word (second key space), when the piece before it has been dropped.  Pieces
  // that begin with lower-case ASCII letters, as nearly all do in text of that alphabet, get it from tables in LDS
  // (l3: the exact length filter by three letters; pair: the ids of the two-letter keys; both of the second key
  // space); the others from the tables in memory, as request() does.
  __device__ __forceinline__ Opening request_next(VocabTable const& t, const int32_t* first_ids, const uint16_t* l3, const int32_t* pair) const
  {
    uint32_t const b   = r[0];
    uint32_t const x   = b & 0x00FFFFFFu;
    uint32_t const low = x & 0x007F7F7Fu;
    // bit 7 of each of the three bytes that is no lower-case letter (bytes past the word are zeros: none of them is)
    uint32_t const bad = (~(low + 0x001F1F1Fu) | (low + 0x00050505u) | x) & 0x00808080u;
    bool const ok3     = bad == 0u;
    bool const ok2     = (bad & 0x00008080u) == 0u;
    uint32_t const c0 = x & 0xFFu, c1 = (x >> 8) & 0xFFu, c2 = x >> 16;
    uint32_t const i2 = c0 * 26u + c1 - 97u * 27u;
    uint32_t const i3 = i2 * 26u + c2 - 97u;
    Opening o;
    o.id1               = first_ids[256 + c0];
    uint32_t const e3   = l3[ok3 ? i3 : 0u];
    int32_t const two   = pair[ok2 ? i2 : 0u];
    uint32_t len3       = (e3 & 0x7Fu) | ((e3 & 0x80u) ? 0xFFFFFF80u : 0u);
    if (((e3 >> (8u + ((b >> 24) & 7u))) & 1u) == 0u) len3 &= 1u;  // no key with this fourth byte: three bytes at most
    o.lens              = ok3 ? len3 : 0xFFFFFFFFu;
    o.id2               = ok2 ? two : kNone;
    if (!ok3 && rem >= 3) o.lens = piece_filter_word(t.lens[length_filter_index(1u, x) & t.lens_mask], b);
    if (!ok2 && rem >= 2) o.id2 = t.short_ids[65536 + (b & 0xFFFFu)];
    return o;
  }

  // The piece at start begins: its candidate lengths are those on a character boundary, no longer than the rest of
  // the word or the longest key, and not ruled out by the length filter of its first three bytes.
  // (What the opening holds is not looked at here but when the next trip begins: by then its reads have arrived.)
  __device__ __forceinline__ void open_piece(VocabTable const& t, uint32_t kind, Opening const& o)
  {
    uint32_t const lim = min(min(rem, t.max_len[kind]), 16u);
    cand               = (bnd >> 1) & ((1u << lim) - 1u);
    lens               = o.lens;
    id1                = o.id1;
    id2                = o.id2;
  }

  // probed: the whole word has been looked up and is known to be absent
  // ascii (the same in every lane): no byte of any of the lanes' words has bit 7 set
  __device__ __forceinline__ void begin(VocabTable const& t, const int32_t* first_ids, const uint32_t (&head)[4], uint32_t len, bool probed, bool ascii)
  {
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = head[k];
    rem   = len;
    count = 0;
    done  = false;
    uint32_t cont = 0;
    if (!ascii)
      cont = gather_byte_flags(continuation_bytes(r[0])) | (gather_byte_flags(continuation_bytes(r[1])) << 4) |
             (gather_byte_flags(continuation_bytes(r[2])) << 8) | (gather_byte_flags(continuation_bytes(r[3])) << 12);
    bnd = (~cont & ((1u << len) - 1u)) | (1u << len);
    open_piece(t, 0, request(t, first_ids, 0, 0));
    if (probed) cand &= ~(1u << (len - 1));
  }

  __device__ __forceinline__ Probe probe_of(VocabTable const& t, const uint4* trim, uint32_t kind, uint32_t l) const
  {
    Probe pr;
    uint4 const keep = trim[l];  // (l <= 16)
    pr.k0            = r[0] & keep.x;
    pr.k1            = r[1] & keep.y;
    // (the third and fourth dword of a key of up to 8 bytes are zeros after the trim: they add nothing)
    uint64_t const h = key_hash_next(key_hash_first(kind, pr.k0, pr.k1), r[2] & keep.z, r[3] & keep.w, 1u);
    HashParts const hp = hash_parts(h, t.bucket_bits);
    pr.want            = slot_word0(hp.tag, kind, l);
    pr.fp              = hp.fp;
    pr.bucket          = hp.bucket;
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

  // One trip: looks up the longest remaining candidate of three bytes and more; when none of those is left, the
  // candidates of two bytes and of one byte are settled from the ids the opening gave, without hashing or further
  // reads.  (The length filter leaves few candidates: a piece that has any has 1.4 on average, so a second lookup in
  // the same trip would mostly be wasted work.)
  // (Measured and left out: requesting, in the same breath, the openings of the pieces that could come next, so that no
  // trip waits twice: 18 % slower, the scattered reads cost more than the waits they save; settling pieces that need
  // no lookup several to a trip, also with their openings coming from LDS: fewer trips, each slower by more, and the
  // registers it takes cost wavefronts per SIMD, which this loop needs: 1.03 ms with 8 of them, 1.07 with 6, 1.28 with 4.)
  template <typename Emit>
  __device__ __forceinline__ void step(VocabTable const& t, const int32_t* first_ids, const uint16_t* l3, const int32_t* pair, const uint4* trim,
                                       Emit&& emit)
  {
    uint32_t const kind = count ? 1u : 0u;
    cand &= (lens << 2) | 3u;
    lens                  = 0xFFFFFFFFu;
    uint32_t const longer = cand & ~3u;
    bool const has_a      = longer != 0;
    uint32_t const la     = 32u - static_cast<uint32_t>(__builtin_clz(has_a ? longer : 4u));
    Probe pa;
    uint4 a0 = make_uint4(0u, 0u, 0u, 0u), a1 = a0;
    if (has_a) {
      pa = probe_of(t, trim, kind, la);
      a0 = t.slots[2 * pa.bucket];
      a1 = t.slots[2 * pa.bucket + 1];
    }
    // where the word would go on from if this trip settles a piece: after the candidate, or, when it is the last one of
    // three bytes and more (or there is none), after two bytes or one
    uint32_t const longer_left = has_a ? longer ^ (1u << (la - 1)) : 0u;  // after a miss
    bool const two             = (cand & 2u) != 0 && id2 != kNone;
    bool const one             = (cand & 1u) != 0 && id1 != kNone;
    uint32_t const short_len   = two ? 2u : 1u;
    int32_t ida = kNone;
    uint32_t va = has_a ? verdict(pa, a0, a1, la, &ida) : 0u;
    if (va == 2u && la > 8) {  // a key of 9 to 16 bytes with the right tag: its bytes decide
      uint32_t k[4] = {r[0], r[1], r[2], r[3]};
      trim_key8(8u, k[0], k[1]);
      trim_key8(la - 8u, k[2], k[3]);
      va = verdict_16(t, pa, a0, a1, k, &ida);
    }
    if (va == 2u) {  // the general lookup (keys of more than 16 bytes, keys carried past their bucket)
      RegWord const rw{{r[0], r[1], r[2], r[3]}};
      ida = lookup_slow(t, kind, rw, 0u, la);
      va  = ida == kNone ? 0u : 1u;
    }
    bool const hit_a = has_a && va == 1u;
    // two bytes, then one byte; else no prefix of the word matched (375-379), or a later piece has no match and the
    // word collapses (396-404): either way a single unknown token
    bool const settle  = !hit_a && longer_left == 0;
    bool const hit     = hit_a || (settle && (two || one));
    bool const unknown = settle && !(two || one);
    uint32_t const len = hit_a ? la : short_len;
    int32_t const id   = hit_a ? ida : two ? id2 : id1;
    if (hit || unknown) emit(unknown ? 0u : count, unknown ? t.unk_id : id);
    count = unknown ? 1u : count + (hit ? 1u : 0u);
    done  = unknown || (hit && len == rem);
    cand  = longer_left | (cand & 3u);
    if (hit && !done) {
      advance(len);  // next piece: the rest of the word (381-395)
      open_piece(t, 1, request_next(t, first_ids, l3, pair));
    }
  }
};

// ------------------------------------------------------------------ the passes
// The column's bytes, from the 16-byte aligned address at or below its first byte, are cut into tiles of TILE
// bytes without regard to rows; kRangeTiles consecutive tiles form a range.
//   * word pass: a wavefront takes one range at a time and walks its tiles in order, so that the rows that start in
//     them are met in order too.  Per tile: find the words, look each one up whole.  Every word gets one slot of the
//     range's part of the word arena, in order: its token, or a marker with the index of its entry in the queue of
//     words that are not in the vocabulary as they stand.
//   * out-of-vocabulary pass: one lane per queued word; the result takes the place of the queue entry.
//   * emit pass: a wavefront per range expands the word slots into the tokens and gives every row that starts in the
//     range its list offset.
// Tiles per range that nvtext_amd_profile_set_range_tiles asked for (0: sized by the column).
std::atomic<int> g_forced_range_tiles{0};
// Whether a call sizes its first attempt from a sample of the column (nvtext_amd_profile_set_sizing_sample).
std::atomic<int> g_sizing_sample{1};
constexpr int kRangeTiles    = 8;     // tiles per range at most (a large column); a small column has fewer, so that every wavefront gets several ranges
constexpr int kOverBlocks    = 16;   // 16-byte blocks staged past the tile: a word that starts in the tile ends in them, or is kMaxWord bytes or more
constexpr uint32_t kQueueChunk = 512;  // queue entries a wavefront of the word pass reserves at a time
// A word slot: the token id (0 .. 2^31-1, or -1 for an absent [UNK]), or kOovMark | index of the word's queue entry
// (never 0xFFFFFFFF: the queue has fewer than 2^31 - 1 entries).
constexpr uint32_t kOovMark = 0x80000000u;

// A queued word (32 bytes).  The out-of-vocabulary pass puts the word's result in its place: up to kOovKeep tokens and
// their number; for a word with more tokens, only the number (the emit pass tokenizes it again, into place, from where
// and how long the word is, which stay).
struct OovEntry {
  uint32_t head[4];    // the word's first 16 bytes, zero padded: most words are tokenized without reading the chars again
  uint32_t len_flags;  // bytes in the word (1..199) | kUnprobed; 0: an unused entry
  uint32_t range;      // the range the word begins in
  uint32_t coord[2];   // coordinate of its first byte (low, high)
};
struct OovResult {
  int32_t tok[kOovKeep];  // count <= kOovKeep: the tokens.  More: tok[4..6] = len_flags, range, coord[0] of the entry; tok[3] = coord[1]
  uint32_t count;
};
static_assert(sizeof(OovEntry) == 32 && sizeof(OovResult) == 32, "a queue record is two 16-byte stores");
constexpr uint32_t kUnprobed = 0x100u;  // the word has not been looked up whole (more than 16 bytes; a key that may have been carried past its bucket)

template <int TILE>
struct TileLds {
  static constexpr int kBlocks = TILE / 16;
  alignas(16) uint32_t bytes[(16 + TILE + 16 * kOverBlocks) / 4 + 4];  // tile position x at byte 16 + x; key reads run a few bytes past a word
  uint32_t bound[kBlocks + kOverBlocks + 1];  // per block: bit i = a row starts at byte i; bit 16 + i = the words that a row's limit drops begin / stop here
  uint32_t masks[kBlocks];                    // per block: bit i = a word starts at byte i, bit 16 + i = a word ends at byte i
  uint32_t prefix[kBlocks + 1];               // word starts before the block | word ends before the block << 16
  static constexpr uint32_t kWordCap = TILE / 4;
  uint32_t word_guard[1];                     // (takes the end of the word that ran into the tile)
  uint32_t word[kWordCap];                    // per word: start | end << 16
};

struct TileArgs {
  ColView col;
  VocabTable table;
  const uint4* abase;      // 16-byte aligned address at or below the first byte of the view; coordinates count bytes from here
  int64_t first_offset;    // offsets[0] of the view
  int64_t cend;            // coordinate past the view's last byte
  int64_t ntiles;
  uint32_t cbeg;           // coordinate of the view's first byte (0..15)
  uint32_t nranges;
  int32_t max_words;
  int32_t range_tiles;     // tiles of a range
  uint32_t range_cap;      // word slots of a range
  const uint32_t* range_first_row;
  uint32_t* arena;         // the word slots of range g from arena[g * range_cap], densely, in order
  uint32_t* range_words;   // words of range g
  uint32_t* range_tokens;  // tokens of range g (here: of its words that are in the vocabulary; the next pass adds the others')
  int32_t* offsets_out;    // per row: words of its range before the row
  OovEntry* queue;
  uint32_t queue_cap;
  uint32_t* queue_size;    // entries reserved so far
  uint32_t* counter;       // next range to hand out
  uint32_t* overflow;      // set when a range has more words than range_cap
};

// The flag words of a tokenize call (indices of 32-bit words; what is asked for with atomics has a 128-byte line of its own):
constexpr uint32_t kCounterGroups = 8;
constexpr uint32_t kFlagLine      = 32;
constexpr uint32_t kFlagOverflow  = 1;                                          // a range had more words than slots
constexpr uint32_t kFlagQueueSize = 2;                                          // queue entries reserved
constexpr uint32_t kFlagLonger    = 1 * kFlagLine;                              // words of more than 16 bytes
constexpr uint32_t kFlagAgain     = 2 * kFlagLine;                              // words of more tokens than a queue record keeps
constexpr uint32_t kFlagWordUnits = 3 * kFlagLine;                              // kCounterGroups work counters of the word pass, a line each
constexpr uint32_t kFlagOovUnits  = kFlagWordUnits + kCounterGroups * kFlagLine;  // and of the out-of-vocabulary pass
constexpr uint32_t kFlagWords     = kFlagOovUnits + kCounterGroups * kFlagLine;

// The next unit of work for a wavefront of a persistent kernel: its first one is its own number in the grid, the
// following ones come from a counter.  Atomics on one address run at about 150 M/s: eight thousand wavefronts that all
// begin by asking one counter wait 55 microseconds between them, which was a tenth of a call on two million short
// rows; and with units small enough to even out the end of the kernel (ranges of 16 KB: a hundred thousand requests
// and more per GB of text), one counter made the word pass 16 % slower than it is with kCounterGroups of them, each in
// a line of its own: counter g serves the wavefronts g, g + kCounterGroups, .. and hands out the units g,
// g + kCounterGroups, .. (it starts at the number of those wavefronts).  (Looking at the counter with a coherent load
// before asking, to spare the one request too many that every wavefront ends with, made the passes two to four times
// slower.)
__device__ __forceinline__ uint32_t next_unit(uint32_t* counters, bool first, uint32_t my_number, int lane)
{
  // (my_number is the same in every lane, which the compiler cannot know: as a scalar, so that what depends on it stays scalar)
  uint32_t const me = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(my_number)));
  if (first) return me;
  uint32_t const g = me % kCounterGroups;
  uint32_t n       = 0xFFFFFFFFu / kCounterGroups - 1u;
  if (lane == 0) n = atomicAdd(counters + g * kFlagLine, 1u);
  return wave_bcast(n, 0) * kCounterGroups + g;
}

__device__ __forceinline__ void wave_lds_sync()
{
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// bit i = byte i of the sixteen is a space
__device__ __forceinline__ uint32_t space_mask16(uint4 const& v)
{
  return gather_byte_flags(space_bytes(v.x)) | (gather_byte_flags(space_bytes(v.y)) << 4) | (gather_byte_flags(space_bytes(v.z)) << 8) |
         (gather_byte_flags(space_bytes(v.w)) << 12);
}

// bit i = coordinate g0 + i lies outside [lo, hi)
__device__ __forceinline__ uint32_t outside_mask16(int64_t g0, int64_t lo, int64_t hi)
{
  int64_t const a  = lo - g0, b = hi - g0;
  uint32_t const l = a <= 0 ? 0u : a >= 16 ? 16u : static_cast<uint32_t>(a);
  uint32_t const h = b <= 0 ? 0u : b >= 16 ? 16u : static_cast<uint32_t>(b);
  return ~(((1u << h) - 1u) & ~((1u << l) - 1u)) & 0xFFFFu;
}

// Words that start in coordinates [from, to) (bytes outside count as spaces), counted by the whole wavefront, 1 KiB
// a step; stops once `limit` is reached.  Same value in every lane.
__device__ __forceinline__ uint32_t count_word_starts(const uint4* abase, int64_t from, int64_t to, uint32_t limit)
{
  int const lane      = lane_id();
  uint32_t total      = 0;
  uint32_t prev_space = 1;
  for (int64_t g = from & ~static_cast<int64_t>(15); g < to && total < limit; g += 16 * kWave) {
    int64_t const g0 = g + 16 * lane;
    uint4 v          = make_uint4(0u, 0u, 0u, 0u);
    if (g0 < to && g0 + 16 > from) v = abase[g0 >> 4];
    uint32_t const sp     = (space_mask16(v) | outside_mask16(g0, from, to)) & 0xFFFFu;
    uint32_t const before = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(static_cast<int>(prev_space), static_cast<int>(sp >> 15), 0x138, 0xf, 0xf, false));
    uint32_t const starts = ~sp & ((sp << 1) | before) & 0xFFFFu;
    total += wave_bcast(wave_inclusive_scan(static_cast<uint32_t>(__builtin_popcount(starts))), kWave - 1);
    prev_space = wave_bcast(sp >> 15, kWave - 1);
  }
  return total;
}

// range_first_row[g] = the first row (0..rows) that starts at or after the first byte of range g; [nranges] = rows.
// The first workgroup also sets the flag words of the call: zeros, but for the work counters, which start past the
// units that the wavefronts take by their place in the grid (counter g serves the wavefronts g, g + kCounterGroups, ..
// and hands out the units g, g + kCounterGroups, ..).
__global__ void range_first_row_kernel(ColView col, int64_t first_offset, uint32_t cbeg, int64_t range_bytes, uint32_t nranges,
                                       uint32_t* __restrict__ range_first_row, uint32_t* __restrict__ flags, uint32_t word_waves,
                                       uint32_t oov_waves)
{
  if (blockIdx.x == 0) {
    for (uint32_t i = threadIdx.x; i < kFlagWords; i += blockDim.x) {
      uint32_t v = 0;
      if (i >= kFlagWordUnits && i % kFlagLine == 0) {
        uint32_t const c = (i - kFlagWordUnits) / kFlagLine;
        v = ((c < kCounterGroups ? word_waves : oov_waves) + kCounterGroups - 1u - c % kCounterGroups) / kCounterGroups;
      }
      flags[i] = v;
    }
  }
  uint32_t const g = blockIdx.x * blockDim.x + threadIdx.x;
  if (g > nranges) return;
  int64_t const target = static_cast<int64_t>(g) * range_bytes;
  uint32_t lo = 0, hi = static_cast<uint32_t>(col.size);
  if (g == nranges) lo = hi;
  while (lo < hi) {
    uint32_t const mid = lo + ((hi - lo) >> 1);
    if (col.off(mid) - first_offset + cbeg < target) lo = mid + 1;
    else hi = mid;
  }
  range_first_row[g] = lo;
}

// One tile at a time per wavefront: stage its bytes (and the 256 after it) in LDS; mark the row starts in it; find
// word starts and ends (lanes <-> 16-byte blocks: spaces by SWAR, row starts as extra separators); with a word limit,
// drop the words past each row's limit; list the words (word k pairs start k with end k); look all of them up (lanes
// <-> words, one probe each) and write their slots; give every row that starts in the tile the number of words of the
// range before it.
template <int TILE, bool IS64, bool LIMIT>
__global__ void __launch_bounds__(kTokThreads, 6) wordpiece_word_kernel(TileArgs a)
{
  constexpr int kBlocks       = TILE / 16;
  constexpr int kSubs         = kBlocks / kWave;
  constexpr uint32_t kWordCap = TileLds<TILE>::kWordCap;
  static_assert(kBlocks % kWave == 0, "whole wavefronts of blocks");
  __shared__ TileLds<TILE> lds_all[kTokWaves];
  __shared__ uint4 trim[17];
  fill_trim_table(trim);
  __syncthreads();
  TileLds<TILE>& lds  = lds_all[threadIdx.x / kWave];
  int const lane      = lane_id();
  uint32_t const rows = static_cast<uint32_t>(a.col.size);
  int64_t const cbeg  = a.cbeg, cend = a.cend;
  VocabTable const& table = a.table;
  int64_t const cadj      = cbeg - a.first_offset;
  auto coord = [&](uint32_t r) -> int64_t {
    int64_t const i = static_cast<int64_t>(r) + a.col.offset;
    return (IS64 ? static_cast<const int64_t*>(a.col.offsets)[i] : static_cast<int64_t>(static_cast<const int32_t*>(a.col.offsets)[i])) + cadj;
  };
  // wordpiece_tokenize.cu:776-781: with a word limit, null rows have no words and the limit is
  // min(max_words, size_bytes / 2); without one, validity is not consulted (503-568).
  auto word_cap = [&](uint32_t r, int64_t bytes) -> uint32_t {
    return a.col.valid(r) ? static_cast<uint32_t>(min(static_cast<int64_t>(a.max_words), bytes / 2)) : 0u;
  };
  const uint8_t* const lds_byte = reinterpret_cast<const uint8_t*>(lds.bytes);
  uint16_t* const word16        = reinterpret_cast<uint16_t*>(lds.word);
  uint32_t q_pos = 0, q_lim = 0;  // this wavefront's reserved queue entries [q_pos, q_lim)

  uint32_t const my_number = blockIdx.x * kTokWaves + threadIdx.x / kWave;
  for (bool first = true;; first = false) {
    uint32_t const range = next_unit(a.counter, first, my_number, lane);
    if (range >= a.nranges) break;
    int64_t t           = static_cast<int64_t>(range) * a.range_tiles;
    int64_t const t_end = min(t + a.range_tiles, a.ntiles);
    uint32_t r_cur      = a.range_first_row[range];
    uint32_t cursor     = 0;  // words of this range so far
    uint32_t known      = 0;  // of them, in the vocabulary (or too long: one unknown token each)
    uint32_t open_left  = 0;  // words the row that runs into the tile may still have (with a word limit)
    uint32_t* const region = a.arena + static_cast<int64_t>(range) * a.range_cap;
    bool spill             = false;
    if (LIMIT && r_cur > 0) {
      uint32_t const ro  = r_cur - 1;
      int64_t const c0   = coord(ro), c1 = coord(ro + 1);
      uint32_t const cap = word_cap(ro, c1 - c0);
      uint32_t const used = cap ? count_word_starts(a.abase, c0, t * TILE, cap) : 0u;
      open_left           = cap - min(cap, used);
    }

    // the bytes of a tile, the 16 before them and the 256 after them, as 16-byte blocks: block j of lane l is l - 1 + 64 j
    constexpr int kStageLoads = (kBlocks + kOverBlocks + 1 + kWave - 1) / kWave;
    uint4 ahead[kStageLoads];
    auto request_tile = [&](int64_t tile) {
      int64_t const tile_begin = tile * TILE;
#pragma unroll
      for (int i = 0; i < kStageLoads; ++i) {
        int64_t const g0 = tile_begin + 16 * (lane - 1 + i * kWave);
        ahead[i]         = make_uint4(0u, 0u, 0u, 0u);
        if (g0 + 16 > cbeg && g0 < cend) ahead[i] = load_stream(a.abase + (g0 >> 4));
      }
    };
    request_tile(t);
    for (; t < t_end; ++t) {
      int64_t const tb     = t * TILE;
      bool const last_tile = t + 1 == a.ntiles;
      bool const edge      = tb < 16 + cbeg || tb + TILE + 16 * kOverBlocks > cend;  // some staged byte lies outside the view

      // ---- stage the bytes (requested while the tile before was being worked on), and request the next tile's
#pragma unroll
      for (int i = 0; i < kStageLoads; ++i) {
        int const j = lane - 1 + i * kWave;
        if (j < kBlocks + kOverBlocks) *reinterpret_cast<uint4*>(&lds.bytes[4 * (j + 1)]) = ahead[i];
      }
      if (t + 1 < t_end) request_tile(t + 1);
      for (int i = lane; i < kBlocks + kOverBlocks + 1; i += kWave) lds.bound[i] = 0;
      wave_lds_sync();

      // ---- the rows that start in the tile: [r_first, r_end)
      uint32_t const r_first = r_cur;
      int64_t crow           = 0;  // where row r_first + lane begins (kept for the passes over the rows below)
      for (;;) {
        uint32_t const r = r_cur + lane;
        int64_t const c  = r <= rows ? coord(r) : std::numeric_limits<int64_t>::max();
        int64_t const p  = r <= rows ? c - tb : c;
        if (r_cur == r_first) crow = c;
        bool const in    = r < rows && (last_tile || p < TILE);
        if (p < TILE + 16 * kOverBlocks) atomicOr(&lds.bound[p >> 4], 1u << (p & 15));
        uint32_t const n = static_cast<uint32_t>(__builtin_popcountll(ballot64(in)));
        r_cur += n;
        if (n < kWave) break;
      }
      uint32_t const r_end = r_cur;
      wave_lds_sync();

      // ---- word starts and ends
      uint32_t nw = 0, ne = 0, inside0 = 0;  // words that start in the tile, words that end in it, the tile begins inside a word
      {
        uint32_t base = 0;
#pragma unroll
        for (int s = 0; s < kSubs; ++s) {
          int const b     = s * kWave + lane;
          uint4 const v   = *reinterpret_cast<const uint4*>(&lds.bytes[4 * (b + 1)]);
          uint32_t sp     = space_mask16(v);
          uint32_t before = lds_byte[16 + 16 * b - 1] == 0x20u, after = lds_byte[16 + 16 * b + 16] == 0x20u;
          if (edge) {
            int64_t const g0 = tb + 16 * b;
            sp |= outside_mask16(g0, cbeg, cend);
            before |= (g0 - 1 < cbeg || g0 - 1 >= cend);
            after |= (g0 + 16 < cbeg || g0 + 16 >= cend);
          }
          uint32_t const bd = lds.bound[b] & 0xFFFFu;
          after |= lds.bound[b + 1] & 1u;
          uint32_t const word   = ~sp & 0xFFFFu;
          uint32_t const starts = word & ((sp << 1) | before | bd);
          uint32_t const ends   = word & ((sp >> 1) | (after << 15) | (bd >> 1));
          if (s == 0) inside0 = wave_bcast(word & ~starts & 1u, 0);
          lds.masks[b]          = starts | (ends << 16);
          uint32_t const cnt    = static_cast<uint32_t>(__builtin_popcount(starts)) | (static_cast<uint32_t>(__builtin_popcount(ends)) << 16);
          uint32_t const incl   = wave_inclusive_scan(cnt);
          lds.prefix[b]         = base + incl - cnt;
          base += wave_bcast(incl, kWave - 1);
        }
        if (lane == 0) lds.prefix[kBlocks] = base;
        nw = base & 0xFFFFu;
        ne = base >> 16;
      }
      wave_lds_sync();

      // word starts at positions below x (0 <= x)
      auto words_before = [&](uint32_t x) -> uint32_t {
        if (x >= TILE) return nw;
        uint32_t const b = x >> 4;
        return (lds.prefix[b] & 0xFFFFu) + static_cast<uint32_t>(__builtin_popcount(lds.masks[b] & ((1u << (x & 15u)) - 1u)));
      };

      // ---- a word limit: the words of a row past its limit are dropped.  The first such word and the row's end are
      // marked; a prefix parity over the marks gives the bytes whose word starts and ends go.
      if (LIMIT) {
        // position of word start k (k < nw)
        auto word_start = [&](uint32_t k) -> uint32_t {
          uint32_t b = 0;
#pragma unroll
          for (uint32_t step = kBlocks / 2; step > 0; step >>= 1)
            if ((lds.prefix[b + step] & 0xFFFFu) <= k) b += step;
          uint32_t m = lds.masks[b] & 0xFFFFu;
          for (uint32_t j = k - (lds.prefix[b] & 0xFFFFu); j > 0; --j) m &= m - 1u;
          return 16u * b + static_cast<uint32_t>(__builtin_ctz(m | 0x10000u));
        };
        bool cut = false;
        auto drop_from = [&](uint32_t k, int64_t e) {  // from word start k up to position e
          uint32_t const at = word_start(k);
          atomicXor(&lds.bound[at >> 4], 0x10000u << (at & 15u));
          if (e < TILE) atomicXor(&lds.bound[e >> 4], 0x10000u << (e & 15));
          cut = true;
        };
        for (uint32_t i = 0; r_first + i < r_end; i += kWave) {
          uint32_t const r = r_first + i + lane;
          // (the first 64 rows' beginnings are at hand; a row ends where the next begins)
          int64_t c_next = static_cast<int64_t>((static_cast<uint64_t>(static_cast<uint32_t>(__shfl_down(static_cast<int>(static_cast<uint64_t>(crow) >> 32), 1))) << 32) |
                                                static_cast<uint32_t>(__shfl_down(static_cast<int>(static_cast<uint32_t>(crow)), 1)));
          if (r < r_end) {
            int64_t const c0 = i == 0 ? crow : coord(r);
            int64_t const c1 = i == 0 && lane < kWave - 1 ? c_next : coord(r + 1);
            if (c1 > c0) {
              int64_t const p = c0 - tb, e = c1 - tb;  // (p < TILE: the rows past the last tile's end are empty)
              uint32_t const cap = word_cap(r, c1 - c0);
              uint32_t const wp  = words_before(static_cast<uint32_t>(p));
              uint32_t const we  = words_before(e < TILE ? static_cast<uint32_t>(e) : static_cast<uint32_t>(TILE));
              if (wp + cap < we) drop_from(wp + cap, e);
            }
          }
        }
        // the row that runs into the tile
        int64_t const e0   = r_first < r_end ? static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(crow), 0)) - tb : static_cast<int64_t>(TILE);
        uint32_t const we0 = words_before(e0 < TILE ? static_cast<uint32_t>(e0) : static_cast<uint32_t>(TILE));
        if (lane == 0 && open_left < we0) drop_from(open_left, e0);
        // and the row that runs out of it
        if (r_first < r_end) {
          uint32_t const rl   = r_end - 1;
          uint32_t const il   = rl - r_first;
          int64_t const c0    = il < kWave ? static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(crow), static_cast<int>(il))) : coord(rl);
          int64_t const c1    = il + 1 < kWave ? static_cast<int64_t>(wave_bcast64(static_cast<uint64_t>(crow), static_cast<int>(il + 1))) : coord(rl + 1);
          int64_t const p     = c0 - tb;
          uint32_t const cap  = word_cap(rl, c1 - c0);
          uint32_t const used = nw - words_before(p < TILE ? static_cast<uint32_t>(p) : static_cast<uint32_t>(TILE));
          open_left           = cap - min(cap, used);
        } else {
          open_left -= min(open_left, nw);
        }
        if (ballot64(cut) != 0) {
          wave_lds_sync();
          uint32_t base = 0, carry = 0;
#pragma unroll
          for (int s = 0; s < kSubs; ++s) {
            int const b      = s * kWave + lane;
            uint32_t const m = lds.masks[b];
            uint32_t px      = lds.bound[b] >> 16;
            px ^= px << 1;
            px ^= px << 2;
            px ^= px << 4;
            px ^= px << 8;
            px &= 0xFFFFu;
            uint64_t const odd  = ballot64((px >> 15) != 0);
            uint32_t const flip = (lanes_below(odd) & 1u) ^ carry;
            carry ^= static_cast<uint32_t>(__builtin_popcountll(odd)) & 1u;
            uint32_t const dead   = flip ? (~px & 0xFFFFu) : px;
            uint32_t const starts = m & 0xFFFFu & ~dead, ends = (m >> 16) & ~dead;
            lds.masks[b]          = starts | (ends << 16);
            uint32_t const cnt    = static_cast<uint32_t>(__builtin_popcount(starts)) | (static_cast<uint32_t>(__builtin_popcount(ends)) << 16);
            uint32_t const incl   = wave_inclusive_scan(cnt);
            lds.prefix[b]         = base + incl - cnt;
            base += wave_bcast(incl, kWave - 1);
          }
          if (lane == 0) lds.prefix[kBlocks] = base;
          nw = base & 0xFFFFu;
          ne = base >> 16;
          wave_lds_sync();
        }
      }
      // ---- the rows that start in the tile: the words of the range before them
      for (uint32_t i = 0; r_first + i < r_end; i += kWave) {
        uint32_t const r = r_first + i + lane;
        if (r < r_end) {
          int64_t const p  = (i == 0 ? crow : coord(r)) - tb;
          a.offsets_out[r] = static_cast<int32_t>(cursor + words_before(p < TILE ? static_cast<uint32_t>(p) : static_cast<uint32_t>(TILE)));
        }
      }

      // ---- the words, at most kWordCap at a time (only a tile of one- and two-byte rows or words has more)
      for (uint32_t w_lo = 0;; w_lo += kWordCap) {
        uint32_t const w_hi = min(nw, w_lo + kWordCap);
        uint32_t const nwc  = w_hi - w_lo;
        // start k pairs with end k (after the end of the word that ran into the tile)
        if (nw <= kWordCap) {
#pragma unroll
          for (int s = 0; s < kSubs; ++s) {
            int const b       = s * kWave + lane;
            uint32_t const m  = lds.masks[b];
            uint32_t const pf = lds.prefix[b];
            uint32_t ks       = pf & 0xFFFFu;
            uint32_t ke       = (pf >> 16) - inside0;  // (the end without a start comes first: it goes to slot -1, which is the entry before lds.word)
            for (uint32_t st = m & 0xFFFFu; st; st &= st - 1u, ++ks) word16[2 * ks] = static_cast<uint16_t>(16 * b + __builtin_ctz(st));
            for (uint32_t en = m >> 16; en; en &= en - 1u, ++ke) word16[2 * static_cast<int32_t>(ke) + 1] = static_cast<uint16_t>(16 * b + __builtin_ctz(en));
          }
        } else {
#pragma unroll
          for (int s = 0; s < kSubs; ++s) {
            int const b       = s * kWave + lane;
            uint32_t const m  = lds.masks[b];
            uint32_t const pf = lds.prefix[b];
            uint32_t ks       = pf & 0xFFFFu;
            int32_t ke        = static_cast<int32_t>(pf >> 16) - static_cast<int32_t>(inside0);
            for (uint32_t st = m & 0xFFFFu; st; st &= st - 1u, ++ks)
              if (ks >= w_lo && ks < w_hi) word16[2 * (ks - w_lo)] = static_cast<uint16_t>(16 * b + __builtin_ctz(st));
            for (uint32_t en = m >> 16; en; en &= en - 1u, ++ke)
              if (ke >= static_cast<int32_t>(w_lo) && ke < static_cast<int32_t>(w_hi)) word16[2 * (ke - w_lo) + 1] = static_cast<uint16_t>(16 * b + __builtin_ctz(en));
          }
        }
        if (w_hi == nw && nwc > 0 && nw + inside0 > ne) {
          // the last word ends past the tile: at the byte before the first space, row start or end of the view
          uint32_t sep = 0;
          if (lane < kOverBlocks) {
            int const b   = kBlocks + lane;
            uint4 const v = *reinterpret_cast<const uint4*>(&lds.bytes[4 * (b + 1)]);
            sep           = space_mask16(v) | (lds.bound[b] & 0xFFFFu);
            if (edge) sep |= outside_mask16(tb + 16 * b, cbeg, cend);
          }
          uint64_t const sm = ballot64(sep != 0);
          uint32_t endpos   = TILE + 16 * kOverBlocks - 1;
          if (sm != 0) {
            int const fl = __builtin_ctzll(sm);
            endpos       = TILE + 16 * fl + __builtin_ctz(wave_bcast(sep, fl)) - 1;
          }
          if (lane == 0) word16[2 * (nwc - 1) + 1] = static_cast<uint16_t>(endpos);
        }
        wave_lds_sync();

        // ---- look the words up; the ones that are not in the vocabulary, or not decided here, go to the queue.
        // A round of 64 words has ten such words on average, too few for the work of building and storing their
        // records: a round only gives each its place in the queue (which its slot names) and lists it, at the front
        // of the list of words itself (entry c of the listed words never lies behind the word it came from); the
        // records of all of them are built and stored afterwards, lanes <-> listed words.
        if (cursor + nwc > a.range_cap) spill = true;
        uint32_t const room = q_lim - q_pos;  // left of the reserved entries: used up before the next ones are begun
        uint32_t fresh      = 0;              // where the next ones begin, once they are needed
        bool have_fresh     = false;
        uint32_t listed     = 0;
        auto queue_place = [&](uint32_t c) { return c < room ? q_pos + c : fresh + (c - room); };
        for (uint32_t k0 = 0; k0 < nwc; k0 += kWave) {
          uint32_t const k   = k0 + lane;
          bool const active  = k < nwc;
          uint32_t const rec = lds.word[active ? k : 0u];
          uint32_t const s   = rec & 0xFFFFu;
          uint32_t const wl  = (rec >> 16) - s + 1u;
          // straight-line code: every lane reads a bucket (of whatever its first bytes are), and what it makes of it
          // depends on the word's length afterwards; only a key of 9 to 16 bytes with the right tag needs a second
          // read, of the key's bytes
          TileWord const tw{lds.bytes, 16u + s};
          uint32_t head[4];
          tw.head16(head);
          uint32_t const wl16 = min(wl, 16u);
          uint4 const keep    = trim[wl16];
          head[0] &= keep.x;
          head[1] &= keep.y;
          head[2] &= keep.z;
          head[3] &= keep.w;
          Probe pr;
          pr.k0             = head[0];
          pr.k1             = head[1];
          // (the third and fourth dword of a word of up to 8 bytes are zeros after the trim: they add nothing)
          uint64_t const h = key_hash_next(key_hash_first(0u, pr.k0, pr.k1), head[2], head[3], 1u);
          HashParts const hp = hash_parts(h, table.bucket_bits);
          pr.want            = slot_word0(hp.tag, 0u, wl16);
          pr.fp              = hp.fp;
          pr.bucket          = hp.bucket;
          uint4 const s0 = table.slots[2 * pr.bucket];
          uint4 const s1 = table.slots[2 * pr.bucket + 1];
          int32_t id  = kNone;
          uint32_t vd = verdict(pr, s0, s1, wl16, &id);
          if (vd == 2u && wl > 8 && wl <= 16) vd = verdict_16(table, pr, s0, s1, head, &id);
          bool const too_long = wl >= kMaxWord;  // wordpiece_tokenize.cu:442-445, 738-741: one unknown token
          bool const found    = wl <= 16 && vd == 1u;
          // 1: not in the vocabulary; 2: not decided here (more than 16 bytes; a key that may have been carried past its bucket)
          uint32_t const defer = !active || too_long || found ? 0u : (wl > 16 || (vd == 2u && wl <= table.max_len[0])) ? 2u : 1u;
          uint32_t value       = too_long ? static_cast<uint32_t>(table.unk_id) : static_cast<uint32_t>(id);
          uint64_t const mm    = ballot64(defer != 0);
          uint32_t const nm    = static_cast<uint32_t>(__builtin_popcountll(mm));
          if (listed + nm > room && !have_fresh) {
            if (lane == 0) fresh = atomicAdd(a.queue_size, kQueueChunk);
            fresh      = wave_bcast(fresh, 0);
            have_fresh = true;
          }
          if (defer != 0) {
            uint32_t const c = listed + lanes_below(mm);
            lds.word[c]      = rec | (defer << 12);  // (a word starts below 2048: bits 12 and 13 of its entry are free)
            value            = kOovMark | queue_place(c);
          }
          listed += nm;
          known += static_cast<uint32_t>(__builtin_popcountll(ballot64(active && defer == 0)));
          if (active && !spill) region[cursor + k] = value;
        }
        wave_lds_sync();
        // the records of the listed words: the word's first 16 bytes, its length, its range and where it begins
        for (uint32_t c0 = 0; c0 < listed; c0 += kWave) {
          uint32_t const c = c0 + lane;
          if (c < listed) {
            uint32_t const entry = lds.word[c];
            uint32_t const s     = entry & 0xFFFu;
            uint32_t const wl    = (entry >> 16) - s + 1u;
            uint32_t const defer = (entry >> 12) & 3u;
            TileWord const tw{lds.bytes, 16u + s};
            uint32_t head[4];
            tw.head16(head);
            uint4 const keep = trim[min(wl, 16u)];
            int64_t const at = tb + s;
            uint32_t const q = queue_place(c);
            if (q < a.queue_cap) {
              uint4* const dst = reinterpret_cast<uint4*>(a.queue + q);
              store_stream(dst, make_uint4(head[0] & keep.x, head[1] & keep.y, head[2] & keep.z, head[3] & keep.w));
              store_stream(dst + 1, make_uint4(wl | (defer == 2u ? kUnprobed : 0u), range, static_cast<uint32_t>(at),
                                               static_cast<uint32_t>(static_cast<uint64_t>(at) >> 32)));
            }
          }
        }
        if (listed > room) {
          q_pos = fresh + (listed - room);
          q_lim = fresh + kQueueChunk;
        } else {
          q_pos += listed;
        }
        cursor += nwc;
        wave_lds_sync();
        if (w_hi == nw) break;
      }
    }
    if (lane == 0) {
      a.range_words[range]  = cursor;
      a.range_tokens[range] = known;
      if (spill) *a.overflow = 1u;
    }
  }
  // the reserved entries that no word took
  for (uint32_t q = q_pos + lane; q < q_lim; q += kWave)
    if (q < a.queue_cap) a.queue[q].len_flags = 0;
}

// ------------------------------------------------------------------ out-of-vocabulary pass
// One lane per queued word, and a lane that finishes its word stores the result and takes the next one.  A wavefront
// takes kOovBlock queue entries at a time (one atomic), brings them into LDS 64 at a time with whole-record reads (the
// next 64 are requested while these are worked on) and lets its idle lanes take entries from there every trip.  Words
// of up to 16 bytes, whole in their queue record, run in registers; the few longer ones are set aside and done, one
// lane each, by the general state machine over the chars in memory, 64 and more at a time or at the end.
constexpr uint32_t kOovBlock = 512;
constexpr int kRefillAt      = 32;
constexpr int kOovWaves      = 16;  // (two workgroups to a CU, 73 KB of LDS each, 8 wavefronts per SIMD)
constexpr int kOovThreads    = kOovWaves * kWave;
constexpr int kRareThreads   = 256;  // the kernels for the few words that this one leaves
struct OovLds {
  alignas(16) uint4 staged[kWave][2];  // 64 queue entries
};

__global__ void __launch_bounds__(kOovThreads, 8) wordpiece_oov_kernel(VocabTable table, const uint4* abase, OovEntry* __restrict__ queue,
                                                                    const uint32_t* __restrict__ queue_size, uint32_t queue_cap,
                                                                    uint32_t* __restrict__ range_tokens, uint32_t* __restrict__ counter,
                                                                    uint32_t* __restrict__ longer, uint32_t* __restrict__ longer_count)
{
  __shared__ OovLds lds_all[kOovWaves];
  __shared__ int32_t first_ids[512];  // the ids of the one-byte keys of both key spaces: looked at whenever a piece of a word begins
  __shared__ int32_t pair_ids[kLetters2];  // the ids of the keys of two lower-case letters, second key space
  __shared__ uint16_t letters3[kLetters3];
  __shared__ uint4 trim[17];
  // an empty queue (a small call, text that is all in the vocabulary), or one that was too small (the host repeats the
  // passes with a larger one): nothing to do, and the tables need not be fetched
  if (*queue_size == 0 || *queue_size > queue_cap) return;
  fill_trim_table(trim);
  for (int i = threadIdx.x; i < 512; i += kOovThreads) first_ids[i] = table.short_ids[2 * 65536 + i];
  for (uint32_t i = threadIdx.x; i < kLetters2; i += kOovThreads) pair_ids[i] = table.short_ids[65536 + ((i / 26u + 'a') | ((i % 26u + 'a') << 8))];
  for (uint32_t i = threadIdx.x; i < kLetters3 / 2; i += kOovThreads)
    reinterpret_cast<uint32_t*>(letters3)[i] = reinterpret_cast<const uint32_t*>(table.letters3)[i];
  __syncthreads();
  uint32_t const total = *queue_size;
  OovLds& lds          = lds_all[threadIdx.x / kWave];
  int const lane       = lane_id();

  ShortWord sw;
  sw.done   = true;
  sw.count  = 0;
  bool busy = false;
  uint32_t mine = 0, mine_range = 0;  // my word's queue entry and range
  uint32_t acc_range = 0, acc_count = 0;
  int32_t tok[kOovKeep];
  auto keep_token = [&](uint32_t j, int32_t id) {
#pragma unroll
    for (int i = 0; i < kOovKeep; ++i)
      if (j == static_cast<uint32_t>(i)) tok[i] = id;
  };
  // the result takes the place of the entry
  auto deliver = [&](uint32_t q, uint32_t count, uint4 const& entry_tail) {
    uint4* const dst = reinterpret_cast<uint4*>(queue + q);
    if (count <= kOovKeep) {
      store_stream(dst, make_uint4(static_cast<uint32_t>(tok[0]), static_cast<uint32_t>(tok[1]), static_cast<uint32_t>(tok[2]), static_cast<uint32_t>(tok[3])));
      store_stream(dst + 1, make_uint4(static_cast<uint32_t>(tok[4]), static_cast<uint32_t>(tok[5]), static_cast<uint32_t>(tok[6]), count));
    } else {
      // more tokens than a record keeps: where and how long the word is stays, for the emit pass
      store_stream(dst, make_uint4(0u, 0u, 0u, entry_tail.w));
      store_stream(dst + 1, make_uint4(entry_tail.x, entry_tail.y, entry_tail.z, count));
    }
  };
  // the lanes named add their acc_count to the token count of their acc_range, one atomic per range among them
  auto add_together = [&](bool which) {
    uint64_t pending = ballot64(which);
    while (pending != 0) {
      uint32_t const r   = wave_bcast(acc_range, __builtin_ctzll(pending));
      bool const same    = which && acc_range == r;
      uint32_t const sum = wave_bcast(wave_inclusive_scan(same ? acc_count : 0u), kWave - 1);
      if (lane == 0) atomicAdd(&range_tokens[r], sum);
      pending &= ~ballot64(same);
    }
  };
  uint4 mine_tail = make_uint4(0u, 0u, 0u, 0u);  // the second half of my word's entry

  // the queue entries being fetched: [f_base, f_base + f_n), one per lane; they come from the block [.., q_end) that
  // this wavefront has taken, and a new block is taken when that one is used up
  uint32_t next_fetch = 0, q_end = 0, f_base = 0, f_n = 0;
  bool no_more = false, first_block = true;
  uint32_t const my_number = blockIdx.x * kOovWaves + threadIdx.x / kWave;
  uint4 pa = make_uint4(0u, 0u, 0u, 0u), pb = pa;
  auto start_fetch = [&] {
    f_n = 0;
    if (next_fetch >= q_end && !no_more) {
      uint32_t const block   = next_unit(counter, first_block, my_number, lane);
      first_block            = false;
      uint64_t const b_begin = static_cast<uint64_t>(block) * kOovBlock;
      if (b_begin >= total) {
        no_more = true;
      } else {
        next_fetch = static_cast<uint32_t>(b_begin);
        q_end      = static_cast<uint32_t>(min(b_begin + kOovBlock, static_cast<uint64_t>(total)));
      }
    }
    if (next_fetch < q_end) {
      f_base = next_fetch;
      f_n    = min(static_cast<uint32_t>(kWave), q_end - next_fetch);
      next_fetch += f_n;
      if (static_cast<uint32_t>(lane) < f_n) {
        const uint4* const src = reinterpret_cast<const uint4*>(queue + f_base + lane);
        pa = load_stream(src);
        pb = load_stream(src + 1);
      }
    }
  };
  uint32_t st_base = 0, st_next = 0, st_end = 0;  // the staged entries still to be taken are queue[st_base + st_next .. st_base + st_end)
  start_fetch();
  for (;;) {
    // Lanes that have finished wait until kRefillAt of them are free (or nobody is working): storing results and
    // taking new words is code that the whole wavefront runs through, whether for one lane or for sixty-four.
    uint64_t const working = ballot64(busy && !sw.done);
    if (kWave - __builtin_popcountll(working) >= kRefillAt || working == 0) {
      bool const finished = busy && sw.done;
      if (finished) {
        deliver(mine, sw.count, mine_tail);
        busy = false;
      }
      // The tokens of a range are added up per lane as long as the lane's words are of the same range (the queue holds
      // the words of a range side by side), and the lanes that move on to another range add what they have together:
      // the lanes of a wavefront are mostly on the same range, and their sixty-four atomics on its one counter, one
      // after the other, were a tenth of this pass.
      add_together(finished && mine_range != acc_range && acc_count != 0);
      if (finished) {
        if (mine_range != acc_range) {
          acc_range = mine_range;
          acc_count = 0;
        }
        acc_count += sw.count;
      }
      if (st_next >= st_end && f_n > 0) {
        // the staged entries are used up: the fetched ones take their place, and the next are requested
        wave_lds_sync();
        lds.staged[lane][0] = pa;
        lds.staged[lane][1] = pb;
        st_base = f_base;
        st_next = 0;
        st_end  = f_n;
        wave_lds_sync();
        start_fetch();
      }
      uint32_t const left = st_end - st_next;
      if (left > 0) {
        uint64_t const idle = ballot64(!busy);
        if (idle != 0) {
          uint32_t const rank = lanes_below(idle);
          bool is_long        = false;
          uint32_t at         = 0;
          // no byte of any word taken now has bit 7 set: every position of theirs is a character boundary
          bool const taking = !busy && rank < left;
          uint4 const ha    = lds.staged[taking ? st_next + rank : 0u][0];
          bool const ascii  = ballot64(taking && ((ha.x | ha.y | ha.z | ha.w) & 0x80808080u) != 0) == 0;
          if (taking) {
            at            = st_next + rank;
            uint4 const a = ha, b = lds.staged[at][1];
            uint32_t const wl = b.x & 0xFFu;
            if (wl != 0) {  // (0: an entry that no word took)
              if (wl <= 16) {
                uint32_t const head[4] = {a.x, a.y, a.z, a.w};
                sw.begin(table, first_ids, head, wl, (b.x & kUnprobed) == 0, ascii);
                busy       = true;
                mine       = st_base + at;
                mine_range = b.y;
                mine_tail  = b;
              } else {
                is_long = true;
              }
            }
          }
          st_next += min(static_cast<uint32_t>(__builtin_popcountll(idle)), left);
          uint64_t const lm = ballot64(is_long);
          if (lm != 0) {
            // words of more than 16 bytes: listed for the kernel that does those
            uint32_t first = 0;
            if (lane == 0) first = atomicAdd(longer_count, static_cast<uint32_t>(__builtin_popcountll(lm)));
            first = wave_bcast(first, 0);
            if (is_long) longer[first + lanes_below(lm)] = st_base + at;
          }
        }
      }
    }
    bool const drained = st_next >= st_end && f_n == 0;
    if (ballot64(busy && !sw.done) == 0) {
      if (drained && ballot64(busy) == 0) break;
      continue;
    }
    if (busy && !sw.done) sw.step(table, first_ids, letters3, pair_ids, trim, keep_token);
  }
  add_together(acc_count != 0);
}

// The queued words of more than 16 bytes, which the kernel above has listed: one lane per word, the general state
// machine over the chars in memory.
__global__ void __launch_bounds__(kRareThreads) wordpiece_oov_long_kernel(VocabTable table, const uint4* abase, OovEntry* __restrict__ queue,
                                                                         const uint32_t* __restrict__ queue_size, uint32_t queue_cap,
                                                                         const uint32_t* __restrict__ longer, const uint32_t* __restrict__ longer_count,
                                                                         uint32_t* __restrict__ range_tokens)
{
  if (*queue_size > queue_cap) return;  // (see wordpiece_oov_kernel)
  uint32_t const n = *longer_count;
  for (uint32_t i = blockIdx.x * kRareThreads + threadIdx.x; i < n; i += gridDim.x * kRareThreads) {
    uint32_t const q   = longer[i];
    OovEntry const e   = queue[q];
    uint32_t const wl  = e.len_flags & 0xFFu;
    int64_t const at   = static_cast<int64_t>((static_cast<uint64_t>(e.coord[1]) << 32) | e.coord[0]);
    int32_t tok[kOovKeep];
    uint32_t const cnt = tokenize_oov_word(table, GlobalWord{reinterpret_cast<const uint8_t*>(abase) + at}, wl, [&](uint32_t j, int32_t id) {
#pragma unroll
      for (int k = 0; k < kOovKeep; ++k)
        if (j == static_cast<uint32_t>(k)) tok[k] = id;
    });
    uint4* const dst = reinterpret_cast<uint4*>(queue + q);
    if (cnt <= kOovKeep) {
      dst[0] = make_uint4(static_cast<uint32_t>(tok[0]), static_cast<uint32_t>(tok[1]), static_cast<uint32_t>(tok[2]), static_cast<uint32_t>(tok[3]));
      dst[1] = make_uint4(static_cast<uint32_t>(tok[4]), static_cast<uint32_t>(tok[5]), static_cast<uint32_t>(tok[6]), cnt);
    } else {
      dst[0] = make_uint4(0u, 0u, 0u, e.coord[1]);
      dst[1] = make_uint4(e.len_flags, e.range, e.coord[0], cnt);
    }
    atomicAdd(&range_tokens[e.range], cnt);
  }
}

// ------------------------------------------------------------------ emit pass
// A wavefront takes a range: walks its word slots 128 at a time, in order, two neighbouring words per lane; a word
// from the queue has its tokens (or their number) in its queue record; a wave scan of the lanes' token counts places
// the tokens, and every lane writes its own words'.  The rows that start in the range (the word pass left each the
// number of the range's words before it) are walked alongside: a row that begins at one of the 128 words gets that
// word's place as its list offset.
// Two things decide the pass' speed.  The counter a wavefront waits on counts reads and writes alike, out of order
// between the two, so every wait for a read is a wait for everything, and what a wavefront has in flight is what one
// round asks for: hence two words per lane (0.21 -> 0.16 ms on two million short rows of known words).  And a vector
// memory instruction takes the address unit about as long for a few lanes as for sixty-four: written word by word, the
// second to seventh tokens of the words that have them were an instruction each for a handful of lanes; put side by
// side in LDS first and written 64 at a time, the same tokens take a third of the instructions (0.69 -> 0.55 ms on
// 3.2 GB of text with one word in seven from the queue).
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__global__ void __launch_bounds__(kTokThreads, 8) wordpiece_emit_kernel(uint32_t nranges, const uint32_t* __restrict__ arena, uint32_t range_cap,
                                                                     const uint32_t* __restrict__ range_words, const int64_t* __restrict__ range_base,
                                                                     const uint32_t* __restrict__ range_first_row, OovEntry* __restrict__ queue,
                                                                     int32_t* __restrict__ offsets, int32_t* __restrict__ child,
                                                                     uint32_t* __restrict__ again, uint32_t* __restrict__ again_count)
{
  constexpr uint32_t kRound = 2 * kWave;
  constexpr uint32_t kStage = 768;  // tokens of a round that are put in order in LDS before they are written
  __shared__ uint32_t stage_all[kTokWaves][kStage];
  uint32_t* const stage     = stage_all[threadIdx.x / kWave];
  int const lane            = lane_id();
  uint32_t const my_number  = blockIdx.x * kTokWaves + threadIdx.x / kWave;
  // The ranges cost this pass about the same, so every wavefront takes every W-th one (W wavefronts in the grid):
  // faster here than taking them from a counter as they go, as the other two passes do (0.71 against 0.77 ms on
  // 3.2 GB of text, 0.21 against 0.26 ms on two million short rows).
  uint32_t const stride_units = gridDim.x * kTokWaves;
  for (uint32_t range = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(my_number))); range < nranges;
       range += stride_units) {
    // (a range's slots begin at an even index, and so does a lane's pair)
    const uint32_t* const slots = arena + static_cast<int64_t>(range) * range_cap;
    uint32_t const nwords       = range_words[range];
    int64_t const base          = range_base[range];
    int32_t* const dst0         = child + base;
    uint32_t r_win              = range_first_row[range];  // the 64 rows being placed: r_win + lane, the first row_used of them done
    uint32_t const r_end        = range_first_row[range + 1];
    uint32_t row_used           = 0;
    uint32_t done               = 0;  // tokens of the range so far
    // the words of the range before my row
    uint32_t row_k = r_win + lane < r_end ? static_cast<uint32_t>(offsets[r_win + lane]) : 0xFFFFFFFFu;
    // in flight: the slots two rounds ahead, the queue records of the next round's words from the queue, this round's writes
    auto load_slots = [&](uint32_t k) -> uint2 {  // slots k, k + 1 (k even; the second may lie past the range's words: not looked at then)
      if (k >= nwords) return make_uint2(0u, 0u);
      u32x2_t const v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(slots + k));
      return make_uint2(v.x, v.y);
    };
    auto from_queue = [&](uint32_t k, uint32_t v) { return k < nwords && (v & kOovMark) != 0 && v != 0xFFFFFFFFu; };
    auto load_record = [&](uint32_t k, uint32_t v, uint4& ra, uint4& rb) {
      if (from_queue(k, v)) {
        const uint4* const src = reinterpret_cast<const uint4*>(queue + (v & ~kOovMark));
        ra = src[0];
        rb = src[1];
      }
    };
    uint2 v_nxt = load_slots(2u * lane), v_far = load_slots(kRound + 2u * lane);
    uint4 a0_nxt = make_uint4(0u, 0u, 0u, 0u), b0_nxt = a0_nxt, a1_nxt = a0_nxt, b1_nxt = a0_nxt;
    load_record(2u * lane, v_nxt.x, a0_nxt, b0_nxt);
    load_record(2u * lane + 1u, v_nxt.y, a1_nxt, b1_nxt);
    for (uint32_t j0 = 0; j0 < nwords; j0 += kRound) {
      uint32_t const k  = j0 + 2u * lane;
      uint2 const v     = v_nxt;
      uint4 const ra0 = a0_nxt, rb0 = b0_nxt, ra1 = a1_nxt, rb1 = b1_nxt;
      v_nxt = v_far;
      load_record(k + kRound, v_nxt.x, a0_nxt, b0_nxt);
      load_record(k + kRound + 1u, v_nxt.y, a1_nxt, b1_nxt);
      v_far = load_slots(k + 2u * kRound);
      bool const act0 = k < nwords, act1 = k + 1u < nwords;
      bool const q0 = from_queue(k, v.x), q1 = from_queue(k + 1u, v.y);
      uint32_t const c0   = !act0 ? 0u : q0 ? rb0.w : 1u;
      uint32_t const c1   = !act1 ? 0u : q1 ? rb1.w : 1u;
      uint32_t const incl = wave_inclusive_scan(c0 + c1);
      uint32_t const ex   = incl - (c0 + c1);  // tokens of the round before my first word
      uint32_t const tot  = wave_bcast(incl, kWave - 1);
      int32_t* const dst  = dst0 + done + ex;
      if (ballot64(q0 || q1) == 0) {
        // no word of the round comes from the queue: a token each, the pair side by side
        if (act1) {
          uint32_t const w[2] = {v.x, v.y};
          __builtin_memcpy(dst, w, 8);  // (one 8-byte store; dst is 4-byte aligned)
        } else if (act0) {
          dst[0] = static_cast<int32_t>(v.x);
        }
      } else if (tot <= kStage) {
        // the tokens of the round side by side in LDS, then written 64 at a time
        auto stage_word = [&](bool active, bool queued, uint32_t slot, uint32_t cnt, uint4 const& ra, uint4 const& rb, uint32_t at) {
          if (queued && cnt > kOovKeep) {
            // more tokens than a record keeps (seldom): noted for wordpiece_retokenize_kernel, with the place of the
            // word's first token in the child left in its record (what is written there now is overwritten then)
            uint32_t const q                  = slot & ~kOovMark;
            again[atomicAdd(again_count, 1u)] = q;
            queue[q].head[0]                  = static_cast<uint32_t>(base + done + at);
          } else if (active) {
            stage[at] = queued ? ra.x : slot;
            if (ballot64(queued && cnt > 1u) != 0) {
              if (queued && cnt > 1u) stage[at + 1] = ra.y;
              if (queued && cnt > 2u) stage[at + 2] = ra.z;
              if (ballot64(queued && cnt > 3u) != 0) {
                if (queued && cnt > 3u) stage[at + 3] = ra.w;
                if (queued && cnt > 4u) stage[at + 4] = rb.x;
                if (queued && cnt > 5u) stage[at + 5] = rb.y;
                if (queued && cnt > 6u) stage[at + 6] = rb.z;
              }
            }
          }
        };
        wave_lds_sync();  // (the writes of the round before have read their tokens)
        stage_word(act0, q0, v.x, c0, ra0, rb0, ex);
        stage_word(act1, q1, v.y, c1, ra1, rb1, ex + c0);
        wave_lds_sync();
        int32_t* const out = dst0 + done;
        for (uint32_t i = lane; i < tot; i += kWave) out[i] = static_cast<int32_t>(stage[i]);
      } else {
        auto write_word = [&](bool active, bool queued, uint32_t slot, uint32_t cnt, uint4 const& ra, uint4 const& rb, int32_t* d) {
          if (queued && cnt > kOovKeep) {
            // more tokens than a record keeps (seldom): noted for wordpiece_retokenize_kernel, with the place of the
            // word's first token in the child left in its record
            uint32_t const q                  = slot & ~kOovMark;
            again[atomicAdd(again_count, 1u)] = q;
            queue[q].head[0]                  = static_cast<uint32_t>(d - child);
          } else if (active) {
            d[0] = static_cast<int32_t>(queued ? ra.x : slot);
            if (ballot64(queued && cnt > 1u) != 0) {
              if (queued && cnt > 1u) d[1] = static_cast<int32_t>(ra.y);
              if (queued && cnt > 2u) d[2] = static_cast<int32_t>(ra.z);
              if (ballot64(queued && cnt > 3u) != 0) {
                if (queued && cnt > 3u) d[3] = static_cast<int32_t>(ra.w);
                if (queued && cnt > 4u) d[4] = static_cast<int32_t>(rb.x);
                if (queued && cnt > 5u) d[5] = static_cast<int32_t>(rb.y);
                if (queued && cnt > 6u) d[6] = static_cast<int32_t>(rb.z);
              }
            }
          }
        };
        write_word(act0, q0, v.x, c0, ra0, rb0, dst);
        write_word(act1, q1, v.y, c1, ra1, rb1, dst + c0);
      }
      // rows that begin at one of these words (or, in the last round, after the last word: the positions past it
      // hold the round's total)
      uint32_t const places = ex | (c0 << 16);  // (a round has fewer than 2^16 tokens: 128 words of fewer than 200 each)
      for (;;) {
        bool const mine   = lane >= static_cast<int>(row_used) && row_k < j0 + kRound;  // (row_k >= j0: the rows are in order)
        uint32_t const at = row_k - j0;
        uint32_t const pl = static_cast<uint32_t>(__shfl(static_cast<int>(places), static_cast<int>((at >> 1) & 63u)));
        uint32_t const e  = (pl & 0xFFFFu) + ((at & 1u) != 0 ? pl >> 16 : 0u);
        if (mine) offsets[r_win + lane] = static_cast<int32_t>(base + done + e);
        row_used += static_cast<uint32_t>(__builtin_popcountll(ballot64(mine)));
        if (row_used < kWave) break;
        // all 64 are placed: the next 64
        r_win += kWave;
        row_used = 0;
        row_k    = r_win + lane < r_end ? static_cast<uint32_t>(offsets[r_win + lane]) : 0xFFFFFFFFu;
      }
      done += tot;
    }
    // the rows after the range's last word; after the last range's, the end of the last row
    for (; r_win < r_end; r_win += kWave, row_used = 0)
      if (lane >= static_cast<int>(row_used) && r_win + lane < r_end) offsets[r_win + lane] = static_cast<int32_t>(base + done);
    if (range + 1 == nranges && lane == 0) offsets[r_end] = static_cast<int32_t>(base + done);
  }
}

// The words that have more tokens than a queue record keeps (the emit pass has listed them in again[0 .. *again_count)
// and left the index of each one's first token in the child in its record, beside where and how long the word is):
// tokenized again, straight into place.  One lane per word; kept apart from the emit pass so that that is compiled for
// its common case.
__global__ void __launch_bounds__(kRareThreads) wordpiece_retokenize_kernel(VocabTable table, const uint4* abase, const OovEntry* __restrict__ queue,
                                                                           const uint32_t* __restrict__ again, const uint32_t* __restrict__ again_count,
                                                                           int32_t* __restrict__ child)
{
  uint32_t const n = *again_count;
  for (uint32_t i = blockIdx.x * kRareThreads + threadIdx.x; i < n; i += gridDim.x * kRareThreads) {
    OovEntry const e   = queue[again[i]];  // head[0] = place in the child, head[3] = coord[1], len_flags, range, coord[0] as they were; coord[1] = the count
    uint32_t const cnt = e.coord[1];
    int64_t const at   = static_cast<int64_t>((static_cast<uint64_t>(e.head[3]) << 32) | e.coord[0]);
    int32_t* const d   = child + e.head[0];
    tokenize_oov_word(table, GlobalWord{reinterpret_cast<const uint8_t*>(abase) + at}, e.len_flags & 0xFFu, [&](uint32_t j, int32_t id) {
      if (j < cnt) d[j] = id;
    });
  }
}

// ------------------------------------------------------------------ a sample of the column, for sizing
// How many words a byte of this column has, and how many of them will be queued, decides the sizes of the word slots
// and of the queue; text in another language than the vocabulary's, or of very short words, needs several times what
// ordinary text does, and finding that out by running out of room costs the word pass a second time.  So the call
// first looks at kSampleWindows windows of kSampleBytes spread evenly over the column's bytes, one wavefront each:
// words as maximal runs of bytes that are not spaces (rows and the word limit are left aside: an estimate), each
// looked up whole.  It runs on the offsets alone, before the host knows where the bytes begin, and leaves the view's
// first and last offset for the host as well: the call synchronises once for both.
constexpr int kSampleWindows = 512;
constexpr int kSampleBytes   = 512;
constexpr int kSampleTail    = 208;  // bytes staged past a window: a word that starts in it ends there, or is kMaxWord bytes or more
static_assert(3 * kSampleWindows <= kHostSampleWords, "a window's three counts fit the pinned words");

__global__ void __launch_bounds__(kWave) wordpiece_sample_kernel(ColView col, VocabTable table, uint64_t* __restrict__ first_last,
                                                               uint32_t* __restrict__ counts)
{
  __shared__ uint32_t staged[(kSampleBytes + kSampleTail + 8) / 4 + 4];  // byte 4 + x of it: byte x of the window; byte 3: the one before
  int const lane      = lane_id();
  int64_t const first = col.off(0), last = col.off(col.size);
  if (blockIdx.x == 0 && lane == 0) {
    first_last[0] = static_cast<uint64_t>(first);
    first_last[1] = static_cast<uint64_t>(last);
  }
  int64_t const span    = last - first;
  int64_t const windows = min(static_cast<int64_t>(kSampleWindows), (span + kSampleBytes - 1) / kSampleBytes);
  uint32_t words = 0, queued = 0, bytes = 0;
  if (static_cast<int64_t>(blockIdx.x) < windows) {
    int64_t const begin = first + span / windows * blockIdx.x;
    int64_t const end   = min(last, begin + kSampleBytes);
    bytes               = static_cast<uint32_t>(end - begin);
    uint8_t* const sb   = reinterpret_cast<uint8_t*>(staged);
    for (int i = lane; i < 4 + kSampleBytes + kSampleTail + 8; i += kWave) {
      int64_t const g = begin + i - 4;
      sb[i]           = (g >= first && g < last) ? col.chars[g] : uint8_t{0x20};  // outside the view: a space
    }
    wave_lds_sync();
    // a lane takes eight byte positions and the words that start there
    constexpr uint32_t kMine = kSampleBytes / kWave;
    for (uint32_t p = kMine * lane; p < kMine * lane + kMine && p < bytes; ++p) {
      if (sb[4 + p] == 0x20u || sb[3 + p] != 0x20u) continue;
      uint32_t len = 1;
      while (len < kMaxWord && sb[4 + p + len] != 0x20u) ++len;
      ++words;
      if (len >= kMaxWord) continue;  // one unknown token, never queued
      if (len > 16) {
        ++queued;
        continue;
      }
      // queued as the word pass queues: whatever the word's home bucket does not settle
      TileWord const tw{staged, 4u + p};
      uint32_t k[4];
      tw.head16(k);
      trim_key8(min(len, 8u), k[0], k[1]);
      trim_key8(len > 8 ? len - 8u : 0u, k[2], k[3]);
      Probe const pr = make_probe(table, 0u, tw, 0u, len, k[0], k[1]);
      uint4 const s0 = table.slots[2 * pr.bucket], s1 = table.slots[2 * pr.bucket + 1];
      int32_t id;
      uint32_t vd = verdict(pr, s0, s1, len, &id);
      if (vd == 2u && len > 8) vd = verdict_16(table, pr, s0, s1, k, &id);
      if (vd != 1u) ++queued;
    }
  }
  uint32_t const w = wave_bcast(wave_inclusive_scan(words), kWave - 1), q = wave_bcast(wave_inclusive_scan(queued), kWave - 1);
  if (lane == 0) {
    counts[3 * blockIdx.x]     = w;
    counts[3 * blockIdx.x + 1] = q;
    counts[3 * blockIdx.x + 2] = bytes;
  }
}

// What the host needs to know before the emit pass: the number of tokens, whether a range ran out of word slots, the
// queue entries reserved.
__global__ void publish_state_kernel(const uint64_t* __restrict__ total, const uint32_t* __restrict__ flags, uint64_t* __restrict__ dst)
{
  if (threadIdx.x == 0) dst[0] = *total;
  if (threadIdx.x == 1) dst[1] = flags[kFlagOverflow];
  if (threadIdx.x == 2) dst[2] = flags[kFlagQueueSize];
}

struct RangeTokensOf {
  const uint32_t* counts;
  __device__ uint64_t operator()(int64_t i) const { return counts[i]; }
};

// ------------------------------------------------------------------ vocabulary construction (device)
// The reference inserts the entries into its two maps on the device (cpp/src/text/wordpiece_tokenize.cu:213-282); so
// does this: a kernel that counts the keys and the bytes of the longer ones (the host sizes the tables from that, its
// one wait), a kernel that enters every key into the table, the length filter and the direct tables with atomics, a
// kernel that settles entries that occur twice (the first one wins, as when a host enters them in order), one that
// packs the length filter and looks up the unknown token.  An entry gives up to two keys: itself, and, when it begins
// with "##", what follows (cpp/src/text/wordpiece_tokenize.cu:184-192).
struct VocabKey {
  const uint8_t* bytes;
  uint32_t len;  // 0: no key
};
__device__ __forceinline__ VocabKey vocabulary_key(ColView const& v, int64_t entry, uint32_t kind)
{
  int64_t const b = v.off(entry), e = v.off(entry + 1);
  int64_t const n = e - b;
  VocabKey k{v.chars + b, 0u};
  // entries of kMaxWord bytes or more can never equal a tokenizable word or piece; empty ones are never looked up
  if (kind == 0) {
    if (n >= 1 && n < kMaxWord) k.len = static_cast<uint32_t>(n);
  } else if (n >= 3 && n - 2 < kMaxWord && v.chars[b] == '#' && v.chars[b + 1] == '#') {
    k.bytes += 2;
    k.len = static_cast<uint32_t>(n - 2);
  }
  return k;
}

struct VocabCounts {
  unsigned long long pool_bytes;  // keys of more than 8 bytes, each padded to whole 8-byte blocks
  uint32_t keys;
  uint32_t max_len[2];
  uint32_t pool_cursor;           // (build kernel) the next free byte of the pool
  int32_t unk_id;                 // (last kernel)
};

__global__ void vocabulary_measure_kernel(ColView v, VocabCounts* __restrict__ counts)
{
  int64_t const t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= 2 * static_cast<int64_t>(v.size)) return;
  uint32_t const kind = static_cast<uint32_t>(t & 1);
  VocabKey const k    = vocabulary_key(v, t >> 1, kind);
  if (k.len == 0) return;
  atomicAdd(&counts->keys, 1u);
  if (k.len > 8) atomicAdd(&counts->pool_bytes, static_cast<unsigned long long>((k.len + 7u) & ~7u));
  atomicMax(&counts->max_len[kind], k.len);
}

// A key's bytes [p, p + 8) as two dwords, zero padded past the key.
__device__ __forceinline__ void vocabulary_key8(VocabKey const& k, uint32_t p, uint32_t* lo, uint32_t* hi)
{
  uint32_t w[2] = {0u, 0u};
  for (uint32_t i = 0; i < 8 && p + i < k.len; ++i) w[i >> 2] |= static_cast<uint32_t>(k.bytes[p + i]) << (8 * (i & 3u));
  *lo = w[0];
  *hi = w[1];
}
__device__ __forceinline__ uint64_t vocabulary_hash(VocabKey const& k, uint32_t kind)
{
  uint32_t lo, hi;
  vocabulary_key8(k, 0, &lo, &hi);
  uint64_t h = key_hash_first(kind, lo, hi);
  for (uint32_t done = 8; done < k.len; done += 8) {
    vocabulary_key8(k, done, &lo, &hi);
    h = key_hash_next(h, lo, hi, done >> 3);
  }
  return h;
}

struct VocabBuild {
  uint32_t* slots;      // the table as dwords: slot s at [4 s, 4 s + 4)
  uint8_t* pool;
  uint32_t* lens32;     // the length filter, a 32-bit word per entry (packed afterwards)
  uint32_t* lens_final; // the filter as the lookups read it: the fourth-byte bits are set here, the packed lengths join them at the end
  uint32_t* short_ids;  // as VocabTable::short_ids, "no such key" = 0x80000000 (above every id)
  uint32_t* letters3;   // as VocabTable::letters3, two entries to a word
  uint32_t bucket_mask, bucket_bits, lens_mask;
};

// The table is filled in three steps so that, among the keys with one home bucket, the two that come first in the
// vocabulary get its two slots (vocabulary files list their most frequent entries first, and a word that is not in its
// home bucket costs the tokenizer a second look): every key bids for slot 0 of its home with an atomic minimum of its
// number (step 1); the winners write their slots, the others bid for slot 1 (step 2); those winners write theirs,
// and what is left, the keys that are carried past their home, takes the first slot from the next bucket on that nobody
// has won or taken (step 3, compare-and-swap).
constexpr uint32_t kNoBid = 0xFFFFFFFFu;

struct VocabKeyParts {
  VocabKey key;
  uint32_t k0, k1;   // key bytes [0, 8)
  HashParts hp;
  uint32_t w0;       // slot.x of the key
  uint32_t number;   // 2 * entry + key space: the order of the vocabulary
};
__device__ __forceinline__ bool vocabulary_key_parts(ColView const& v, VocabBuild const& t, VocabKeyParts* p)
{
  int64_t const th = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (th >= 2 * static_cast<int64_t>(v.size)) return false;
  uint32_t const kind = static_cast<uint32_t>(th & 1);
  p->number           = static_cast<uint32_t>(th);
  p->key              = vocabulary_key(v, th >> 1, kind);
  if (p->key.len == 0) return false;
  vocabulary_key8(p->key, 0, &p->k0, &p->k1);
  p->hp = hash_parts(vocabulary_hash(p->key, kind), t.bucket_bits);
  p->w0 = slot_word0(p->hp.tag, kind, p->key.len);
  return true;
}
// Writes the key into a slot that is its alone.  (Slot 0 of a bucket may be getting its flags at this moment: its first
// two words are or-ed in; the slots start as zeros.)
__device__ __forceinline__ void vocabulary_write_slot(VocabBuild const& t, VocabCounts* counts, VocabKeyParts const& p, uint32_t* slot, bool claimed)
{
  uint32_t pool_off = 0;
  if (p.key.len > 8) {
    pool_off = atomicAdd(&counts->pool_cursor, (p.key.len + 7u) & ~7u);
    for (uint32_t i = 0; i < p.key.len; ++i) t.pool[pool_off + i] = p.key.bytes[i];  // (the pool starts as zeros: the padding)
  }
  if (!claimed) atomicOr(slot, p.w0);
  atomicOr(slot + 1, p.number >> 1);
  slot[2] = p.key.len <= 8 ? p.k0 : pool_off;
  slot[3] = p.key.len <= 8 ? p.k1 : 0u;
}

// step 1; also the length filter and the direct tables
__global__ void vocabulary_bid_kernel(ColView v, VocabBuild t, uint32_t* __restrict__ bid0)
{
  VocabKeyParts p;
  if (!vocabulary_key_parts(v, t, &p)) return;
  uint32_t const kind = p.number & 1u, id = p.number >> 1, k0 = p.k0;
  VocabKey const& k = p.key;
  // the length filter over the first three bytes, and its exact twin for pieces of lower-case letters
  if (k.len >= 3) {
    uint32_t const entry = length_filter_index(kind, k0 & 0x00FFFFFFu) & t.lens_mask;
    atomicOr(&t.lens32[entry], 1u << length_filter_bit(k.len));
    if (k.len >= 4) atomicOr(&t.lens_final[entry], 0x10000u << ((k0 >> 24) & 15u));
    uint32_t const c0 = k0 & 0xFFu, c1 = (k0 >> 8) & 0xFFu, c2 = (k0 >> 16) & 0xFFu;
    auto letter = [](uint32_t c) { return c >= 'a' && c <= 'z'; };
    if (kind == 1 && letter(c0) && letter(c1) && letter(c2)) {
      uint32_t const at   = ((c0 - 'a') * 26u + (c1 - 'a')) * 26u + (c2 - 'a');
      uint32_t const bits = (k.len <= 9 ? 1u << (k.len - 3) : 0x80u) | (k.len >= 4 ? 0x100u << ((k0 >> 24) & 7u) : 0u);
      atomicOr(&t.letters3[at >> 1], bits << (16u * (at & 1u)));
    }
  }
  // the direct tables of the keys of one and two bytes: the first entry with a key wins
  if (k.len <= 2) {
    uint32_t const at = k.len == 2 ? kind * 65536u + (k0 & 0xFFFFu) : 2u * 65536u + kind * 256u + (k0 & 0xFFu);
    atomicMin(&t.short_ids[at], id);
  }
  atomicMin(&bid0[p.hp.bucket], p.number);
}

// step 2
__global__ void vocabulary_first_slot_kernel(ColView v, VocabBuild t, VocabCounts* __restrict__ counts, const uint32_t* __restrict__ bid0,
                                             uint32_t* __restrict__ bid1)
{
  VocabKeyParts p;
  if (!vocabulary_key_parts(v, t, &p)) return;
  if (bid0[p.hp.bucket] == p.number)
    vocabulary_write_slot(t, counts, p, t.slots + 8 * static_cast<size_t>(p.hp.bucket), false);
  else
    atomicMin(&bid1[p.hp.bucket], p.number);
}

// step 3
__global__ void vocabulary_other_slots_kernel(ColView v, VocabBuild t, VocabCounts* __restrict__ counts, const uint32_t* __restrict__ bid0,
                                              const uint32_t* __restrict__ bid1)
{
  VocabKeyParts p;
  if (!vocabulary_key_parts(v, t, &p)) return;
  uint32_t const home = p.hp.bucket;
  if (bid0[home] == p.number) return;
  if (bid1[home] == p.number) {
    vocabulary_write_slot(t, counts, p, t.slots + 8 * static_cast<size_t>(home) + 4, false);
    return;
  }
  // both slots of the home bucket went to keys that come earlier in the vocabulary: carried on
  for (uint32_t b = home;;) {
    atomicOr(t.slots + 8 * static_cast<size_t>(b) + 1, kSearchOn);  // the key is carried past this bucket
    atomicOr(t.slots + 8 * static_cast<size_t>(b), p.hp.fp);
    b = (b + 1) & t.bucket_mask;
    // a slot that some key has won is (or will be) full; the first of the others that is empty is taken
    uint32_t* const slot0 = t.slots + 8 * static_cast<size_t>(b);
    if (bid0[b] == kNoBid && atomicCAS(slot0, 0u, p.w0) == 0u) {
      vocabulary_write_slot(t, counts, p, slot0, true);
      return;
    }
    if (bid1[b] == kNoBid && atomicCAS(slot0 + 4, 0u, p.w0) == 0u) {
      vocabulary_write_slot(t, counts, p, slot0 + 4, true);
      return;
    }
  }
}

// Entries that occur twice: every one of them looks for the first slot on its way that holds its key and leaves the
// smaller id there (lookups stop at that slot; the other slots with the key are never reached).
__global__ void vocabulary_settle_kernel(ColView v, VocabBuild t)
{
  int64_t const th = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (th >= 2 * static_cast<int64_t>(v.size)) return;
  uint32_t const kind = static_cast<uint32_t>(th & 1);
  uint32_t const id   = static_cast<uint32_t>(th >> 1);
  VocabKey const k    = vocabulary_key(v, th >> 1, kind);
  if (k.len == 0) return;
  uint32_t k0, k1;
  vocabulary_key8(k, 0, &k0, &k1);
  HashParts const hp = hash_parts(vocabulary_hash(k, kind), t.bucket_bits);
  uint32_t const w0  = slot_word0(hp.tag, kind, k.len);
  for (uint32_t b = hp.bucket;; b = (b + 1) & t.bucket_mask) {
    for (uint32_t j = 0; j < 2; ++j) {
      uint32_t* const slot = t.slots + 4 * (2 * static_cast<size_t>(b) + j);
      uint32_t const x     = slot[0];
      if (x == 0) return;  // (cannot happen: the key is in the table)
      if ((x & ~kCarried) != w0) continue;
      bool same = slot[2] == k0 && slot[3] == k1;
      if (k.len > 8) {
        same = true;
        for (uint32_t i = 0; same && i < k.len; ++i) same = t.pool[slot[2] + i] == k.bytes[i];
      }
      if (!same) continue;
      for (uint32_t seen = slot[1];;) {
        uint32_t const want = (seen & kSearchOn) | min(seen & ~kSearchOn, id);
        uint32_t const was  = atomicCAS(slot + 1, seen, want);
        if (was == seen) break;
        seen = was;
      }
      return;
    }
  }
}

// The length filter in its stored form, "no such key" of the direct tables as the lookups expect it, and the id of
// the unknown token (cpp/src/text/wordpiece_tokenize.cu:199-209, 273-275: "[UNK]", else "[unk]", else -1).
__global__ void vocabulary_finish_kernel(VocabTable table, const uint32_t* __restrict__ lens32, uint32_t* __restrict__ lens_final, uint32_t lens_size,
                                         int32_t* __restrict__ short_ids, VocabCounts* __restrict__ counts)
{
  uint32_t const stride = gridDim.x * blockDim.x;
  uint32_t const t      = blockIdx.x * blockDim.x + threadIdx.x;
  for (uint32_t i = t; i < lens_size; i += stride) lens_final[i] |= packed_filter_word(lens32[i]);
  for (uint32_t i = t; i < kShortIds; i += stride)
    if (static_cast<uint32_t>(short_ids[i]) == 0x80000000u) short_ids[i] = kNone;  // (the same bits: kNone is INT32_MIN)
  if (t == 0) {
    int32_t unk = kNone;
    for (int which = 0; which < 2 && unk == kNone; ++which) {
      // "[UNK]" / "[unk]" as two dwords
      RegWord const w{{which == 0 ? 0x4B4E555Bu : 0x6B6E755Bu, 0x0000005Du, 0u, 0u}};
      unk = lookup(table, 0u, w, 0u, 5u, w.r[0], w.r[1]);
    }
    counts->unk_id = unk == kNone ? -1 : unk;
  }
}

}  // namespace
}  // namespace nvtext_amd

extern "C" {

nvtext_amd_status nvtext_amd_wordpiece_vocabulary_create(const nvtext_amd_strings_column* vocabulary, void* stream_, const nvtext_amd_allocator* mr,
                                                         nvtext_amd_wordpiece_vocabulary** out)
{
  using namespace nvtext_amd;
  EntryScope const entry("nvtext_amd_wordpiece_vocabulary_create");
  if (!vocabulary || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  // cpp/src/text/wordpiece_tokenize.cu:217-218
  if (vocabulary->size == 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary must not be empty");
  if (vocabulary->null_count > 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary must not have nulls");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Mr const temp_mr{mr, stream};
  int32_t const V = vocabulary->size;
  ColView const entries = make_view(*vocabulary);
  unsigned const key_grid = static_cast<unsigned>((2 * static_cast<int64_t>(V) + 255) / 256);

  // how many keys, how many bytes of keys that do not fit a slot: the host's one wait before the tables exist
  Temp counts_mem(temp_mr, sizeof(VocabCounts));
  if (!counts_mem.ok()) return fail(NVTEXT_AMD_ALLOC_FAILED, "vocabulary allocation failed");
  VocabCounts* const d_counts = counts_mem.as<VocabCounts>();
  launch_fill_u32(reinterpret_cast<uint32_t*>(d_counts), 0u, sizeof(VocabCounts) / sizeof(uint32_t), stream);
  hipLaunchKernelGGL(vocabulary_measure_kernel, dim3(key_grid), dim3(256), 0, stream, entries, d_counts);
  VocabCounts counts{};
  NVTEXT_HIP_TRY(hipGetLastError());
  NVTEXT_HIP_TRY(hipMemcpyAsync(&counts, d_counts, sizeof(counts), hipMemcpyDeviceToHost, stream));
  NVTEXT_HIP_TRY(hipStreamSynchronize(stream));
  if (counts.pool_bytes > 0xFFFFFFF0ull) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary too large");

  // both key spaces share one table (wordpiece_tokenize.cu:224-263 builds two maps of capacity 2x each)
  size_t const keys = counts.keys;
  size_t capacity   = 64;
  while (capacity < 2 * keys) capacity <<= 1;
  if (capacity > (size_t{1} << 31)) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary too large");
  uint32_t const mask = static_cast<uint32_t>(capacity / 2 - 1);  // buckets of two slots
  uint32_t bucket_bits = 0;
  while ((1u << bucket_bits) < capacity / 2) ++bucket_bits;
  size_t lens_size = 1024;
  while (lens_size < 4 * keys) lens_size <<= 1;

  auto* v = new nvtext_amd_wordpiece_vocabulary;
  v->entries    = V;
  v->slot_bytes = capacity * sizeof(uint4);
  v->pool_bytes = static_cast<size_t>(counts.pool_bytes) + 16;
  v->store.bind(mr, stream);
  v->d_slots   = v->store.allocate(v->slot_bytes);
  v->d_pool    = v->store.allocate(v->pool_bytes);
  v->d_lens    = v->store.allocate(lens_size * sizeof(uint32_t));
  v->d_short   = v->store.allocate(kShortIds * sizeof(int32_t));
  v->d_letters = v->store.allocate(kLetters3 * sizeof(uint16_t));
  Temp lens32(temp_mr, lens_size * sizeof(uint32_t));
  Temp bids(temp_mr, capacity * sizeof(uint32_t));  // per bucket: who gets slot 0, who gets slot 1
  if (!v->d_slots || !v->d_pool || !v->d_lens || !v->d_short || !v->d_letters || !lens32.ok() || !bids.ok()) {
    nvtext_amd_wordpiece_vocabulary_destroy(v);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "vocabulary allocation failed");
  }
  launch_fill_u32(static_cast<uint32_t*>(v->d_slots), 0u, static_cast<int64_t>(capacity) * 4, stream);
  launch_fill_u32(static_cast<uint32_t*>(v->d_pool), 0u, static_cast<int64_t>(v->pool_bytes / 4), stream);  // (the sizes are multiples of 8)
  launch_fill_u32(lens32.as<uint32_t>(), 0u, static_cast<int64_t>(lens_size), stream);
  launch_fill_u32(static_cast<uint32_t*>(v->d_lens), 0u, static_cast<int64_t>(lens_size), stream);
  launch_fill_u32(bids.as<uint32_t>(), kNoBid, static_cast<int64_t>(capacity), stream);
  launch_fill_u32(static_cast<uint32_t*>(v->d_short), 0x80000000u, kShortIds, stream);
  launch_fill_u32(static_cast<uint32_t*>(v->d_letters), 0u, kLetters3 / 2, stream);

  v->table.slots       = static_cast<const uint4*>(v->d_slots);
  v->table.pool        = static_cast<const uint8_t*>(v->d_pool);
  v->table.bucket_mask = mask;
  v->table.bucket_bits = bucket_bits;
  v->table.unk_id      = -1;
  v->table.max_len[0]  = counts.max_len[0];
  v->table.max_len[1]  = counts.max_len[1];
  v->table.lens        = static_cast<const uint32_t*>(v->d_lens);
  v->table.lens_mask   = static_cast<uint32_t>(lens_size - 1);
  v->table.short_ids   = static_cast<const int32_t*>(v->d_short);
  v->table.letters3    = static_cast<const uint16_t*>(v->d_letters);

  VocabBuild build{};
  build.slots       = static_cast<uint32_t*>(v->d_slots);
  build.pool        = static_cast<uint8_t*>(v->d_pool);
  build.lens32      = lens32.as<uint32_t>();
  build.lens_final  = static_cast<uint32_t*>(v->d_lens);
  build.short_ids   = static_cast<uint32_t*>(v->d_short);
  build.letters3    = static_cast<uint32_t*>(v->d_letters);
  build.bucket_mask = mask;
  build.bucket_bits = bucket_bits;
  build.lens_mask   = static_cast<uint32_t>(lens_size - 1);
  hipLaunchKernelGGL(vocabulary_bid_kernel, dim3(key_grid), dim3(256), 0, stream, entries, build, bids.as<uint32_t>());
  hipLaunchKernelGGL(vocabulary_first_slot_kernel, dim3(key_grid), dim3(256), 0, stream, entries, build, d_counts, bids.as<uint32_t>(),
                     bids.as<uint32_t>() + capacity / 2);
  hipLaunchKernelGGL(vocabulary_other_slots_kernel, dim3(key_grid), dim3(256), 0, stream, entries, build, d_counts, bids.as<uint32_t>(),
                     bids.as<uint32_t>() + capacity / 2);
  hipLaunchKernelGGL(vocabulary_settle_kernel, dim3(key_grid), dim3(256), 0, stream, entries, build);
  hipLaunchKernelGGL(vocabulary_finish_kernel, dim3(256), dim3(256), 0, stream, v->table, lens32.as<uint32_t>(), static_cast<uint32_t*>(v->d_lens),
                     static_cast<uint32_t>(lens_size), static_cast<int32_t*>(v->d_short), d_counts);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipMemcpyAsync(&counts, d_counts, sizeof(counts), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);  // (the id of the unknown token; the temporaries are still in use until here)
  if (e != hipSuccess) {
    nvtext_amd_wordpiece_vocabulary_destroy(v);
    return fail(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
  }
  v->table.unk_id = counts.unk_id;
  *out            = v;
  return NVTEXT_AMD_SUCCESS;
}

void nvtext_amd_wordpiece_vocabulary_destroy(nvtext_amd_wordpiece_vocabulary* v)
{
  delete v;  // the store hands the tables back
}

void nvtext_amd_profile_set_range_tiles(int32_t tiles)
{
  nvtext_amd::g_forced_range_tiles.store(tiles == 1 || tiles == 2 || tiles == 4 || tiles == 8 ? tiles : 0, std::memory_order_relaxed);
}

void nvtext_amd_profile_set_sizing_sample(int32_t on) { nvtext_amd::g_sizing_sample.store(on != 0 ? 1 : 0, std::memory_order_relaxed); }

int32_t nvtext_amd_wordpiece_vocabulary_unk_id(const nvtext_amd_wordpiece_vocabulary* v) { return v ? v->table.unk_id : -1; }

nvtext_amd_status nvtext_amd_wordpiece_tokenize(const nvtext_amd_strings_column* input, const nvtext_amd_wordpiece_vocabulary* vocabulary,
                                                int32_t max_words_per_row, void* stream_, const nvtext_amd_allocator* mr_,
                                                nvtext_amd_list_column* out)
{
  using namespace nvtext_amd;
  EntryScope const entry("nvtext_amd_wordpiece_tokenize");
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
  auto give_up = [&](nvtext_amd_status st, const char* what) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(st, what);
  };

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
    if (!out->offsets || !out->null_mask) return give_up(NVTEXT_AMD_ALLOC_FAILED, "allocation failed");
    launch_fill_u32(reinterpret_cast<uint32_t*>(out->offsets), 0u, rows + 1, stream);
    launch_fill_u32(out->null_mask, 0u, static_cast<int64_t>(out->null_mask_bytes / 4), stream);
    if (hipGetLastError() != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, "kernel launch failed");
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
    if (!out->null_mask) return give_up(NVTEXT_AMD_ALLOC_FAILED, "mask allocation failed");
    launch_copy_bitmask(out->null_mask, input->null_mask, input->offset, rows, stream);
  }

  ColView const v = make_view(*input);
  // first and last offset of the view (the reference reads the same two scalars, cpp/src/strings/utilities.cu:180-190):
  // the bytes between them are what is tokenized
  size_t const ow = input->offsets_is_int64 ? 8 : 4;
  int64_t first_offset = 0, last_offset = 0;
  uint64_t* const scalars = host_scalars();  // pinned words that kernels write for the host (nullptr: copy instead)
  bool const sampling     = g_sizing_sample.load(std::memory_order_relaxed) != 0;
  double sample_words = 0, sample_queued = 0, sample_bytes = 0;  // what the sample found (nothing without the pinned words)
  if (scalars) {
    uint32_t* const counts = reinterpret_cast<uint32_t*>(scalars + 8);
    if (sampling)
      hipLaunchKernelGGL(wordpiece_sample_kernel, dim3(kSampleWindows), dim3(kWave), 0, stream, v, vocabulary->table, scalars, counts);
    else
      launch_read_two_offsets(input->offsets, input->offsets_is_int64 != 0, input->offset, static_cast<int64_t>(input->offset) + rows, scalars, stream);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
    first_offset = static_cast<int64_t>(scalars[0]);
    last_offset  = static_cast<int64_t>(scalars[1]);
    for (int i = 0; sampling && i < kSampleWindows; ++i) {
      sample_words += counts[3 * i];
      sample_queued += counts[3 * i + 1];
      sample_bytes += counts[3 * i + 2];
    }
  } else {
    unsigned char buf[16] = {0};
    const uint8_t* d_off  = static_cast<const uint8_t*>(input->offsets) + static_cast<size_t>(input->offset) * ow;
    hipError_t e          = hipMemcpyAsync(buf, d_off, ow, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipMemcpyAsync(buf + 8, d_off + static_cast<size_t>(rows) * ow, ow, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
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
  if (last_offset < first_offset) return give_up(NVTEXT_AMD_INVALID_ARGUMENT, "offsets are not monotone");
  if (last_offset == first_offset) {  // rows without bytes: no tokens
    launch_fill_u32(reinterpret_cast<uint32_t*>(out->offsets), 0u, rows + 1, stream);
    if (hipGetLastError() != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, "kernel launch failed");
    return NVTEXT_AMD_SUCCESS;
  }

  constexpr int kTile         = 2048;
  const uint8_t* const first_byte = v.chars + first_offset;
  uint32_t const cbeg             = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(first_byte) & 15u);
  int64_t const cend              = cbeg + (last_offset - first_offset);
  int64_t const ntiles            = (cend + kTile - 1) / kTile;

  int device = 0, cus = 256;
  (void)hipGetDevice(&device);
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
  // persistent kernels: as many workgroups as can be resident at once
  // (asked of the runtime once per kernel and device: the answer does not change, and a call on a small column is
  // short enough for three such questions to show)
  auto resident = [&](const void* kernel, int threads, int which) -> int64_t {
    static std::atomic<int> known[16][6];
    int per_cu = device >= 0 && device < 16 ? known[device][which].load(std::memory_order_relaxed) : 0;
    if (per_cu == 0) {
      if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess || per_cu < 1) per_cu = 2;
      if (device >= 0 && device < 16) known[device][which].store(per_cu, std::memory_order_relaxed);
    }
    return static_cast<int64_t>(per_cu) * cus;
  };
  bool const is64  = input->offsets_is_int64 != 0;
  bool const limit = max_words_per_row > 0;
  void (*const word_kernel)(TileArgs) = is64 ? (limit ? wordpiece_word_kernel<kTile, true, true> : wordpiece_word_kernel<kTile, true, false>)
                                             : (limit ? wordpiece_word_kernel<kTile, false, true> : wordpiece_word_kernel<kTile, false, false>);
  int64_t const word_resident = resident(reinterpret_cast<const void*>(word_kernel), kTokThreads, (is64 ? 2 : 0) + (limit ? 1 : 0));
  // A range is what a wavefront works through by itself, one tile after the other: kRangeTiles tiles when that still
  // leaves every wavefront of the word pass eight ranges or more (the last ones then end close together), fewer in a
  // smaller column (2M rows of 120 bytes: 0.34 -> 0.30 ms for the word pass).
  int range_tiles = kRangeTiles;
  while (range_tiles > 1 && ntiles / range_tiles < 8 * word_resident * kTokWaves) range_tiles >>= 1;
  // (tests, which have no column of a gigabyte to give, set the size through nvtext_amd_profile_set_range_tiles)
  if (int const want = g_forced_range_tiles.load(std::memory_order_relaxed)) range_tiles = want;
  int64_t const kRange    = static_cast<int64_t>(kTile) * range_tiles;
  int64_t const nranges64 = (ntiles + range_tiles - 1) / range_tiles;
  if (nranges64 > 0x7FFFFFF0) return give_up(NVTEXT_AMD_LOGIC_ERROR, "words exceed internal limit");
  uint32_t const nranges = static_cast<uint32_t>(nranges64);
  unsigned const word_grid = static_cast<unsigned>(
    std::min<int64_t>((static_cast<int64_t>(nranges) + kTokWaves - 1) / kTokWaves, word_resident));
  unsigned const oov_grid  = static_cast<unsigned>(resident(reinterpret_cast<const void*>(wordpiece_oov_kernel), kOovThreads, 4));
  unsigned const emit_grid = static_cast<unsigned>(
    std::min<int64_t>((static_cast<int64_t>(nranges) + kTokWaves - 1) / kTokWaves, resident(reinterpret_cast<const void*>(wordpiece_emit_kernel), kTokThreads, 5)));

  TileArgs args{};
  args.col          = v;
  args.table        = vocabulary->table;
  args.abase        = reinterpret_cast<const uint4*>(first_byte - cbeg);
  args.first_offset = first_offset;
  args.cend         = cend;
  args.ntiles       = ntiles;
  args.cbeg         = cbeg;
  args.nranges      = nranges;
  args.range_tiles  = range_tiles;
  args.max_words    = max_words_per_row;

  // Word slots per range and queue entries.  A range of ordinary text has a word per five or six bytes, and about a
  // word in forty of a large column is not in the vocabulary; the first attempt has room for five words per sixteen
  // bytes and queues a word per 32 bytes.  A column with more (rows or words of a byte or two; text in another
  // language than the vocabulary's) makes the attempt fail, and the second has what the first found to be needed:
  // room for a word per byte, the exact number of queue entries.
  uint32_t range_cap      = static_cast<uint32_t>(kRange * 5 / 16);
  uint64_t queue_capacity = static_cast<uint64_t>((last_offset - first_offset) >> 5) + static_cast<uint64_t>(word_grid) * kTokWaves * kQueueChunk + 4096;
  if (sample_bytes > 0) {
    // what the sample calls for, with half as much again for the ranges that are denser than the column as a whole
    // (never less than the sizes above: a sample can miss; the second attempt remains)
    double const per_byte_words  = std::max(sample_words / sample_bytes, static_cast<double>(rows) / static_cast<double>(last_offset - first_offset));
    double const per_byte_queued = sample_queued / sample_bytes;
    range_cap = static_cast<uint32_t>(std::min<double>(static_cast<double>(kRange + 8), std::max<double>(range_cap, per_byte_words * 1.5 * static_cast<double>(kRange) + 256)));
    range_cap = (range_cap + 1u) & ~1u;  // (a range's slots begin at an even index)
    queue_capacity = std::max<uint64_t>(queue_capacity, static_cast<uint64_t>(per_byte_queued * 1.25 * static_cast<double>(last_offset - first_offset)) +
                                                          static_cast<uint64_t>(word_grid) * kTokWaves * kQueueChunk + 4096);
  }
  uint64_t total = 0;
  for (int attempt = 0;; ++attempt) {
    if (queue_capacity > 0x7FFFFFF0ull) queue_capacity = 0x7FFFFFF0ull;
    uint32_t const qcap        = static_cast<uint32_t>(queue_capacity);
    size_t const temp_bytes[9] = {static_cast<size_t>(nranges) * range_cap * sizeof(uint32_t),
                                  (static_cast<size_t>(nranges) + 1) * sizeof(uint32_t),
                                  static_cast<size_t>(nranges) * sizeof(uint32_t),
                                  static_cast<size_t>(nranges) * sizeof(uint32_t),
                                  (static_cast<size_t>(nranges) + 1) * sizeof(int64_t),
                                  scan_temp_bytes(nranges),
                                  kFlagWords * sizeof(uint32_t),
                                  static_cast<size_t>(qcap) * sizeof(OovEntry),
                                  static_cast<size_t>(qcap) * sizeof(uint32_t)};
    TempParts<9> const temps(mr, temp_bytes);
    if (!temps.ok()) return give_up(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    uint32_t* const arena     = temps.part<uint32_t>(0);
    uint32_t* const first_row = temps.part<uint32_t>(1);
    uint32_t* const words     = temps.part<uint32_t>(2);
    uint32_t* const tokens    = temps.part<uint32_t>(3);
    int64_t* const bases      = temps.part<int64_t>(4);
    uint64_t* const scan_tmp  = temps.part<uint64_t>(5);
    uint32_t* const flags     = temps.part<uint32_t>(6);
    OovEntry* const queue     = temps.part<OovEntry>(7);
    uint32_t* const longer    = temps.part<uint32_t>(8);  // queue indices of the words of more than 16 bytes
    args.range_cap       = range_cap;
    args.range_first_row = first_row;
    args.arena           = arena;
    args.range_words     = words;
    args.range_tokens    = tokens;
    args.offsets_out     = out->offsets;
    args.queue           = queue;
    args.queue_cap       = qcap;
    args.queue_size      = flags + kFlagQueueSize;
    args.counter         = flags + kFlagWordUnits;
    args.overflow        = flags + kFlagOverflow;
    hipLaunchKernelGGL(range_first_row_kernel, dim3((nranges + 1 + 255) / 256), dim3(256), 0, stream, v, first_offset, cbeg, kRange, nranges, first_row,
                       flags, word_grid * kTokWaves, oov_grid * kOovWaves);
    {
      ProfileScope ps("wordpiece_word_kernel", stream);
      hipLaunchKernelGGL(word_kernel, dim3(word_grid), dim3(kTokThreads), 0, stream, args);
    }
    {
      ProfileScope ps("wordpiece_oov_kernel", stream);
      hipLaunchKernelGGL(wordpiece_oov_kernel, dim3(oov_grid), dim3(kOovThreads), 0, stream, vocabulary->table, args.abase, queue, flags + kFlagQueueSize, qcap, tokens,
                         flags + kFlagOovUnits, longer, flags + kFlagLonger);
    }
    {
      ProfileScope ps("wordpiece_oov_long_kernel", stream);
      hipLaunchKernelGGL(wordpiece_oov_long_kernel, dim3(static_cast<unsigned>(cus)), dim3(kRareThreads), 0, stream, vocabulary->table, args.abase, queue,
                         flags + kFlagQueueSize, qcap, longer, flags + kFlagLonger, tokens);
    }
    // where the tokens of each range go; the total decides the child size
    // (cpp/include/cudf/detail/sizes_to_offsets_iterator.cuh:302-339)
    device_exclusive_scan(RangeTokensOf{tokens}, static_cast<int64_t>(nranges), bases, scan_tmp, stream);
    // the total (the last word of the scan's temporaries) and the first flag words: written to the pinned words by a
    // kernel of one wavefront, or, without those, fetched in one copy (the flags lie right behind the scan's temporaries)
    uint32_t state[3] = {0, 0, 0};
    if (scalars) {
      hipLaunchKernelGGL(publish_state_kernel, dim3(1), dim3(kWave), 0, stream, scan_tmp + scan_tiles(nranges), flags, scalars + 2);
      hipError_t e = hipGetLastError();
      if (e == hipSuccess) e = hipStreamSynchronize(stream);
      if (e != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
      total    = scalars[2];
      state[1] = static_cast<uint32_t>(scalars[3]);
      state[2] = static_cast<uint32_t>(scalars[4]);
    } else {
      const char* const from = reinterpret_cast<const char*>(scan_tmp + scan_tiles(nranges));
      size_t const span      = static_cast<size_t>(reinterpret_cast<const char*>(flags + 3) - from);
      alignas(8) char both[256 + 8 + sizeof(state)];
      if (span > sizeof(both)) return give_up(NVTEXT_AMD_LOGIC_ERROR, "unexpected layout of the temporaries");
      hipError_t e = hipMemcpyAsync(both, from, span, hipMemcpyDeviceToHost, stream);
      if (e == hipSuccess) e = hipStreamSynchronize(stream);
      if (e != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
      std::memcpy(&total, both, sizeof(total));
      std::memcpy(state, both + span - sizeof(state), sizeof(state));
    }
    bool const words_over = state[1] != 0, queue_over = state[2] > qcap;
    if (words_over || queue_over) {
      if (attempt > 0 || state[2] > 0x7FFFFFF0u) return give_up(NVTEXT_AMD_LOGIC_ERROR, "words exceed internal limit");
      if (words_over) range_cap = static_cast<uint32_t>(kRange + 8);
      // state[2] counts the chunks of kQueueChunk entries that the wavefronts reserved, the unused rest of each
      // wavefront's last chunk included; which ranges a wavefront gets differs from one attempt to the next, and with it
      // that rest: a chunk per wavefront on top of what this attempt reserved covers every assignment.
      queue_capacity = std::max<uint64_t>(queue_capacity, static_cast<uint64_t>(state[2]) + static_cast<uint64_t>(word_grid) * kTokWaves * kQueueChunk);
      continue;
    }
    if (total > static_cast<uint64_t>(std::numeric_limits<int32_t>::max())) return give_up(NVTEXT_AMD_OVERFLOW, "Size of output exceeds the column size limit");
    out->child_size  = static_cast<int64_t>(total);
    out->child_bytes = static_cast<size_t>(total) * sizeof(int32_t);
    if (total) {
      out->child = mr.allocate(out->child_bytes);
      if (!out->child) return give_up(NVTEXT_AMD_ALLOC_FAILED, "child allocation failed");
    }
    {
      ProfileScope ps("wordpiece_emit_kernel", stream);
      hipLaunchKernelGGL(wordpiece_emit_kernel, dim3(emit_grid), dim3(kTokThreads), 0, stream, nranges, arena, range_cap, words, bases, first_row, queue,
                         out->offsets, static_cast<int32_t*>(out->child), longer, flags + kFlagAgain);
      // (the list of longer words has served its purpose by now: its memory takes the list of words to do again, at most
      // one entry per queued word)
      hipLaunchKernelGGL(wordpiece_retokenize_kernel, dim3(static_cast<unsigned>(cus)), dim3(kRareThreads), 0, stream, vocabulary->table, args.abase, queue,
                         longer, flags + kFlagAgain, static_cast<int32_t*>(out->child));
    }
    break;
  }
  if (hipGetLastError() != hipSuccess) return give_up(NVTEXT_AMD_DEVICE_ERROR, "kernel launch failed");
  return NVTEXT_AMD_SUCCESS;
}

}  // extern "C"

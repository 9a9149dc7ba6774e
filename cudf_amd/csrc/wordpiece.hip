// wordpiece_vocabulary + wordpiece_tokenize for gfx950.
//
// The reference (cpp/src/text/wordpiece_tokenize.cu) keeps two cuco hash maps keyed by
// MurmurHash3 of the candidate substring and re-hashes every shrinking prefix (O(L^2) per
// out-of-vocabulary word, 349-407), marks word starts with a copy_if over all bytes, merges
// them with the row offsets and writes tokens into a 4-byte-per-input-byte temporary that is
// then counted and compacted (503-568, 462-491, 877-881).
//
// Here:
//   * one open-addressing table (16-byte slots, load <= 0.5, linear probing) holds both key
//     spaces: whole entries (kind 0) and "##" entries without their prefix (kind 1).  Keys of
//     up to 8 bytes sit inside the slot, so a hit costs one 16-byte load; the table for a
//     30k-entry vocabulary is 2 MiB and stays in L2.
//   * the key hash is polynomial (H <- H*B + byte mod 2^32), so dropping the last byte of a
//     candidate is one subtract and one multiply by B^-1: prefixes are never re-hashed.
//   * a wavefront owns a row: 256-byte chunks (+200-byte halo, the longest tokenizable word)
//     are staged in LDS with bytes outside the row replaced by spaces, word starts are found
//     with lanes <-> bytes and a DPP scan, then lanes <-> words tokenize in parallel.
//   * output is two-pass size-then-fill: pass 1 counts tokens per row, a device-wide scan
//     makes the int32 list offsets, pass 2 writes the tokens in place.  No chars-sized temporary.
#include "common.cuh"

#include <cstring>
#include <limits>
#include <string>
#include <vector>

namespace nvtext_amd {
namespace {

constexpr uint32_t kMaxWord  = 200;  // wordpiece_tokenize.cu:300: words this long become one [UNK]
constexpr uint32_t kHashB    = 0x01000193u;
constexpr uint32_t kSeedSub  = 0x9747b28cu;  // initial hash of the "##" key space

constexpr uint32_t inv_mod_2_32(uint32_t a)
{
  uint32_t x = a;  // Newton iteration: correct to 3 bits, doubles every step
  for (int i = 0; i < 5; ++i) x *= 2u - a * x;
  return x;
}
constexpr uint32_t kHashBInv = inv_mod_2_32(kHashB);
static_assert(kHashB * kHashBInv == 1u, "B^-1 mod 2^32");

__host__ __device__ __forceinline__ uint32_t mix32(uint32_t h)
{
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}

// slot.x = (tag23 << 9) | (kind << 8) | len   (0 = empty; len in 1..199)
// slot.y = token id
// slot.z, slot.w = the key itself when len <= 8 (zero padded), else (offset into the pool, 0)
struct VocabTable {
  const uint4* slots;
  const uint8_t* pool;
  uint32_t mask;  // capacity - 1
  int32_t unk_id;
};

__host__ __device__ __forceinline__ uint32_t slot_word0(uint32_t h, uint32_t kind, uint32_t len, uint32_t* start)
{
  uint32_t const x = mix32(h + len * 0x9E3779B9u);
  *start           = x;
  return (x & 0xFFFFFE00u) | (kind << 8) | len;
}

}  // namespace
}  // namespace nvtext_amd

struct nvtext_amd_wordpiece_vocabulary {
  nvtext_amd::VocabTable table{};
  void* d_slots     = nullptr;
  void* d_pool      = nullptr;
  size_t slot_bytes = 0;
  size_t pool_bytes = 0;
  int32_t entries   = 0;
};

namespace nvtext_amd {
namespace {

// ------------------------------------------------------------------ device-side lookup
// Bytes [0, 8) at byte offset `o` of the LDS dword array, zero padded past len.
__device__ __forceinline__ void inline_key(const uint32_t* w, uint32_t o, uint32_t len, uint32_t* k0, uint32_t* k1)
{
  uint32_t const i  = o >> 2;
  uint32_t const sh = (o & 3u) * 8u;
  uint32_t const d0 = w[i], d1 = w[i + 1], d2 = w[i + 2];
  uint32_t lo       = __builtin_amdgcn_alignbit(d1, d0, sh);
  uint32_t hi       = __builtin_amdgcn_alignbit(d2, d1, sh);
  if (len < 4) lo &= (1u << (8 * len)) - 1u;
  if (len <= 4) hi = 0;
  else if (len < 8) hi &= (1u << (8 * (len - 4))) - 1u;
  *k0 = lo;
  *k1 = hi;
}

// Returns the token id of key bytes [o, o+len) (LDS) in key space `kind`, or INT32_MIN if absent.
__device__ __forceinline__ int32_t lookup(VocabTable const& t, uint32_t kind, uint32_t h, const uint32_t* w, uint32_t o, uint32_t len)
{
  uint32_t idx;
  uint32_t const want = slot_word0(h, kind, len, &idx);
  uint32_t k0 = 0, k1 = 0;
  if (len <= 8) inline_key(w, o, len, &k0, &k1);
  const uint8_t* q = reinterpret_cast<const uint8_t*>(w) + o;
  for (;;) {
    idx &= t.mask;
    uint4 const s = t.slots[idx];
    if (s.x == 0) return std::numeric_limits<int32_t>::min();
    if (s.x == want) {
      if (len <= 8) {
        if (s.z == k0 && s.w == k1) return static_cast<int32_t>(s.y);
      } else {
        const uint8_t* e = t.pool + s.z;
        uint32_t i       = 0;
        while (i < len && e[i] == q[i]) ++i;
        if (i == len) return static_cast<int32_t>(s.y);
      }
    }
    ++idx;
  }
}

// cpp/src/text/wordpiece_tokenize.cu:307-317: length after dropping the last UTF-8 character.
__device__ __forceinline__ uint32_t remove_last_char(const uint8_t* p, uint32_t n)
{
  if (n < 2) return 0;
  uint32_t e = n - 1;
  while (e > 0 && is_utf8_continuation(p[e])) --e;
  return e;
}

// Collects the tokens of one word: the count, and the first kKeep ids in registers.
constexpr int kKeep = 4;
struct KeepTokens {
  int32_t tok[kKeep];
  uint32_t count = 0;
  __device__ __forceinline__ void emit(int32_t id)
  {
#pragma unroll
    for (int k = 0; k < kKeep; ++k)
      if (count == static_cast<uint32_t>(k)) tok[k] = id;
    ++count;
  }
  __device__ __forceinline__ void collapse(int32_t id)
  {
    tok[0] = id;
    count  = 1;
  }
};
// Writes the tokens of one word straight to their final place.
struct WriteTokens {
  int32_t* dst;
  uint32_t count = 0;
  __device__ __forceinline__ void emit(int32_t id) { dst[count++] = id; }
  __device__ __forceinline__ void collapse(int32_t id)
  {
    dst[0] = id;
    count  = 1;
  }
};

// Greedy longest-match-first tokenization of word bytes [o, o+len) of the LDS array `w`
// (cpp/src/text/wordpiece_tokenize.cu:349-407).  len in [1, 199].
template <typename Out>
__device__ __forceinline__ void wp_tokenize(VocabTable const& t, const uint32_t* w, uint32_t o, uint32_t len, Out& out)
{
  const uint8_t* p = reinterpret_cast<const uint8_t*>(w) + o;
  constexpr int32_t none = std::numeric_limits<int32_t>::min();
  // whole word, then ever shorter prefixes, in the full key space
  uint32_t h = 0;
  for (uint32_t i = 0; i < len; ++i) h = h * kHashB + p[i];
  int32_t id = lookup(t, 0, h, w, o, len);
  if (id != none) {
    out.emit(id);
    return;
  }
  uint32_t piece = len;
  for (;;) {
    uint32_t const shorter = remove_last_char(p, piece);
    if (shorter == 0) {  // nothing matched: one unknown token (375-379)
      out.emit(t.unk_id);
      return;
    }
    for (uint32_t i = piece; i > shorter; --i) h = (h - p[i - 1]) * kHashBInv;
    piece = shorter;
    id    = lookup(t, 0, h, w, o, piece);
    if (id != none) break;
  }
  out.emit(id);
  // the rest, piece by piece, in the "##" key space (381-395)
  uint32_t start = piece;
  while (start < len) {
    const uint8_t* r = p + start;
    uint32_t rl      = len - start;
    h                = kSeedSub;
    for (uint32_t i = 0; i < rl; ++i) h = h * kHashB + r[i];
    for (;;) {
      id = lookup(t, 1, h, w, o + start, rl);
      if (id != none) break;
      uint32_t const shorter = remove_last_char(r, rl);
      if (shorter == 0) {  // 396-404: the word collapses to a single unknown token
        out.collapse(t.unk_id);
        return;
      }
      for (uint32_t i = rl; i > shorter; --i) h = (h - r[i - 1]) * kHashBInv;
      rl = shorter;
    }
    out.emit(id);
    start += rl;
  }
}

// ------------------------------------------------------------------ row kernel
constexpr int kTokWaves   = 4;
constexpr int kTokThreads = kTokWaves * kWave;
constexpr int kChunk      = 256;                       // bytes per wavefront step (4 per lane)
constexpr int kChunkWords = (kChunk + kMaxWord + 12) / 4;  // + halo + over-read of inline_key

struct TokLds {
  uint32_t bytes[kChunkWords];
  uint16_t starts[kChunk / 2 + 2];
};

// One wavefront per row.  FILL == false: counts[r] = tokens of row r.
// FILL == true: writes the tokens at out_tokens + offsets[r].
template <bool FILL>
__global__ void __launch_bounds__(kTokThreads) wordpiece_rows_kernel(ColView col, VocabTable table, int32_t max_words, int32_t* __restrict__ counts,
                                                                     const int32_t* __restrict__ offsets, int32_t* __restrict__ out_tokens)
{
  __shared__ TokLds lds_all[kTokWaves];
  int const lane  = lane_id();
  int const wave  = threadIdx.x / kWave;
  int64_t const r = static_cast<int64_t>(blockIdx.x) * kTokWaves + wave;
  if (r >= col.size) return;
  TokLds& lds = lds_all[wave];

  int64_t const o = col.off(r);
  int64_t const n = col.off(r + 1) - o;
  // wordpiece_tokenize.cu:776-781: with a word limit, null rows have no words and the limit is
  // min(max_words, size_bytes / 2); without one, validity is not consulted (503-568).
  int64_t cap = std::numeric_limits<int64_t>::max();
  if (max_words > 0) cap = col.valid(r) ? min(static_cast<int64_t>(max_words), n / 2) : 0;

  const uint8_t* row   = col.chars + o;
  uint32_t const mis   = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row) & 3u);
  const uint32_t* arow = reinterpret_cast<const uint32_t*>(row - mis);
  int64_t const aend   = static_cast<int64_t>(mis) + n;  // row end in aligned coordinates
  int32_t* dst         = FILL ? out_tokens + offsets[r] : nullptr;

  int64_t words_done = 0;
  uint32_t tokens_done = 0;
  uint32_t prev_last = 0x20;  // byte before the chunk (a row starts as if after a space)
  for (int64_t cbase = 0; cbase < aend && words_done < cap; cbase += kChunk) {
    // stage aligned bytes [cbase, cbase + kChunk + kMaxWord) with everything outside the row as ' '
    uint32_t mine = 0x20202020u;
    for (int i = lane; i < (kChunk + static_cast<int>(kMaxWord) + 3) / 4; i += kWave) {
      int64_t const a0 = cbase + 4 * i;  // aligned coordinate of this dword's first byte
      uint32_t v       = 0x20202020u;
      if (a0 < aend && a0 + 4 > static_cast<int64_t>(mis)) {
        v = arow[a0 >> 2];
        if (a0 < static_cast<int64_t>(mis)) {  // bytes before the row
          uint32_t const k = static_cast<uint32_t>(mis - a0);
          uint32_t const m = (1u << (8 * k)) - 1u;
          v                = (v & ~m) | (0x20202020u & m);
        }
        if (a0 + 4 > aend) {  // bytes after the row
          uint32_t const k = static_cast<uint32_t>(aend - a0);
          uint32_t const m = (1u << (8 * k)) - 1u;
          v                = (v & m) | (0x20202020u & ~m);
        }
      }
      lds.bytes[i] = v;
      if (i == lane) mine = v;
    }
    // word starts among this lane's 4 bytes: a non-space byte after a space (wordpiece_tokenize.cu:519-522)
    uint32_t const up = static_cast<uint32_t>(__shfl_up(static_cast<int>(mine >> 24), 1));
    uint32_t before   = lane == 0 ? prev_last : up;
    uint32_t sbits    = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t const b = (mine >> (8 * j)) & 0xffu;
      if (b != 0x20u && before == 0x20u) sbits |= 1u << j;
      before = b;
    }
    prev_last            = wave_bcast(mine >> 24, kWave - 1);
    uint32_t const ns    = __builtin_popcount(sbits);
    uint32_t const incl  = wave_inclusive_scan(ns);
    uint32_t const total = wave_bcast(incl, kWave - 1);
    uint32_t slot        = incl - ns;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (sbits & (1u << j)) lds.starts[slot++] = static_cast<uint16_t>(4 * lane + j);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    int64_t const allowed = min(static_cast<int64_t>(total), cap - words_done);
    for (uint32_t w0 = 0; w0 < allowed; w0 += kWave) {
      uint32_t const wi = w0 + lane;
      bool const active = wi < allowed;
      KeepTokens kt;
      uint32_t wo = 0, wl = 0;
      if (active) {
        wo               = lds.starts[wi];
        const uint8_t* p = reinterpret_cast<const uint8_t*>(lds.bytes) + wo;
        while (wl < kMaxWord && p[wl] != 0x20u) ++wl;
        if (wl >= kMaxWord) {
          kt.emit(table.unk_id);  // wordpiece_tokenize.cu:442-445, 738-741
        } else {
          wp_tokenize(table, lds.bytes, wo, wl, kt);
        }
      }
      uint32_t const cnt  = active ? kt.count : 0;
      uint32_t const inc2 = wave_inclusive_scan(cnt);
      if (FILL && active) {
        int32_t* d = dst + tokens_done + (inc2 - cnt);
        if (cnt <= kKeep) {
#pragma unroll
          for (int k = 0; k < kKeep; ++k)
            if (static_cast<uint32_t>(k) < cnt) d[k] = kt.tok[k];
        } else {
          WriteTokens wt{d};
          wp_tokenize(table, lds.bytes, wo, wl, wt);
        }
      }
      tokens_done += wave_bcast(inc2, kWave - 1);
    }
    words_done += allowed;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  if (!FILL && lane == 0) counts[r] = static_cast<int32_t>(tokens_done);
}

struct CountOf {
  const int32_t* counts;
  __device__ uint64_t operator()(int64_t i) const { return static_cast<uint64_t>(counts[i]); }
};

// ------------------------------------------------------------------ vocabulary construction (host)
struct HostSlot {
  uint32_t x, y, z, w;
};

void host_insert(std::vector<HostSlot>& slots, uint32_t mask, const std::vector<uint8_t>& pool, uint32_t kind, const uint8_t* key, uint32_t len,
                 uint32_t pool_off, int32_t id)
{
  uint32_t h = kind ? kSeedSub : 0u;
  for (uint32_t i = 0; i < len; ++i) h = h * kHashB + key[i];
  uint32_t idx;
  uint32_t const w0 = slot_word0(h, kind, len, &idx);
  uint32_t k0 = 0, k1 = 0;
  if (len <= 8) {
    uint8_t buf[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    std::memcpy(buf, key, len);
    std::memcpy(&k0, buf, 4);
    std::memcpy(&k1, buf + 4, 4);
  }
  for (;;) {
    idx &= mask;
    HostSlot& s = slots[idx];
    if (s.x == 0) {
      s.x = w0;
      s.y = static_cast<uint32_t>(id);
      s.z = len <= 8 ? k0 : pool_off;
      s.w = len <= 8 ? k1 : 0u;
      return;
    }
    if (s.x == w0) {  // same key already present?  The first entry wins (duplicates are undefined in the reference).
      bool same = len <= 8 ? (s.z == k0 && s.w == k1) : (std::memcmp(pool.data() + s.z, key, len) == 0);
      if (same) return;
    }
    ++idx;
  }
}

int32_t host_find(const std::vector<HostSlot>& slots, uint32_t mask, const std::vector<uint8_t>& pool, const char* text)
{
  uint32_t const len = static_cast<uint32_t>(std::strlen(text));
  const uint8_t* key = reinterpret_cast<const uint8_t*>(text);
  uint32_t h         = 0;
  for (uint32_t i = 0; i < len; ++i) h = h * kHashB + key[i];
  uint32_t idx;
  uint32_t const w0 = slot_word0(h, 0, len, &idx);
  uint32_t k0 = 0, k1 = 0;
  uint8_t buf[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  std::memcpy(buf, key, len < 8 ? len : 8);
  std::memcpy(&k0, buf, 4);
  std::memcpy(&k1, buf + 4, 4);
  for (;;) {
    idx &= mask;
    HostSlot const& s = slots[idx];
    if (s.x == 0) return -1;
    if (s.x == w0 && (len <= 8 ? (s.z == k0 && s.w == k1) : std::memcmp(pool.data() + s.z, key, len) == 0)) return static_cast<int32_t>(s.y);
    ++idx;
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
  uint32_t const mask = static_cast<uint32_t>(capacity - 1);
  std::vector<HostSlot> slots(capacity, HostSlot{0, 0, 0, 0});
  for (int32_t i = 0; i < V; ++i) {
    int64_t const b = off_at(i) - first, e = off_at(i + 1) - first;
    int64_t const len = e - b;
    // entries of 200 bytes or more can never equal a tokenizable word or piece; empty ones are never looked up
    if (len >= 1 && len < kMaxWord) host_insert(slots, mask, pool, 0, pool.data() + b, static_cast<uint32_t>(len), static_cast<uint32_t>(b), i);
    // wordpiece_tokenize.cu:184-192: "##" entries also live, without the prefix, in the second key space
    if (len >= 3 && len - 2 < kMaxWord && pool[b] == '#' && pool[b + 1] == '#')
      host_insert(slots, mask, pool, 1, pool.data() + b + 2, static_cast<uint32_t>(len - 2), static_cast<uint32_t>(b + 2), i);
  }
  if (pool.size() > 0xFFFFFFFFull) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "vocabulary too large");

  auto* v = new nvtext_amd_wordpiece_vocabulary;
  v->entries = V;
  // wordpiece_tokenize.cu:199-209, 273-275
  int32_t unk = host_find(slots, mask, pool, "[UNK]");
  if (unk < 0) unk = host_find(slots, mask, pool, "[unk]");
  v->slot_bytes = capacity * sizeof(HostSlot);
  v->pool_bytes = pool.size() + 16;
  if (hipMalloc(&v->d_slots, v->slot_bytes) != hipSuccess || hipMalloc(&v->d_pool, v->pool_bytes) != hipSuccess) {
    nvtext_amd_wordpiece_vocabulary_destroy(v);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "vocabulary allocation failed");
  }
  hipError_t e1 = hipMemcpyAsync(v->d_slots, slots.data(), v->slot_bytes, hipMemcpyHostToDevice, stream);
  hipError_t e2 = pool.empty() ? hipSuccess : hipMemcpyAsync(v->d_pool, pool.data(), pool.size(), hipMemcpyHostToDevice, stream);
  hipError_t e3 = hipStreamSynchronize(stream);  // host vectors die at return
  if (e1 != hipSuccess || e2 != hipSuccess || e3 != hipSuccess) {
    nvtext_amd_wordpiece_vocabulary_destroy(v);
    return fail(NVTEXT_AMD_DEVICE_ERROR, "vocabulary upload failed");
  }
  v->table.slots  = static_cast<const uint4*>(v->d_slots);
  v->table.pool   = static_cast<const uint8_t*>(v->d_pool);
  v->table.mask   = mask;
  v->table.unk_id = unk;
  *out            = v;
  return NVTEXT_AMD_SUCCESS;
}

void nvtext_amd_wordpiece_vocabulary_destroy(nvtext_amd_wordpiece_vocabulary* v)
{
  if (!v) return;
  if (v->d_slots) (void)hipFree(v->d_slots);
  if (v->d_pool) (void)hipFree(v->d_pool);
  delete v;
}

int32_t nvtext_amd_wordpiece_vocabulary_unk_id(const nvtext_amd_wordpiece_vocabulary* v) { return v ? v->table.unk_id : -1; }

nvtext_amd_status nvtext_amd_wordpiece_tokenize(const nvtext_amd_strings_column* input, const nvtext_amd_wordpiece_vocabulary* vocabulary,
                                                int32_t max_words_per_row, void* stream_, const nvtext_amd_allocator* mr_,
                                                nvtext_amd_list_column* out)
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
  Temp counts(mr, static_cast<size_t>(rows) * sizeof(int32_t));
  Temp scan_tmp(mr, scan_temp_bytes(rows));
  if (!counts.ok() || !scan_tmp.ok()) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
  }
  unsigned const blocks = static_cast<unsigned>((static_cast<int64_t>(rows) + kTokWaves - 1) / kTokWaves);
  {
    ProfileScope ps("wordpiece_rows_kernel<count>", stream);
    hipLaunchKernelGGL(HIP_KERNEL_NAME(wordpiece_rows_kernel<false>), dim3(blocks), dim3(kTokThreads), 0, stream, v, vocabulary->table,
                       max_words_per_row, counts.as<int32_t>(), static_cast<const int32_t*>(nullptr), static_cast<int32_t*>(nullptr));
  }
  // int32 list offsets; the total decides the child size (cpp/include/cudf/detail/sizes_to_offsets_iterator.cuh:302-339)
  device_exclusive_scan(CountOf{counts.as<int32_t>()}, static_cast<int64_t>(rows), out->offsets, scan_tmp.as<uint64_t>(), stream);
  uint64_t total = 0;
  hipError_t e   = hipMemcpyAsync(&total, scan_tmp.as<uint64_t>() + scan_tiles(rows), sizeof(uint64_t), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  if (e != hipSuccess) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_DEVICE_ERROR, hipGetErrorString(e));
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
    ProfileScope ps("wordpiece_rows_kernel<fill>", stream);
    hipLaunchKernelGGL(HIP_KERNEL_NAME(wordpiece_rows_kernel<true>), dim3(blocks), dim3(kTokThreads), 0, stream, v, vocabulary->table,
                       max_words_per_row, static_cast<int32_t*>(nullptr), out->offsets, static_cast<int32_t*>(out->child));
  }
  NVTEXT_HIP_TRY(hipGetLastError());
  return NVTEXT_AMD_SUCCESS;
}

}  // extern "C"

// wordpiece_vocabulary + wordpiece_tokenize for gfx950.
//
// The reference (cpp/src/text/wordpiece_tokenize.cu) keeps two cuco hash maps keyed by
// MurmurHash3 of the candidate substring and re-hashes every shrinking prefix (O(L^2) per
// out-of-vocabulary word, 349-407), marks word starts with a copy_if over all bytes, merges
// them with the row offsets and writes tokens into a 4-byte-per-input-byte temporary that is
// then counted and compacted (503-568, 462-491, 877-881).
//
// Here:
//   * one open-addressing table of 2-slot buckets (16-byte slots, load <= 0.5) holds both key
//     spaces: whole entries (kind 0) and "##" entries without their prefix (kind 1).  Keys of
//     up to 8 bytes sit inside the slot, so a probe is one 32-byte read; the table for a
//     30k-entry vocabulary is 2 MiB and stays in L2.
//   * the key hash is polynomial (H <- H*B + byte mod 2^32).  A wavefront owns a row and walks
//     it in 256-byte chunks with lanes <-> bytes: a segmented DPP scan over (multiplier, value)
//     pairs gives the hash of every word prefix at once, so no lane ever loops over the bytes of
//     its word, and the hash of any inner piece is P[e] - P[p] * B^(e-p).
//   * words are handled in the chunk where they END; the previous chunk stays in a 512-byte LDS
//     ring so a word (< 200 bytes) is always whole.  Then lanes <-> words: one probe settles an
//     in-vocabulary word, the rest follow the greedy longest-match rule with O(1) hashes.
//     Tokens are written over the word's own prefix-hash slots (a word never has more tokens than
//     bytes) and copied out after a DPP scan of the per-word counts.
//   * pass 1 tokenizes every row once into an arena with floor(bytes/2)+1 slots per row and
//     records the counts; a device-wide scan makes the int32 list offsets; pass 2 copies the
//     arena rows into place (a row that overflowed its arena slots is tokenized again, directly).
#include "common.cuh"

#include <cstring>
#include <limits>
#include <string>
#include <vector>

namespace nvtext_amd {
namespace {

constexpr uint32_t kMaxWord = 200;  // wordpiece_tokenize.cu:300: words this long become one [UNK]
constexpr uint32_t kHashB   = 0x01000193u;

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
// Bucket b = slots[2b], slots[2b+1]; a bucket fills slot 0 first, overflow goes to the next bucket.
struct VocabTable {
  const uint4* slots;
  const uint8_t* pool;
  uint32_t bucket_mask;  // buckets - 1
  int32_t unk_id;
  uint32_t max_len[2];   // longest key of each key space (longer candidates cannot match)
};

__host__ __device__ __forceinline__ uint32_t slot_word0(uint32_t h, uint32_t kind, uint32_t len, uint32_t* bucket)
{
  uint32_t const x = mix32(h + len * 0x9E3779B9u + kind * 0x7F4A7C15u);
  *bucket          = x;
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

constexpr int kTokWaves   = 4;
constexpr int kTokThreads = kTokWaves * kWave;
constexpr int kChunk      = 256;  // bytes per wavefront step (4 per lane)
constexpr int kRing       = 512;  // two chunks: the current one and the one before it
constexpr int32_t kNone   = std::numeric_limits<int32_t>::min();

struct TokLds {
  uint32_t bytes[kRing / 4];       // row bytes (everything outside the row is ' ')
  uint32_t pt[kRing];              // prefix hash of each byte's word up to that byte; later the word's tokens
  uint16_t wend[kChunk / 2 + 2];   // ring index of the last byte of each word ending in the chunk
  uint16_t wlen[kChunk / 2 + 2];   // its length in bytes (clamped to kMaxWord)
};

// One word inside the ring: byte k of the word is ring byte (start + k) & 511.
struct Word {
  const TokLds* lds;
  uint32_t start;
  __device__ __forceinline__ uint32_t byte(uint32_t k) const { return reinterpret_cast<const uint8_t*>(lds->bytes)[(start + k) & (kRing - 1)]; }
  // hash of word bytes [0, k]
  __device__ __forceinline__ uint32_t prefix_hash(uint32_t k) const { return lds->pt[(start + k) & (kRing - 1)]; }
  // word bytes [p, p+8) as two dwords, zero padded past len
  __device__ __forceinline__ void key8(uint32_t p, uint32_t len, uint32_t* k0, uint32_t* k1) const
  {
    uint32_t const o  = (start + p) & (kRing - 1);
    uint32_t const i  = o >> 2;
    uint32_t const sh = (o & 3u) * 8u;
    uint32_t const d0 = lds->bytes[i], d1 = lds->bytes[(i + 1) & (kRing / 4 - 1)], d2 = lds->bytes[(i + 2) & (kRing / 4 - 1)];
    uint32_t lo       = __builtin_amdgcn_alignbit(d1, d0, sh);
    uint32_t hi       = __builtin_amdgcn_alignbit(d2, d1, sh);
    if (len < 4) lo &= (1u << (8 * len)) - 1u;
    if (len <= 4) hi = 0;
    else if (len < 8) hi &= (1u << (8 * (len - 4))) - 1u;
    *k0 = lo;
    *k1 = hi;
  }
};

__device__ __forceinline__ bool slot_matches(VocabTable const& t, uint4 const& s, uint32_t want, uint32_t len, uint32_t k0, uint32_t k1, Word const& w,
                                             uint32_t p)
{
  if (s.x != want) return false;
  if (len <= 8) return s.z == k0 && s.w == k1;
  const uint8_t* e = t.pool + s.z;
  uint32_t i       = 0;
  while (i < len && e[i] == w.byte(p + i)) ++i;
  return i == len;
}

// Token id of word bytes [p, p+len) in key space `kind` (hash h), or kNone.
__device__ __forceinline__ int32_t lookup(VocabTable const& t, uint32_t kind, uint32_t h, Word const& w, uint32_t p, uint32_t len)
{
  uint32_t b;
  uint32_t const want = slot_word0(h, kind, len, &b);
  uint32_t k0 = 0, k1 = 0;
  if (len <= 8) w.key8(p, len, &k0, &k1);
  for (;;) {
    b &= t.bucket_mask;
    uint4 const s0 = t.slots[2 * b];
    uint4 const s1 = t.slots[2 * b + 1];
    if (slot_matches(t, s0, want, len, k0, k1, w, p)) return static_cast<int32_t>(s0.y);
    if (s0.x == 0) return kNone;
    if (slot_matches(t, s1, want, len, k0, k1, w, p)) return static_cast<int32_t>(s1.y);
    if (s1.x == 0) return kNone;
    ++b;
  }
}

// cpp/src/text/wordpiece_tokenize.cu:307-317 on word bytes [p, e): the end after dropping the last
// UTF-8 character; returns p when nothing is left.
__device__ __forceinline__ uint32_t drop_last_char(Word const& w, uint32_t p, uint32_t e)
{
  if (e - p < 2) return p;
  uint32_t x = e - 1;
  while (x > p && is_utf8_continuation(w.byte(x))) --x;
  return x;
}

// Greedy longest-match-first tokenization of one word of `len` bytes (1..199)
// (cpp/src/text/wordpiece_tokenize.cu:349-407).  Tokens go to tok[(start + j) & 511]; returns the count.
// `pw[k]` = B^k.
__device__ __forceinline__ uint32_t wp_tokenize(VocabTable const& t, TokLds& lds, const uint32_t* pw, uint32_t start, uint32_t len)
{
  Word const w{&lds, start};
  uint32_t* const tok = lds.pt;
  auto put            = [&](uint32_t j, int32_t id) { tok[(start + j) & (kRing - 1)] = static_cast<uint32_t>(id); };
  // whole word, then ever shorter prefixes, in the full key space
  int32_t id = len <= t.max_len[0] ? lookup(t, 0, w.prefix_hash(len - 1), w, 0, len) : kNone;
  if (id != kNone) {
    put(0, id);
    return 1;
  }
  uint32_t e = len;
  for (;;) {
    e = drop_last_char(w, 0, e);
    if (e == 0) {  // nothing matched: one unknown token (375-379)
      put(0, t.unk_id);
      return 1;
    }
    if (e > t.max_len[0]) continue;
    id = lookup(t, 0, w.prefix_hash(e - 1), w, 0, e);
    if (id != kNone) break;
  }
  uint32_t hp = w.prefix_hash(e - 1);  // hash of bytes [0, p)
  put(0, id);
  uint32_t count = 1;
  uint32_t p     = e;
  // the rest, piece by piece, in the "##" key space (381-395)
  while (p < len) {
    e = len;
    for (;;) {
      uint32_t const pl = e - p;
      if (pl <= t.max_len[1]) {
        uint32_t const he = w.prefix_hash(e - 1);
        id                = lookup(t, 1, he - hp * pw[pl], w, p, pl);
        if (id != kNone) {
          hp = he;  // read before the token below may overwrite that slot
          break;
        }
      }
      e = drop_last_char(w, p, e);
      if (e == p) {  // 396-404: the word collapses to a single unknown token
        put(0, t.unk_id);
        return 1;
      }
    }
    put(count++, id);
    p = e;
  }
  return count;
}

template <int CTRL, int ROW_MASK, int OLD>
__device__ __forceinline__ uint32_t dpp_old(uint32_t v)
{
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(OLD, static_cast<int>(v), CTRL, ROW_MASK, 0xf, false));
}

// Inclusive scan across the wavefront of hash blocks (m, v) under (m1,v1).(m2,v2) = (m1*m2, v1*m2 + v2):
// appending block 2 to a prefix of hash v1 gives v1*m2 + v2.  Lanes without a source compose with (1, 0).
__device__ __forceinline__ void wave_scan_hash(uint32_t& m, uint32_t& v)
{
#define NVTEXT_HASH_STEP(CTRL, RM)                          \
  {                                                         \
    uint32_t const ms = dpp_old<CTRL, RM, 1>(m);            \
    uint32_t const vs = dpp_old<CTRL, RM, 0>(v);            \
    v                 = vs * m + v;                         \
    m                 = ms * m;                             \
  }
  NVTEXT_HASH_STEP(0x111, 0xf)
  NVTEXT_HASH_STEP(0x112, 0xf)
  NVTEXT_HASH_STEP(0x114, 0xf)
  NVTEXT_HASH_STEP(0x118, 0xf)
  NVTEXT_HASH_STEP(0x142, 0xa)
  NVTEXT_HASH_STEP(0x143, 0xc)
#undef NVTEXT_HASH_STEP
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

// value of the lane below (lane 0 gets `first`)
template <int FIRST>
__device__ __forceinline__ uint32_t from_lane_below(uint32_t v)
{
  return dpp_old<0x138, 0xf, FIRST>(v);  // wave_shr:1
}

// Tokenizes row r with one wavefront.  Tokens are delivered in order to dst[0 .. ) but only while
// the running index is below `slots`; returns the row's token count (which may exceed slots).
__device__ __forceinline__ uint32_t tokenize_row(ColView const& col, VocabTable const& table, int32_t max_words, int64_t r, TokLds& lds,
                                                 const uint32_t* pw, int32_t* dst, int64_t slots, int lane)
{
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

  // aligned dword at coordinate a0 with every byte outside the row replaced by ' '
  auto load_clean = [&](int64_t a0) -> uint32_t {
    uint32_t v = 0x20202020u;
    if (a0 < aend && a0 + 4 > static_cast<int64_t>(mis)) {
      v = arow[a0 >> 2];
      if (a0 < static_cast<int64_t>(mis)) {
        uint32_t const m = (1u << (8 * static_cast<uint32_t>(mis - a0))) - 1u;
        v                = (v & ~m) | (0x20202020u & m);
      }
      if (a0 + 4 > aend) {
        uint32_t const m = (1u << (8 * static_cast<uint32_t>(aend - a0))) - 1u;
        v                = (v & m) | (0x20202020u & ~m);
      }
    }
    return v;
  };

  int64_t words_done   = 0;
  uint32_t tokens_done = 0;
  uint32_t carry_hash  = 0;     // hash of the word running into the chunk (0 after a space)
  uint32_t carry_start = 0;     // 1 + aligned coordinate of the start of that word
  uint32_t prev_last   = 0x20;  // byte before the chunk
  for (int64_t cbase = 0; cbase < aend && words_done < cap; cbase += kChunk) {
    int64_t const a0    = cbase + 4 * lane;
    uint32_t const mine = load_clean(a0);
    uint32_t const ring0 = static_cast<uint32_t>(a0) & (kRing - 1);
    lds.bytes[ring0 >> 2] = mine;
    // neighbours: the byte before my four and the byte after them
    uint32_t before = from_lane_below<0>(mine >> 24);
    if (lane == 0) before = prev_last;
    uint32_t after = static_cast<uint32_t>(__shfl_down(static_cast<int>(mine & 0xffu), 1));
    if (lane == kWave - 1) after = load_clean(a0 + 4) & 0xffu;
    prev_last = wave_bcast(mine >> 24, kWave - 1);

    // per byte: hash block of my bytes so far, word starts and word ends
    uint32_t bm[4], bv[4];
    uint32_t m = 1, v = 0, smax = 0, ends = 0;
    uint32_t prevb = before;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t const b    = (mine >> (8 * j)) & 0xffu;
      uint32_t const next = j < 3 ? (mine >> (8 * (j + 1))) & 0xffu : after;
      bool const sp       = b == 0x20u;
      uint32_t const em   = sp ? 0u : kHashB;
      uint32_t const ev   = sp ? 0u : b;
      v                   = v * em + ev;
      m                   = m * em;
      bm[j]               = m;
      bv[j]               = v;
      if (!sp && prevb == 0x20u) smax = static_cast<uint32_t>(a0) + j + 1;  // word start (1-based coordinate)
      if (!sp && next == 0x20u) ends |= 1u << j;
      prevb = b;
    }
    // prefix over the lanes below (exclusive), seeded with the carry from the previous chunk
    uint32_t im = m, iv = v;
    wave_scan_hash(im, iv);
    uint32_t xm = from_lane_below<1>(im);
    uint32_t xv = from_lane_below<0>(iv);
    xv          = carry_hash * xm + xv;
    uint32_t const is   = wave_scan_max(smax);
    uint32_t xs         = max(from_lane_below<0>(is), carry_start);
    carry_hash          = carry_hash * wave_bcast(im, kWave - 1) + wave_bcast(iv, kWave - 1);
    carry_start         = max(carry_start, wave_bcast(is, kWave - 1));

    uint32_t const ne   = __builtin_popcount(ends);
    uint32_t const incl = wave_inclusive_scan(ne);
    uint32_t const total = wave_bcast(incl, kWave - 1);
    uint32_t slot        = incl - ne;
    uint32_t prevb2      = before;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t const b = (mine >> (8 * j)) & 0xffu;
      lds.pt[ring0 + j] = xv * bm[j] + bv[j];
      if (b != 0x20u && prevb2 == 0x20u) xs = static_cast<uint32_t>(a0) + j + 1;
      if (ends & (1u << j)) {
        uint32_t const wl = static_cast<uint32_t>(a0) + j + 1 - xs + 1;
        lds.wend[slot]    = static_cast<uint16_t>(ring0 + j);
        lds.wlen[slot]    = static_cast<uint16_t>(min(wl, kMaxWord));
        ++slot;
      }
      prevb2 = b;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    int64_t const allowed = min(static_cast<int64_t>(total), cap - words_done);
    for (uint32_t w0 = 0; w0 < allowed; w0 += kWave) {
      uint32_t const wi = w0 + lane;
      bool const active = wi < allowed;
      uint32_t cnt = 0, wstart = 0;
      if (active) {
        uint32_t const wl = lds.wlen[wi];
        wstart            = (static_cast<uint32_t>(lds.wend[wi]) + kRing + 1 - wl) & (kRing - 1);
        if (wl >= kMaxWord) {
          // wordpiece_tokenize.cu:442-445, 738-741.  The clamped length no longer locates the word start,
          // so the single token is parked on the word's last byte.
          wstart         = lds.wend[wi];
          lds.pt[wstart] = static_cast<uint32_t>(table.unk_id);
          cnt            = 1;
        } else {
          cnt = wp_tokenize(table, lds, pw, wstart, wl);
        }
      }
      uint32_t const inc2 = wave_inclusive_scan(cnt);
      if (active) {
        int64_t at = static_cast<int64_t>(tokens_done) + (inc2 - cnt);
        for (uint32_t k = 0; k < cnt; ++k, ++at)
          if (at < slots) dst[at] = static_cast<int32_t>(lds.pt[(wstart + k) & (kRing - 1)]);
      }
      tokens_done += wave_bcast(inc2, kWave - 1);
    }
    words_done += allowed;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  return tokens_done;
}

// Arena layout: row r owns the slots [arena_pos(r), arena_pos(r+1)), at least floor(bytes/2) + 1 of them.
__device__ __forceinline__ int64_t arena_pos(ColView const& col, int64_t first_offset, int64_t r) { return ((col.off(r) - first_offset) >> 1) + r; }

__device__ __forceinline__ void init_powers(uint32_t* pw)
{
  // pw[k] = B^k mod 2^32 for k < kMaxWord, by square-and-multiply
  for (uint32_t k = threadIdx.x; k < kMaxWord; k += blockDim.x) {
    uint32_t r = 1, b = kHashB;
    for (uint32_t e = k; e; e >>= 1) {
      if (e & 1u) r *= b;
      b *= b;
    }
    pw[k] = r;
  }
  __syncthreads();
}

// Pass 1: one wavefront per row tokenizes into the arena; counts[r] = tokens of row r.
__global__ void __launch_bounds__(kTokThreads) wordpiece_tokenize_kernel(ColView col, VocabTable table, int32_t max_words, int64_t first_offset,
                                                                         int32_t* __restrict__ arena, int32_t* __restrict__ counts)
{
  __shared__ TokLds lds_all[kTokWaves];
  __shared__ uint32_t pw[kMaxWord];
  init_powers(pw);
  int const lane  = lane_id();
  int const wave  = threadIdx.x / kWave;
  int64_t const r = static_cast<int64_t>(blockIdx.x) * kTokWaves + wave;
  if (r >= col.size) return;
  int64_t const ap    = arena_pos(col, first_offset, r);
  int64_t const slots = arena_pos(col, first_offset, r + 1) - ap;
  uint32_t const n    = tokenize_row(col, table, max_words, r, lds_all[wave], pw, arena + ap, slots, lane);
  if (lane == 0) counts[r] = static_cast<int32_t>(n);
}

// Pass 2: copy each row's tokens from the arena to out + offsets[r]; a row with more tokens than
// arena slots is tokenized again straight into place.
__global__ void __launch_bounds__(kTokThreads) wordpiece_gather_kernel(ColView col, VocabTable table, int32_t max_words, int64_t first_offset,
                                                                       const int32_t* __restrict__ arena, const int32_t* __restrict__ offsets,
                                                                       int32_t* __restrict__ out)
{
  __shared__ TokLds lds_all[kTokWaves];
  __shared__ uint32_t pw[kMaxWord];
  init_powers(pw);
  int const lane  = lane_id();
  int const wave  = threadIdx.x / kWave;
  int64_t const r = static_cast<int64_t>(blockIdx.x) * kTokWaves + wave;
  if (r >= col.size) return;
  int32_t const begin = offsets[r];
  int32_t const n     = offsets[r + 1] - begin;
  int64_t const ap    = arena_pos(col, first_offset, r);
  int64_t const slots = arena_pos(col, first_offset, r + 1) - ap;
  if (n <= slots) {
    for (int32_t k = lane; k < n; k += kWave) out[begin + k] = arena[ap + k];
  } else {
    tokenize_row(col, table, max_words, r, lds_all[wave], pw, out + begin, std::numeric_limits<int64_t>::max(), lane);
  }
}

struct CountOf {
  const int32_t* counts;
  __device__ uint64_t operator()(int64_t i) const { return static_cast<uint64_t>(counts[i]); }
};

// ------------------------------------------------------------------ vocabulary construction (host)
struct HostSlot {
  uint32_t x, y, z, w;
};

uint32_t host_hash(const uint8_t* key, uint32_t len)
{
  uint32_t h = 0;
  for (uint32_t i = 0; i < len; ++i) h = h * kHashB + key[i];
  return h;
}

void host_key8(const uint8_t* key, uint32_t len, uint32_t* k0, uint32_t* k1)
{
  uint8_t buf[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  std::memcpy(buf, key, len < 8 ? len : 8);
  std::memcpy(k0, buf, 4);
  std::memcpy(k1, buf + 4, 4);
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
      if (host_same(s, w0, pool, key, len, k0, k1)) return static_cast<int32_t>(s.y);
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
  for (int32_t i = 0; i < V; ++i) {
    int64_t const b = off_at(i) - first, e = off_at(i + 1) - first;
    int64_t const len = e - b;
    // entries of 200 bytes or more can never equal a tokenizable word or piece; empty ones are never looked up
    if (len >= 1 && len < kMaxWord) {
      host_insert(slots, mask, pool, 0, pool.data() + b, static_cast<uint32_t>(len), static_cast<uint32_t>(b), i);
      max_len[0] = std::max(max_len[0], static_cast<uint32_t>(len));
    }
    // wordpiece_tokenize.cu:184-192: "##" entries also live, without the prefix, in the second key space
    if (len >= 3 && len - 2 < kMaxWord && pool[b] == '#' && pool[b + 1] == '#') {
      host_insert(slots, mask, pool, 1, pool.data() + b + 2, static_cast<uint32_t>(len - 2), static_cast<uint32_t>(b + 2), i);
      max_len[1] = std::max(max_len[1], static_cast<uint32_t>(len - 2));
    }
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
  v->table.bucket_mask = mask;
  v->table.unk_id      = unk;
  v->table.max_len[0]  = max_len[0];
  v->table.max_len[1]  = max_len[1];
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
  // first and last offset of the view (the reference reads the same two scalars,
  // cpp/src/strings/utilities.cu:180-190); they size the token arena
  size_t const ow = input->offsets_is_int64 ? 8 : 4;
  int64_t first_offset = 0, last_offset = 0;
  {
    unsigned char buf[16] = {0};
    const uint8_t* d_off  = static_cast<const uint8_t*>(input->offsets) + static_cast<size_t>(input->offset) * ow;
    hipError_t e          = hipMemcpyAsync(buf, d_off, ow, hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipMemcpyAsync(buf + 8, d_off + static_cast<size_t>(rows) * ow, ow, hipMemcpyDeviceToHost, stream);
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
  size_t const arena_slots = static_cast<size_t>((last_offset - first_offset) >> 1) + static_cast<size_t>(rows) + 1;
  Temp arena(mr, arena_slots * sizeof(int32_t));
  Temp counts(mr, static_cast<size_t>(rows) * sizeof(int32_t));
  Temp scan_tmp(mr, scan_temp_bytes(rows));
  if (!arena.ok() || !counts.ok() || !scan_tmp.ok()) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
  }
  unsigned const blocks = static_cast<unsigned>((static_cast<int64_t>(rows) + kTokWaves - 1) / kTokWaves);
  {
    ProfileScope ps("wordpiece_tokenize_kernel", stream);
    hipLaunchKernelGGL(wordpiece_tokenize_kernel, dim3(blocks), dim3(kTokThreads), 0, stream, v, vocabulary->table, max_words_per_row,
                       first_offset, arena.as<int32_t>(), counts.as<int32_t>());
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
    ProfileScope ps("wordpiece_gather_kernel", stream);
    hipLaunchKernelGGL(wordpiece_gather_kernel, dim3(blocks), dim3(kTokThreads), 0, stream, v, vocabulary->table, max_words_per_row, first_offset,
                       arena.as<int32_t>(), out->offsets, static_cast<int32_t*>(out->child));
  }
  NVTEXT_HIP_TRY(hipGetLastError());
  return NVTEXT_AMD_SUCCESS;
}

}  // extern "C"

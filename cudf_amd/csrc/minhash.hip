// minhash / minhash64 for gfx950.
//
// Replaces the reference's three-kernel pipeline (cpp/src/text/minhash.cu:87-157 seed
// hashes into a chars-sized temporary, 281-376 permutation kernel re-reading it,
// 390-424 size partitioning) with one fused pass and no chars-sized temporary:
//
//   * a wavefront owns a section of a row.  Per 256-position tile it stages the bytes
//     in LDS (coalesced aligned dword loads), hashes the windows with lanes <-> window
//     starts, and compacts the hashes into LDS;
//   * it then switches to lanes <-> parameters: every lane keeps K (a, b) pairs and
//     K running minima in registers and streams the tile's hashes through LDS
//     broadcast reads, so the inner loop is v_mad_u64_u32 + v_min only;
//   * a workgroup takes four rows: a row of up to 1 KiB belongs to one wavefront alone; the 4
//     wavefronts split the first 16 KiB of a longer row and combine in LDS (plain store); the
//     rest of a still longer row is covered by extra workgroups that merge with atomic min, so
//     no output pre-initialisation is needed;
//   * in a tile with characters of more than one byte the wavefront lists the characters first,
//     so that a lane takes a character and reads its window's length instead of walking to it;
//     hashes that the wavefront has folded lately are dropped (a minimum does not mind).
//
// Null rows get no output slot (the reference drops them with purge_nonempty_nulls,
// minhash.cu:626-628), empty rows are all zeros (minhash.cu:318).
#include "common.cuh"
#include "murmur.cuh"
#include "windows.cuh"

#include <limits>
#include <mutex>
#include <type_traits>

// Scratch of nvtext_amd_minhash_preallocated, the entry point that allocates nothing: the extra-span counts of the
// rows (rows + 1 values) and behind them the tile sums of the scans.  Every device holds its own copy of the array
// for as long as the library is loaded (4.2 MB).
constexpr int32_t kPreallocatedMaxRows = NVTEXT_AMD_MINHASH_PREALLOCATED_MAX_ROWS;
constexpr size_t kScratchPrefixBytes   = (static_cast<size_t>(kPreallocatedMaxRows) + 1 + 63) / 64 * 64 * sizeof(uint32_t);
constexpr size_t kScratchScanBytes     = (static_cast<size_t>(kPreallocatedMaxRows) / nvtext_amd::kScanTile + 2) * sizeof(uint64_t);
static __device__ __align__(256) unsigned char scratch[kScratchPrefixBytes + kScratchScanBytes];

namespace nvtext_amd {
namespace {

template <typename T>
struct HashTraits;
template <>
struct HashTraits<uint32_t> {
  template <typename Src>
  static __device__ __forceinline__ uint32_t hash(Src const& src, uint32_t len, uint32_t seed)
  {
    return murmur3_x86_32(src, len, seed);
  }
  // Permutation (minhash.cu:350-351) in uint32 arithmetic: the product and sum wrap mod 2^32, after
  // which "% (2^61-1)" and "& max" change nothing: (hv * a + b), see Fold<uint32_t>.
};
template <>
struct HashTraits<uint64_t> {
  template <typename Src>
  static __device__ __forceinline__ uint64_t hash(Src const& src, uint32_t len, uint64_t seed)
  {
    return murmur3_x64_128_lo(src, len, seed);  // minhash.cu:138: first word of the 128-bit hash
  }
  // Permutation (minhash.cu:350-351): ((hv*a + b) mod 2^64) % (2^61-1), see Fold<uint64_t>.
};

// ((h * a + b) mod 2^64) folded once mod 2^61 - 1, that is (x & p) + (x >> 61) for the 64-bit x: at most p + 7; for two
// hashes and one (a, b).  x = h.lo * a.lo + b is one 64-bit multiply-add; the two cross products, of which only the low
// dwords count, are two more, chained (h.lo * a.hi, then h.hi * a.lo added to it), and their sum goes to the high dword
// of x with a plain 32-bit add, which issues in half the cycles of a multiply or of a three-operand add (left to itself
// the compiler makes them two multiplies and a three-operand add).  The fold is a shift and a mask of that dword and
// one more multiply-add (q * 1 + x) for the carry.  Eight instructions per hash, none that only moves a value.  The
// chained pairs of the two hashes stand interleaved in one block of assembly, so that neither waits for its own first
// half; everything else is left to the compiler, which puts an idle cycle between instructions it cannot see into.
__device__ __forceinline__ void permute_fold_u64_pair(uint64_t h0, uint64_t h1, uint64_t a, uint64_t b, uint32_t one, uint64_t* y0,
                                                      uint64_t* y1)
{
  uint32_t const al = static_cast<uint32_t>(a), ah = static_cast<uint32_t>(a >> 32);
  uint32_t const l0 = static_cast<uint32_t>(h0), u0 = static_cast<uint32_t>(h0 >> 32);
  uint32_t const l1 = static_cast<uint32_t>(h1), u1 = static_cast<uint32_t>(h1 >> 32);
  uint64_t c0, c1;
  asm("v_mad_u64_u32 %0, vcc, %2, %6, 0\n\t"
      "v_mad_u64_u32 %1, vcc, %4, %6, 0\n\t"
      "v_mad_u64_u32 %0, vcc, %3, %7, %0\n\t"
      "v_mad_u64_u32 %1, vcc, %5, %7, %1"
      : "=&v"(c0), "=&v"(c1)
      : "v"(l0), "v"(u0), "v"(l1), "v"(u1), "v"(ah), "v"(al)
      : "vcc");
  uint64_t const x0 = static_cast<uint64_t>(l0) * al + b;
  uint64_t const x1 = static_cast<uint64_t>(l1) * al + b;
  uint32_t xh0      = static_cast<uint32_t>(x0 >> 32) + static_cast<uint32_t>(c0);
  uint32_t xh1      = static_cast<uint32_t>(x1 >> 32) + static_cast<uint32_t>(c1);
  uint32_t const q0 = xh0 >> 29, q1 = xh1 >> 29;
  xh0 &= 0x1FFFFFFFu;
  xh1 &= 0x1FFFFFFFu;
  *y0 = static_cast<uint64_t>(q0) * one + ((static_cast<uint64_t>(xh0) << 32) | static_cast<uint32_t>(x0));
  *y1 = static_cast<uint64_t>(q1) * one + ((static_cast<uint64_t>(xh1) << 32) | static_cast<uint32_t>(x1));
}

// min of two values below 2^62 in one instruction: such bit patterns are non-negative finite doubles
// (or denormals, which this code object keeps: float_denorm_mode_16_64 = 3), and those order like the
// integers.  An operand that is all ones (the "no hash yet" start value, a NaN pattern) loses to the other.
__device__ __forceinline__ uint64_t min_below_2_62(uint64_t m, uint64_t y)
{
  uint64_t r;
  asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(m), "v"(y));
  return r;
}

// Folds the compacted hashes first, first + 1, .. of every `stride` (the count padded to a multiple of the stride)
// into m[K]; lanes <-> parameters.  A wavefront whose lanes all hold different parameters folds every hash
// (first 0, stride = the hashes of one trip); with few parameters the lanes form groups that hold the same
// parameters and fold every other trip each (see Packing).
template <typename T, int K>
struct Fold;

// How the lanes of a wavefront share the work when there are at most 32 parameters: `groups` sets of `ppad` lanes
// (both powers of two, groups <= 16), lane l holding parameter l % ppad and folding the trips l / ppad,
// l / ppad + groups, ...  The sets are combined with a butterfly of minima before the results leave the registers.
struct Packing {
  int32_t ppad;    // lanes per set; 64 when every lane has its own parameter
  int32_t groups;  // sets per wavefront
  __device__ __forceinline__ int param_lane(int lane) const { return lane & (ppad - 1); }
  __device__ __forceinline__ uint32_t first(int lane, uint32_t per_trip) const { return static_cast<uint32_t>(lane / ppad) * per_trip; }
  __device__ __forceinline__ uint32_t stride(uint32_t per_trip) const { return static_cast<uint32_t>(groups) * per_trip; }
  template <typename T>
  __device__ __forceinline__ T combine(T m) const
  {
    for (int d = ppad; d < kWave; d <<= 1) {
      T const other = __shfl_xor(m, d);
      m             = min(m, other);
    }
    return m;
  }
};

__host__ __device__ inline Packing packing_for(int32_t P)
{
  if (P > 32) return Packing{kWave, 1};
  int32_t ppad = 4;  // at most 16 sets, so that the padding of a tile's hashes fits one wavefront-wide store
  while (ppad < P) ppad <<= 1;
  return Packing{ppad, kWave / ppad};
}

template <int K>
struct Fold<uint32_t, K> {
  static constexpr uint32_t kPerTrip = 4;
  static __device__ __forceinline__ void run(const uint32_t* hashes, uint32_t padded, uint32_t first, uint32_t stride,
                                             const uint32_t (&a)[K], const uint32_t (&b)[K], uint32_t (&m)[K])
  {
    for (uint32_t i = first; i < padded; i += stride) {
      uint32_t const h0 = hashes[i], h1 = hashes[i + 1], h2 = hashes[i + 2], h3 = hashes[i + 3];
#pragma unroll
      for (int k = 0; k < K; ++k) {
        // one v_mad_u64_u32 per product, one v_min3_u32 per two products
        uint32_t const r0 = h0 * a[k] + b[k];
        uint32_t const r1 = h1 * a[k] + b[k];
        uint32_t const r2 = h2 * a[k] + b[k];
        uint32_t const r3 = h3 * a[k] + b[k];
        m[k]              = min(min(m[k], r0), r1);
        m[k]              = min(min(m[k], r2), r3);
      }
    }
  }
};

template <int K>
struct Fold<uint64_t, K> {
  static constexpr uint64_t p = (1ull << 61) - 1;
  // x mod p for x < 2^64: x = q*2^61 + r with q <= 7, so y = r + q <= p + 7.
  static __device__ __forceinline__ uint64_t fold_once(uint64_t x) { return (x & p) + (x >> 61); }

  // hashes per trip: four (with two, and two and more sets of parameters, the loop issued 3 to 5 % less: fewer
  // independent products between a trip's LDS read and its dependent minima)
  static constexpr uint32_t kPerTrip = 4;
  static __device__ __forceinline__ void run(const uint64_t* hashes, uint32_t padded, uint32_t first, uint32_t stride,
                                             const uint64_t (&a)[K], const uint64_t (&b)[K], uint64_t (&m)[K])
  {
    // Fast pass: the final "subtract p if y >= p" is left out.  y >= p needs the top dword of y to be
    // at least 0x1FFFFFFF (one chance in 2^29 per product), which is tracked with a running maximum;
    // if it ever happens the tile is folded again exactly.  Unreduced values are >= p, above every
    // reduced value, so they can never displace a correct minimum.
    uint32_t top = 0;
    uint32_t one;  // the number 1 where the compiler does not see it: q * one + x stays one multiply-add
    asm("s_mov_b32 %0, 1" : "=s"(one));
    for (uint32_t i = first; i < padded; i += stride) {
      uint64_t h[kPerTrip];
#pragma unroll
      for (uint32_t j = 0; j < kPerTrip; ++j) h[j] = hashes[i + j];
#pragma unroll
      for (int k = 0; k < K; ++k) {
#pragma unroll
        for (uint32_t j = 0; j < kPerTrip; j += 2) {
          uint64_t y0, y1;
          permute_fold_u64_pair(h[j], h[j + 1], a[k], b[k], one, &y0, &y1);
          top               = max(max(top, static_cast<uint32_t>(y0 >> 32)), static_cast<uint32_t>(y1 >> 32));
          m[k]              = min_below_2_62(min_below_2_62(m[k], y0), y1);
        }
      }
    }
    if (ballot64(top >= 0x1FFFFFFFu) != 0) {
      // every lane folds every hash here: a minimum does not mind the hashes of the other sets
      for (uint32_t i = 0; i < padded; ++i) {
        uint64_t const h = hashes[i];
#pragma unroll
        for (int k = 0; k < K; ++k) {
          uint64_t const y = fold_once(h * a[k] + b[k]);
          m[k]             = min(m[k], y >= p ? y - p : y);
        }
      }
    }
  }
};

// The parameters beyond the last full set of 64, when there are at most 32 of them: one more (a, b) pair per lane,
// shared out over sets of lanes as Packing describes, so that they cost the fold a share of a full set (4 parameters
// beyond 256: a sixteenth) instead of a whole one.
template <typename T>
struct TailParams {
  T a[1], b[1], m[1];
  Packing pk;
};
struct NoTail {};

template <typename T, int K, typename Tail = NoTail>
__device__ __forceinline__ void fold_hashes(T* hashes, uint32_t count, const T (&a)[K], const T (&b)[K], T (&m)[K], int lane, Packing pk, Tail& tail)
{
  constexpr bool kHasTail = !std::is_same<Tail, NoTail>::value;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (count == 0) return;
  // a duplicate never changes a minimum
  uint32_t stride = K > 1 ? Fold<T, K>::kPerTrip : pk.stride(Fold<T, K>::kPerTrip);  // a power of two, at most 64
  if constexpr (kHasTail) stride = max(stride, tail.pk.stride(Fold<T, 1>::kPerTrip));
  uint32_t const padded = (count + stride - 1u) & ~(stride - 1u);
  if (lane < static_cast<int>(padded - count)) hashes[count + lane] = hashes[0];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  // the usual case keeps the loop counter out of the vector registers
  if (K > 1 || pk.groups == 1)
    Fold<T, K>::run(hashes, padded, 0u, Fold<T, K>::kPerTrip, a, b, m);
  else
    Fold<T, K>::run(hashes, padded, pk.first(lane, Fold<T, K>::kPerTrip), pk.stride(Fold<T, K>::kPerTrip), a, b, m);
  if constexpr (kHasTail)
    Fold<T, 1>::run(hashes, padded, tail.pk.first(lane, Fold<T, 1>::kPerTrip), tail.pk.stride(Fold<T, 1>::kPerTrip), tail.a, tail.b, tail.m);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
template <typename T, int K>
__device__ __forceinline__ void fold_hashes(T* hashes, uint32_t count, const T (&a)[K], const T (&b)[K], T (&m)[K], int lane,
                                            Packing pk = Packing{kWave, 1})
{
  NoTail none;
  fold_hashes<T, K, NoTail>(hashes, count, a, b, m, lane, pk, none);
}

// Whether the wavefront has met this hash lately (it is noted either way).  Called by the lanes that have a hash.
template <typename T>
__device__ __forceinline__ bool seen_lately(WaveLds<T>& lds, T hv)
{
  T* const at  = &lds.recent[static_cast<uint32_t>(hv) & (recent_entries<T>() - 1)];
  T const was  = *at;
  *at          = hv;
  return was == hv;
}
template <typename T>
__device__ __forceinline__ void forget_hashes(WaveLds<T>& lds, int lane)
{
  for (int i = lane; i < recent_entries<T>(); i += kWave) lds.recent[i] = T{0};
}

// Processes the window starts [s_begin, s_end) of one row with one wavefront and folds the
// permuted hashes into m[K].  Lane l owns parameters chunk_base + l + 64*k.
template <typename T, int K, typename Tail>
__device__ __forceinline__ void process_section(const uint8_t* row, int64_t n, int64_t s_begin, int64_t s_end, T seed, int32_t width,
                                                const T (&a)[K], const T (&b)[K], T (&m)[K], WaveLds<T>& lds, int lane, Packing pk, Tail& tail)
{
  using H = HashTraits<T>;
  if (static_cast<int64_t>(width) * 4 <= kHalo) {
    // usual case: a window (<= 4*width bytes) fits the halo staged behind every tile
    uint32_t const halo = static_cast<uint32_t>(width) * 4u;
    forget_hashes(lds, lane);  // (the wave barrier after the first tile's staging comes before the first look)
    for (int64_t base = s_begin; base < s_end; base += kTile) {
      uint32_t const cnt = static_cast<uint32_t>(min(static_cast<int64_t>(kTile), s_end - base));
      uint32_t const len = static_cast<uint32_t>(min(n - base, static_cast<int64_t>(cnt + halo)));
      bool all_ascii;
      uint32_t const mis = stage_bytes(row, base, len, lds.bytes, lane, &all_ascii);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      uint32_t count = 0;  // compacted hashes so far (wave-uniform)
      // In a tile of one-byte characters of a row of at least `width` bytes every window is `width` bytes long: the
      // hash then runs with a length that the compiler knows to be the same in every lane (its loops over the
      // blocks and the tail become scalar branches instead of masked ones).
      bool const plain         = all_ascii && n >= static_cast<int64_t>(width);
      uint32_t const width_all = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(width));
      if (plain) {
        for (uint32_t q = 0; q < cnt; q += kWave) {
          uint32_t const p = q + lane;
          bool valid = p < cnt && n - (base + p) >= static_cast<int64_t>(width_all);
          T hv       = 0;
          if (valid) {
            WordSrc const src{lds.bytes, mis + p};
            hv = H::hash(src, width_all, seed);
            hv = hv < 1 ? T{1} : hv;  // minhash.cu:141
          }
          valid             = valid && !seen_lately(lds, hv);
          uint64_t const vm = ballot64(valid);
          if (valid) lds.hashes[count + lanes_below(vm)] = hv;
          count += static_cast<uint32_t>(__builtin_popcountll(vm));
        }
      } else {
        // A tile with longer characters: all of them are found at once, and where they follow one another without a gap
        // a lane takes a character, not a byte, and reads its window's length from the list of characters instead of
        // walking.  (A row shorter than `width` comes here too, whatever its bytes.)
        CharMap map;
        map.exact = false;
        if (!all_ascii) map.build(lds.bytes, mis, len, cnt, base + len == n, lds.chars, lane);
        uint32_t const items = map.exact ? map.windows : cnt;  // characters, or byte positions
        for (uint32_t q = 0; q < items; q += kWave) {
          uint32_t const item = q + lane;
          bool valid          = false;
          T hv                = 0;
          if (item < items) {
            uint32_t p = item, hlen;
            if (map.exact) {
              valid = map.window(item, len, base == 0, width, lds.chars, &p, &hlen);
            } else {
              int64_t const gpos = base + p;
              WordSrc const at{lds.bytes, mis + p};
              valid = window_at(at, row + gpos, n - gpos, len - p, gpos == 0, all_ascii, width, &hlen);
            }
            if (valid) {
              WordSrc const src{lds.bytes, mis + p};
              hv = H::hash(src, hlen, seed);
              hv = hv < 1 ? T{1} : hv;  // minhash.cu:141
            }
          }
          valid             = valid && !seen_lately(lds, hv);
          uint64_t const vm = ballot64(valid);
          if (valid) lds.hashes[count + lanes_below(vm)] = hv;
          count += static_cast<uint32_t>(__builtin_popcountll(vm));
        }
      }
      fold_hashes<T, K, Tail>(lds.hashes, count, a, b, m, lane, pk, tail);
    }
  } else {
    // very wide windows: 64 starts at a time, bytes read straight from global memory
    for (int64_t base = s_begin; base < s_end; base += kWave) {
      int64_t const gpos = base + lane;
      bool valid         = false;
      T hv               = 0;
      if (gpos < s_end) {
        int64_t const remaining = n - gpos;
        BoundedSrc const src{row + gpos, remaining};
        uint32_t hlen;
        uint32_t const readable = static_cast<uint32_t>(min(remaining, static_cast<int64_t>(width) * 4));
        valid = window_at(src, row + gpos, remaining, readable, gpos == 0, false, width, &hlen);
        if (valid) {
          hv = H::hash(src, hlen, seed);
          hv = hv < 1 ? T{1} : hv;
        }
      }
      uint64_t const vm = ballot64(valid);
      if (valid) lds.hashes[lanes_below(vm)] = hv;
      fold_hashes<T, K, Tail>(lds.hashes, static_cast<uint32_t>(__builtin_popcountll(vm)), a, b, m, lane, pk, tail);
    }
  }
}

template <typename T, int K>
__device__ __forceinline__ void load_params(const T* pa, const T* pb, int32_t P, int32_t chunk_base, int lane, T (&a)[K], T (&b)[K], T (&m)[K])
{
#pragma unroll
  for (int k = 0; k < K; ++k) {
    int32_t const j = chunk_base + lane + kWave * k;
    a[k]            = j < P ? pa[j] : T{0};
    b[k]            = j < P ? pb[j] : T{0};
    m[k]            = std::numeric_limits<T>::max();
  }
}

// One workgroup per (group of consecutive rows, parameter chunk).  A row of up to kSoloBytes (kSoloBytesMany when a
// wavefront takes several) is done by one wavefront alone (wavefront w takes the rows w, w + 4, .. of the group, `solo_per_wave` of them: nothing to combine, the minima go
// from the registers to the result); a longer row is shared by the four wavefronts, which split its first kSpan bytes
// and combine through LDS, one such row after the other.  The groups lie along x and, beyond kMaxRowBlocks of them,
// along z.
// Rows differ in length, and a workgroup lasts as long as its slowest wavefront: with one short row per wavefront the
// others waited for the longest of four (8 M rows of about 500 bytes: 88 ms; four rows per wavefront 80 ms, sixteen
// 77 ms).  More rows per workgroup mean fewer workgroups, and a column of few rows needs them all to fill the device
// and to even out its end: the host asks for as many rows per wavefront (a power of two, at most kMaxSoloPerWave) as
// leave at least kMinRowGroups groups.
constexpr int64_t kSoloBytes      = 1024;   // with one row to a wavefront
constexpr int64_t kSoloBytesMany  = 4096;   // with several: their sum evens out, and a row done alone needs no barrier (2 M rows of 2 KB: 2 % faster than 1024)
constexpr int kMaxSoloPerWave     = 16;
constexpr int32_t kMinRowGroups   = 16384;  // sixteen times the workgroups that 256 CUs hold at four apiece
inline int solo_rows_per_wave(int32_t rows)
{
  int spw = 1;
  while (spw < kMaxSoloPerWave && rows / (2 * spw * kWaves) >= kMinRowGroups) spw *= 2;
  return spw;
}

// The tail of a launch with TAIL: the P - 64 K parameters (1..32) beyond the K full sets of the one chunk.
template <typename T, int K, bool TAIL>
struct TailOf {
  using type = NoTail;
  static __device__ __forceinline__ void load(type&, const T*, const T*, int32_t, int) {}
  static __device__ __forceinline__ void reset(type&) {}
  static __device__ __forceinline__ void finish(type&) {}
  static __device__ __forceinline__ T value(type const&) { return T{0}; }
};
template <typename T, int K>
struct TailOf<T, K, true> {
  using type = TailParams<T>;
  static __device__ __forceinline__ void load(type& t, const T* pa, const T* pb, int32_t P, int lane)
  {
    t.pk            = packing_for(P - K * kWave);
    int32_t const j = K * kWave + t.pk.param_lane(lane);
    t.a[0]          = j < P ? pa[j] : T{0};
    t.b[0]          = j < P ? pb[j] : T{0};
    t.m[0]          = std::numeric_limits<T>::max();
  }
  static __device__ __forceinline__ void reset(type& t) { t.m[0] = std::numeric_limits<T>::max(); }
  static __device__ __forceinline__ void finish(type& t) { t.m[0] = t.pk.combine(t.m[0]); }  // every set of lanes then holds the minima
  static __device__ __forceinline__ T value(type const& t) { return t.m[0]; }
};

template <typename T, int K, bool TAIL>
__global__ void __launch_bounds__(kThreads, sizeof(T) == 4 ? 7 : 4) minhash_rows_kernel(ColView col, T seed, const T* __restrict__ pa, const T* __restrict__ pb, int32_t P,
                                                                int32_t width, const int32_t* __restrict__ out_offsets, T* __restrict__ out,
                                                                int solo_per_wave)
{
  using TailT = TailOf<T, K, TAIL>;
  constexpr int kSets = K + (TAIL ? 1 : 0);
  __shared__ WaveLds<T> lds[kWaves];
  __shared__ T red[kWaves][kSets * kWave];
  __shared__ uint32_t next_row;

  int const group_rows     = solo_per_wave * kWaves;
  int64_t const solo_bytes = solo_per_wave > 1 ? kSoloBytesMany : kSoloBytes;
  int64_t const r0     = (static_cast<int64_t>(blockIdx.z) * gridDim.x + blockIdx.x) * group_rows;
  if (r0 >= col.size) return;
  int const lane           = lane_id();
  int const wave           = threadIdx.x / kWave;
  int32_t const chunk_base = blockIdx.y * (K * kWave);  // (with TAIL there is one chunk)
  int32_t const in_chunk   = min(kSets * kWave, P - chunk_base);
  Packing const pk         = K == 1 ? packing_for(P) : Packing{kWave, 1};
  T a[K], b[K], m[K];
  load_params<T, K>(pa, pb, P, chunk_base, pk.param_lane(lane), a, b, m);
  typename TailT::type tail;
  TailT::load(tail, pa, pb, P, lane);

  int const rows_here = static_cast<int>(min(static_cast<int64_t>(group_rows), col.size - r0));
  if (threadIdx.x == 0) next_row = 0;
  __syncthreads();

  // First the short rows of the group: a wavefront takes the next one whenever it is done with one (a counter in LDS),
  // so that the four are done with their short rows at about the same time whatever the rows' lengths.  Then, from
  // `together` = 0 on, its part of the rows that are too long for that, one after the other.
  int together = -1;
  for (;;) {
    int i;
    if (together < 0) {
      int t = 0;
      if (lane == 0) t = static_cast<int>(atomicAdd(&next_row, 1u));
      i = __builtin_amdgcn_readfirstlane(t);  // (the same in every lane: what depends on it stays scalar)
      if (i >= rows_here) {
        together = 0;
        continue;
      }
    } else {
      if (together >= rows_here) break;
      i = together++;
    }
    bool const solo = together < 0;
    if (!col.valid(r0 + i)) continue;
    int64_t const o = col.off(r0 + i);
    int64_t const n = col.off(r0 + i + 1) - o;
    if (solo != (n <= solo_bytes)) continue;
#pragma unroll
    for (int k = 0; k < K; ++k) m[k] = std::numeric_limits<T>::max();
    TailT::reset(tail);
    int64_t sb = 0, se = n;
    if (!solo) {
      int64_t const span = min(n, static_cast<int64_t>(kSpan));
      int64_t sec        = (span + kWaves - 1) / kWaves;
      sec                = (sec + kWave - 1) / kWave * kWave;
      sb                 = min(span, wave * sec);
      se                 = min(span, sb + sec);
    }
    if (sb < se) process_section<T, K>(col.chars + o, n, sb, se, seed, width, a, b, m, lds[wave], lane, pk, tail);
    if (K == 1) m[0] = pk.combine(m[0]);
    TailT::finish(tail);
    T* const dst = out + static_cast<int64_t>(out_offsets[r0 + i]) + chunk_base;
    if (solo) {
      // nothing to combine: the minima go from the registers to the result; an empty row is zeros (minhash.cu:318)
#pragma unroll
      for (int k = 0; k < K; ++k) {
        int32_t const j = lane + kWave * k;  // (with fewer than 64 parameters the first lanes hold one each, in order)
        if (j < in_chunk) dst[j] = n > 0 ? m[k] : T{0};
      }
      if (TAIL && K * kWave + lane < in_chunk) dst[K * kWave + lane] = n > 0 ? TailT::value(tail) : T{0};
    } else {
      __syncthreads();  // (the row before has been read out of red)
#pragma unroll
      for (int k = 0; k < K; ++k) red[wave][k * kWave + lane] = m[k];
      if (TAIL) red[wave][K * kWave + lane] = TailT::value(tail);
      __syncthreads();
      for (int j = threadIdx.x; j < in_chunk; j += kThreads) {
        T v = red[0][j];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v = min(v, red[w][j]);
        dst[j] = v;
      }
    }
  }
}

// Extra parts of rows longer than kSpan: task t covers bytes [part*kSpan, (part+1)*kSpan) of its row.
// extra_prefix[r] = number of extra parts in rows < r (rows+1 entries).
// (uint32: held to the registers of six wavefronts per SIMD, which left to itself the compiler exceeds with four and
// five sets of parameters: the reference's 260-parameter shapes 3 to 5 % faster; uint64 gains nothing from it.)
template <typename T, int K, bool TAIL>
__global__ void __launch_bounds__(kThreads, sizeof(T) == 4 ? 6 : 1) minhash_extra_kernel(ColView col, T seed, const T* __restrict__ pa, const T* __restrict__ pb, int32_t P,
                                                                 int32_t width, const int32_t* __restrict__ out_offsets,
                                                                 const uint32_t* __restrict__ extra_prefix, T* __restrict__ out)
{
  using TailT = TailOf<T, K, TAIL>;
  constexpr int kSets = K + (TAIL ? 1 : 0);
  __shared__ WaveLds<T> lds[kWaves];
  __shared__ T red[kWaves][kSets * kWave];
  uint32_t const total     = extra_prefix[col.size];
  int32_t const chunk_base = blockIdx.y * (K * kWave);
  int32_t const in_chunk   = min(kSets * kWave, P - chunk_base);
  int const lane           = lane_id();
  int const wave           = threadIdx.x / kWave;
  Packing const pk         = K == 1 ? packing_for(P) : Packing{kWave, 1};
  for (uint32_t t = blockIdx.x; t < total; t += gridDim.x) {
    // last row r with extra_prefix[r] <= t
    int64_t lo = 0, hi = col.size;
    while (hi - lo > 1) {
      int64_t const mid = (lo + hi) >> 1;
      if (extra_prefix[mid] <= t) lo = mid; else hi = mid;
    }
    int64_t const r    = lo;
    int64_t const part = static_cast<int64_t>(t - extra_prefix[r]) + 1;
    int64_t const o    = col.off(r);
    int64_t const n    = col.off(r + 1) - o;
    T a[K], b[K], m[K];
    load_params<T, K>(pa, pb, P, chunk_base, pk.param_lane(lane), a, b, m);
    typename TailT::type tail;
    TailT::load(tail, pa, pb, P, lane);
    int64_t const pb0  = part * kSpan;
    int64_t const pe0  = min(n, pb0 + kSpan);
    int64_t const sec  = kSpan / kWaves;
    int64_t const sb   = min(pe0, pb0 + wave * sec);
    int64_t const se   = min(pe0, sb + sec);
    if (sb < se) process_section<T, K>(col.chars + o, n, sb, se, seed, width, a, b, m, lds[wave], lane, pk, tail);
    if (K == 1) m[0] = pk.combine(m[0]);
    TailT::finish(tail);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < K; ++k) red[wave][k * kWave + lane] = m[k];
    if (TAIL) red[wave][K * kWave + lane] = TailT::value(tail);
    __syncthreads();
    T* dst = out + static_cast<int64_t>(out_offsets[r]) + chunk_base;
    for (int j = threadIdx.x; j < in_chunk; j += kThreads) {
      T v = red[0][j];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) v = min(v, red[w][j]);
      if (v != std::numeric_limits<T>::max()) atomicMin(&dst[j], v);
    }
  }
}

struct ValidTimesP {
  ColView col;
  int32_t P;
  __device__ uint64_t operator()(int64_t i) const { return col.valid(i) ? static_cast<uint64_t>(P) : 0; }
};

struct ExtraParts {
  ColView col;
  __device__ uint64_t operator()(int64_t i) const
  {
    if (!col.valid(i)) return 0;
    int64_t const n = col.off(i + 1) - col.off(i);
    return n > kSpan ? static_cast<uint64_t>((n + kSpan - 1) / kSpan - 1) : 0;
  }
};

__global__ void uniform_offsets_kernel(int32_t* out, int32_t rows, int32_t P)
{
  int64_t const i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i <= rows) out[i] = static_cast<int32_t>(i * P);
}

constexpr int32_t kMaxRowBlocks = 1 << 15;  // groups along x (a launch of 4 M rows, 64 to a group, has two layers along z: the tests reach them)

template <typename T, int K, bool TAIL>
void launch_kernels(const ColView& v, T seed, const T* a, const T* b, int32_t P, int32_t width, const int32_t* offsets,
                    const uint32_t* extra_prefix, T* child, hipStream_t stream)
{
  int32_t const chunks = TAIL ? 1 : (P + K * kWave - 1) / (K * kWave);
  int const solo_per_wave = solo_rows_per_wave(v.size);
  int32_t const groups    = (v.size + solo_per_wave * kWaves - 1) / (solo_per_wave * kWaves);
  dim3 grid(static_cast<unsigned>(std::min(groups, kMaxRowBlocks)), static_cast<unsigned>(chunks),
            static_cast<unsigned>((groups + kMaxRowBlocks - 1) / kMaxRowBlocks));
  {
    ProfileScope ps("minhash_rows_kernel", stream);
    hipLaunchKernelGGL(HIP_KERNEL_NAME(minhash_rows_kernel<T, K, TAIL>), grid, dim3(kThreads), 0, stream, v, seed, a, b, P, width, offsets, child,
                       solo_per_wave);
  }
  dim3 grid2(4096, static_cast<unsigned>(chunks));
  {
    ProfileScope ps("minhash_extra_kernel", stream);
    hipLaunchKernelGGL(HIP_KERNEL_NAME(minhash_extra_kernel<T, K, TAIL>), grid2, dim3(kThreads), 0, stream, v, seed, a, b, P, width, offsets,
                       extra_prefix, child);
  }
}

// How the parameters are shared out: chunks of K sets of 64 (every chunk hashes the windows again, and a lane without
// a parameter still folds), or, for 65 to 288 parameters of which at most 32 lie beyond the last full set, one chunk of
// K full sets and a tail that costs the fold the share `lanes of a tail set / 64` of a set.  Costs in 64ths of a set.
struct Sharing {
  int k;
  bool tail;
};
inline Sharing sharing_for(int32_t P)
{
  Sharing best{1, false};
  int64_t best_cost = std::numeric_limits<int64_t>::max();
  for (int k = 1; k <= 5; ++k) {  // the larger K (fewer hashing passes) on a tie
    int64_t const cost = static_cast<int64_t>((P + k * kWave - 1) / (k * kWave)) * k * kWave;
    if (cost <= best_cost) { best_cost = cost; best = Sharing{k, false}; }
  }
  int const full = P / kWave, rest = P % kWave;
  if (full >= 1 && full <= 4 && rest >= 1 && rest <= 32) {
    int64_t const cost = static_cast<int64_t>(full) * kWave + packing_for(rest).ppad;
    if (cost < best_cost) best = Sharing{full, true};
  }
  return best;
}

// The launches of one minhash call: the row offsets of the result, the number of extra workgroup-spans of every
// row, then the two hashing kernels.  extra_prefix holds rows + 1 values, scan_tmp scan_temp_bytes(rows) bytes.
template <typename T>
void run_minhash(const ColView& v, T seed, const T* a, const T* b, int32_t P, int32_t width, int32_t* offsets, T* child, int64_t child_size,
                 uint32_t* extra_prefix, uint64_t* scan_tmp, hipStream_t stream)
{
  int32_t const rows = v.size;
  if (v.use_mask) {
    device_exclusive_scan(ValidTimesP{v, P}, static_cast<int64_t>(rows), offsets, scan_tmp, stream);
  } else {
    hipLaunchKernelGGL(uniform_offsets_kernel, dim3((rows + 1 + 255) / 256), dim3(256), 0, stream, offsets, rows, P);
  }
  device_exclusive_scan(ExtraParts{v}, static_cast<int64_t>(rows), extra_prefix, scan_tmp, stream);

  if (child_size > 0) {
    Sharing const sh = sharing_for(P);
    switch (sh.k * 2 + (sh.tail ? 1 : 0)) {
      case 10: launch_kernels<T, 5, false>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 9: launch_kernels<T, 4, true>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 8: launch_kernels<T, 4, false>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 7: launch_kernels<T, 3, true>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 6: launch_kernels<T, 3, false>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 5: launch_kernels<T, 2, true>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 4: launch_kernels<T, 2, false>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      case 3: launch_kernels<T, 1, true>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
      default: launch_kernels<T, 1, false>(v, seed, a, b, P, width, offsets, extra_prefix, child, stream); break;
    }
  }
}

template <typename T>
nvtext_amd_status minhash_impl(const nvtext_amd_strings_column* input, T seed, const T* a, const T* b, int64_t a_count, int64_t b_count,
                               int32_t width, void* stream_, const nvtext_amd_allocator* mr_, nvtext_amd_list_column* out, int32_t type_id)
{
  EntryScope const entry(sizeof(T) == 4 ? "nvtext_amd_minhash" : "nvtext_amd_minhash64");
  if (!input || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nvtext_amd_list_column{};
  // cpp/src/text/minhash.cu:435-446, same order and messages
  if (width < 2) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameter width should be an integer value of 2 or greater");
  if (a_count <= 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameters A and B cannot be empty");
  if (a_count != b_count) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameters A and B should have the same number of elements");
  if (static_cast<uint64_t>(input->size) * static_cast<uint64_t>(a_count) >= static_cast<uint64_t>(std::numeric_limits<int32_t>::max()))
    return fail(NVTEXT_AMD_OVERFLOW, "The number of parameters times the number of input rows exceeds the column size limit");
  if (input->size < 0 || input->null_count < 0 || input->null_count > input->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "invalid column sizes");
  if (input->null_count > 0 && !input->null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");

  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Mr mr{mr_, stream};
  int32_t const rows = input->size;
  int32_t const P    = static_cast<int32_t>(a_count);
  out->child_type    = type_id;
  out->size          = rows;
  out->null_count    = input->null_count;
  out->offsets_size  = rows + 1;
  out->offsets_bytes = static_cast<size_t>(rows + 1) * sizeof(int32_t);
  out->offsets       = static_cast<int32_t*>(mr.allocate(out->offsets_bytes));
  if (!out->offsets) return fail(NVTEXT_AMD_ALLOC_FAILED, "offsets allocation failed");
  if (rows == 0) {  // minhash.cu:449 then 616: zero rows, offsets = [0], empty child
    launch_fill_u32(reinterpret_cast<uint32_t*>(out->offsets), 0u, 1, stream);
    NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_list_column_free(out, stream_, mr_));
    return NVTEXT_AMD_SUCCESS;
  }
  out->child_size  = static_cast<int64_t>(rows - input->null_count) * P;
  out->child_bytes = static_cast<size_t>(out->child_size) * sizeof(T);
  if (out->child_bytes) {
    out->child = mr.allocate(out->child_bytes);
    if (!out->child) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "child allocation failed");
    }
  }
  if (input->null_mask) {  // copy_bitmask(input): cpp/src/bitmask/null_mask.cu:381-391
    out->null_mask_bytes = mask_alloc_bytes(rows);
    out->null_mask       = static_cast<uint32_t*>(mr.allocate(out->null_mask_bytes));
    if (!out->null_mask) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "mask allocation failed");
    }
    launch_copy_bitmask(out->null_mask, input->null_mask, input->offset, rows, stream);
  }

  ColView const v = make_view(*input);
  Temp scan_tmp(mr, scan_temp_bytes(rows));
  Temp extra(mr, static_cast<size_t>(rows + 1) * sizeof(uint32_t));
  if (!scan_tmp.ok() || !extra.ok()) {
    nvtext_amd_list_column_free(out, stream_, mr_);
    return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
  }
  run_minhash<T>(v, seed, a, b, P, width, out->offsets, static_cast<T*>(out->child), out->child_size, extra.as<uint32_t>(),
                 scan_tmp.as<uint64_t>(), stream);
  NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_list_column_free(out, stream_, mr_));
  return NVTEXT_AMD_SUCCESS;
}


// ------------------------------------------------------------------ minhash_ngrams / minhash64_ngrams
// LIST<STRING> rows: the hashed items are runs of consecutive list elements instead of character windows
// (cpp/src/text/minhash.cu:182-250); the permutation and the minimum are the ones above.
struct ListView {
  const int32_t* offsets;  // element index of the first element of row i + offset
  const uint32_t* mask;
  int32_t size;
  int32_t offset;
  int32_t use_mask;
  ColView child;           // the elements

  __device__ __forceinline__ int64_t off(int64_t i) const { return offsets[i + offset]; }
  __device__ __forceinline__ bool valid(int64_t i) const
  {
    if (!use_mask) return true;
    int64_t const b = i + offset;
    return (mask[b >> 5] >> (b & 31)) & 1u;
  }
};

// Byte source over global memory through aligned dword loads that overlap [p, p + len) only.
struct AlignedSrc {
  const uint32_t* w;  // aligned address at or below the first byte
  uint32_t mis;       // first byte inside w[0]
  uint32_t end;       // mis + len
  __device__ __forceinline__ AlignedSrc(const uint8_t* p, uint32_t len)
  {
    mis = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p) & 3u);
    w   = reinterpret_cast<const uint32_t*>(p - mis);
    end = mis + len;
  }
  __device__ __forceinline__ uint32_t byte(uint32_t i) const { return reinterpret_cast<const uint8_t*>(w)[mis + i]; }
  __device__ __forceinline__ uint32_t u32(uint32_t i) const
  {
    uint32_t const o  = mis + i;
    uint32_t const j  = o >> 2;
    uint32_t const lo = w[j];
    uint32_t const hi = 4u * (j + 1u) < end ? w[j + 1] : 0u;
    return __builtin_amdgcn_alignbit(hi, lo, (o & 3u) * 8u);
  }
};

constexpr uint32_t kNgramStageBytes = 4096;                             // longest stretch of chars hashed out of LDS
constexpr uint32_t kNgramStageWords = (kNgramStageBytes + 4 + 28) / 4;  // + misalignment, + over-read of the hash tail

// One workgroup per (group of consecutive rows, parameter chunk), as in minhash_rows_kernel: a row of up to
// kNgramSoloPositions positions is done by one wavefront alone, 64 positions a trip (wavefront w takes the rows w, w + 4, .. of the group,
// `solo_per_wave` of them), and its minima go from the registers to the result; a row of more positions is shared by the
// four wavefronts, which take its positions 64 at a time in turn and combine through LDS, one such row after the other.
// A column of fewer than 131,072 rows keeps one row to a workgroup, every row shared by the four wavefronts
// (solo_per_wave 0): it needs its workgroups to fill the device and to even out its end (20,000 rows of 3,000 elements:
// four rows to a workgroup were 8 % slower).
constexpr int64_t kNgramSoloPositions = 2048;
template <typename T, int K>
__global__ void __launch_bounds__(kThreads) minhash_ngrams_kernel(ListView in, int32_t ngrams, T seed, const T* __restrict__ pa,
                                                                  const T* __restrict__ pb, int32_t P, const int32_t* __restrict__ out_offsets,
                                                                  T* __restrict__ out, int solo_per_wave)
{
  using H = HashTraits<T>;
  __shared__ alignas(16) T hashes[kWaves][2 * kWave];  // 64 hashes a trip, padded to the stride of the fold (at most 64 more)
  __shared__ T red[kWaves][K * kWave];
  // the chars of the elements a wavefront is hashing (32-bit hash only: measured 13 % faster there, 9 % slower for the
  // 64-bit hash, whose 16-byte steps cost more to assemble out of LDS than they save)
  constexpr bool kStageRuns = sizeof(T) == 4;
  __shared__ uint32_t run_bytes[kWaves][kStageRuns ? kNgramStageWords : 1];
  __shared__ uint32_t next_row;

  int const group_rows = solo_per_wave > 0 ? solo_per_wave * kWaves : 1;
  int64_t const r0     = (static_cast<int64_t>(blockIdx.z) * gridDim.x + blockIdx.x) * group_rows;  // groups along x, then z
  if (r0 >= in.size) return;
  int64_t const solo_positions = solo_per_wave > 0 ? kNgramSoloPositions : -1;
  int32_t const chunk_base     = blockIdx.y * (K * kWave);
  int32_t const in_chunk       = min(K * kWave, P - chunk_base);
  int const lane               = lane_id();
  int const wave               = threadIdx.x / kWave;
  T a[K], b[K], m[K];
  load_params<T, K>(pa, pb, P, chunk_base, lane, a, b, m);

  int const rows_here = static_cast<int>(min(static_cast<int64_t>(group_rows), in.size - r0));
  if (threadIdx.x == 0) next_row = 0;
  __syncthreads();
  // the short rows of the group first, each wavefront taking the next one whenever it is done with one; then, from
  // `together` = 0 on, the rows that all four do together, one after the other (see minhash_rows_kernel)
  int together = -1;
  for (;;) {
    int i;
    if (together < 0) {
      int t = 0;
      if (lane == 0) t = static_cast<int>(atomicAdd(&next_row, 1u));
      i = __builtin_amdgcn_readfirstlane(t);
      if (i >= rows_here) {
        together = 0;
        continue;
      }
    } else {
      if (together >= rows_here) break;
      i = together++;
    }
    bool const solo = together < 0;
    if (!in.valid(r0 + i)) continue;
    int64_t const first = in.off(r0 + i);
    int64_t const n     = in.off(r0 + i + 1) - first;
    // minhash.cu:311-314 with width = ngrams: the positions that the permutation looks at
    int64_t const positions = max(static_cast<int64_t>(1), n - ngrams + 1);
    if (solo != (positions <= solo_positions)) continue;
#pragma unroll
    for (int k = 0; k < K; ++k) m[k] = std::numeric_limits<T>::max();
    if (n > 0) {
      int64_t const trip = solo ? kWave : kWaves * kWave;
      for (int64_t base = solo ? 0 : static_cast<int64_t>(wave) * kWave; base < positions; base += trip) {
        int64_t const idx = base + lane;
        bool valid        = false;
        T hv              = 0;
        int64_t bo = 0, eo = 0;
        if (idx < positions && in.child.valid(first + idx)) {  // 213-216: a null element starts no run
          // 218-222: the run ends at element idx + ngrams, clamped to the row; a clamped run counts only at idx 0
          int64_t const next = min(idx + ngrams, n - 1);
          if (idx == 0 || next - idx >= ngrams) {
            // 224-229: the bytes from the start of element idx to the end of element next
            bo    = in.child.off(first + idx);
            eo    = in.child.off(first + next + 1);
            valid = true;
          }
        }
        // The runs of these 64 elements overlap and lie side by side in the chars: fetch that stretch once, with
        // coalesced loads, and hash out of LDS (the hash walks a run dword by dword, each step a dependent read).
        // A stretch too long for the buffer is hashed straight from memory.
        int64_t const span_begin = kStageRuns ? in.child.off(first + base) : 0;
        int64_t const span_end   = kStageRuns ? in.child.off(first + min(base + kWave + ngrams, n)) : 0;
        if (kStageRuns && span_end - span_begin <= static_cast<int64_t>(kNgramStageBytes)) {
          bool ascii;
          uint32_t const mis = stage_bytes(in.child.chars, span_begin, static_cast<uint32_t>(span_end - span_begin), run_bytes[wave], lane, &ascii);
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          if (valid) {
            WordSrc const src{run_bytes[wave], mis + static_cast<uint32_t>(bo - span_begin)};
            hv = H::hash(src, static_cast<uint32_t>(eo - bo), seed);
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
        } else if (valid) {
          AlignedSrc const src(in.child.chars + bo, static_cast<uint32_t>(eo - bo));
          hv = H::hash(src, static_cast<uint32_t>(eo - bo), seed);
        }
        if (valid) hv = hv < 1 ? T{1} : hv;  // 237
        uint64_t const vm = ballot64(valid);
        if (valid) hashes[wave][lanes_below(vm)] = hv;
        fold_hashes<T, K>(hashes[wave], static_cast<uint32_t>(__builtin_popcountll(vm)), a, b, m, lane);
      }
    }
    T* const dst = out + static_cast<int64_t>(out_offsets[r0 + i]) + chunk_base;
    if (solo) {
      // an empty row is zeros (minhash.cu:318); a row whose every run was skipped keeps the all-ones start value
#pragma unroll
      for (int k = 0; k < K; ++k) {
        int32_t const j = lane + kWave * k;
        if (j < in_chunk) dst[j] = n > 0 ? m[k] : T{0};
      }
    } else {
      __syncthreads();  // (the row before has been read out of red)
#pragma unroll
      for (int k = 0; k < K; ++k) red[wave][k * kWave + lane] = m[k];
      __syncthreads();
      for (int j = threadIdx.x; j < in_chunk; j += kThreads) {
        T v = red[0][j];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v = min(v, red[w][j]);
        dst[j] = n > 0 ? v : T{0};
      }
    }
  }
}

struct ListValidTimesP {
  ListView in;
  int32_t P;
  __device__ uint64_t operator()(int64_t i) const { return in.valid(i) ? static_cast<uint64_t>(P) : 0; }
};

template <typename T, int K>
void launch_ngrams(const ListView& v, int32_t ngrams, T seed, const T* a, const T* b, int32_t P, const int32_t* offsets, T* child,
                   hipStream_t stream)
{
  int32_t const chunks    = (P + K * kWave - 1) / (K * kWave);
  int const solo_per_wave = v.size >= 131072 ? solo_rows_per_wave(v.size) : 0;
  int32_t const group     = solo_per_wave > 0 ? solo_per_wave * kWaves : 1;
  int32_t const groups    = (v.size + group - 1) / group;
  dim3 grid(static_cast<unsigned>(std::min(groups, kMaxRowBlocks)), static_cast<unsigned>(chunks),
            static_cast<unsigned>((groups + kMaxRowBlocks - 1) / kMaxRowBlocks));
  ProfileScope ps("minhash_ngrams_kernel", stream);
  hipLaunchKernelGGL(HIP_KERNEL_NAME(minhash_ngrams_kernel<T, K>), grid, dim3(kThreads), 0, stream, v, ngrams, seed, a, b, P, offsets, child,
                     solo_per_wave);
}

template <typename T>
nvtext_amd_status minhash_ngrams_impl(const nvtext_amd_list_strings_column* input, int32_t ngrams, T seed, const T* a, const T* b,
                                      int64_t a_count, int64_t b_count, void* stream_, const nvtext_amd_allocator* mr_,
                                      nvtext_amd_list_column* out, int32_t type_id)
{
  EntryScope const entry(sizeof(T) == 4 ? "nvtext_amd_minhash_ngrams" : "nvtext_amd_minhash64_ngrams");
  if (!input || !out) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  *out = nvtext_amd_list_column{};
  // cpp/src/text/minhash.cu:524-536, same order and messages
  if (ngrams < 2) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameter ngrams should be an integer value of 2 or greater");
  if (a_count <= 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameters A and B cannot be empty");
  if (a_count != b_count) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameters A and B should have the same number of elements");
  if (static_cast<uint64_t>(input->size) * static_cast<uint64_t>(a_count) >= static_cast<uint64_t>(std::numeric_limits<int32_t>::max()))
    return fail(NVTEXT_AMD_OVERFLOW, "The number of parameters times the number of input rows exceeds the column size limit");
  if (input->size < 0 || input->null_count < 0 || input->null_count > input->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "invalid column sizes");
  if (input->null_count > 0 && !input->null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");
  if (input->size > 0 && !input->offsets) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "a list column with rows needs offsets");
  if (input->child.null_count > 0 && !input->child.null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");

  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Mr mr{mr_, stream};
  int32_t const rows = input->size;
  int32_t const P    = static_cast<int32_t>(a_count);
  out->child_type    = type_id;
  out->size          = rows;
  out->null_count    = input->null_count;
  out->offsets_size  = rows + 1;
  out->offsets_bytes = static_cast<size_t>(rows + 1) * sizeof(int32_t);
  out->offsets       = static_cast<int32_t*>(mr.allocate(out->offsets_bytes));
  if (!out->offsets) return fail(NVTEXT_AMD_ALLOC_FAILED, "offsets allocation failed");
  if (rows == 0) {  // minhash.cu:539 then 616
    launch_fill_u32(reinterpret_cast<uint32_t*>(out->offsets), 0u, 1, stream);
    NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_list_column_free(out, stream_, mr_));
    return NVTEXT_AMD_SUCCESS;
  }
  out->child_size  = static_cast<int64_t>(rows - input->null_count) * P;
  out->child_bytes = static_cast<size_t>(out->child_size) * sizeof(T);
  if (out->child_bytes) {
    out->child = mr.allocate(out->child_bytes);
    if (!out->child) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "child allocation failed");
    }
  }
  if (input->null_mask) {
    out->null_mask_bytes = mask_alloc_bytes(rows);
    out->null_mask       = static_cast<uint32_t*>(mr.allocate(out->null_mask_bytes));
    if (!out->null_mask) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "mask allocation failed");
    }
    launch_copy_bitmask(out->null_mask, input->null_mask, input->offset, rows, stream);
  }

  ListView v;
  v.offsets  = input->offsets;
  v.mask     = input->null_mask;
  v.size     = rows;
  v.offset   = input->offset;
  v.use_mask = (input->null_mask != nullptr && input->null_count > 0) ? 1 : 0;
  v.child    = make_view(input->child);
  if (v.use_mask) {
    Temp scan_tmp(mr, scan_temp_bytes(rows));
    if (!scan_tmp.ok()) {
      nvtext_amd_list_column_free(out, stream_, mr_);
      return fail(NVTEXT_AMD_ALLOC_FAILED, "temporary allocation failed");
    }
    device_exclusive_scan(ListValidTimesP{v, P}, static_cast<int64_t>(rows), out->offsets, scan_tmp.as<uint64_t>(), stream);
  } else {
    hipLaunchKernelGGL(uniform_offsets_kernel, dim3((rows + 1 + 255) / 256), dim3(256), 0, stream, out->offsets, rows, P);
  }
  T* child = static_cast<T*>(out->child);
  if (out->child_size > 0) {
    if (P > 2 * kWave)
      launch_ngrams<T, 4>(v, ngrams, seed, a, b, P, out->offsets, child, stream);
    else if (P > kWave)
      launch_ngrams<T, 2>(v, ngrams, seed, a, b, P, out->offsets, child, stream);
    else
      launch_ngrams<T, 1>(v, ngrams, seed, a, b, P, out->offsets, child, stream);
  }
  NVTEXT_HIP_TRY_OR(hipGetLastError(), nvtext_amd_list_column_free(out, stream_, mr_));
  return NVTEXT_AMD_SUCCESS;
}

// ------------------------------------------------------------------ minhash without allocations
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void* g_scratch_ptr[kMaxDevices] = {};

// The address of this device's copy of the array (the array's name means nothing to host code).
nvtext_amd_status scratch_of_current_device(unsigned char** out)
{
  int device = -1;
  NVTEXT_HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "device index out of range");
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    NVTEXT_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[device] = p;
  }
  *out = static_cast<unsigned char*>(g_scratch_ptr[device]);
  return NVTEXT_AMD_SUCCESS;
}

}  // namespace
}  // namespace nvtext_amd

extern "C" {

nvtext_amd_status nvtext_amd_minhash_preallocated(const nvtext_amd_strings_column* input, uint32_t seed, const uint32_t* a, const uint32_t* b,
                                                  int64_t a_count, int64_t b_count, int32_t width, void* stream_, int32_t* out_offsets,
                                                  uint32_t* out_child, int64_t out_child_capacity, uint32_t* out_null_mask)
{
  using namespace nvtext_amd;
  EntryScope const entry("nvtext_amd_minhash_preallocated");
  if (!input || !out_offsets) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null argument");
  if (width < 2) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameter width should be an integer value of 2 or greater");
  if (a_count <= 0) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameters A and B cannot be empty");
  if (a_count != b_count) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "Parameters A and B should have the same number of elements");
  if (input->size < 0 || input->null_count < 0 || input->null_count > input->size) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "invalid column sizes");
  if (static_cast<uint64_t>(input->size) * static_cast<uint64_t>(a_count) >= static_cast<uint64_t>(std::numeric_limits<int32_t>::max()))
    return fail(NVTEXT_AMD_OVERFLOW, "The number of parameters times the number of input rows exceeds the column size limit");
  if (input->null_count > 0 && !input->null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "null_count > 0 requires a null mask");
  if (input->size > kPreallocatedMaxRows)
    return fail(NVTEXT_AMD_INVALID_ARGUMENT, "more rows than nvtext_amd_minhash_preallocated takes (NVTEXT_AMD_MINHASH_PREALLOCATED_MAX_ROWS)");
  int32_t const rows       = input->size;
  int32_t const P          = static_cast<int32_t>(a_count);
  int64_t const child_size = static_cast<int64_t>(rows - input->null_count) * P;
  if (child_size > out_child_capacity || (child_size > 0 && !out_child)) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "out_child is too small");
  if (input->null_mask && !out_null_mask) return fail(NVTEXT_AMD_INVALID_ARGUMENT, "the input has a null mask: out_null_mask is needed");

  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (rows == 0) {
    launch_fill_u32(reinterpret_cast<uint32_t*>(out_offsets), 0u, 1, stream);
    NVTEXT_HIP_TRY(hipGetLastError());
    return NVTEXT_AMD_SUCCESS;
  }
  unsigned char* base = nullptr;
  nvtext_amd_status const st = scratch_of_current_device(&base);
  if (st != NVTEXT_AMD_SUCCESS) return st;
  uint32_t* const extra_prefix = reinterpret_cast<uint32_t*>(base);
  uint64_t* const scan_tmp     = reinterpret_cast<uint64_t*>(base + kScratchPrefixBytes);

  if (input->null_mask) launch_copy_bitmask(out_null_mask, input->null_mask, input->offset, rows, stream);
  ColView const v = make_view(*input);
  // every value of the scratch that the kernels read is written earlier in this same call: nothing to clear
  run_minhash<uint32_t>(v, seed, a, b, P, width, out_offsets, out_child, child_size, extra_prefix, scan_tmp, stream);
  NVTEXT_HIP_TRY(hipGetLastError());
  return NVTEXT_AMD_SUCCESS;
}

nvtext_amd_status nvtext_amd_minhash(const nvtext_amd_strings_column* input, uint32_t seed, const uint32_t* a, const uint32_t* b, int64_t a_count,
                                     int64_t b_count, int32_t width, void* stream, const nvtext_amd_allocator* mr, nvtext_amd_list_column* out)
{
  return nvtext_amd::minhash_impl<uint32_t>(input, seed, a, b, a_count, b_count, width, stream, mr, out, NVTEXT_AMD_TYPE_UINT32);
}

nvtext_amd_status nvtext_amd_minhash64(const nvtext_amd_strings_column* input, uint64_t seed, const uint64_t* a, const uint64_t* b, int64_t a_count,
                                       int64_t b_count, int32_t width, void* stream, const nvtext_amd_allocator* mr, nvtext_amd_list_column* out)
{
  return nvtext_amd::minhash_impl<uint64_t>(input, seed, a, b, a_count, b_count, width, stream, mr, out, NVTEXT_AMD_TYPE_UINT64);
}

nvtext_amd_status nvtext_amd_minhash_ngrams(const nvtext_amd_list_strings_column* input, int32_t ngrams, uint32_t seed, const uint32_t* a,
                                            const uint32_t* b, int64_t a_count, int64_t b_count, void* stream, const nvtext_amd_allocator* mr,
                                            nvtext_amd_list_column* out)
{
  return nvtext_amd::minhash_ngrams_impl<uint32_t>(input, ngrams, seed, a, b, a_count, b_count, stream, mr, out, NVTEXT_AMD_TYPE_UINT32);
}

nvtext_amd_status nvtext_amd_minhash64_ngrams(const nvtext_amd_list_strings_column* input, int32_t ngrams, uint64_t seed, const uint64_t* a,
                                              const uint64_t* b, int64_t a_count, int64_t b_count, void* stream, const nvtext_amd_allocator* mr,
                                              nvtext_amd_list_column* out)
{
  return nvtext_amd::minhash_ngrams_impl<uint64_t>(input, ngrams, seed, a, b, a_count, b_count, stream, mr, out, NVTEXT_AMD_TYPE_UINT64);
}

}  // extern "C"

// Seeded synthetic workloads for the nvtext hot path (host only, multithreaded).
//
// Everything is a pure function of (seed, row index): a counter-based generator
// (splitmix64 over a key made of seed, row and draw number) so that the output does not
// depend on the number of threads.  Rows are single-space separated words with no leading,
// trailing or double spaces; a null row is zero-length with its validity bit cleared.
//
// Build: make -C cudf_amd/datagen
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <unordered_set>
#include <vector>

namespace {

inline uint64_t splitmix64(uint64_t x)
{
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

struct Rng {
  uint64_t key;
  uint64_t ctr = 0;
  Rng(uint64_t seed, uint64_t stream) : key(splitmix64(seed ^ splitmix64(stream + 0x1234567ull))) {}
  uint64_t next() { return splitmix64(key + (ctr++) * 0xD1342543DE82EF95ull); }
  double uniform() { return double(next() >> 11) * (1.0 / 9007199254740992.0); }  // [0,1)
  uint64_t below(uint64_t n) { return uint64_t(uniform() * double(n)); }         // n < 2^53
  double normal()
  {
    double u1 = uniform(), u2 = uniform();
    if (u1 < 1e-300) u1 = 1e-300;
    return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
  }
};

struct Vocab {
  std::string chars;
  std::vector<int64_t> offsets{0};
  void add(const std::string& s)
  {
    chars += s;
    offsets.push_back(int64_t(chars.size()));
  }
  size_t size() const { return offsets.size() - 1; }
};

std::string utf8(uint32_t cp)
{
  std::string s;
  if (cp < 0x80) {
    s += char(cp);
  } else if (cp < 0x800) {
    s += char(0xC0 | (cp >> 6));
    s += char(0x80 | (cp & 0x3F));
  } else if (cp < 0x10000) {
    s += char(0xE0 | (cp >> 12));
    s += char(0x80 | ((cp >> 6) & 0x3F));
    s += char(0x80 | (cp & 0x3F));
  } else {
    s += char(0xF0 | (cp >> 18));
    s += char(0x80 | ((cp >> 12) & 0x3F));
    s += char(0x80 | ((cp >> 6) & 0x3F));
    s += char(0x80 | (cp & 0x3F));
  }
  return s;
}

std::string random_letters(Rng& g, int lo, int hi)
{
  int const n = lo + int(g.below(uint64_t(hi - lo + 1)));
  std::string s;
  for (int i = 0; i < n; ++i) s += char('a' + g.below(26));
  return s;
}

// Latin-1 accented lower-case letters U+00E0..U+00FF except the division sign U+00F7
std::string random_latin1(Rng& g, int lo, int hi)
{
  int const n = lo + int(g.below(uint64_t(hi - lo + 1)));
  std::string s;
  for (int i = 0; i < n; ++i) {
    if (g.below(3) == 0) {
      uint32_t cp = 0xE0 + uint32_t(g.below(32));
      if (cp == 0xF7) cp = 0xE9;
      s += utf8(cp);
    } else {
      s += char('a' + g.below(26));
    }
  }
  return s;
}

constexpr uint32_t kCjkBase  = 0x4E00;
constexpr uint32_t kCjkCount = 3000;
const char* const kPunct[]   = {".", ",", ";", ":", "!", "?", "'", "\"", "(", ")", "-"};
constexpr int kPunctCount    = 11;

// kind 0: BERT-like ASCII vocabulary: [PAD] [UNK] [CLS] [SEP], a..z, ##a..##z, then unique random
//         2-8 letter stems (2 of 3) and "##" + 1-6 letter suffixes (1 of 3).
// kind 1: lexicon: unique random 2-10 letter words only.
// kind 2: multilingual: kind 0's head, punctuation, 3000 single CJK characters and their "##" forms,
//         then stems/suffixes that are ASCII (60 %), Latin-1 accented (25 %) or 2-3 CJK characters (15 %).
Vocab make_vocab(int kind, int64_t V, uint64_t seed)
{
  Vocab v;
  std::unordered_set<std::string> seen;
  auto add = [&](const std::string& s) {
    if (int64_t(v.size()) < V && seen.insert(s).second) v.add(s);
  };
  Rng g(seed, 0xABCDEFull + uint64_t(kind));
  if (kind != 1) {
    for (auto s : {"[PAD]", "[UNK]", "[CLS]", "[SEP]"}) add(s);
    for (char c = 'a'; c <= 'z'; ++c) add(std::string(1, c));
    for (char c = 'a'; c <= 'z'; ++c) add(std::string("##") + c);
  }
  if (kind == 2) {
    for (int i = 0; i < kPunctCount; ++i) add(kPunct[i]);
    for (uint32_t i = 0; i < kCjkCount; ++i) add(utf8(kCjkBase + i));
    for (uint32_t i = 0; i < kCjkCount; ++i) add("##" + utf8(kCjkBase + i));
    for (uint32_t cp = 0xE0; cp <= 0xFF; ++cp)
      if (cp != 0xF7) {
        add(utf8(cp));
        add("##" + utf8(cp));
      }
  }
  uint64_t n = 0;
  while (int64_t(v.size()) < V) {
    bool const suffix = (kind != 1) && (n++ % 3 == 2);
    std::string s;
    if (kind == 2) {
      double const u = g.uniform();
      if (u < 0.60) {
        s = suffix ? random_letters(g, 1, 6) : random_letters(g, 2, 8);
      } else if (u < 0.85) {
        s = suffix ? random_latin1(g, 1, 6) : random_latin1(g, 2, 8);
      } else {
        int const c = 2 + int(g.below(2));
        for (int i = 0; i < c; ++i) s += utf8(kCjkBase + uint32_t(g.below(kCjkCount)));
      }
    } else if (kind == 1) {
      s = random_letters(g, 2, 10);
    } else {
      s = suffix ? random_letters(g, 1, 6) : random_letters(g, 2, 8);
    }
    add(suffix ? "##" + s : s);
  }
  return v;
}

struct RowsConfig {
  int64_t rows;
  uint64_t seed;
  double mean_bytes;    // lognormal mean of the row length in bytes
  double sigma;         // lognormal sigma
  int64_t cap_bytes;    // hard cap on the row length
  int64_t min_bytes;    // rows shorter than this are regenerated at this target
  double zipf_s;        // Zipf exponent over the word list
  double p_oov;         // probability of a random out-of-vocabulary word
  double p_null;        // probability of a null row
  double p_empty;       // probability of an empty (valid) row
  int32_t words_lo;     // if > 0: the row is words_lo..words_hi words (uniform) instead of a byte target
  int32_t words_hi;
  int32_t oov_lo, oov_hi;  // length range of OOV random strings
  int32_t multilingual;    // 1: script mix 70/20/10 with punctuation words
  int32_t uniform_words;   // 1: words are uniform random 1..12 letter strings (config 1), no lexicon
};

struct WordList {
  std::vector<std::string> words;      // Zipf rank order = list order
  std::vector<std::string> latin, cjk; // multilingual only
  std::vector<double> cdf, cdf_latin, cdf_cjk;
};

std::vector<double> zipf_cdf(size_t n, double s)
{
  std::vector<double> c(n);
  double acc = 0;
  for (size_t i = 0; i < n; ++i) {
    acc += 1.0 / std::pow(double(i + 1), s);
    c[i] = acc;
  }
  for (auto& x : c) x /= acc;
  return c;
}

inline size_t sample(const std::vector<double>& cdf, double u)
{
  size_t const i = size_t(std::lower_bound(cdf.begin(), cdf.end(), u) - cdf.begin());
  return i < cdf.size() ? i : cdf.size() - 1;
}

bool is_ascii(const std::string& s)
{
  for (unsigned char c : s)
    if (c >= 0x80) return false;
  return true;
}

WordList make_wordlist(const uint8_t* chars, const int64_t* offsets, int64_t V, double s, bool multilingual)
{
  WordList w;
  for (int64_t i = 0; i < V; ++i) {
    std::string e(reinterpret_cast<const char*>(chars) + offsets[i], size_t(offsets[i + 1] - offsets[i]));
    if (e.empty() || e[0] == '[' || (e.size() >= 2 && e[0] == '#' && e[1] == '#')) continue;
    if (e.size() == 1) continue;  // single ASCII letters are pieces, not lexicon words
    if (!multilingual || is_ascii(e)) {
      bool punct = false;
      for (int k = 0; k < kPunctCount; ++k) punct |= (e == kPunct[k]);
      if (!punct) w.words.push_back(e);
    } else if ((unsigned char)e[0] >= 0xE0) {
      w.cjk.push_back(e);
    } else {
      w.latin.push_back(e);
    }
  }
  w.cdf = zipf_cdf(w.words.size(), s);
  if (multilingual) {
    w.cdf_latin = zipf_cdf(w.latin.size(), s);
    w.cdf_cjk   = zipf_cdf(w.cjk.size(), s);
  }
  return w;
}

void gen_word(const RowsConfig& c, const WordList& w, Rng& g, std::string& out)
{
  out.clear();
  if (c.uniform_words) {
    out = random_letters(g, 1, 12);
    return;
  }
  if (c.multilingual) {
    if (g.uniform() < 0.08) {
      out = kPunct[g.below(kPunctCount)];
      return;
    }
    double const u = g.uniform();
    if (g.uniform() < c.p_oov) {
      if (u < 0.7) out = random_letters(g, c.oov_lo, c.oov_hi);
      else if (u < 0.9) out = random_latin1(g, c.oov_lo, c.oov_hi);
      else {
        int const k = 1 + int(g.below(4));
        for (int i = 0; i < k; ++i) out += utf8(kCjkBase + uint32_t(g.below(kCjkCount + 500)));
      }
      return;
    }
    if (u < 0.7 || w.latin.empty() || w.cjk.empty()) out = w.words[sample(w.cdf, g.uniform())];
    else if (u < 0.9) out = w.latin[sample(w.cdf_latin, g.uniform())];
    else out = w.cjk[sample(w.cdf_cjk, g.uniform())];
    return;
  }
  if (g.uniform() < c.p_oov) {
    out = random_letters(g, c.oov_lo, c.oov_hi);
    return;
  }
  out = w.words[sample(w.cdf, g.uniform())];
}

struct RowsJob {
  RowsConfig cfg;
  WordList words;
  int nthreads;
  std::vector<std::string> part_chars;
  std::vector<std::vector<int64_t>> part_lens;  // -1 = null
  int64_t total_bytes = 0;
  int64_t nulls       = 0;
};

void gen_rows_range(RowsJob& job, int t, int64_t lo, int64_t hi)
{
  const RowsConfig& c = job.cfg;
  std::string& buf    = job.part_chars[size_t(t)];
  auto& lens          = job.part_lens[size_t(t)];
  lens.reserve(size_t(hi - lo));
  buf.reserve(size_t(double(hi - lo) * c.mean_bytes * 1.05) + 1024);
  double const mu = std::log(c.mean_bytes) - 0.5 * c.sigma * c.sigma;
  std::string word;
  for (int64_t r = lo; r < hi; ++r) {
    Rng g(c.seed, uint64_t(r));
    double const u = g.uniform();
    if (u < c.p_null) {
      lens.push_back(-1);
      continue;
    }
    if (u < c.p_null + c.p_empty) {
      lens.push_back(0);
      continue;
    }
    size_t const start = buf.size();
    if (c.words_lo > 0) {
      int const nw = c.words_lo + int(g.below(uint64_t(c.words_hi - c.words_lo + 1)));
      for (int i = 0; i < nw; ++i) {
        gen_word(c, job.words, g, word);
        if (i) buf += ' ';
        buf += word;
      }
    } else {
      double target = std::exp(mu + c.sigma * g.normal());
      if (target > double(c.cap_bytes)) target = double(c.cap_bytes);
      if (target < double(c.min_bytes)) target = double(c.min_bytes);
      int64_t const tb = int64_t(target);
      for (;;) {
        gen_word(c, job.words, g, word);
        int64_t const cur = int64_t(buf.size() - start);
        int64_t const add = int64_t(word.size()) + (cur ? 1 : 0);
        if (cur && cur + add > tb) break;
        if (cur) buf += ' ';
        buf += word;
        if (int64_t(buf.size() - start) >= tb) break;
      }
      // a first word longer than the cap is cut at a character boundary
      while (int64_t(buf.size() - start) > c.cap_bytes) {
        buf.pop_back();
        while (buf.size() > start && (uint8_t(buf.back()) & 0xC0) == 0x80) buf.pop_back();
        if (buf.size() > start && uint8_t(buf.back()) >= 0xC0) buf.pop_back();
      }
      while (buf.size() > start && buf.back() == ' ') buf.pop_back();
    }
    lens.push_back(int64_t(buf.size() - start));
  }
}

}  // namespace

extern "C" {

// ---- vocabulary / lexicon
void* datagen_vocab_create(int kind, int64_t V, uint64_t seed, int64_t* nchars)
{
  auto* v = new Vocab(make_vocab(kind, V, seed));
  *nchars = int64_t(v->chars.size());
  return v;
}

void datagen_vocab_finish(void* h, uint8_t* chars, int64_t* offsets)
{
  auto* v = static_cast<Vocab*>(h);
  if (!v->chars.empty()) std::memcpy(chars, v->chars.data(), v->chars.size());
  std::memcpy(offsets, v->offsets.data(), v->offsets.size() * sizeof(int64_t));
  delete v;
}

// ---- rows.  `lex_*`: the vocabulary / lexicon the words are drawn from (host buffers, int64 offsets).
void* datagen_rows_begin(const RowsConfig* cfg, const uint8_t* lex_chars, const int64_t* lex_offsets, int64_t lex_size, int nthreads,
                         int64_t* total_bytes, int64_t* null_count)
{
  auto* job     = new RowsJob;
  job->cfg      = *cfg;
  job->nthreads = std::max(1, nthreads);
  if (!cfg->uniform_words) job->words = make_wordlist(lex_chars, lex_offsets, lex_size, cfg->zipf_s, cfg->multilingual != 0);
  job->part_chars.resize(size_t(job->nthreads));
  job->part_lens.resize(size_t(job->nthreads));
  std::vector<std::thread> ts;
  for (int t = 0; t < job->nthreads; ++t) {
    int64_t const lo = cfg->rows * t / job->nthreads, hi = cfg->rows * (t + 1) / job->nthreads;
    ts.emplace_back([=] { gen_rows_range(*job, t, lo, hi); });
  }
  for (auto& t : ts) t.join();
  for (int t = 0; t < job->nthreads; ++t) {
    job->total_bytes += int64_t(job->part_chars[size_t(t)].size());
    for (auto l : job->part_lens[size_t(t)]) job->nulls += (l < 0);
  }
  *total_bytes = job->total_bytes;
  *null_count  = job->nulls;
  return job;
}

// chars: total_bytes; offsets: rows+1 int64; mask: ceil(rows/32) uint32 words (may be NULL when there are no nulls)
void datagen_rows_finish(void* h, uint8_t* chars, int64_t* offsets, uint32_t* mask)
{
  auto* job    = static_cast<RowsJob*>(h);
  int64_t row  = 0, pos = 0;
  int64_t const words = (job->cfg.rows + 31) / 32;
  if (mask)
    for (int64_t i = 0; i < words; ++i) mask[i] = 0;
  for (int t = 0; t < job->nthreads; ++t) {
    auto const& buf = job->part_chars[size_t(t)];
    if (!buf.empty()) std::memcpy(chars + pos, buf.data(), buf.size());
    for (auto l : job->part_lens[size_t(t)]) {
      offsets[row] = pos;
      if (l >= 0) {
        pos += l;
        if (mask) mask[row >> 5] |= 1u << (row & 31);
      }
      ++row;
    }
    std::string().swap(job->part_chars[size_t(t)]);
  }
  offsets[row] = pos;
  delete job;
}

}  // extern "C"

// Exercises the C++ mirror of the nvtext API (cudf_amd/include) on the GPU with the cases of the
// reference's gtests: cpp/tests/text/minhash_tests.cpp (Permuted, PermutedWide, EmptyTest, ErrorsTest, Ngrams, NgramsWide,
// NgramsSliced), cpp/tests/text/jaccard_tests.cpp (Basic, WithNulls, Errors)
// cpp/tests/text/normalize_tests.cpp (NormalizeEmptyTest, AllNullStrings, SomeNullStrings, WithNormalizer, SpecialTokens,
// NormalizeSlicedColumn) and cpp/tests/text/subword_tests.cpp (all seven).  Own tiny harness: prints one line per case and
// exits non-zero on the first failure.
#include <cudf/column/column.hpp>
#include <cudf/lists/lists_column_view.hpp>
#include <cudf/strings/strings_column_view.hpp>
#include <hip/hip_runtime.h>
#include <nvtext/jaccard.hpp>
#include <nvtext/minhash.hpp>
#include <nvtext/normalize.hpp>
#include <nvtext/wordpiece_tokenize.hpp>

#include <cstdio>
#include <cstdlib>
#include <optional>
#include <string>
#include <vector>

#define HIP_OK(x)                                                                    \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                                  \
    }                                                                                \
  } while (0)

static int g_failures = 0;
#define CHECK(cond)                                                     \
  do {                                                                  \
    if (!(cond)) {                                                      \
      std::printf("  FAILED: %s (%s:%d)\n", #cond, __FILE__, __LINE__); \
      ++g_failures;                                                     \
    }                                                                   \
  } while (0)
#define EXPECT_THROW(stmt, type)                                                     \
  do {                                                                               \
    bool thrown_ = false;                                                            \
    try { stmt; } catch (type const&) { thrown_ = true; } catch (...) {}             \
    if (!thrown_) { std::printf("  FAILED: expected " #type " from " #stmt "\n"); ++g_failures; } \
  } while (0)

using Text = std::optional<std::string>;

// Device memory owned by the test, freed at exit.
static std::vector<void*> g_allocs;
template <typename T>
T* upload(std::vector<T> const& h)
{
  void* d = nullptr;
  HIP_OK(hipMalloc(&d, std::max<size_t>(h.size() * sizeof(T), 16)));
  if (!h.empty()) HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
  g_allocs.push_back(d);
  return static_cast<T*>(d);
}

// strings column as cudf::test::strings_column_wrapper builds it (null rows are zero-length)
struct StringsColumn {
  cudf::column_view view;
};
StringsColumn make_strings(std::vector<Text> const& rows)
{
  std::vector<char> chars;
  std::vector<int32_t> offsets{0};
  std::vector<uint32_t> mask((rows.size() + 31) / 32, 0);
  int nulls = 0;
  for (size_t i = 0; i < rows.size(); ++i) {
    if (rows[i]) {
      chars.insert(chars.end(), rows[i]->begin(), rows[i]->end());
      mask[i / 32] |= 1u << (i % 32);
    } else {
      ++nulls;
    }
    offsets.push_back(static_cast<int32_t>(chars.size()));
  }
  using namespace cudf;
  if (rows.empty()) return {column_view{data_type{type_id::STRING}, 0, nullptr, nullptr, 0}};  // childless empty column
  column_view off{data_type{type_id::INT32}, static_cast<size_type>(offsets.size()), upload(offsets), nullptr, 0};
  return {column_view{data_type{type_id::STRING}, static_cast<size_type>(rows.size()), upload(chars), nulls ? upload(mask) : nullptr,
                      nulls, 0, {off}}};
}
cudf::column_view slice(cudf::column_view const& c, int lo, int hi)  // cudf::slice on a column without nulls
{
  std::vector<cudf::column_view> kids;
  for (int i = 0; i < c.num_children(); ++i) kids.push_back(c.child(i));
  return cudf::column_view{c.type(), hi - lo, c.head<void>(), c.null_mask(), 0, c.offset() + lo, kids};
}
template <typename T>
cudf::column_view make_fixed(std::vector<T> const& v)
{
  return cudf::column_view{cudf::data_type{cudf::type_to_id<T>()}, static_cast<cudf::size_type>(v.size()), upload(v), nullptr, 0};
}

template <typename T>
struct HostList {
  std::vector<std::optional<std::vector<T>>> rows;
};
template <typename T>
HostList<T> download(cudf::column const& col)
{
  HIP_OK(hipDeviceSynchronize());
  HostList<T> out;
  cudf::lists_column_view lv(col.view());
  int const n = lv.size();
  std::vector<int32_t> off(lv.offsets().size());
  if (!off.empty()) HIP_OK(hipMemcpy(off.data(), lv.offsets().head<void>(), off.size() * 4, hipMemcpyDeviceToHost));
  std::vector<T> child(lv.child().size());
  if (!child.empty()) HIP_OK(hipMemcpy(child.data(), lv.child().head<void>(), child.size() * sizeof(T), hipMemcpyDeviceToHost));
  std::vector<uint32_t> mask((n + 31) / 32, 0xFFFFFFFFu);
  if (lv.null_mask() && n) HIP_OK(hipMemcpy(mask.data(), lv.null_mask(), mask.size() * 4, hipMemcpyDeviceToHost));
  for (int i = 0; i < n; ++i) {
    if (!((mask[i / 32] >> (i % 32)) & 1u)) {
      out.rows.emplace_back(std::nullopt);
    } else {
      out.rows.emplace_back(std::vector<T>(child.begin() + off[i], child.begin() + off[i + 1]));
    }
  }
  return out;
}
template <typename T>
bool same(HostList<T> const& got, std::vector<std::optional<std::vector<T>>> const& exp)
{
  if (got.rows.size() != exp.size()) return false;
  for (size_t i = 0; i < exp.size(); ++i) {
    if (got.rows[i].has_value() != exp[i].has_value()) return false;
    if (exp[i] && *got.rows[i] != *exp[i]) return false;
  }
  return true;
}
template <typename T>
using L = std::vector<std::optional<std::vector<T>>>;

void test_minhash_permuted()
{
  std::printf("MinHashTest.Permuted\n");
  auto input = make_strings({"doc 1", "this is doc 2", "doc 3", "d", "The quick brown fox jump\xC3\xA9" "d over the lazy brown dog.",
                             "line six", "line seven", "line eight", "line nine", "line ten"});
  auto view  = cudf::strings_column_view(input.view);
  auto params = make_fixed<uint32_t>({10, 11, 12});
  auto results = nvtext::minhash(view, 0, params, params, 4);
  L<uint32_t> expected{{{1392101586u, 394869177u, 811528444u}}, {{211415830u, 187088503u, 130291444u}},
                       {{2098117052u, 394869177u, 799753544u}}, {{2264583304u, 2920538364u, 3576493424u}},
                       {{253327882u, 41747273u, 302030804u}},   {{2109809594u, 1017470651u, 326988172u}},
                       {{1303819864u, 850676747u, 147107852u}}, {{736021564u, 720812292u, 1405158760u}},
                       {{902780242u, 134064807u, 1613944636u}}, {{547084870u, 1748895564u, 656501844u}}};
  CHECK(same(download<uint32_t>(*results), expected));
  CHECK(results->type().id() == cudf::type_id::LIST && results->child(1).type().id() == cudf::type_id::UINT32);
  auto params64  = make_fixed<uint64_t>({10, 11, 12});
  auto results64 = nvtext::minhash64(view, 0, params64, params64, 4);
  L<uint64_t> expected64{{{827364888116975697ul, 1601854279692781452ul, 70500662054893256ul}},
                         {{18312093741021833ul, 133793446674258329ul, 21974512489226198ul}},
                         {{22474244732520567ul, 1638811775655358395ul, 949306297364502264ul}},
                         {{1332357434996402861ul, 2157346081260151330ul, 676491718310205848ul}},
                         {{65816830624808020ul, 43323600380520789ul, 63511816333816345ul}},
                         {{629657184954525200ul, 49741036507643002ul, 97466271004074331ul}},
                         {{301611977846331113ul, 101188874709594830ul, 97466271004074331ul}},
                         {{121498891461700668ul, 171065800427907402ul, 97466271004074331ul}},
                         {{54617739511834072ul, 231454301607238929ul, 97466271004074331ul}},
                         {{576418665851990314ul, 231454301607238929ul, 97466271004074331ul}}};
  CHECK(same(download<uint64_t>(*results64), expected64));
}

void test_minhash_wide()
{
  std::printf("MinHashTest.PermutedWide\n");
  auto input  = make_strings({std::string(2 << 10, 'x'), std::string(2 << 19, 'y')});
  auto view   = cudf::strings_column_view(input.view);
  auto params = make_fixed<uint32_t>({20, 21, 22});
  L<uint32_t> expected{{{1731998032u, 315359380u, 3193688024u}}, {{1293098788u, 2860992281u, 133918478u}}};
  CHECK(same(download<uint32_t>(*nvtext::minhash(view, 0, params, params, 4)), expected));
  auto params64 = make_fixed<uint64_t>({20, 21, 22});
  L<uint64_t> expected64{{{1818322427062143853ul, 641024893347719371ul, 1769570368846988848ul}},
                         {{1389920339306667795ul, 421787002125838902ul, 1759496674158703968ul}}};
  CHECK(same(download<uint64_t>(*nvtext::minhash64(view, 0, params64, params64, 4)), expected64));
}

void test_minhash_empty_and_errors()
{
  std::printf("MinHashTest.EmptyTest / ErrorsTest\n");
  auto empty  = make_strings({});
  auto eview  = cudf::strings_column_view(empty.view);
  auto params = make_fixed<uint32_t>({1, 2, 3});
  CHECK(nvtext::minhash(eview, 0, params, params, 4)->size() == 0);
  auto params64 = make_fixed<uint64_t>({1, 2, 3});
  CHECK(nvtext::minhash64(eview, 0, params64, params64, 4)->size() == 0);

  auto input = make_strings({"this string intentionally left blank"});
  auto view  = cudf::strings_column_view(input.view);
  auto none  = make_fixed<uint32_t>({});
  auto none64 = make_fixed<uint64_t>({});
  EXPECT_THROW(nvtext::minhash(view, 0, none, none, 0), std::invalid_argument);
  EXPECT_THROW(nvtext::minhash64(view, 0, none64, none64, 0), std::invalid_argument);
  EXPECT_THROW(nvtext::minhash(view, 0, none, none, 4), std::invalid_argument);
  EXPECT_THROW(nvtext::minhash64(view, 0, none64, none64, 4), std::invalid_argument);
  // a column of the wrong type does not convert to the span (column_view.hpp:445-452)
  EXPECT_THROW(nvtext::minhash(view, 0, params64, params64, 4), cudf::logic_error);

  std::vector<Text> blanks(50000, std::string());
  auto big    = make_strings(blanks);
  auto bview  = cudf::strings_column_view(big.view);
  auto zeros  = make_fixed<uint32_t>(std::vector<uint32_t>(50000, 0));
  auto zeros64 = make_fixed<uint64_t>(std::vector<uint64_t>(50000, 0));
  EXPECT_THROW(nvtext::minhash(bview, 0, zeros, zeros, 4), std::overflow_error);
  EXPECT_THROW(nvtext::minhash64(bview, 0, zeros64, zeros64, 4), std::overflow_error);
}

// lists column of strings as cudf::test::lists_column_wrapper<cudf::string_view> builds it
cudf::column_view make_list_strings(std::vector<std::vector<Text>> const& rows)
{
  using namespace cudf;
  std::vector<Text> flat;
  std::vector<int32_t> offsets{0};
  for (auto const& r : rows) {
    flat.insert(flat.end(), r.begin(), r.end());
    offsets.push_back(static_cast<int32_t>(flat.size()));
  }
  if (rows.empty()) return column_view{data_type{type_id::LIST}, 0, nullptr, nullptr, 0};
  column_view off{data_type{type_id::INT32}, static_cast<size_type>(offsets.size()), upload(offsets), nullptr, 0};
  return column_view{data_type{type_id::LIST}, static_cast<size_type>(rows.size()), nullptr, nullptr, 0, 0, {off, make_strings(flat).view}};
}

void test_minhash_ngrams()
{
  std::printf("minhash_ngrams (Ngrams, NgramsWide, NgramsSliced, errors)\n");
  std::vector<Text> const row_a{"The", "quick", "brown", "fox", "jump\xc3\xa9" "d", "over", "the", "lazy", "brown", "dog."};
  std::vector<Text> const row_b{"The", "quick", "brown", "fox", "jump\xc3\xa9" "d", "over", "the", "lazy", "", "dog."};
  std::vector<Text> const row_c{"short", "row"};
  std::vector<Text> const ignored{"ignored", "row"};
  std::vector<uint32_t> const p32{10, 11, 12};
  std::vector<uint64_t> const p64{10, 11, 12};
  auto const a32 = make_fixed(p32);
  auto const a64 = make_fixed(p64);
  L<uint32_t> const e32{{{230924604u, 55492793u, 963436400u}}, {{230924604u, 367515795u, 963436400u}}, {{2380648568u, 1330223236u, 279797904u}}};
  L<uint64_t> const e64{{{208926840193078200ul, 576399628675212695ul, 312927673584437419ul}},
                        {{677038498284219393ul, 326338087730412201ul, 298455901014050223ul}},
                        {{1493265692486268500ul, 720255058049417768ul, 2253087432826260995ul}}};
  {
    auto const input = make_list_strings({row_a, row_b, row_c});
    cudf::lists_column_view view(input);
    CHECK(same(download<uint32_t>(*nvtext::minhash_ngrams(view, 4, 0, a32, a32)), e32));
    CHECK(same(download<uint64_t>(*nvtext::minhash64_ngrams(view, 4, 0, a64, a64)), e64));
  }
  {
    auto const input = make_list_strings({ignored, row_a, row_b, row_c, ignored});
    cudf::lists_column_view view(slice(input, 1, 4));
    CHECK(same(download<uint32_t>(*nvtext::minhash_ngrams(view, 4, 0, a32, a32)), e32));
    CHECK(same(download<uint64_t>(*nvtext::minhash64_ngrams(view, 4, 0, a64, a64)), e64));
  }
  {
    std::vector<Text> const many(512, Text{"hello"});
    auto const input = make_list_strings({many, many});
    cudf::lists_column_view view(input);
    L<uint32_t> const w32{{{571536396u, 2346676954u, 4121817512u}}, {{571536396u, 2346676954u, 4121817512u}}};
    L<uint64_t> const w64{{{1947142336021414174ul, 1219519365938078011ul, 491896395854741840ul}},
                          {{1947142336021414174ul, 1219519365938078011ul, 491896395854741840ul}}};
    CHECK(same(download<uint32_t>(*nvtext::minhash_ngrams(view, 4, 0, a32, a32)), w32));
    CHECK(same(download<uint64_t>(*nvtext::minhash64_ngrams(view, 4, 0, a64, a64)), w64));
  }
  {
    auto const empty_list = make_list_strings({});
    cudf::lists_column_view lview(empty_list);
    auto const e  = make_fixed(std::vector<uint32_t>{});
    auto const ee = make_fixed(std::vector<uint64_t>{});
    EXPECT_THROW(nvtext::minhash_ngrams(lview, 0, 0, e, e), std::invalid_argument);
    EXPECT_THROW(nvtext::minhash64_ngrams(lview, 0, 0, ee, ee), std::invalid_argument);
    EXPECT_THROW(nvtext::minhash_ngrams(lview, 4, 0, e, e), std::invalid_argument);
    EXPECT_THROW(nvtext::minhash64_ngrams(lview, 4, 0, ee, ee), std::invalid_argument);
    CHECK(nvtext::minhash_ngrams(lview, 4, 0, a32, a32)->size() == 0);
    CHECK(nvtext::minhash64_ngrams(lview, 4, 0, a64, a64)->size() == 0);
    std::vector<std::vector<Text>> const big(50000, std::vector<Text>{Text{""}});
    auto const input = make_list_strings(big);
    cudf::lists_column_view view(input);
    auto const z32 = make_fixed(std::vector<uint32_t>(50000, 0u));
    auto const z64 = make_fixed(std::vector<uint64_t>(50000, 0ul));
    EXPECT_THROW(nvtext::minhash_ngrams(view, 4, 0, z32, z32), std::overflow_error);
    EXPECT_THROW(nvtext::minhash64_ngrams(view, 4, 0, z64, z64), std::overflow_error);
  }
}

void test_jaccard()
{
  std::printf("JaccardTest.Basic / WithNulls / Errors\n");
  auto fetch = [](cudf::column const& col, std::vector<float>& values, std::vector<bool>& valid) {
    HIP_OK(hipDeviceSynchronize());
    auto const v = col.view();
    values.assign(v.size(), 0.f);
    if (v.size()) HIP_OK(hipMemcpy(values.data(), v.head<void>(), v.size() * sizeof(float), hipMemcpyDeviceToHost));
    std::vector<uint32_t> mask((v.size() + 31) / 32, 0xFFFFFFFFu);
    if (v.null_mask() && v.size()) HIP_OK(hipMemcpy(mask.data(), v.null_mask(), mask.size() * 4, hipMemcpyDeviceToHost));
    valid.clear();
    for (int i = 0; i < v.size(); ++i) valid.push_back((mask[i / 32] >> (i % 32)) & 1u);
  };
  std::vector<float> values;
  std::vector<bool> valid;
  {
    auto input1 = make_strings({"the quick brown fox", "jumped over the lazy dog."});
    auto input2 = make_strings({"the slowest brown cat", "crawled under the jumping fox"});
    cudf::strings_column_view view1(input1.view), view2(input2.view);
    auto results = nvtext::jaccard_index(view1, view2, 5);
    fetch(*results, values, valid);
    CHECK(results->type().id() == cudf::type_id::FLOAT32 && results->null_count() == 0);
    CHECK(values == (std::vector<float>{0.103448279f, 0.0697674453f}));
    fetch(*nvtext::jaccard_index(view1, view1, 5), values, valid);
    CHECK(values == (std::vector<float>{1.0f, 1.0f}));
    fetch(*nvtext::jaccard_index(view2, view2, 10), values, valid);
    CHECK(values == (std::vector<float>{1.0f, 1.0f}));
  }
  {
    auto input1 = make_strings({"brown fox", "jumps over dog", std::nullopt, ""});
    auto input2 = make_strings({"brown cat", "jumps on fox", "", std::nullopt});
    cudf::strings_column_view view1(input1.view), view2(input2.view);
    auto results = nvtext::jaccard_index(view1, view2, 5);
    fetch(*results, values, valid);
    CHECK(values[0] == 0.25f && values[1] == 0.200000003f);
    CHECK(valid == (std::vector<bool>{true, true, false, false}) && results->null_count() == 2);
    results = nvtext::jaccard_index(view1, view1, 7);
    fetch(*results, values, valid);
    CHECK(values[0] == 1.0f && values[1] == 1.0f && values[3] == 0.f);
    CHECK(valid == (std::vector<bool>{true, true, false, true}) && results->null_count() == 1);
  }
  {
    auto input  = make_strings({"1", "2", "3"});
    auto input2 = make_strings({"1", "2"});
    cudf::strings_column_view view(input.view), view2(input2.view);
    EXPECT_THROW(nvtext::jaccard_index(view, view, 1), std::invalid_argument);
    EXPECT_THROW(nvtext::jaccard_index(view, view2, 5), std::invalid_argument);
  }
}

// rows of a STRING column, nullopt for nulls
std::vector<Text> download_strings(cudf::column const& col)
{
  HIP_OK(hipDeviceSynchronize());
  auto const v = col.view();
  int const n  = v.size();
  std::vector<Text> rows;
  if (n == 0) return rows;
  std::vector<int32_t> off(n + 1);
  HIP_OK(hipMemcpy(off.data(), v.child(0).head<void>(), off.size() * 4, hipMemcpyDeviceToHost));
  std::vector<char> chars(off[n]);
  if (!chars.empty()) HIP_OK(hipMemcpy(chars.data(), v.head<void>(), chars.size(), hipMemcpyDeviceToHost));
  std::vector<uint32_t> mask((n + 31) / 32, 0xFFFFFFFFu);
  if (v.null_mask()) HIP_OK(hipMemcpy(mask.data(), v.null_mask(), mask.size() * 4, hipMemcpyDeviceToHost));
  for (int i = 0; i < n; ++i) {
    if ((mask[i / 32] >> (i % 32)) & 1u) rows.emplace_back(std::string(chars.begin() + off[i], chars.begin() + off[i + 1]));
    else rows.emplace_back(std::nullopt);
  }
  return rows;
}

void test_normalize()
{
  std::printf("TextNormalizeTest.NormalizeEmptyTest / AllNullStrings / SomeNullStrings / WithNormalizer / SpecialTokens / NormalizeSlicedColumn\n");
  std::string const long_row = "this entry is intended to pad out past 256 bytes which is currently the block size";
  {
    auto empty      = make_strings({});
    auto normalizer = nvtext::create_character_normalizer(true);
    CHECK(nvtext::normalize_characters(cudf::strings_column_view(empty.view), *normalizer)->size() == 0);
    auto nulls   = make_strings({std::nullopt, std::nullopt, std::nullopt});
    auto results = nvtext::normalize_characters(cudf::strings_column_view(nulls.view), *normalizer);
    CHECK(download_strings(*results) == (std::vector<Text>{std::nullopt, std::nullopt, std::nullopt}) && results->null_count() == 3);
    auto some = make_strings({std::nullopt, ".", "a"});
    results   = nvtext::normalize_characters(cudf::strings_column_view(some.view), *normalizer);
    CHECK(download_strings(*results) == (std::vector<Text>{std::nullopt, " . ", "a"}));
  }
  {
    auto input = make_strings({"abc\xC2\xA3" "def", std::nullopt, "\xC3\xA9\xC3\xA8 \xC3\xA2 \xC3\xAE\xC3\xB4\taeio",
                               "\t\xC4\x82\xC4\x86\xC4\x96\xC3\x91  \xC3\x9C", "ACEN U", "P^NP", "$41.07", "[a,b]",
                               "\xE4\xB8\x8F\xE4\xB8\x9F", "", long_row, long_row, long_row});
    cudf::strings_column_view sv(input.view);
    auto normalizer = nvtext::create_character_normalizer(true);
    std::vector<Text> const lower{"abc\xC2\xA3" "def", std::nullopt, "ee a io aeio", " acen  u", "acen u", "p ^ np", " $ 41 . 07", " [ a , b ] ",
                                  " \xE4\xB8\x8F  \xE4\xB8\x9F ", "", long_row, long_row, long_row};
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == lower);
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == lower);  // normalizer re-use
    normalizer = nvtext::create_character_normalizer(false);
    std::vector<Text> const keep{"abc\xC2\xA3" "def", std::nullopt, "\xC3\xA9\xC3\xA8 \xC3\xA2 \xC3\xAE\xC3\xB4 aeio",
                                 " \xC4\x82\xC4\x86\xC4\x96\xC3\x91  \xC3\x9C", "ACEN U", "P ^ NP", " $ 41 . 07", " [ a , b ] ",
                                 " \xE4\xB8\x8F  \xE4\xB8\x9F ", "", long_row, long_row, long_row};
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == keep);
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == keep);
  }
  {
    auto input  = make_strings({"[BOS]Some strings with [PAD] special[SEP]tokens[EOS]", "[bos]these should[sep]work for lowercase[eos]",
                                "some[non]tokens[eol]too", long_row, long_row, long_row});
    auto tokens = make_strings({"[BOS]", "[EOS]", "[SEP]", "[PAD]"});
    cudf::strings_column_view sv(input.view), stv(tokens.view);
    auto normalizer = nvtext::create_character_normalizer(true, stv);
    std::vector<Text> const lower{" [BOS] some strings with  [PAD]  special [SEP] tokens [EOS] ", " [BOS] these should [SEP] work for lowercase [EOS] ",
                                  "some [ non ] tokens [ eol ] too", long_row, long_row, long_row};
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == lower);
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == lower);
    normalizer = nvtext::create_character_normalizer(false, stv);
    std::vector<Text> const keep{" [BOS] Some strings with  [PAD]  special [SEP] tokens [EOS] ",
                                 " [ bos ] these should [ sep ] work for lowercase [ eos ] ", "some [ non ] tokens [ eol ] too", long_row, long_row,
                                 long_row};
    CHECK(download_strings(*nvtext::normalize_characters(sv, *normalizer)) == keep);
    auto with_null = make_strings({"[PAD]", std::nullopt});
    EXPECT_THROW(nvtext::create_character_normalizer(true, cudf::strings_column_view(with_null.view)), std::invalid_argument);
  }
  {
    auto input = make_strings({"abc\xC2\xA3" "def", "\xC3\xA9\xC3\xA8 \xC3\xA2 \xC3\xAE\xC3\xB4\taeio", "ACEN U", "P^NP", "$41.07", "[a,b]",
                               "\xE4\xB8\x8F\xE4\xB8\x9F"});
    auto normalizer = nvtext::create_character_normalizer(true);
    auto results    = nvtext::normalize_characters(cudf::strings_column_view(slice(input.view, 0, 4)), *normalizer);
    CHECK(download_strings(*results) == (std::vector<Text>{"abc\xC2\xA3" "def", "ee a io aeio", "acen u", "p ^ np"}));
    normalizer = nvtext::create_character_normalizer(false);
    results    = nvtext::normalize_characters(cudf::strings_column_view(slice(input.view, 4, 7)), *normalizer);
    CHECK(download_strings(*results) == (std::vector<Text>{" $ 41 . 07", " [ a , b ] ", " \xE4\xB8\x8F  \xE4\xB8\x9F "}));
  }
}

void test_wordpiece()
{
  std::printf("TextSubwordTest.WordPiece / WordPieceSliced\n");
  auto vocabulary = make_strings({"ate", "brown", "cheese", "dog", "fox", "jumped", "lazy", "quick", "over", "the", "[UNK]"});
  auto vocab      = nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(vocabulary.view));
  auto input = make_strings({"the quick brown fox jumped over", "the  lazy  brown  dog",
                             " ate brown cheese dog fox jumped lazy quick over the [UNK] "});
  auto sv    = cudf::strings_column_view(input.view);
  L<int32_t> expected{{{9, 7, 1, 4, 5, 8}}, {{9, 6, 1, 3}}, {{0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10}}};
  L<int32_t> expected5{{{9, 7, 1, 4, 5}}, {{9, 6, 1, 3}}, {{0, 1, 2, 3, 4}}};
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab)), expected));
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab, 5)), expected5));

  auto wide = make_strings({" ate the cheese dog quick over  lazy day ", "the quick brown fox jumped over", "the  lazy  brown  dog",
                            " ate brown cheese dog fox jumped lazy quick over the [UNK] ", " ate the cheese dog quick over  lazy day "});
  auto sliced = cudf::strings_column_view(slice(wide.view, 1, 4));
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sliced, *vocab)), expected));
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sliced, *vocab, 5)), expected5));
}

void test_wordpiece_subwords()
{
  std::printf("TextSubwordTest.WordPieceWithSubwords\n");
  auto vocabulary = make_strings({"", "[UNK]", "!", "a", "I", "G", "have", "##P", "##U"});
  auto vocab      = nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(vocabulary.view));
  auto input      = make_strings({"I have a GPU ! ", "do not have a gpu", "no gpu"});
  auto sv         = cudf::strings_column_view(input.view);
  L<int32_t> expected{{{4, 6, 3, 5, 7, 8, 2}}, {{1, 1, 6, 3, 1}}, {{1, 1}}};
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab)), expected));
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab, 6)), expected));  // max applies to words, not tokens
  L<int32_t> expected4{{{4, 6, 3, 5, 7, 8}}, {{1, 1, 6, 3}}, {{1, 1}}};
  CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab, 4)), expected4));
}

void test_wordpiece_edges()
{
  std::printf("TextSubwordTest.WordPieceEmpty / AllNulls / NoTokens / Errors\n");
  {
    auto vocabulary = make_strings({""});
    auto vocab      = nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(vocabulary.view));
    auto empty      = make_strings({});
    auto sv         = cudf::strings_column_view(empty.view);
    CHECK(nvtext::wordpiece_tokenize(sv, *vocab)->size() == 0);
    CHECK(nvtext::wordpiece_tokenize(sv, *vocab, 10)->size() == 0);
    auto nulls = make_strings({std::nullopt, std::nullopt, std::nullopt});
    auto nv    = cudf::strings_column_view(nulls.view);
    L<int32_t> all_null{std::nullopt, std::nullopt, std::nullopt};
    auto r = nvtext::wordpiece_tokenize(nv, *vocab);
    CHECK(same(download<int32_t>(*r), all_null));
    CHECK(r->null_count() == 3);
    CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(nv, *vocab, 10)), all_null));
  }
  {
    auto vocabulary = make_strings({"x"});
    auto vocab      = nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(vocabulary.view));
    auto input      = make_strings({"  ", " www ", "xxxx"});
    auto sv         = cudf::strings_column_view(input.view);
    L<int32_t> expected{{{}}, {{-1}}, {{-1}}};  // -1: no [UNK] in the vocabulary
    CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab)), expected));
    CHECK(same(download<int32_t>(*nvtext::wordpiece_tokenize(sv, *vocab, 10)), expected));
    auto blank = make_strings({"  "});
    EXPECT_THROW(nvtext::wordpiece_tokenize(cudf::strings_column_view(blank.view), *vocab, -1), std::invalid_argument);
  }
  auto empty = make_strings({});
  EXPECT_THROW(nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(empty.view)), std::invalid_argument);
  auto nulls = make_strings({std::nullopt, std::nullopt, std::nullopt});
  EXPECT_THROW(nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(nulls.view)), std::invalid_argument);
}

// A memory resource that counts what is out: the vocabulary and the normalizer must take their tables from the
// resource given to them and give every byte back when they die, as results and temporaries do.
struct CountingResource final : rmm::mr::device_memory_resource {
  long live_buffers = 0, live_bytes = 0, requests = 0;
  void* allocate_async(std::size_t bytes, cuda::stream_ref) override
  {
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) return nullptr;
    ++live_buffers, ++requests, live_bytes += static_cast<long>(bytes);
    return p;
  }
  void deallocate_async(void* p, std::size_t bytes, cuda::stream_ref) noexcept override
  {
    (void)hipDeviceSynchronize();
    (void)hipFree(p);
    --live_buffers, live_bytes -= static_cast<long>(bytes);
  }
};

void test_objects_use_the_callers_resource()
{
  std::printf("objects take their tables from the caller's memory resource\n");
  CountingResource mr;
  {
    auto vocabulary = make_strings({"ate", "brown", "cheese", "dog", "fox", "jumped", "lazy", "quick", "over", "the", "[UNK]"});
    auto vocab      = nvtext::load_wordpiece_vocabulary(cudf::strings_column_view(vocabulary.view), cudf::get_default_stream(), mr);
    CHECK(mr.live_buffers >= 1 && mr.live_bytes > 0);
    long const held = mr.live_bytes;
    auto input      = make_strings({"the quick brown fox jumped over the lazy dog", "the quick brown fox quacked"});
    {
      auto result = nvtext::wordpiece_tokenize(cudf::strings_column_view(input.view), *vocab, 0, cudf::get_default_stream(), mr);
      L<int32_t> expected{{{9, 7, 1, 4, 5, 8, 9, 6, 3}}, {{9, 7, 1, 4, 10}}};
      CHECK(same(download<int32_t>(*result), expected));
      CHECK(mr.live_bytes > held);
    }
    CHECK(mr.live_bytes == held);  // the result and the temporaries are back, the tables are not
  }
  CHECK(mr.live_buffers == 0 && mr.live_bytes == 0);
  {
    auto normalizer = nvtext::create_character_normalizer(true, nvtext::detail::no_special_tokens(), cudf::get_default_stream(), mr);
    CHECK(mr.live_bytes > 14000000);  // the code point tables
    long const held = mr.live_bytes;
    auto input      = make_strings({"Hello, World"});
    {
      auto result = nvtext::normalize_characters(cudf::strings_column_view(input.view), *normalizer, cudf::get_default_stream(), mr);
      CHECK(download_strings(*result) == std::vector<Text>{Text{"hello ,  world"}});
    }
    CHECK(mr.live_bytes == held);
  }
  CHECK(mr.live_buffers == 0 && mr.live_bytes == 0);
}

int main()
{
  int devices = 0;
  if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
    std::printf("no GPU\n");
    return 77;
  }
  test_minhash_permuted();
  test_minhash_wide();
  test_minhash_empty_and_errors();
  test_minhash_ngrams();
  test_jaccard();
  test_normalize();
  test_wordpiece();
  test_wordpiece_subwords();
  test_wordpiece_edges();
  test_objects_use_the_callers_resource();
  HIP_OK(hipDeviceSynchronize());
  for (void* p : g_allocs) (void)hipFree(p);
  std::printf(g_failures ? "FAILED (%d checks)\n" : "ALL PASSED\n", g_failures);
  return g_failures ? 1 : 0;
}

/*
 * nvtext_amd.h -- C ABI of the MI355X (gfx950) implementation of libcudf's nvtext
 * text-dedup hot path: minhash / minhash64 over character windows and
 * wordpiece_tokenize with its wordpiece_vocabulary, plus the calls either side of them
 * (minhash_ngrams, jaccard_index, normalize_characters).
 *
 * Plain pointers and sizes only.  Every pointer named "device" is HIP device memory
 * that must stay valid until the work queued on `stream` has completed.  All work is
 * queued on the caller's stream; results are valid once that stream is synchronised
 * (wordpiece_tokenize synchronises it once internally to learn the token total).
 *
 * Each entry point cites the reference interface it replaces (paths relative to the
 * cudf source tree).
 */
#ifndef NVTEXT_AMD_H
#define NVTEXT_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  The C++ shim rethrows them as the reference's exception types
 * (cpp/include/cudf/utilities/error.hpp:35-103,182-199,280-284). */
typedef enum nvtext_amd_status {
  NVTEXT_AMD_SUCCESS          = 0,
  NVTEXT_AMD_INVALID_ARGUMENT = 1, /* std::invalid_argument */
  NVTEXT_AMD_OVERFLOW         = 2, /* std::overflow_error   */
  NVTEXT_AMD_LOGIC_ERROR      = 3, /* cudf::logic_error     */
  NVTEXT_AMD_DEVICE_ERROR     = 4, /* cudf::cuda_error      */
  NVTEXT_AMD_ALLOC_FAILED     = 5  /* std::bad_alloc        */
} nvtext_amd_status;

/* cudf::type_id values used by this path (cpp/include/cudf/types.hpp:185-217). */
enum {
  NVTEXT_AMD_TYPE_INT32  = 3,
  NVTEXT_AMD_TYPE_UINT32 = 7,
  NVTEXT_AMD_TYPE_UINT64 = 8,
  NVTEXT_AMD_TYPE_FLOAT32 = 9
};

/* Non-owning view of an Arrow-layout strings column as libcudf lays it out
 * (cudf::strings_column_view, cpp/include/cudf/strings/strings_column_view.hpp:27-114;
 *  cudf::column_view, cpp/include/cudf/column/column_view.hpp:44-293).
 * Row i is chars[offsets[i+offset] .. offsets[i+offset+1]); bit (i+offset) of
 * null_mask (uint32 words, LSB first) is its validity. */
typedef struct nvtext_amd_strings_column {
  const char*     chars;            /* device; may be NULL when there are no bytes            */
  const void*     offsets;          /* device; element 0 of the offsets child; NULL if size 0 */
  int32_t         offsets_is_int64; /* 0: int32 offsets, 1: int64 offsets                     */
  const uint32_t* null_mask;        /* device or NULL                                         */
  int32_t         size;             /* rows in this view                                      */
  int32_t         offset;           /* first row of the view inside the parent buffers        */
  int32_t         null_count;       /* nulls in the view (>= 0)                               */
} nvtext_amd_strings_column;

/* Stream-ordered allocator for results and temporaries; the counterpart of
 * rmm::device_async_resource_ref in the reference signatures.  A NULL allocator (or
 * NULL members) selects hipMallocAsync / hipFreeAsync on `stream`. */
typedef struct nvtext_amd_allocator {
  void* ctx;
  void* (*allocate)(void* ctx, size_t bytes, void* stream);
  void  (*deallocate)(void* ctx, void* ptr, size_t bytes, void* stream);
} nvtext_amd_allocator;

/* Owning result: a LIST column (cudf::make_lists_column,
 * cpp/src/lists/lists_column_factories.cu:106-129).  Buffers come from the allocator
 * given to the call and belong to the caller afterwards. */
typedef struct nvtext_amd_list_column {
  int32_t   size;            /* rows                                                        */
  int32_t   null_count;
  int32_t   child_type;      /* NVTEXT_AMD_TYPE_*                                           */
  int32_t   offsets_size;    /* size+1, or 0 for the canonical empty list column            */
  int32_t*  offsets;         /* device, offsets_size entries (NULL if 0)                    */
  void*     child;           /* device, child_size elements of child_type (NULL if 0)       */
  int64_t   child_size;
  uint32_t* null_mask;       /* device or NULL; bit i = row i                               */
  size_t    offsets_bytes;   /* allocation sizes, for deallocate()                          */
  size_t    child_bytes;
  size_t    null_mask_bytes;
} nvtext_amd_list_column;

/* LIST<STRING> input column (cpp/include/cudf/lists/lists_column_view.hpp:33-120): int32 list offsets
 * (size + offset + 1 entries) that index the elements of `child`, optional row validity, and the view's
 * offset / size for a sliced column.  `child` describes all the elements (its own offset applies on top). */
typedef struct nvtext_amd_list_strings_column {
  const int32_t*  offsets;
  const uint32_t* null_mask;
  int32_t         size;
  int32_t         offset;
  int32_t         null_count;
  nvtext_amd_strings_column child;
} nvtext_amd_list_strings_column;

/* Fixed-width result column (cudf::make_numeric_column, cpp/include/cudf/column/column_factories.hpp):
 * `size` values of `type`, optional validity.  The buffers come from the caller's allocator and are
 * returned with nvtext_amd_fixed_column_free. */
typedef struct nvtext_amd_fixed_column {
  int32_t   type;            /* NVTEXT_AMD_TYPE_* */
  int32_t   size;
  int32_t   null_count;
  void*     data;
  uint32_t* null_mask;       /* NULL when the column has no nulls */
  size_t    data_bytes;
  size_t    null_mask_bytes;
} nvtext_amd_fixed_column;

/* Owning result: a STRING column (cudf::make_strings_column, cpp/include/cudf/column/column_factories.hpp).
 * The offsets are int32 unless the chars reach INT32_MAX bytes, then int64 (large strings:
 * cpp/include/cudf/strings/detail/strings_children.cuh:164-175, cpp/src/strings/utilities.cu:150-157).
 * The buffers come from the caller's allocator and are returned with nvtext_amd_strings_result_free. */
typedef struct nvtext_amd_strings_result {
  int32_t   size;            /* rows                                                        */
  int32_t   null_count;
  int32_t   offsets_size;    /* size+1, or 0 for the canonical empty strings column         */
  int32_t   offsets_is_int64;
  void*     offsets;         /* device, offsets_size entries (NULL if 0)                    */
  char*     chars;           /* device, chars_size bytes (NULL if 0)                        */
  int64_t   chars_size;
  uint32_t* null_mask;       /* device or NULL; bit i = row i                               */
  size_t    offsets_bytes;   /* allocation sizes, for deallocate()                          */
  size_t    chars_bytes;
  size_t    null_mask_bytes;
} nvtext_amd_strings_result;

typedef struct nvtext_amd_wordpiece_vocabulary nvtext_amd_wordpiece_vocabulary;
typedef struct nvtext_amd_character_normalizer nvtext_amd_character_normalizer;

/* Library version (major*10000 + minor*100 + patch). */
int32_t nvtext_amd_version(void);

/* Message of the last failure on the calling thread ("" if none). */
const char* nvtext_amd_last_error(void);

/* Replaces nvtext::minhash (cpp/include/nvtext/minhash.hpp:62-69; cpp/src/text/minhash.cu:691-701).
 * MurmurHash3_x86_32(seed) of every `width`-character window, permuted by
 * (hash*a[j]+b[j]) in uint32 arithmetic, minimum per j.  Result: LIST<UINT32>,
 * param_count values per valid row, none for a null row, zeros for an empty row.
 * a, b: device arrays of param_count values. */
nvtext_amd_status nvtext_amd_minhash(const nvtext_amd_strings_column* input,
                                     uint32_t seed,
                                     const uint32_t* a,
                                     const uint32_t* b,
                                     int64_t a_count,
                                     int64_t b_count,
                                     int32_t width,
                                     void* stream,
                                     const nvtext_amd_allocator* mr,
                                     nvtext_amd_list_column* out);

/* Replaces nvtext::minhash64 (cpp/include/nvtext/minhash.hpp:109-116; cpp/src/text/minhash.cu:716-726).
 * MurmurHash3_x64_128(seed) word 0; permutation ((hash*a+b) mod 2^64) % (2^61-1).  Result: LIST<UINT64>. */
nvtext_amd_status nvtext_amd_minhash64(const nvtext_amd_strings_column* input,
                                       uint64_t seed,
                                       const uint64_t* a,
                                       const uint64_t* b,
                                       int64_t a_count,
                                       int64_t b_count,
                                       int32_t width,
                                       void* stream,
                                       const nvtext_amd_allocator* mr,
                                       nvtext_amd_list_column* out);

/* nvtext_amd_minhash for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid it).  It has no counterpart in the reference.  The caller brings the result buffers:
 * out_offsets (input->size + 1 values), out_child (room for out_child_capacity values; the call needs
 * (size - null_count) * param_count of them) and, when the input has a null mask, out_null_mask
 * ((size + 31) / 32 words, bit i = row i of the view).  The values are those of nvtext_amd_minhash.
 * Temporaries live in an array inside the library, one copy per device, so the call makes no allocation and
 * releases nothing; in exchange it takes at most NVTEXT_AMD_MINHASH_PREALLOCATED_MAX_ROWS rows (more is
 * NVTEXT_AMD_INVALID_ARGUMENT), and two calls that overlap in time on one device race on that array: keep the
 * calls of a device on one stream, or order them otherwise.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress, under a lock): make one call on every device outside of any stream capture before the calls
 * that are captured. */
#define NVTEXT_AMD_MINHASH_PREALLOCATED_MAX_ROWS 1048576
nvtext_amd_status nvtext_amd_minhash_preallocated(const nvtext_amd_strings_column* input,
                                                  uint32_t seed,
                                                  const uint32_t* a,
                                                  const uint32_t* b,
                                                  int64_t a_count,
                                                  int64_t b_count,
                                                  int32_t width,
                                                  void* stream,
                                                  int32_t* out_offsets,
                                                  uint32_t* out_child,
                                                  int64_t out_child_capacity,
                                                  uint32_t* out_null_mask);

/* Replaces nvtext::minhash_ngrams (cpp/include/nvtext/minhash.hpp:156-163; cpp/src/text/minhash.cu:703-714).
 * The hashed items are runs of consecutive strings of a LIST<STRING> row: for element i the bytes from the
 * start of element i to the end of element min(i + ngrams, last) (adjacent elements are contiguous in the
 * child's chars), MurmurHash3_x86_32(seed), for i in [0, max(1, elements - ngrams + 1)); a run that the row
 * cuts short counts only at i = 0, a null element starts no run.  Permutation, minimum and result layout
 * as nvtext_amd_minhash: LIST<UINT32>, param_count values per valid row, zeros for an empty row. */
nvtext_amd_status nvtext_amd_minhash_ngrams(const nvtext_amd_list_strings_column* input,
                                            int32_t ngrams,
                                            uint32_t seed,
                                            const uint32_t* a,
                                            const uint32_t* b,
                                            int64_t a_count,
                                            int64_t b_count,
                                            void* stream,
                                            const nvtext_amd_allocator* mr,
                                            nvtext_amd_list_column* out);

/* Replaces nvtext::minhash64_ngrams (cpp/include/nvtext/minhash.hpp:203-210; cpp/src/text/minhash.cu:728-739).
 * MurmurHash3_x64_128(seed) word 0; permutation ((hash*a+b) mod 2^64) % (2^61-1).  Result: LIST<UINT64>. */
nvtext_amd_status nvtext_amd_minhash64_ngrams(const nvtext_amd_list_strings_column* input,
                                              int32_t ngrams,
                                              uint64_t seed,
                                              const uint64_t* a,
                                              const uint64_t* b,
                                              int64_t a_count,
                                              int64_t b_count,
                                              void* stream,
                                              const nvtext_amd_allocator* mr,
                                              nvtext_amd_list_column* out);

/* Replaces nvtext::jaccard_index (cpp/include/nvtext/jaccard.hpp:66-71; cpp/src/text/jaccard.cu:490-498).
 * For every row r: A, B = the sets of non-zero MurmurHash3_x86_32(seed 0) values of the `width`-character
 * windows of input1[r], input2[r] (the window rule of nvtext_amd_minhash); result[r] = |A n B| / |A u B| as
 * float32 (0 when both sets are empty).  A row that is null in either input is null in the result (its value
 * is unspecified); the result has a null mask only if an input has nulls.  Synchronises the stream once.
 * Limit: two rows of one pair may have 2^32 / 3 bytes together (1.43 GB); beyond that NVTEXT_AMD_OVERFLOW. */
nvtext_amd_status nvtext_amd_jaccard_index(const nvtext_amd_strings_column* input1,
                                           const nvtext_amd_strings_column* input2,
                                           int32_t width,
                                           void* stream,
                                           const nvtext_amd_allocator* mr,
                                           nvtext_amd_fixed_column* out);

/* Returns the buffers of a fixed-width result to the allocator they came from. */
void nvtext_amd_fixed_column_free(nvtext_amd_fixed_column* col, void* stream, const nvtext_amd_allocator* mr);

/* Replaces nvtext::load_wordpiece_vocabulary / wordpiece_vocabulary::wordpiece_vocabulary
 * (cpp/include/nvtext/wordpiece_tokenize.hpp:26-66; cpp/src/text/wordpiece_tokenize.cu:213-293).
 * Token id = row index.  Fails with INVALID_ARGUMENT for an empty vocabulary or one with nulls.
 * The object owns a device copy of the entries and its lookup tables, allocated through `mr` on `stream`
 * (NULL: hipMalloc) and handed back the same way by _destroy, so the allocator's ctx and the stream must
 * outlive the object, as a memory resource must outlive what it allocated.  It is immutable and may be
 * shared by concurrent calls. */
nvtext_amd_status nvtext_amd_wordpiece_vocabulary_create(const nvtext_amd_strings_column* vocabulary,
                                                         void* stream,
                                                         const nvtext_amd_allocator* mr,
                                                         nvtext_amd_wordpiece_vocabulary** out);

/* Replaces wordpiece_vocabulary::~wordpiece_vocabulary (cpp/src/text/wordpiece_tokenize.cu:284). */
void nvtext_amd_wordpiece_vocabulary_destroy(nvtext_amd_wordpiece_vocabulary* vocabulary);

/* Id of "[UNK]" (else "[unk]", else -1): cpp/src/text/wordpiece_tokenize.cu:199-209,273-275. */
int32_t nvtext_amd_wordpiece_vocabulary_unk_id(const nvtext_amd_wordpiece_vocabulary* vocabulary);

/* Replaces nvtext::wordpiece_tokenize (cpp/include/nvtext/wordpiece_tokenize.hpp:68-111;
 * cpp/src/text/wordpiece_tokenize.cu:839-899).  Result: LIST<INT32> of token ids per row.
 * max_words_per_row == 0 tokenizes every word; > 0 only the first
 * min(max_words_per_row, row_bytes/2) words of each valid row; < 0 is INVALID_ARGUMENT. */
nvtext_amd_status nvtext_amd_wordpiece_tokenize(const nvtext_amd_strings_column* input,
                                                const nvtext_amd_wordpiece_vocabulary* vocabulary,
                                                int32_t max_words_per_row,
                                                void* stream,
                                                const nvtext_amd_allocator* mr,
                                                nvtext_amd_list_column* out);

/* Replaces nvtext::create_character_normalizer / character_normalizer::character_normalizer
 * (cpp/include/nvtext/normalize.hpp:170-213; cpp/src/text/normalize.cu:219-256).  The object owns the device
 * tables that say, per Unicode code point, whether it is padded with spaces (punctuation, CJK ideographs),
 * removed (control and format characters; accents when lower-casing), replaced by a space (whitespace) or
 * replaced by its lower-cased, accent-stripped form of one to three code points.  special_tokens (NULL or
 * empty for none) are bracketed tokens such as "[PAD]" that keep their case and their brackets unpadded;
 * nulls among them give INVALID_ARGUMENT.  The tables (14.4 MB) come from `mr` on `stream` (NULL: hipMalloc)
 * and go back the same way in _destroy: the allocator's ctx and the stream must outlive the object.  Belongs to
 * the device that is current at creation; immutable and shareable between concurrent calls. */
nvtext_amd_status nvtext_amd_character_normalizer_create(int32_t do_lower_case,
                                                         const nvtext_amd_strings_column* special_tokens,
                                                         void* stream,
                                                         const nvtext_amd_allocator* mr,
                                                         nvtext_amd_character_normalizer** out);

/* Replaces character_normalizer::~character_normalizer (cpp/src/text/normalize.cu:247). */
void nvtext_amd_character_normalizer_destroy(nvtext_amd_character_normalizer* normalizer);

/* Replaces nvtext::normalize_characters (cpp/include/nvtext/normalize.hpp:215-254;
 * cpp/src/text/normalize.cu:491-573): the BERT basic-tokenizer clean-up that precedes wordpiece_tokenize.
 * Works on the bytes between the first and the last offset of the view as one flat sequence, so a null row
 * keeps whatever its offsets span and the result has the input's validity.  Result: STRING column (int64
 * offsets when it holds INT32_MAX bytes or more).  Synchronises the stream twice (the byte range of the view,
 * the size of the result). */
nvtext_amd_status nvtext_amd_normalize_characters(const nvtext_amd_strings_column* input,
                                                  const nvtext_amd_character_normalizer* normalizer,
                                                  void* stream,
                                                  const nvtext_amd_allocator* mr,
                                                  nvtext_amd_strings_result* out);

/* Returns the buffers of a strings result to the allocator they came from. */
void nvtext_amd_strings_result_free(nvtext_amd_strings_result* col, void* stream, const nvtext_amd_allocator* mr);

/* Releases the buffers of a result through the allocator that produced them. */
void nvtext_amd_list_column_free(nvtext_amd_list_column* col, void* stream, const nvtext_amd_allocator* mr);

#ifdef __cplusplus
}
#endif
#endif /* NVTEXT_AMD_H */

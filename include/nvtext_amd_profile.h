/*
 * nvtext_amd_profile.h -- kernel timing hooks of libnvtext_amd.so for benchmarks and profiling scripts.
 * Not part of the product interface in nvtext_amd.h: the record behind these calls is one global list,
 * not safe against entry-point calls on other threads.
 */
#ifndef NVTEXT_AMD_PROFILE_H
#define NVTEXT_AMD_PROFILE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Kernel timing for benchmarks.  The reference marks these entry points with NVTX ranges
 * (CUDF_FUNC_RANGE, cpp/src/text/minhash.cu:699, cpp/src/text/wordpiece_tokenize.cu:897) and is
 * timed from outside with Nsight; here the library itself brackets each of its kernels with HIP
 * events on the caller's stream while profiling is on.  nvtext_amd_profile_read synchronises the
 * recorded events, returns up to `capacity` (name, milliseconds) pairs in launch order and clears
 * the record; the names are static strings.  Off by default; not thread-safe against concurrent
 * entry-point calls. */
void    nvtext_amd_profile_enable(int32_t on);
int32_t nvtext_amd_profile_read(const char** names, float* milliseconds, int32_t capacity);

/* Test knob.  nvtext_amd_wordpiece_tokenize hands its wavefronts ranges of 1, 2, 4 or 8 tiles of 2048 bytes, the
 * fewer the smaller the column, so only a column of hundreds of megabytes runs with the largest.  tiles = 1, 2, 4 or 8
 * makes every later call of the process use that size whatever the column's, so that small test columns cover the code
 * as a large column runs it; any other value gives the choice back to the library.  Results do not depend on it. */
void    nvtext_amd_profile_set_range_tiles(int32_t tiles);

/* Test knob.  nvtext_amd_wordpiece_tokenize sizes the temporaries of its first attempt from a sample of the column and
 * repeats its passes with larger ones when a range or the queue runs out of room all the same.  on = 0 makes every later
 * call of the process skip the sample, so that columns which the sample sizes correctly still reach the second attempt;
 * any other value switches it back on (the default).  Results do not depend on it. */
void    nvtext_amd_profile_set_sizing_sample(int32_t on);

#ifdef __cplusplus
}
#endif
#endif /* NVTEXT_AMD_PROFILE_H */

// Entry points that allocate nothing.
//
// They have no counterpart in the reference (mini_llm leaves every allocation to torch).  They are for
// callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, and
// harnesses that forbid hipMalloc.  Such an entry point is a variant of an existing one whose scratch
// memory, instead of coming in as a workspace argument, lies in a file-scope device array of a stated
// maximum size; it calls no hipMalloc, hipFree or allocating library routine, and refuses sizes beyond
// the maximum with an error.  The caller still passes inputs and outputs.
#pragma once

#include <stdint.h>

#ifndef LRS_API
#define LRS_API extern "C" __attribute__((visibility("default")))
#endif

// Most (row, slice) pairs a call may ask for: rows x parts <= this.  The scratch holds one float and one
// int per pair: 128 KB on every GPU the library runs on, kept until the process ends.
#define LRS_CHOOSE_STATIC_MAX_PARTS 16384

// lrs_choose_tokens_split() without its two scratch arguments: out[r] = the chosen token of row r of
// logits [rows, vocab] (float32, row stride `row_stride`); temperature == nullptr or temperature[r] == 0
// picks the lowest index among the largest logits, else a draw keyed by (seeds[r], counters[r]).  A row that
// holds a value that is not finite comes out as -1 (`filtered` != 0: rows of positive temperature may hold -inf,
// as lrs_filter_logits() leaves them).  Each row is
// cut into `parts` slices, one workgroup each; rows x parts must not exceed LRS_CHOOSE_STATIC_MAX_PARTS.
// Results equal lrs_choose_tokens_split()'s for the same `parts`.  Every call on a GPU uses that GPU's one
// scratch array (nothing in it needs clearing between calls): calls that overlap on one GPU race, so
// keep them on one stream or order them yourself.  Returns 0, or 1 with a message for lrs_last_error().
LRS_API int lrs_choose_tokens_static(int* out, const float* logits, int64_t row_stride, int rows, int vocab,
                                     const float* temperature, const uint64_t* seeds, const uint32_t* counters,
                                     int parts, int filtered, void* stream);

// Looks up the current device's copy of the scratch array now (otherwise the first call on a device does
// it): call it once per device before a capture begins.  Safe to call again.
LRS_API int lrs_choose_tokens_static_init();

// LRS_CHOOSE_STATIC_MAX_PARTS, for callers that load the library at run time.
LRS_API int lrs_choose_tokens_static_max_parts();

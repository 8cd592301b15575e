// Launch plans: a recorded sequence of this library's own launches, made again by one call.
//
// A plan is an array of 64-bit words: for every launch the number of its entry point (its place in
// ops.PLAN_OPS on the Python side) followed by its arguments, one word each, in the entry point's own
// order and without the stream (pointers and integers as they are, floats as their 32 bits).
// lrs_plan_run() walks the array and calls each entry point with the stream it is given.  The entry points
// check their arguments as they always do; the first that fails ends the run, and its message (with the
// launch's place in the plan) is what lrs_last_error() returns.
#include "common.h"

#include <string.h>

static inline float word_as_float(uint64_t word) {
  const uint32_t bits = (uint32_t)word;
  float value;
  memcpy(&value, &bits, sizeof(value));
  return value;
}

#define LRS_PLAN_DECLARATIONS
#include "plan_dispatch.inc"
#undef LRS_PLAN_DECLARATIONS

static int short_plan(const char* name) { return lrs_fail("plan_run: the plan ends inside the arguments of %s", name); }

LRS_API const char* lrs_last_error();

LRS_API int lrs_plan_run(const uint64_t* words, int64_t length, int launches, void* stream) {
  LRS_REQUIRE(words != nullptr && length > 0 && launches > 0, "plan_run: an empty plan");
  int64_t at = 0;
  for (int launch = 0; launch < launches; ++launch) {
    LRS_REQUIRE(at < length, "plan_run: the plan ends after %d of %d launches", launch, launches);
    const uint64_t op = words[at++];
    const uint64_t* w = words + at;
    const int64_t left = length - at;
    int taken = 0, rc = 0;
    switch (op) {
#define LRS_PLAN_CASES
#include "plan_dispatch.inc"
#undef LRS_PLAN_CASES
      default:
        return lrs_fail("plan_run: launch %d names entry point %llu, which no plan may hold", launch, (unsigned long long)op);
    }
    if (rc != 0) {
      char message[900];
      snprintf(message, sizeof(message), "%s", lrs_last_error());
      return lrs_fail("plan_run: launch %d of %d failed: %s", launch, launches, message);
    }
    at += taken;
  }
  LRS_REQUIRE(at == length, "plan_run: %lld words left over after the last launch", (long long)(length - at));
  return 0;
}

// Entry points of the sampler (sampling.hip), and the arguments they share.
#pragma once
#include "common.h"

// Per-request options live in the request's state slot, written once when the
// request is admitted: fparams[slot] = {temperature, top_p, min_p, repetition,
// presence, frequency, -, -}; iparams[slot] = {top_k, -}; seeds[slot] = {seed,
// index of the next draw}. The kernel advances the draw index itself.
struct SampleArgs {
  const float* logits;      // [R, V]
  float* work;              // [R, V] processed logits (scratch, returned to the caller)
  const int* counts;        // [slots, V] occurrences of each id in prompt + output, or null
  const int* slot;          // [R] state slot of each row
  const float* fparams;     // [slots, 8]
  const int* iparams;       // [slots, 2]
  unsigned long long* seeds;  // [slots, 2]
  int* out_token;           // [R]
  float* out_logprob;       // [R]
  int rows, vocab;
  int write_work;           // also keep the processed logits of greedy rows
  float* partials;          // [R, parts, 4]: maximum, sum of exp(value - maximum), first index of the maximum
  int parts;                // > 0: the first pass ran in sample_first_pass_kernel, `parts` blocks per row
};

// One token per row; two launches at most (the first pass in parts, then the rest). When
// `parts` > 0 the caller brings `partials`.
extern "C" int qrt_sample(const SampleArgs* args, hipStream_t stream);

// The same, for callers that cannot allocate device memory: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference
// (yuzheng310/qwen3-runtime samples with torch calls, which allocate as they please). The
// `partials` field of the arguments is ignored: the partial results of the first pass live in
// a buffer that is part of the library's image, QRT_SAMPLE_SCRATCH_BYTES per GPU, held until
// the process ends. rows * parts * 16 bytes must fit in it (64 rows in 64 parts each do);
// more is refused with a message. Nothing in the buffer has to start at zero: the first pass
// writes every entry the second reads. It keeps the last call's contents, and every call on a
// GPU shares that GPU's buffer, so calls that overlap on one GPU (two streams, two threads)
// race; calls on one stream are ordered and safe. The caller still passes every input and
// output (logits, work, options, seeds, token and log-probability rows). Calls no hipMalloc,
// hipFree or allocating library routine.
#define QRT_SAMPLE_SCRATCH_BYTES (64 * 1024)
extern "C" int qrt_sample_noalloc(const SampleArgs* args, hipStream_t stream);

// Looks the built-in buffer's address up for the current device now (once per device; later calls
// return at once), so that the first qrt_sample_noalloc on that device, which may sit inside a
// stream capture, makes no runtime query. Optional: qrt_sample_noalloc does the same at its first
// call on a device. Returns 0, or -1 with qrt_last_error().
extern "C" int qrt_sample_noalloc_setup();

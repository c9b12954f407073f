// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code that runs
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The two-pass argmax needs a
// place for the first pass's results (per row and chunk of 4,096 columns the chunk's best value and its index);
// nnis_argmax takes that place from the caller, nnis_argmax_static keeps it in a fixed array in device memory
// that the library holds on every GPU it has run on, until the process ends.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// 4-byte words of the fixed array: 256 KB a GPU.  A call needs 2 * rows * ceil(vocab / 4096) of them
// (nnis_argmax_scratch(rows, vocab)): 64 rows of a vocabulary of 2 million, or 2,048 rows of 65,536.
#define NNIS_STATIC_SCRATCH_WORDS 65536

// out[r] = index of the largest of logits[r, 0..vocab), the lowest index on ties, as nnis_argmax gives it, on
// `stream` of the current device.  Calls hipMalloc, hipFree or any allocating routine never.  Returns non-zero
// with a message for nnis_last_error() when nnis_argmax_scratch(rows, vocab) exceeds NNIS_STATIC_SCRATCH_WORDS
// (nothing is launched then).  Nothing in the array has to start at zero: the first pass writes every word the
// second reads.  Every call on a GPU uses that GPU's one array, so calls that overlap on one GPU (two streams,
// two threads) race: a caller keeps them in order on one stream, or waits between them.
int nnis_argmax_static(const float* logits, int* out, int rows, int vocab, void* stream);

#ifdef __cplusplus
}
#endif

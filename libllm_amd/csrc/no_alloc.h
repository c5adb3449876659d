// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
// code that runs under HIP graph capture, tight serving loops, and harnesses that forbid
// hipMalloc.  llm_argmax (sampling.hip) needs two scratch arrays that its caller allocates, one
// entry for every slice of every row; llm_argmax_static computes the same result with the same
// kernels and keeps those arrays in a file-scope device array of LLM_ARGMAX_STATIC_BYTES bytes,
// which every GPU that the library runs on holds until the process ends.
//
// Limits and rules:
//  * rows * llm_argmax_parts(vocab) must not exceed LLM_ARGMAX_STATIC_ENTRIES; beyond that the
//    call launches nothing and returns LLM_ERR_TOO_LARGE (llm_argmax_static_max_rows tells the
//    most rows for a vocabulary).
//  * The stream must belong to the device that is current at the call.  The array's address on
//    that device is looked up once, at the first call there (or by llm_argmax_static_init, for a
//    caller that wants the look-up done before it begins a capture).
//  * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams,
//    two threads) race and give wrong tokens.  Calls on one stream are ordered and safe.  The
//    array keeps the last call's contents; nothing in it has to start at zero, since the first
//    kernel writes every entry that the second reads.
//  * It calls no hipMalloc, hipFree or allocating library routine.
#pragma once
#include <hip/hip_runtime.h>

#define LLM_ARGMAX_STATIC_ENTRIES 32768
#define LLM_ARGMAX_STATIC_BYTES (LLM_ARGMAX_STATIC_ENTRIES * 8)    // a float and an int an entry: 256 KiB

extern "C" {
// out[r] = index of the largest of logits[r, 0..vocab) (the lowest index wins a tie), r < rows;
// logits float32 [rows, vocab], out int32 [rows], both on the current device.  Returns LLM_OK,
// LLM_ERR_ARG, LLM_ERR_TOO_LARGE or LLM_ERR_LAUNCH.
int llm_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t stream);
// Looks up the array's address on the current device (idempotent).  LLM_OK or LLM_ERR_LAUNCH.
int llm_argmax_static_init(void);
// The most rows llm_argmax_static takes for this vocabulary (0 for a vocabulary it refuses).
int llm_argmax_static_max_rows(int vocab);
}

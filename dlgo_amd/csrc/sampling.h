// What the sampling library exports.  Every function returns nullptr on success, else a message that names
// what was refused; launches go to `stream` and nothing waits for them.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

// out[r] = index of the first maximum of row r of float32 logits [n_rows, V] (row stride ld).
// partial: device scratch of n_rows * 512 bytes that the caller brings.
const char* dlgo_argmax(const float* logits, int ld, int n_rows, int V, void* partial, long long partial_bytes, int32_t* out,
                        hipStream_t stream);

// The same result as dlgo_argmax without a scratch argument and without allocating anything, for callers that
// cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
// counterpart in computerex/dlgo.  The candidates of the first stage go to a fixed array in device memory
// (DLGO_ARGMAX_NOALLOC_ROWS * 512 bytes = 128 KB, held by every GPU the library runs on until the process ends);
// more rows than DLGO_ARGMAX_NOALLOC_ROWS are refused.  Nothing in the array has to start at zero: the first stage
// writes every entry that the second reads.  All calls on one GPU share the array, so calls that overlap there
// (two streams, two threads) race; calls on one stream are ordered and safe.
// The array's address on a device is asked of the runtime (hipGetSymbolAddress) the first time it is wanted there, which
// is a call that a capturing stream does not take: a caller that captures calls dlgo_argmax_noalloc_init(), or
// dlgo_argmax_noalloc itself, once on that device before its first capture.  After that the entry point only launches.
#define DLGO_ARGMAX_NOALLOC_ROWS 256
const char* dlgo_argmax_noalloc(const float* logits, int ld, int n_rows, int V, int32_t* out, hipStream_t stream);
// Resolves the array's address for the current device (nothing else); nullptr on success.
const char* dlgo_argmax_noalloc_init();

}  // extern "C"

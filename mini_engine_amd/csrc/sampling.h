// C entry points of the token-choice kernels (sampling.hip), as exported by libme_core.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

extern "C" {

// Token ids for float32 logits [S, V] with row stride `ld`: argmax where temperatures[s] == 0, else
// argmax(logits / T - log E), E ~ Exp(1) hashed from (keys[s], vocabulary id). keys: [S, 2] uint32;
// out: [S] int32; scratch: device memory of 2 * S * 32 4-byte words, brought by the caller.
// Returns 0, or a negative code with the message in me_last_error().
int me_sample(const float* logits, int64_t ld, const float* temperatures, const uint32_t* keys,
              int32_t* out, void* scratch, int S, int V, hipStream_t stream);

// The same result as me_sample, for callers that cannot allocate device memory and have no workspace
// to bring: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. It has
// no counterpart in the reference (whose sampler is eager torch ops that allocate their temporaries).
//
// The per-chunk partial results live in a file-scope device array of the library
// (ME_SAMPLE_STATIC_MAX_ROWS * 32 * 2 words = 256 KiB, held by every GPU the library runs on until the
// process ends), so this call allocates and frees nothing, neither directly nor through a library.
// S > ME_SAMPLE_STATIC_MAX_ROWS is refused with an error. Nothing in the array has to start at zero:
// the first kernel writes every word the second reads. All calls on one GPU share that GPU's array:
// calls that overlap in time on one GPU (different streams, or graphs replayed side by side) race;
// calls on one stream, one after the other, are safe.
#define ME_SAMPLE_STATIC_MAX_ROWS 1024
int me_sample_static(const float* logits, int64_t ld, const float* temperatures, const uint32_t* keys,
                     int32_t* out, int S, int V, hipStream_t stream);

}  // extern "C"

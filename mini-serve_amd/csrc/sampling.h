// Entry points of the token sampler (sampling.hip). All return 0 when the kernels were launched,
// 1 for a bad argument, 2 for a size the call does not take, 3 when a launch or a set-up call failed.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Bytes of the scratch buffer ms_sample_rows needs for `rows` rows (-1: too many rows).
int ms_sample_scratch_bytes(int rows);

// tokens[row] from float32 logits [rows, vocab] (rows `row_stride` floats apart): the first maximal
// index where temperature is null or 0 for the row, else argmax(logits / T + Gumbel noise hashed from
// (seed, counter, index)), restricted to the nucleus where top_p < 1. `scratch`: device memory of
// ms_sample_scratch_bytes(rows) bytes that the caller owns; it holds the best candidate of each
// vocabulary part between the two kernels.
int ms_sample_rows(const float* logits, int rows, int vocab, long long row_stride, const float* temperature,
                   const float* top_p, const unsigned* seed, const int* counter, void* scratch, int* tokens,
                   hipStream_t st);

// The most rows one call of ms_sample_rows_static takes.
#define MS_SAMPLE_STATIC_MAX_ROWS 256
int ms_sample_rows_static_max_rows();

// ms_sample_rows without a scratch argument and without any allocation. It has no counterpart in the
// reference (whose sampler allocates [rows, vocab] temporaries with every call). It is for callers
// that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
// that forbid allocation. The candidates between the two kernels lie in an array inside the library
// (MS_SAMPLE_STATIC_MAX_ROWS * 64 parts * 8 bytes = 128 KiB on each GPU the library runs on, held
// until the process ends); the caller passes inputs and outputs only. Same kernels, same result as
// ms_sample_rows. More than MS_SAMPLE_STATIC_MAX_ROWS rows: returns 2 and launches nothing. Every call
// on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race;
// calls on one stream, or ordered by events, do not. The first call on a device looks the array's
// device address up (no allocation); it must be made with that device current, as every call must.
int ms_sample_rows_static(const float* logits, int rows, int vocab, long long row_stride, const float* temperature,
                          const float* top_p, const unsigned* seed, const int* counter, int* tokens, hipStream_t st);

#ifdef __cplusplus
}
#endif

// C entry points of the sampling kernels (sampling.hip, module "core").
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

// Number of chunks a row of V logits is cut into by the two-stage kernels; 0 when rows of this
// length are served by the one-stage kernel, which needs no workspace.
int pi_sample_chunks(int V);

// out[m] = next token of row m of float32 logits [M, V] (rows row_stride apart): the arg max
// (lowest index among equals) where temperature is null or temperature[m] <= 0, otherwise the
// first index whose cumulative softmax(logits / temperature[m]) reaches uniform[m].
// ws: float32 workspace of ws_elems >= M * pi_sample_chunks(V) * 4 for the two-stage kernels
// (with less the one-stage kernel is taken).  Returns 0, or -1 with a message in
// pi_core_last_error().
int pi_sample(int* out, const float* logits, long row_stride, const float* temperature, const float* uniform, int M,
              int V, float* ws, long ws_elems, hipStream_t stream);

// The same operation with the same kernels and the same results as pi_sample with a large enough
// workspace, for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  It
// allocates and frees nothing: the chunk records of the two-stage kernels go to an array that the
// library holds in each GPU's memory from load to process end (PI_SAMPLE_STATIC_FLOATS floats,
// 256 KiB).  Limit: M * pi_sample_chunks(V) * 4 <= PI_SAMPLE_STATIC_FLOATS, i.e. 256 rows of any
// vocabulary above 131072 entries, more rows of shorter ones; rows of up to 16384 logits need no
// workspace and have no limit on M.  Anything larger is refused with an error, nothing is run.
// Every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU (two
// streams, two threads) race on it and must be ordered by the caller.  Nothing in the array has to
// start at zero: each call writes every record before it reads it.
#define PI_SAMPLE_STATIC_FLOATS 65536
int pi_sample_static(int* out, const float* logits, long row_stride, const float* temperature, const float* uniform,
                     int M, int V, hipStream_t stream);

}  // extern "C"

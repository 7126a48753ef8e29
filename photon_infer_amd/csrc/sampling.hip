// Next-token choice from float32 logits [M, V]: greedy or temperature sampling, per row.
//
// Greedy (src/arch/llama_model.cpp:304-328): the largest logit, the lowest index among
// equals -- fixed here for every reduction order, whereas the reference's GPU kernel
// (src/ops/kernels/cuda/sampling_kernel.cu:36-138) leaves ties to the order its 32-lane
// shuffles happen to take.
// Temperature (demo/llama_infer.cpp:77-101): p_i = exp((l_i - max l) / tau) / sum, and the
// first index whose cumulative probability reaches u.  u in [0, 1) is given per row by
// the caller, so a request's draws do not depend on what else is in the batch.  If
// rounding lets the cumulative sum end below u * sum, the last index with p > 0 is taken.
#include "common.h"

#define SAMPLE_THREADS 256

struct ArgMax {
  float v;
  int i;
};

__device__ inline ArgMax better(ArgMax a, ArgMax b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ inline ArgMax wave_argmax(ArgMax a) {
#pragma unroll
  for (int off = PI_WAVE / 2; off > 0; off >>= 1) {
    ArgMax b;
    b.v = __shfl_xor(a.v, off, PI_WAVE);
    b.i = __shfl_xor(a.i, off, PI_WAVE);
    a = better(a, b);
  }
  return a;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(int* __restrict__ out, const float* __restrict__ logits,
                                                                long row_stride, const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform, int V) {
  __shared__ float wv[SAMPLE_THREADS / PI_WAVE];
  __shared__ int wi[SAMPLE_THREADS / PI_WAVE];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ float scratch[16];
  __shared__ int chosen;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* l = logits + (long)row * row_stride;

  ArgMax best = {-INFINITY, 0x7fffffff};
  for (int i = tid; i < V; i += SAMPLE_THREADS) {
    const float v = l[i];
    if (v > best.v) best = {v, i};  // ascending i: the first of equals stays
  }
  best = wave_argmax(best);
  if (tid % PI_WAVE == 0) {
    wv[tid / PI_WAVE] = best.v;
    wi[tid / PI_WAVE] = best.i;
  }
  __syncthreads();
  best = {wv[0], wi[0]};
  for (int w = 1; w < SAMPLE_THREADS / PI_WAVE; ++w) best = better(best, ArgMax{wv[w], wi[w]});
  if (best.i == 0x7fffffff) best = {l[0], 0};  // no finite logit in the row

  const float tau = temperature ? temperature[row] : 0.f;
  if (!(tau > 0.f)) {
    if (tid == 0) out[row] = best.i;
    return;
  }

  // each thread owns a contiguous run of the vocabulary
  const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int c0 = tid * chunk;
  const int c1 = (c0 + chunk < V) ? c0 + chunk : V;
  float local = 0.f;
  for (int i = c0; i < c1; ++i) local += expf((l[i] - best.v) / tau);
  sums[tid] = local;
  if (tid == 0) chosen = -1;
  const float total = block_sum(local, scratch);
  const float target = uniform[row] * total;
  float before = 0.f;
  for (int j = 0; j < tid; ++j) before += sums[j];
  // Runs partition [0, total): exactly one thread has before < target <= before + local
  // (thread 0 also takes target <= 0).  Its scan adds in the order that made `local`,
  // so the last element of the run always satisfies the test.
  if ((before < target || tid == 0) && target <= before + local) {
    float cum = 0.f;
    for (int i = c0; i < c1; ++i) {
      cum += expf((l[i] - best.v) / tau);
      if (target <= before + cum) {
        chosen = i;
        break;
      }
    }
  }
  __syncthreads();
  if (tid == 0) {
    int pick = chosen;
    if (pick < 0) {  // target beyond the last run's end by rounding
      pick = best.i;
      for (int i = V - 1; i >= 0; --i)
        if (expf((l[i] - best.v) / tau) > 0.f) {
          pick = i;
          break;
        }
    }
    out[row] = pick;
  }
}

extern "C" int pi_sample(int* out, const float* logits, long row_stride, const float* temperature, const float* uniform,
                         int M, int V, hipStream_t stream) {
  PI_REQUIRE(M >= 0 && V > 0 && row_stride >= V, "sample: bad sizes M=%d V=%d stride=%ld", M, V, row_stride);
  PI_REQUIRE(temperature == nullptr || uniform != nullptr, "sample: temperatures given without uniform numbers");
  if (M == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SAMPLE_THREADS), 0, stream, out, logits, row_stride, temperature, uniform, V);
  return pi_check_launch("sample");
}

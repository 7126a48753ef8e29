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
#include "sampling.h"

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

// ---- large vocabularies: two stages, so that one row keeps many compute units busy.
// Stage 1: the row is cut into chunks; each block finds its chunk's maximum (lowest index among
// equals) and, for sampled rows, the sum of exp((l - chunk max) / tau).
// Stage 2: one block per row takes the chunk results in chunk order: the global maximum; the total
// sum (chunk sums rescaled to the global maximum); the chunk the draw falls into; and scans that
// chunk for the first index whose cumulative weight reaches the draw.
#define CHUNK_REC 4   // max, index (as float bits), sum, unused
#define TWO_STAGE_FROM 16384
#define MAX_CHUNKS 64

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_stage1_kernel(float* __restrict__ ws, const float* __restrict__ logits,
                                                                       long row_stride, const float* __restrict__ temperature,
                                                                       int V, int chunk) {
  __shared__ float wv[SAMPLE_THREADS / PI_WAVE];
  __shared__ int wi[SAMPLE_THREADS / PI_WAVE];
  __shared__ float scratch[16];
  const int c = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
  const float* l = logits + (long)row * row_stride;
  const int c0 = c * chunk, c1 = min(V, c0 + chunk);
  ArgMax best = {-INFINITY, 0x7fffffff};
  for (int i = c0 + tid; i < c1; i += SAMPLE_THREADS) {
    const float v = l[i];
    if (v > best.v) best = {v, i};
  }
  best = wave_argmax(best);
  if (tid % PI_WAVE == 0) {
    wv[tid / PI_WAVE] = best.v;
    wi[tid / PI_WAVE] = best.i;
  }
  __syncthreads();
  best = {wv[0], wi[0]};
  for (int w = 1; w < SAMPLE_THREADS / PI_WAVE; ++w) best = better(best, ArgMax{wv[w], wi[w]});
  const float tau = temperature ? temperature[row] : 0.f;
  float sum = 0.f;
  if (tau > 0.f && best.i != 0x7fffffff) {
    for (int i = c0 + tid; i < c1; i += SAMPLE_THREADS) sum += expf((l[i] - best.v) / tau);
    sum = block_sum(sum, scratch);
  }
  if (tid == 0) {
    float* rec = ws + ((long)row * gridDim.x + c) * CHUNK_REC;
    rec[0] = best.v;
    rec[1] = __int_as_float(best.i);
    rec[2] = sum;
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_stage2_kernel(int* __restrict__ out, const float* __restrict__ ws,
                                                                       const float* __restrict__ logits, long row_stride,
                                                                       const float* __restrict__ temperature,
                                                                       const float* __restrict__ uniform, int V, int chunk,
                                                                       int chunks) {
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ int chosen;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* l = logits + (long)row * row_stride;
  const float* rec = ws + (long)row * chunks * CHUNK_REC;
  // the chunks' maxima, one per lane (there are at most as many chunks as a wave has lanes): every
  // wave finds the same overall maximum, lowest index among equals, in one trip to memory
  static_assert(MAX_CHUNKS <= PI_WAVE, "one chunk record per lane");
  const int lane = tid % PI_WAVE;
  ArgMax best = lane < chunks ? ArgMax{rec[lane * CHUNK_REC], __float_as_int(rec[lane * CHUNK_REC + 1])} : ArgMax{-INFINITY, 0x7fffffff};
  best = wave_argmax(best);
  if (best.i == 0x7fffffff) best = {l[0], 0};
  const float tau = temperature ? temperature[row] : 0.f;
  if (!(tau > 0.f)) {
    if (tid == 0) out[row] = best.i;
    return;
  }
  // every thread walks the chunk sums the same way (chunks is small): total, then the chunk of the draw
  float total = 0.f;
  for (int c = 0; c < chunks; ++c) {
    const float m = rec[c * CHUNK_REC];
    if (m != -INFINITY) total += rec[c * CHUNK_REC + 2] * expf((m - best.v) / tau);
  }
  const float target = uniform[row] * total;
  float before_chunk = 0.f;
  int pick_chunk = chunks - 1;
  for (int c = 0; c < chunks; ++c) {
    const float m = rec[c * CHUNK_REC];
    const float w = (m != -INFINITY) ? rec[c * CHUNK_REC + 2] * expf((m - best.v) / tau) : 0.f;
    if (target <= before_chunk + w) {
      pick_chunk = c;
      break;
    }
    if (c + 1 < chunks) before_chunk += w;
  }
  // inside the chunk: each thread owns a contiguous run
  const int c0 = pick_chunk * chunk, c1 = min(V, c0 + chunk);
  const int run = (c1 - c0 + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int r0 = min(c1, c0 + tid * run), r1 = min(c1, r0 + run);
  float local = 0.f;
  for (int i = r0; i < r1; ++i) local += expf((l[i] - best.v) / tau);
  sums[tid] = local;
  if (tid == 0) chosen = -1;
  __syncthreads();
  float before = before_chunk;
  for (int j = 0; j < tid; ++j) before += sums[j];
  if ((before < target || (tid == 0 && pick_chunk == 0)) && target <= before + local) {
    float cum = 0.f;
    for (int i = r0; i < r1; ++i) {
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
    if (pick < 0) {
      // rounding between the chunk sums and the scan: the draw lies at an edge of the chunk.
      // Below its first weight: the first index with weight; beyond its last: the last one.
      const bool below = target <= before_chunk;
      pick = -1;
      if (below) {
        for (int i = c0; i < c1 && pick < 0; ++i)
          if (expf((l[i] - best.v) / tau) > 0.f) pick = i;
      } else {
        for (int i = c1 - 1; i >= c0 && pick < 0; --i)
          if (expf((l[i] - best.v) / tau) > 0.f) pick = i;
      }
      if (pick < 0) pick = best.i;
    }
    out[row] = pick;
  }
}

// Rows of more than `two_stage_from` logits use the two-stage kernels and need `ws`
// (float32, M * chunks * 4 with chunks = pi_sample_chunks(V)).
extern "C" int pi_sample_chunks(int V) {
  if (V <= TWO_STAGE_FROM) return 0;
  int chunks = (V + 2047) / 2048;
  return chunks > MAX_CHUNKS ? MAX_CHUNKS : chunks;
}

extern "C" int pi_sample(int* out, const float* logits, long row_stride, const float* temperature, const float* uniform,
                         int M, int V, float* ws, long ws_elems, hipStream_t stream) {
  PI_REQUIRE(M >= 0 && V > 0 && row_stride >= V, "sample: bad sizes M=%d V=%d stride=%ld", M, V, row_stride);
  PI_REQUIRE(temperature == nullptr || uniform != nullptr, "sample: temperatures given without uniform numbers");
  if (M == 0) return 0;
  const int chunks = pi_sample_chunks(V);
  if (chunks == 0 || ws == nullptr || ws_elems < (long)M * chunks * CHUNK_REC || M > 65535) {
    hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SAMPLE_THREADS), 0, stream, out, logits, row_stride, temperature, uniform, V);
    return pi_check_launch("sample");
  }
  const int chunk = (V + chunks - 1) / chunks;
  hipLaunchKernelGGL(sample_stage1_kernel, dim3(chunks, M), dim3(SAMPLE_THREADS), 0, stream, ws, logits, row_stride, temperature, V, chunk);
  if (pi_check_launch("sample_stage1")) return -1;
  hipLaunchKernelGGL(sample_stage2_kernel, dim3(M), dim3(SAMPLE_THREADS), 0, stream, out, ws, logits, row_stride, temperature, uniform, V, chunk, chunks);
  return pi_check_launch("sample_stage2");
}

// ---- the entry point that allocates nothing: the chunk records live in an array of the library's
// own.  Each GPU holds its own copy of the array at its own address; in host code the array's
// name is only a handle for hipGetSymbolAddress, never a pointer a kernel may be given.
static __device__ __align__(256) float sample_static_records[PI_SAMPLE_STATIC_FLOATS];

#define SAMPLE_MAX_DEVICES 64
static float* sample_static_ptr[SAMPLE_MAX_DEVICES] = {nullptr};

// The device address of the array on the current GPU (looked up once per GPU, at the first call there).
static int sample_static_address(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  PI_REQUIRE(e == hipSuccess, "sample_static: hipGetDevice failed: %s", hipGetErrorString(e));
  PI_REQUIRE(dev >= 0 && dev < SAMPLE_MAX_DEVICES, "sample_static: device %d is beyond the %d this library keeps an address for",
             dev, SAMPLE_MAX_DEVICES);
  if (sample_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(sample_static_records));
    PI_REQUIRE(e == hipSuccess && p != nullptr, "sample_static: hipGetSymbolAddress failed on device %d: %s", dev,
               hipGetErrorString(e));
    sample_static_ptr[dev] = (float*)p;
  }
  *ptr = sample_static_ptr[dev];
  return 0;
}

extern "C" int pi_sample_static(int* out, const float* logits, long row_stride, const float* temperature,
                                const float* uniform, int M, int V, hipStream_t stream) {
  PI_REQUIRE(M >= 0 && V > 0 && row_stride >= V, "sample_static: bad sizes M=%d V=%d stride=%ld", M, V, row_stride);
  PI_REQUIRE(temperature == nullptr || uniform != nullptr, "sample_static: temperatures given without uniform numbers");
  if (M == 0) return 0;
  const int chunks = pi_sample_chunks(V);
  if (chunks == 0) return pi_sample(out, logits, row_stride, temperature, uniform, M, V, nullptr, 0, stream);
  PI_REQUIRE(M <= 65535 && (long)M * chunks * CHUNK_REC <= PI_SAMPLE_STATIC_FLOATS,
             "sample_static: %d rows of %d logits need %ld floats of chunk records; the library's array holds %d "
             "(at most %d rows of this length)",
             M, V, (long)M * chunks * CHUNK_REC, PI_SAMPLE_STATIC_FLOATS, PI_SAMPLE_STATIC_FLOATS / (chunks * CHUNK_REC));
  float* records = nullptr;
  if (sample_static_address(&records)) return -1;
  return pi_sample(out, logits, row_stride, temperature, uniform, M, V, records, PI_SAMPLE_STATIC_FLOATS, stream);
}

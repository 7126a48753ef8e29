// General matrix product C[M, N] (+)= A[M, K] . W[N, K]^T for any M, N, K and any mix of
// float32 / bfloat16 operands, with float32 multiply-add throughout (no matrix cores, no
// reduced-precision mode).  It is the whole-model float32 path and the fallback for sizes
// the matrix-core kernels do not take.
//
// Convention (include/photon/ops/kernels/matmul_kernel.hpp:54-129): activations
// row-major [rows, in], weights row-major [out, in], y = x W^T, no bias.
//
// Each output element accumulates over k in ascending order, 16 at a time, so a row's
// result does not depend on which other rows share the launch.
//
// Up to 16 rows of activations (decode steps) take a second kernel that streams the weights:
// a block owns a few weight rows, its waves take turns over k, their lanes four elements at a time (16-byte loads that
// follow the row), the activations of a k chunk are shared through LDS, and every output is
// summed over the lanes and waves at the end.  A lane adds its own k in ascending order and the
// lanes and waves are added in a fixed order, so here too a row's result does not depend on the
// other rows.
#include "common.h"

#define GT 64   // output tile edge
#define GK 16   // reduction slab

template <typename TA, typename TW, typename TC, bool ACCUM>
__global__ __launch_bounds__(256) void gemm_general_kernel(TC* __restrict__ C, long ldc, const TA* __restrict__ A, long lda,
                                                           const TW* __restrict__ W, long ldw, int M, int N, int K) {
  __shared__ float As[GK][GT + 4];
  __shared__ float Ws[GK][GT + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const long m0 = (long)blockIdx.y * GT, n0 = (long)blockIdx.x * GT;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      const int row = idx / GK, kk = idx % GK;
      const long m = m0 + row, n = n0 + row;
      const int k = k0 + kk;
      As[kk][row] = (m < M && k < K) ? to_float(A[m * lda + k]) : 0.f;
      Ws[kk][row] = (n < N && k < K) ? to_float(W[n * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n >= N) continue;
      TC* c = C + m * ldc + n;
      if (ACCUM)
        *c = from_float<TC>(to_float(*c) + acc[i][j]);
      else
        *c = from_float<TC>(acc[i][j]);
    }
  }
}

// ------------------------------------------------------------------ few rows: stream the weights

// MT: rows of activations the kernel holds (M <= MT); R: weight rows per wave.  KW = 1: a block's
// four waves take R rows each; KW = 4: they work on the same R rows, each on every fourth group
// of 256 k, and their sums meet in LDS and are added in wave order (matrices of few rows, which
// would otherwise leave most of the chip idle, and steps of one or two tokens).  K and the row
// strides are multiples of 4 and the operands 16-byte aligned (8-byte for bfloat16).
template <typename TA, typename TW, typename TC, bool ACCUM, int MT, int R, int KW>
__global__ __launch_bounds__(256) void gemm_rows_kernel(TC* __restrict__ C, long ldc, const TA* __restrict__ A, long lda,
                                                        const TW* __restrict__ W, long ldw, int M, int N, int K) {
  static_assert(R * MT <= PI_WAVE, "one lane per output of a wave");
  static_assert(KW == 1 || KW == 4, "the waves of a block share their rows or do not");
  constexpr int ROWS_KC = (8192 / MT) < 1024 ? 1024 : (8192 / MT) > 4096 ? 4096 : (8192 / MT);   // k per chunk of activations in LDS
  constexpr int GROUP = 4 * PI_WAVE;             // k a wave covers with one load per lane and row
  __shared__ __attribute__((aligned(16))) float As[MT][ROWS_KC];
  __shared__ float sums[4][R * MT];
  const int tid = threadIdx.x, lane = tid % PI_WAVE, wave = tid / PI_WAVE;
  const long n0 = KW == 1 ? ((long)blockIdx.x * 4 + wave) * R : (long)blockIdx.x * R;
  const TW* wrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) wrow[r] = W + (n0 + r < N ? n0 + r : (long)N - 1) * ldw;   // rows beyond N: the last row, never stored
  float acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;
  for (int k0 = 0; k0 < K; k0 += ROWS_KC) {
    for (int idx = tid; idx < MT * (ROWS_KC / 4); idx += 256) {
      const int m = idx / (ROWS_KC / 4), kl = (idx % (ROWS_KC / 4)) * 4;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (m < M && k0 + kl < K) load4(A + (long)m * lda + k0 + kl, v);
      *reinterpret_cast<float4*>(&As[m][kl]) = make_float4(v[0], v[1], v[2], v[3]);
    }
    __syncthreads();
#pragma unroll
    for (int sub = 0; sub < ROWS_KC / GROUP / KW; ++sub) {
      const int kl = (KW == 1 ? sub : sub * 4 + wave) * GROUP + lane * 4;      // this wave's group of the chunk
      if (k0 + kl < K) {
        float w[R][4];
#pragma unroll
        for (int r = 0; r < R; ++r) load4(wrow[r] + k0 + kl, w[r]);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float4 a = *reinterpret_cast<const float4*>(&As[m][kl]);
#pragma unroll
          for (int r = 0; r < R; ++r) {
            acc[r][m] = fmaf(a.x, w[r][0], acc[r][m]);
            acc[r][m] = fmaf(a.y, w[r][1], acc[r][m]);
            acc[r][m] = fmaf(a.z, w[r][2], acc[r][m]);
            acc[r][m] = fmaf(a.w, w[r][3], acc[r][m]);
          }
        }
      }
    }
    __syncthreads();
  }
  // every output summed over the lanes of its wave (then over the waves, in wave order); lane
  // (or thread) r * MT + m keeps output (m, n0 + r)
  float mine = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float total = wave_sum(acc[r][m]);
      if (lane == r * MT + m) mine = total;
    }
  if (KW == 4) {
    if (lane < R * MT) sums[wave][lane] = mine;
    __syncthreads();
    if (wave != 0) return;
    if (lane < R * MT) mine = ((sums[0][lane] + sums[1][lane]) + sums[2][lane]) + sums[3][lane];
  }
  const int r = lane / MT, m = lane % MT;
  if (lane < R * MT && m < M && n0 + r < N) {
    TC* c = C + (long)m * ldc + n0 + r;
    *c = ACCUM ? from_float<TC>(to_float(*c) + mine) : from_float<TC>(mine);
  }
}

template <typename TA, typename TW, typename TC>
static int launch_rows(void* C, long ldc, const void* A, long lda, const void* W, long ldw, int M, int N, int K, int accumulate,
                       hipStream_t stream) {
  const dim3 block(256);
#define ROWS_GO(ACC, MT, R, KW) hipLaunchKernelGGL((gemm_rows_kernel<TA, TW, TC, ACC, MT, R, KW>), dim3(ceil_div(N, R * (KW == 1 ? 4 : 1))), block, 0, \
                                                   stream, (TC*)C, ldc, (const TA*)A, lda, (const TW*)W, ldw, M, N, K)
#define ROWS_PICK(MT, R1, R4)                                                                    \
  do {                                                                                           \
    if (few_rows) { if (accumulate) ROWS_GO(true, MT, R4, 4); else ROWS_GO(false, MT, R4, 4); }  \
    else { if (accumulate) ROWS_GO(true, MT, R1, 1); else ROWS_GO(false, MT, R1, 1); }           \
  } while (0)
  // a matrix of few rows gives too few blocks when every wave takes rows of its own: its blocks'
  // waves share their rows and split k instead
  const bool few_rows = N < 8192;
  if (M <= 2) {
    if (accumulate) ROWS_GO(true, 2, 8, 4); else ROWS_GO(false, 2, 8, 4);
  } else if (M <= 8) {
    ROWS_PICK(8, 4, 8);
  } else {
    ROWS_PICK(16, 2, 4);
  }
#undef ROWS_PICK
#undef ROWS_GO
  return pi_check_launch("gemm_rows");
}

template <typename TA, typename TW, typename TC>
static int launch(void* C, long ldc, const void* A, long lda, const void* W, long ldw, int M, int N, int K, int accumulate,
                  hipStream_t stream) {
  if (M <= 16 && K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0 && (long)N < 2147483647L)
    return launch_rows<TA, TW, TC>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
  const dim3 grid(ceil_div(N, GT), ceil_div(M, GT)), block(256);
  if (grid.y > 65535) return pi_fail("gemm: too many rows (%d)", M);
  if (accumulate)
    hipLaunchKernelGGL((gemm_general_kernel<TA, TW, TC, true>), grid, block, 0, stream, (TC*)C, ldc, (const TA*)A, lda, (const TW*)W, ldw, M, N, K);
  else
    hipLaunchKernelGGL((gemm_general_kernel<TA, TW, TC, false>), grid, block, 0, stream, (TC*)C, ldc, (const TA*)A, lda, (const TW*)W, ldw, M, N, K);
  return pi_check_launch("gemm_general");
}

// dtypes: a = activations, w = weights, c = output.  accumulate requires float32 output.
extern "C" int pi_gemm_general(void* C, int c_dtype, long ldc, const void* A, int a_dtype, long lda, const void* W,
                               int w_dtype, long ldw, int M, int N, int K, int accumulate, hipStream_t stream) {
  PI_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  PI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: row strides (%ld, %ld, %ld) smaller than the rows (K=%d, N=%d)", lda, ldw, ldc, K, N);
  PI_REQUIRE(!accumulate || c_dtype == PI_F32, "gemm: accumulation needs a float32 output");
  if (M == 0) return 0;
  const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (key) {
    case 0: return launch<float, float, float>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 1: return launch<float, float, bf16_t>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 2: return launch<float, bf16_t, float>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 3: return launch<float, bf16_t, bf16_t>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 4: return launch<bf16_t, float, float>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 5: return launch<bf16_t, float, bf16_t>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 6: return launch<bf16_t, bf16_t, float>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
    case 7: return launch<bf16_t, bf16_t, bf16_t>(C, ldc, A, lda, W, ldw, M, N, K, accumulate, stream);
  }
  return pi_fail("gemm: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
}

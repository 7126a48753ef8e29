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

template <typename TA, typename TW, typename TC>
static int launch(void* C, long ldc, const void* A, long lda, const void* W, long ldw, int M, int N, int K, int accumulate,
                  hipStream_t stream) {
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

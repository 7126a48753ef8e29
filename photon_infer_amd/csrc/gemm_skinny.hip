// bfloat16 matrix product for few rows (decoding: 1..64 tokens), where the weights are read
// once from HBM and everything else is small:  C[M, N] (+)= X[M, K] . W[N, K]^T.
//
// The weights are the row operand of v_mfma_f32_16x16x32_bf16 and the activations the column
// operand, so a wave produces C^T for 32 weight rows (two row tiles) and up to 64 tokens.
// A lane reads 32 contiguous bytes of a weight row per step; the four lane groups of a row
// cover 128 contiguous bytes.  No LDS on the way in: activations come from L2.
// A block is four waves on the same 32 rows, each on a quarter of the block's k-range; they
// add up through LDS.  The k-range may further be split over blocks (grid.y): each block
// then writes its partial tile to a workspace and the consumer of the product adds the
// partials in split order (deterministic).
//
// Epilogues as in the many-row kernel: store bf16, store f32, add into f32, SwiGLU (gate / up
// rows interleaved by 16, so the two row tiles of a wave are the gate and the up rows of the
// same 16 features; no k-split over blocks in that case).
#include "mfma.h"

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACCUM = 2, EPI_SWIGLU = 3 };

#define ROWS_PER_BLOCK 32
#define KSTEP 64

template <int EPI>
__device__ inline void epilogue_store(void* Cv, long ldc, long m, long n, float v) {
  if (EPI == EPI_BF16) reinterpret_cast<bf16_t*>(Cv)[m * ldc + n] = from_float<bf16_t>(v);
  if (EPI == EPI_F32) reinterpret_cast<float*>(Cv)[m * ldc + n] = v;
  if (EPI == EPI_ACCUM) reinterpret_cast<float*>(Cv)[m * ldc + n] += v;
}

template <int MB, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(void* __restrict__ Cv, long ldc, const bf16_t* __restrict__ X, long ldx,
                                                          const bf16_t* __restrict__ W, long ldw, int M, int N, int K,
                                                          int k_per_block, float* __restrict__ part) {
  __shared__ float red[4][ROWS_PER_BLOCK][MB * 16 + 1];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int lr = lane % 16, lg = lane / 16;
  const long n0 = (long)blockIdx.x * ROWS_PER_BLOCK;
  const int splits = gridDim.y;

  // this wave's k-range: a quarter (rounded up to whole steps) of the block's range
  const int kb0 = blockIdx.y * k_per_block;
  const int kb1 = min(K, kb0 + k_per_block);
  const int per_wave = ((kb1 - kb0 + 4 * KSTEP - 1) / (4 * KSTEP)) * KSTEP;
  const int k0 = kb0 + wave * per_wave;
  const int k1 = min(kb1, k0 + per_wave);

  // rows beyond N / tokens beyond M read the last valid row; their results are never stored
  const bf16_t* wrow[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) wrow[t] = W + min(n0 + t * 16 + lr, (long)N - 1) * ldw + lg * 16;
  const bf16_t* xrow[MB];
#pragma unroll
  for (int c = 0; c < MB; ++c) xrow[c] = X + (long)min(c * 16 + lr, M - 1) * ldx + lg * 16;

  f32x4_t acc[2][MB];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int c = 0; c < MB; ++c) acc[t][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  int kk = k0;
  for (; kk + KSTEP <= k1; kk += KSTEP) {
    Frag w[2][2], x[MB][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      w[t][0] = load_frag(wrow[t] + kk);
      w[t][1] = load_frag(wrow[t] + kk + 8);
    }
#pragma unroll
    for (int c = 0; c < MB; ++c) {
      x[c][0] = load_frag(xrow[c] + kk);
      x[c][1] = load_frag(xrow[c] + kk + 8);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int c = 0; c < MB; ++c) {
        acc[t][c] = mfma16(w[t][0], x[c][0], acc[t][c]);
        acc[t][c] = mfma16(w[t][1], x[c][1], acc[t][c]);
      }
  }
  if (kk < k1) {  // a last, partial step: 8-element chunks beyond k1 count as zero
    const int ka = kk + lg * 16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const bool ok = ka + h * 8 < k1;
      Frag w[2], x[MB];
#pragma unroll
      for (int t = 0; t < 2; ++t) w[t] = ok ? load_frag(wrow[t] + kk + h * 8) : zero_frag();
#pragma unroll
      for (int c = 0; c < MB; ++c) x[c] = ok ? load_frag(xrow[c] + kk + h * 8) : zero_frag();
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c = 0; c < MB; ++c) acc[t][c] = mfma16(w[t], x[c], acc[t][c]);
    }
  }

  // acc[t][c][r] is C^T[n0 + t*16 + lg*4 + r][c*16 + lr]; add the four waves through LDS
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int c = 0; c < MB; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][t * 16 + lg * 4 + r][c * 16 + lr] = acc[t][c][r];
  __syncthreads();

  const int cols = MB * 16;
  if (splits == 1) {
    if (EPI == EPI_SWIGLU) {
      for (int idx = tid; idx < 16 * cols; idx += 256) {
        const int j = idx % 16, m = idx / 16;
        const long n = n0 + j;                     // gate row; up row is n + 16
        if (m >= M || n + 16 >= N) continue;
        const float g = red[0][j][m] + red[1][j][m] + red[2][j][m] + red[3][j][m];
        const float u = red[0][16 + j][m] + red[1][16 + j][m] + red[2][16 + j][m] + red[3][16 + j][m];
        reinterpret_cast<bf16_t*>(Cv)[(long)m * ldc + n0 / 2 + j] = from_float<bf16_t>(g / (1.0f + expf(-g)) * u);
      }
    } else {
      for (int idx = tid; idx < ROWS_PER_BLOCK * cols; idx += 256) {
        const int nl = idx % ROWS_PER_BLOCK, m = idx / ROWS_PER_BLOCK;
        if (m >= M || n0 + nl >= N) continue;
        epilogue_store<EPI>(Cv, ldc, m, n0 + nl, red[0][nl][m] + red[1][nl][m] + red[2][nl][m] + red[3][nl][m]);
      }
    }
    return;
  }

  // k split over blocks: this block's partial tile goes to part[split][m][n]; whoever consumes
  // the product (the reduce kernel below, or a norm / rotation kernel that folds the sum into
  // its own read) adds the splits in split order.  No block waits for or signals another:
  // on a chip of several dies a device-wide fence costs more than a kernel boundary.
  float* mine = part + (long)blockIdx.y * M * N;
  for (int idx = tid; idx < ROWS_PER_BLOCK * cols; idx += 256) {
    const int nl = idx % ROWS_PER_BLOCK, m = idx / ROWS_PER_BLOCK;
    if (m >= M || n0 + nl >= N) continue;
    mine[(long)m * N + n0 + nl] = red[0][nl][m] + red[1][nl][m] + red[2][nl][m] + red[3][nl][m];
  }
}

// C[m][n] (op)= sum over splits of part[s][m][n], in split order.
template <int EPI>
__global__ void splitk_reduce_kernel(void* __restrict__ Cv, long ldc, const float* __restrict__ part, int splits, int M, int N) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)M * N) return;
  const long m = idx / N, n = idx % N;
  float sum = 0.f;
  for (int s = 0; s < splits; ++s) sum += part[(long)s * M * N + idx];
  epilogue_store<EPI>(Cv, ldc, m, n, sum);
}

extern "C" int pi_splitk_reduce(void* C, int epilogue, long ldc, const void* part, int splits, int M, int N, hipStream_t stream) {
  PI_REQUIRE(M > 0 && N > 0 && splits >= 1 && part, "splitk_reduce: bad arguments M=%d N=%d splits=%d", M, N, splits);
  const long total = (long)M * N;
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  switch (epilogue) {
    case EPI_BF16: hipLaunchKernelGGL(splitk_reduce_kernel<EPI_BF16>, grid, block, 0, stream, C, ldc, (const float*)part, splits, M, N); break;
    case EPI_F32: hipLaunchKernelGGL(splitk_reduce_kernel<EPI_F32>, grid, block, 0, stream, C, ldc, (const float*)part, splits, M, N); break;
    case EPI_ACCUM: hipLaunchKernelGGL(splitk_reduce_kernel<EPI_ACCUM>, grid, block, 0, stream, C, ldc, (const float*)part, splits, M, N); break;
    default: return pi_fail("splitk_reduce: unknown epilogue %d", epilogue);
  }
  return pi_check_launch("splitk_reduce");
}

template <int MB>
static int launch_mb(int epi, dim3 grid, hipStream_t stream, void* C, long ldc, const bf16_t* X, long ldx, const bf16_t* W,
                     long ldw, int M, int N, int K, int kpb, float* part) {
#define GO(E) hipLaunchKernelGGL((gemm_skinny_kernel<MB, E>), grid, dim3(256), 0, stream, C, ldc, X, ldx, W, ldw, M, N, K, kpb, part)
  switch (epi) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    case EPI_ACCUM: GO(EPI_ACCUM); break;
    case EPI_SWIGLU: GO(EPI_SWIGLU); break;
    default: return pi_fail("gemm_skinny: unknown epilogue %d", epi);
  }
#undef GO
  return pi_check_launch("gemm_skinny");
}

// splits > 1: the partial products go to `part` (float32 [splits, M, N]) and C is not touched;
// *splits_out tells how many splits were made (no empty ones).
extern "C" int pi_gemm_skinny(void* C, int epilogue, long ldc, const void* X, long ldx, const void* W, long ldw, int M,
                              int N, int K, int splits, void* part, long part_elems, int* splits_out, hipStream_t stream) {
  PI_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: takes 1..64 rows, got M=%d N=%d K=%d", M, N, K);
  PI_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "gemm_skinny: K (%d) and row strides (%ld, %ld) must be multiples of 8", K, ldx, ldw);
  PI_REQUIRE(((uintptr_t)X % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_skinny: operands must be 16-byte aligned");
  PI_REQUIRE(splits >= 1 && splits <= 65535, "gemm_skinny: bad split count %d", splits);
  PI_REQUIRE(epilogue != EPI_SWIGLU || (splits == 1 && N % 32 == 0), "gemm_skinny: the SwiGLU epilogue needs one split and N (%d) a multiple of 32", N);
  const int groups = ceil_div(N, ROWS_PER_BLOCK);
  int kpb = ceil_div(K, splits);
  kpb = ((kpb + KSTEP - 1) / KSTEP) * KSTEP;
  splits = ceil_div(K, kpb);                      // no empty splits
  if (splits > 1)
    PI_REQUIRE(part && part_elems >= (long)splits * M * N, "gemm_skinny: workspace too small (%ld floats for %ld)", part_elems, (long)splits * M * N);
  if (splits_out) *splits_out = splits;
  const dim3 grid(groups, splits);
  const int mb = (M + 15) / 16;
  const bf16_t *x = (const bf16_t*)X, *w = (const bf16_t*)W;
  switch (mb) {
    case 1: return launch_mb<1>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part);
    case 2: return launch_mb<2>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part);
    case 3: return launch_mb<3>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part);
    default: return launch_mb<4>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part);
  }
}

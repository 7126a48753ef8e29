// bfloat16 matrix product on the matrix cores for many rows (prompts):
//   C[M, N] (+)= A[M, K] . W[N, K]^T, float32 accumulation.
// Block tile 128 x 128, reduction slab 64, four waves in 2 x 2, each wave 64 x 64 as 4 x 4
// tiles of v_mfma_f32_16x16x32_bf16.  Slabs go global -> registers -> LDS (double buffered,
// rows padded to 144 bytes so 16-byte fragment reads do not collide on banks).
//
// Epilogues: store bfloat16, store float32, add into float32 (the residual stream), or
// SwiGLU: with gate and up rows interleaved in blocks of 16 in W, a lane holds the gate and
// the up value of the same (row, feature) and stores silu(gate) * up directly.
//
// Any M and N (edges are zero-filled on load and skipped on store); K must be a multiple of
// 8 and row strides multiples of 8 so that 16-byte loads stay aligned.  Each output row
// accumulates over k in the same order whatever the other rows are.
#include "mfma.h"

PI_DEFINE_MODULE(bf16)

#define BM 128
#define BN 128
#define BK 64
#define LDS_ROW (BK + 8)                    // bf16 elements per padded row
#define TILE_ELEMS (BM * LDS_ROW)

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACCUM = 2, EPI_SWIGLU = 3 };

__device__ inline float silu_mul(float g, float u) { return g / (1.0f + expf(-g)) * u; }

template <int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(void* __restrict__ Cv, long ldc, const bf16_t* __restrict__ A, long lda,
                                                        const bf16_t* __restrict__ W, long ldw, int M, int N, int K,
                                                        int tiles_n, int k_per_split) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  uint16_t* As = lds;                       // [2][BM][LDS_ROW]
  uint16_t* Ws = lds + 2 * TILE_ELEMS;      // [2][BN][LDS_ROW]
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  // k split over blocks (gridDim.y > 1, float32 store only): split s owns k in
  // [s * k_per_split, (s + 1) * k_per_split) and writes its piece to C + s * M * N.
  const int k_lo = blockIdx.y * k_per_split;
  const int k_hi = min(K, k_lo + k_per_split);
  if (gridDim.y > 1) Cv = reinterpret_cast<float*>(Cv) + (long)blockIdx.y * M * ldc;
  // Consecutive blocks go to the chip's 8 dies in turn, each with an L2 of its own.  Give every
  // die a contiguous range of weight tiles (columns) and let it walk the row tiles of a column
  // before the next column: a die then streams its slice of W once and re-reads only A.
  const int tiles_m = gridDim.x / tiles_n;
  int tile_m, tile_n;
  if (tiles_n % 8 == 0) {
    const int die = blockIdx.x % 8, local = blockIdx.x / 8;
    tile_n = die * (tiles_n / 8) + local / tiles_m;
    tile_m = local % tiles_m;
  } else {
    tile_m = blockIdx.x / tiles_n;
    tile_n = blockIdx.x % tiles_n;
  }
  const long m0 = (long)tile_m * BM, n0 = (long)tile_n * BN;

  // global -> register staging: thread t moves 16-byte chunk (t % 8) of rows (t / 8) + 32 p
  // (eight lanes move one row's 128 bytes; the next eight lanes take the row 8 further down, so
  // that sixteen lanes land on 64 distinct LDS banks with rows 144 bytes apart)
  const int lgrp = tid / 8, lchunk = tid % 8;
  const int lrow = (lgrp / 16) * 16 + ((lgrp / 8) % 2) * 4 + (lgrp % 8) / 2 + 8 * (lgrp % 2);
  uint4 ra[4], rw[4];
  auto load_slab = [&](int k0) {
    const int k = k0 + lchunk * 8;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const long m = m0 + lrow + 32 * p, n = n0 + lrow + 32 * p;
      ra[p] = (m < M && k < k_hi) ? *reinterpret_cast<const uint4*>(A + m * lda + k) : make_uint4(0, 0, 0, 0);
      rw[p] = (n < N && k < k_hi) ? *reinterpret_cast<const uint4*>(W + n * ldw + k) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int off = (lrow + 32 * p) * LDS_ROW + lchunk * 8;
      *reinterpret_cast<uint4*>(As + buf * TILE_ELEMS + off) = ra[p];
      *reinterpret_cast<uint4*>(Ws + buf * TILE_ELEMS + off) = rw[p];
    }
  };

  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int slabs = (k_hi - k_lo + BK - 1) / BK;
  load_slab(k_lo);
  store_slab(0);
  __syncthreads();
  const int frow = lane % 16, fk = (lane / 16) * 8;
  for (int s = 0; s < slabs; ++s) {
    const int buf = s & 1;
    if (s + 1 < slabs) load_slab(k_lo + (s + 1) * BK);
    const uint16_t* a_base = As + buf * TILE_ELEMS + (wm * 64 + frow) * LDS_ROW + fk;
    const uint16_t* w_base = Ws + buf * TILE_ELEMS + (wn * 64 + frow) * LDS_ROW + fk;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      Frag a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i].q = *reinterpret_cast<const uint4*>(a_base + i * 16 * LDS_ROW + ks * 32);
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j].q = *reinterpret_cast<const uint4*>(w_base + j * 16 * LDS_ROW + ks * 32);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma16(a[i], b[j], acc[i][j]);
    }
    if (s + 1 < slabs) store_slab(buf ^ 1);
    __syncthreads();
  }

  // epilogue: acc[i][j][r] is C[m0 + wm*64 + i*16 + (lane/16)*4 + r][n0 + wn*64 + j*16 + lane%16]
  const int crow = (lane / 16) * 4, ccol = lane % 16;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const long m = m0 + wm * 64 + i * 16 + crow + r;
      if (m >= M) continue;
      if (EPI == EPI_SWIGLU) {
        bf16_t* C = reinterpret_cast<bf16_t*>(Cv);
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
          const long n = n0 + wn * 64 + j * 16 + ccol;        // gate column; up is at n + 16
          if (n + 16 < N) C[m * ldc + (n0 + wn * 64 + j * 16) / 2 + ccol] = from_float<bf16_t>(silu_mul(acc[i][j][r], acc[i][j + 1][r]));
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const long n = n0 + wn * 64 + j * 16 + ccol;
          if (n >= N) continue;
          if (EPI == EPI_BF16) reinterpret_cast<bf16_t*>(Cv)[m * ldc + n] = from_float<bf16_t>(acc[i][j][r]);
          if (EPI == EPI_F32) reinterpret_cast<float*>(Cv)[m * ldc + n] = acc[i][j][r];
          if (EPI == EPI_ACCUM) reinterpret_cast<float*>(Cv)[m * ldc + n] += acc[i][j][r];
        }
      }
    }
  }
}

static const size_t kLdsBytes = 4 * TILE_ELEMS * sizeof(uint16_t);   // 73,728 bytes

template <int EPI>
static int launch(void* C, long ldc, const void* A, long lda, const void* W, long ldw, int M, int N, int K, int splits,
                  hipStream_t stream) {
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_mfma_kernel<EPI>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
    if (e != hipSuccess) return pi_fail("gemm_mfma: cannot reserve %zu bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
    configured = true;
  }
  const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
  int kps = ceil_div(K, splits);
  kps = ((kps + BK - 1) / BK) * BK;
  splits = ceil_div(K, kps);
  hipLaunchKernelGGL((gemm_mfma_kernel<EPI>), dim3((unsigned)tiles_m * tiles_n, splits), dim3(256), kLdsBytes, stream, C, ldc,
                     (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, tiles_n, kps);
  return pi_check_launch("gemm_mfma");
}

// Pieces a k-split into `splits` makes (the kernel rounds a split's range up to whole slabs).
extern "C" int pi_gemm_mfma_pieces(int K, int splits) {
  if (splits < 1 || K < 1) return 0;
  int kps = ceil_div(K, splits);
  kps = ((kps + BK - 1) / BK) * BK;
  return ceil_div(K, kps);
}

// epilogue: 0 store bf16, 1 store f32, 2 add into f32, 3 SwiGLU (W rows interleaved by 16; C is [M, N / 2] bf16)
extern "C" int pi_gemm_mfma(void* C, int epilogue, long ldc, const void* A, long lda, const void* W, long ldw, int M,
                            int N, int K, int splits, hipStream_t stream) {
  PI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma: bad sizes M=%d N=%d K=%d", M, N, K);
  // splits > 1: C is a float32 workspace [splits, M, N] (ldc = N) that receives the pieces; the
  // number of pieces is ceil(K / (ceil(K / splits) rounded up to 64))
  PI_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || (epilogue == EPI_F32 && ldc == N)),
             "gemm_mfma: a k-split (%d) needs the float32 store into a [splits, M, N] workspace", splits);
  PI_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_mfma: K (%d) and row strides (%ld, %ld) must be multiples of 8", K, lda, ldw);
  PI_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_mfma: operands must be 16-byte aligned");
  PI_REQUIRE(epilogue != EPI_SWIGLU || N % 32 == 0, "gemm_mfma: the SwiGLU epilogue needs N (%d) to be a multiple of 32", N);
  PI_REQUIRE((long)ceil_div(M, BM) * ceil_div(N, BN) < 2147483647L, "gemm_mfma: too many tiles");
  switch (epilogue) {
    case EPI_BF16: return launch<EPI_BF16>(C, ldc, A, lda, W, ldw, M, N, K, splits, stream);
    case EPI_F32: return launch<EPI_F32>(C, ldc, A, lda, W, ldw, M, N, K, splits, stream);
    case EPI_ACCUM: return launch<EPI_ACCUM>(C, ldc, A, lda, W, ldw, M, N, K, splits, stream);
    case EPI_SWIGLU: return launch<EPI_SWIGLU>(C, ldc, A, lda, W, ldw, M, N, K, splits, stream);
  }
  return pi_fail("gemm_mfma: unknown epilogue %d", epilogue);
}

// bfloat16 matrix product on the matrix cores for many rows (prompts):
//   C[M, N] (+)= A[M, K] . W[N, K]^T, float32 accumulation.
// Block tile 128 x 128, reduction slab 64, four waves in 2 x 2, each wave 64 x 64 as 2 x 2
// tiles of v_mfma_f32_32x32x16_bf16.  Slabs go global -> registers -> LDS (double buffered,
// rows padded to 144 bytes so 16-byte fragment reads do not collide on banks).
//
// Epilogues: store bfloat16, store float32, add into float32 (the residual stream), or
// SwiGLU: with gate and up rows interleaved in blocks of 16 in W, the gate and the up value of
// the same (row, feature) sit 16 lanes apart; one row swap brings them together and
// silu(gate) * up is stored directly.
//
// Any M and N (edges read zeros and are skipped on store); K must be a multiple of
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

// silu(g) * u for a bfloat16 result: the hardware exponential and reciprocal (1 ulp each) are
// far inside the rounding of the store
__device__ inline float silu_mul(float g, float u) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g)) * u;
}

// Global loads go through buffer descriptors: a scalar base (the block's first row at its first
// k), a byte length, and per-lane 32-bit offsets.  An offset at or beyond the length reads
// zeros, which is how rows beyond the matrix and k beyond the range are filled, without a branch.
#define PI_OUT_OF_RANGE 0x7ffffff0u
#if defined(__HIP_DEVICE_COMPILE__)
__device__ inline __amdgpu_buffer_rsrc_t operand_descriptor(const bf16_t* base, long bytes) {
  // made scalar by hand so that the loads take the descriptor from scalar registers
  const uint64_t v = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  void* p = reinterpret_cast<void*>((static_cast<uint64_t>(hi) << 32) | lo);
  return __builtin_amdgcn_make_buffer_rsrc(p, 0, __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000);
}
#endif

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
  const int a_rows = (int)min((long)BM, M - m0), w_rows = (int)min((long)BN, N - n0);
#if defined(__HIP_DEVICE_COMPILE__)
  const __amdgpu_buffer_rsrc_t a_src = operand_descriptor(A + m0 * lda + k_lo, ((long)(a_rows - 1) * lda + (k_hi - k_lo)) * 2);
  const __amdgpu_buffer_rsrc_t w_src = operand_descriptor(W + n0 * ldw + k_lo, ((long)(w_rows - 1) * ldw + (k_hi - k_lo)) * 2);
#endif
  unsigned a_off[4], w_off[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int row = lrow + 32 * p;
    a_off[p] = row < a_rows ? (unsigned)(row * (int)lda + lchunk * 8) * 2u : PI_OUT_OF_RANGE;
    w_off[p] = row < w_rows ? (unsigned)(row * (int)ldw + lchunk * 8) * 2u : PI_OUT_OF_RANGE;
  }
  u32x4_t ra[4], rw[4];
  auto load_slab = [&](int k0) {
    // k0 is relative to k_lo; this lane's 8 k of the slab may lie beyond the range (last slab)
    const unsigned kb = (unsigned)k0 * 2u;
    const bool k_in = k0 + lchunk * 8 < k_hi - k_lo;
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      ra[p] = __builtin_amdgcn_raw_buffer_load_b128(a_src, k_in ? a_off[p] + kb : PI_OUT_OF_RANGE, 0, 0);
      rw[p] = __builtin_amdgcn_raw_buffer_load_b128(w_src, k_in ? w_off[p] + kb : PI_OUT_OF_RANGE, 0, 0);
    }
#endif
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int off = (lrow + 32 * p) * LDS_ROW + lchunk * 8;
      *reinterpret_cast<u32x4_t*>(As + buf * TILE_ELEMS + off) = ra[p];
      *reinterpret_cast<u32x4_t*>(Ws + buf * TILE_ELEMS + off) = rw[p];
    }
  };

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int slabs = (k_hi - k_lo + BK - 1) / BK;
  load_slab(0);
  store_slab(0);
  __syncthreads();
  // 32 x 32 x 16 instruction: a lane reads row lane % 32, 16 bytes at k = (lane / 32) * 8; with
  // rows 144 bytes apart the 16 lanes served together fall on distinct banks
  const int frow = lane % 32, fk = (lane / 32) * 8;
  for (int s = 0; s < slabs; ++s) {
    const int buf = s & 1;
    if (s + 1 < slabs) load_slab((s + 1) * BK);
    const uint16_t* a_base = As + buf * TILE_ELEMS + (wm * 64 + frow) * LDS_ROW + fk;
    const uint16_t* w_base = Ws + buf * TILE_ELEMS + (wn * 64 + frow) * LDS_ROW + fk;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      Frag a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i].n = *reinterpret_cast<const u32x4_t*>(a_base + i * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int j = 0; j < 2; ++j) b[j].n = *reinterpret_cast<const u32x4_t*>(w_base + j * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(a[i], b[j], acc[i][j]);
    }
    if (s + 1 < slabs) store_slab(buf ^ 1);
    __syncthreads();
  }

  // acc[i][j][v] is C[m0 + wm*64 + i*32 + 8*(v/4) + 4*(lane/32) + v%4][n0 + wn*64 + j*32 + lane%32]
  const int half = lane / 32, ccol = lane % 32;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const long nb = n0 + wn * 64 + j * 32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const long m = m0 + wm * 64 + i * 32 + 8 * (v / 4) + 4 * half + v % 4;
        if (EPI == EPI_SWIGLU) {
          // columns 0..15 of a tile are gate rows of W, 16..31 the up rows of the same features:
          // the swap leaves the gate value in both 16-lane rows of one result and the up value
          // in both rows of the other; the lower rows store
#if defined(__HIP_DEVICE_COMPILE__)
          const unsigned bits = __float_as_uint(acc[i][j][v]);
          auto gu = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
          if (ccol < 16 && m < M && nb + ccol + 16 < N)
            reinterpret_cast<bf16_t*>(Cv)[m * ldc + nb / 2 + ccol] = from_float<bf16_t>(silu_mul(__uint_as_float(gu[0]), __uint_as_float(gu[1])));
#endif
        } else {
          const long n = nb + ccol;
          if (m >= M || n >= N) continue;
          if (EPI == EPI_BF16) reinterpret_cast<bf16_t*>(Cv)[m * ldc + n] = from_float<bf16_t>(acc[i][j][v]);
          if (EPI == EPI_F32) reinterpret_cast<float*>(Cv)[m * ldc + n] = acc[i][j][v];
          if (EPI == EPI_ACCUM) reinterpret_cast<float*>(Cv)[m * ldc + n] += acc[i][j][v];
        }
      }
    }
}

// ---------------------------------------------------------------------------------------------
// The same product with block tile 256 x 256 for problems that have enough of them to fill the
// chip and a k that is a multiple of the slab: four waves in 2 x 2, each 128 x 128 as 4 x 4
// tiles of v_mfma_f32_32x32x16_bf16.  Per 16 k a wave reads 8 fragments from LDS for 16
// matrix-core instructions, half the LDS traffic per flop of the 128 x 128 kernel.  The
// accumulators alone are 256 registers, so there is one wave per SIMD and nothing else to fill
// its idle cycles: every load, LDS access and address computation has to be issued in the
// shadow of a matrix-core instruction (32 cycles each).  Hence no branch in the loop (rows
// beyond the matrix are clamped on load and skipped on store), global loads through a buffer
// descriptor (a scalar base that moves with k plus fixed 32-bit lane offsets, no vector
// arithmetic per slab), and scheduling hints that deal the memory instructions out between
// the matrix-core ones.  A slab's global loads are issued a whole slab before they are stored.
// Per output element the sum over k runs in ascending k, as in the small kernel.
#define GM 256
#define GN 256
#define BIG_TILE_ELEMS (GM * LDS_ROW)
#define PI_SCHED_MFMA 0x008
#define PI_SCHED_VMEM_READ 0x020
#define PI_SCHED_DS_READ 0x100
#define PI_SCHED_DS_WRITE 0x200

template <int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_big_kernel(void* __restrict__ Cv, long ldc, const bf16_t* __restrict__ A, long lda,
                                                            const bf16_t* __restrict__ W, long ldw, int M, int N, int K,
                                                            int tiles_n, int k_per_split) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  uint16_t* As = lds;                           // [2][GM][LDS_ROW]
  uint16_t* Ws = lds + 2 * BIG_TILE_ELEMS;      // [2][GN][LDS_ROW]
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wm = wave / 2, wn = wave % 2;
  const int k_lo = blockIdx.y * k_per_split;
  const int k_hi = min(K, k_lo + k_per_split);
  if (gridDim.y > 1) Cv = reinterpret_cast<float*>(Cv) + (long)blockIdx.y * M * ldc;
  const int tiles_m = gridDim.x / tiles_n;
  int tile_m, tile_n;
  if (tiles_n % 8 == 0) {                       // a die streams its own slice of W, see above
    const int die = blockIdx.x % 8, local = blockIdx.x / 8;
    tile_n = die * (tiles_n / 8) + local / tiles_m;
    tile_m = local % tiles_m;
  } else {
    tile_m = blockIdx.x / tiles_n;
    tile_n = blockIdx.x % tiles_n;
  }
  const long m0 = (long)tile_m * GM, n0 = (long)tile_n * GN;

  // global -> registers: thread t moves 16-byte chunk t % 8 of rows lrow + 32 p of both operands
  const int lgrp = tid / 8, lchunk = tid % 8;
  const int lrow = (lgrp / 16) * 16 + ((lgrp / 8) % 2) * 4 + (lgrp % 8) / 2 + 8 * (lgrp % 2);
  const int a_rows = (int)min((long)GM, M - m0), w_rows = (int)min((long)GN, N - n0);
#if defined(__HIP_DEVICE_COMPILE__)
  const __amdgpu_buffer_rsrc_t a_src = operand_descriptor(A + m0 * lda + k_lo, ((long)(a_rows - 1) * lda + (k_hi - k_lo)) * 2);
  const __amdgpu_buffer_rsrc_t w_src = operand_descriptor(W + n0 * ldw + k_lo, ((long)(w_rows - 1) * ldw + (k_hi - k_lo)) * 2);
#endif
  unsigned a_off[8], w_off[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    a_off[p] = (unsigned)(min(lrow + 32 * p, a_rows - 1) * (int)lda + lchunk * 8) * 2u;
    w_off[p] = (unsigned)(min(lrow + 32 * p, w_rows - 1) * (int)ldw + lchunk * 8) * 2u;
  }
  u32x4_t ra[8], rw[8];
  const int slabs = (k_hi - k_lo) / BK;
  auto load_slab = [&](int s) {
    const int kbytes = min(s, slabs - 1) * BK * 2;     // past the last slab: read it again, unused
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      ra[p] = __builtin_amdgcn_raw_buffer_load_b128(a_src, a_off[p], kbytes, 0);
      rw[p] = __builtin_amdgcn_raw_buffer_load_b128(w_src, w_off[p], kbytes, 0);
    }
#endif
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int off = (lrow + 32 * p) * LDS_ROW + lchunk * 8;
      *reinterpret_cast<u32x4_t*>(As + buf * BIG_TILE_ELEMS + off) = ra[p];
      *reinterpret_cast<u32x4_t*>(Ws + buf * BIG_TILE_ELEMS + off) = rw[p];
    }
  };

  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int frow = lane % 32, fk = (lane / 32) * 8;
  Frag fa[2][4], fb[2][4];
  auto read_frags = [&](int which, int buf, int ks) {   // ks: which 16 k of the slab
    const uint16_t* a_base = As + buf * BIG_TILE_ELEMS + (wm * 128 + frow) * LDS_ROW + fk + ks * 16;
    const uint16_t* w_base = Ws + buf * BIG_TILE_ELEMS + (wn * 128 + frow) * LDS_ROW + fk + ks * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[which][i].n = *reinterpret_cast<const u32x4_t*>(a_base + i * 32 * LDS_ROW);
#pragma unroll
    for (int j = 0; j < 4; ++j) fb[which][j].n = *reinterpret_cast<const u32x4_t*>(w_base + j * 32 * LDS_ROW);
  };
  auto products = [&](int which) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma32(fa[which][i], fb[which][j], acc[i][j]);
  };
  // the order wanted inside one scheduling region: one matrix-core instruction, then one of
  // each kind of memory instruction named, `n` times; the rest of the 16 after that
#define PI_DEAL(n, kind_a, kind_b)                                                   \
  _Pragma("unroll") for (int d_ = 0; d_ < n; ++d_) {                                 \
    __builtin_amdgcn_sched_group_barrier(PI_SCHED_MFMA, 1, 0);                       \
    if (kind_a) __builtin_amdgcn_sched_group_barrier(kind_a, 1, 0);                  \
    if (kind_b) __builtin_amdgcn_sched_group_barrier(kind_b, 1, 0);                  \
  }

  load_slab(0);
  store_slab(0);
  __syncthreads();
  load_slab(1);
  read_frags(0, 0, 0);
  for (int s = 0; s < slabs; ++s) {
    const int buf = s & 1;
    read_frags(1, buf, 1);
    products(0);
    PI_DEAL(8, PI_SCHED_DS_READ, 0)
    PI_DEAL(8, 0, 0)
    read_frags(0, buf, 2);
    products(1);
    PI_DEAL(8, PI_SCHED_DS_READ, 0)
    PI_DEAL(8, 0, 0)
    read_frags(1, buf, 3);
    products(0);
    store_slab(buf ^ 1);            // slab s + 1, loaded during the previous slab's last step
    PI_DEAL(8, PI_SCHED_DS_READ, PI_SCHED_DS_WRITE)
    PI_DEAL(8, PI_SCHED_DS_WRITE, 0)
    __syncthreads();
    load_slab(s + 2);
    read_frags(0, buf ^ 1, 0);
    products(1);
    PI_DEAL(8, PI_SCHED_VMEM_READ, PI_SCHED_DS_READ)
    PI_DEAL(8, PI_SCHED_VMEM_READ, 0)
  }
#undef PI_DEAL

  // acc[i][j][v] is C[m0 + wm*128 + i*32 + 8*(v/4) + 4*(lane/32) + v%4][n0 + wn*128 + j*32 + lane%32].
  // Offsets inside the wave's 128 x 128 corner are 32-bit (the host checks 128 * ldc fits).
  const int half = lane / 32, ccol = lane % 32;
  const long mw = m0 + wm * 128, nw = n0 + wn * 128;
  const int rows_left = (int)min((long)128, M - mw), cols_left = (int)min((long)128, N - nw);   // may be <= 0
  const int ld = (int)ldc;
  if (EPI == EPI_SWIGLU) {
    // columns 0..15 of a tile are gate rows of W, 16..31 the up rows of the same features: bring
    // the two together (the swap leaves the gate value in both 16-lane rows of one result and
    // the up value in both rows of the other); the lower rows store
    bf16_t* C = reinterpret_cast<bf16_t*>(Cv) + mw * ldc + nw / 2;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
#if defined(__HIP_DEVICE_COMPILE__)
          const unsigned bits = __float_as_uint(acc[i][j][v]);
          auto gu = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
          const int rl = i * 32 + 8 * (v / 4) + 4 * half + v % 4;
          if (ccol < 16 && rl < rows_left && j * 32 + ccol + 16 < cols_left)
            C[rl * ld + j * 16 + ccol] = from_float<bf16_t>(silu_mul(__uint_as_float(gu[0]), __uint_as_float(gu[1])));
#endif
        }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int rl = i * 32 + 8 * (v / 4) + 4 * half + v % 4, cl = j * 32 + ccol;
          if (rl >= rows_left || cl >= cols_left) continue;
          const int off = rl * ld + cl;
          if (EPI == EPI_BF16) (reinterpret_cast<bf16_t*>(Cv) + mw * ldc + nw)[off] = from_float<bf16_t>(acc[i][j][v]);
          if (EPI == EPI_F32) (reinterpret_cast<float*>(Cv) + mw * ldc + nw)[off] = acc[i][j][v];
          if (EPI == EPI_ACCUM) (reinterpret_cast<float*>(Cv) + mw * ldc + nw)[off] += acc[i][j][v];
        }
  }
}

static const size_t kBigLdsBytes = 4 * BIG_TILE_ELEMS * sizeof(uint16_t);   // 147,456 bytes
#define BIG_MIN_TILES 192      // enough 256 x 256 tiles (times k pieces) to occupy most of the chip

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
  int kps = ceil_div(K, splits);
  kps = ((kps + BK - 1) / BK) * BK;
  splits = ceil_div(K, kps);
  const long big_tiles = (long)ceil_div(M, GM) * ceil_div(N, GN);
  if (big_tiles * splits >= BIG_MIN_TILES && big_tiles < 2147483647L && ldc < (1L << 23) && K % BK == 0) {
    static bool big_configured = false;
    if (!big_configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_mfma_big_kernel<EPI>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLdsBytes);
      if (e != hipSuccess) return pi_fail("gemm_mfma: cannot reserve %zu bytes of LDS: %s", kBigLdsBytes, hipGetErrorString(e));
      big_configured = true;
    }
    hipLaunchKernelGGL((gemm_mfma_big_kernel<EPI>), dim3((unsigned)big_tiles, splits), dim3(256), kBigLdsBytes, stream, C, ldc,
                       (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, ceil_div(N, GN), kps);
    return pi_check_launch("gemm_mfma_big");
  }
  const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
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
  PI_REQUIRE(256 * lda < (1L << 29) && 256 * ldw < (1L << 29), "gemm_mfma: row strides (%ld, %ld) are too long for 32-bit offsets inside a tile", lda, ldw);
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

// bfloat16 matrix product on the matrix cores for many rows (prompts):
//   C[M, N] (+)= A[M, K] . W[N, K]^T, float32 accumulation.
// Block tile 128 x 128, reduction slab 64, four waves in 2 x 2, each wave 64 x 64 as 2 x 2
// tiles of v_mfma_f32_32x32x16_bf16.  Slabs go from memory straight into LDS (buffer loads
// with the LDS as their destination, double buffered): no registers and no LDS store
// instructions in between.  Such a load writes its 64 lanes' 16 bytes one after the other, so
// rows cannot be padded; instead the 16-byte pieces of a row are turned by (row / 2) % 8, which
// puts the fragment reads of sixteen neighbouring rows on all 64 banks.  (Through registers
// and padded rows, which this kernel did first, the q/k/v product of a 2,048-token prompt took
// 40 us instead of 34 and the 256 x 256 kernel below 133 us instead of 120 on the gate / up
// product: 230 instead of 180 registers, eight LDS stores per slab and thread.)
//
// Epilogues: store bfloat16, store float32, add into float32 (the residual stream), or
// SwiGLU: with gate and up rows interleaved in blocks of 16 in W, the gate and the up value of
// the same (row, feature) sit 16 lanes apart; one row swap brings them together and
// silu(gate) * up is stored directly.
//
// Any M and N (edges read zeros and are skipped on store); K must be a multiple of
// 8 and row strides multiples of 8 so that 16-byte loads stay aligned.  Each output row
// accumulates over k in the same order whatever the other rows are.
#include <type_traits>

#include "addressing.h"
#include "mfma.h"

PI_DEFINE_MODULE(bf16)

#define BM 128
#define BN 128
#define BK 64
#define TILE_ELEMS (BM * BK)                // a tile's slab in LDS: rows of 128 bytes

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACCUM = 2, EPI_SWIGLU = 3 };

// silu(g) * u for a bfloat16 result: the hardware exponential and reciprocal (1 ulp each) are
// far inside the rounding of the store
__device__ inline float silu_mul(float g, float u) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g)) * u;
}

// The epilogue of both kernels: 32 rows x 64 columns of a wave's result, held as two 32 x 32
// accumulator tiles (lane = column, register = row), go through a patch of LDS that belongs to
// the wave alone and come back with eight (bfloat16) or four (float32) neighbouring columns in
// one lane, so that a row leaves as whole 16-byte stores instead of 2- or 4-byte ones.
// `C` points at the corner's first element (for SwiGLU: of the halved output); rows_left and
// cols_left (input columns) may be <= 0 or ragged; `wide` says that 16-byte stores are aligned.
#define PATCH_LD 72                      // floats per patch row: rows r and r + 4 fall on different bank halves
#define PATCH_FLOATS (32 * PATCH_LD)

__device__ inline uint32_t pack2(float a, float b) { return f32x2_to_bf16x2_bits(a, b); }

template <int EPI>
__device__ inline void store_rows32(float* patch, const f32x16_t& acc0, const f32x16_t& acc1, void* C, int ld, int row0,
                                    int rows_left, int cols_left, int lane, bool wide) {
  const int half = lane / 32, ccol = lane % 32;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int r = 8 * (v / 4) + 4 * half + v % 4;
    patch[r * PATCH_LD + ccol] = acc0[v];
    patch[r * PATCH_LD + 32 + ccol] = acc1[v];
  }
  // the wave reads what its own lanes wrote: LDS serves one wave's accesses in order
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (EPI == EPI_SWIGLU) {
    // columns 0..15 of a tile are gate rows of W, 16..31 the up rows of the same features
    bf16_t* out = reinterpret_cast<bf16_t*>(C);
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int id = pass * 64 + lane, r = id / 4, j = (id % 4) / 2, q = id % 2;
      const float* g = patch + r * PATCH_LD + j * 32 + q * 8;
      const int oc = j * 16 + q * 8;                       // output column; its up column in the input is j*32 + 16 + q*8 (+7)
      if (row0 + r >= rows_left || j * 32 + 16 + q * 8 >= cols_left) continue;
      const f32x4_t g0 = *reinterpret_cast<const f32x4_t*>(g), g1 = *reinterpret_cast<const f32x4_t*>(g + 4);
      const f32x4_t u0 = *reinterpret_cast<const f32x4_t*>(g + 16), u1 = *reinterpret_cast<const f32x4_t*>(g + 20);
      float o[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) { o[e] = silu_mul(g0[e], u0[e]); o[4 + e] = silu_mul(g1[e], u1[e]); }
      bf16_t* dst = out + (row0 + r) * ld + oc;
      if (wide && j * 32 + 16 + q * 8 + 8 <= cols_left) {
        *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{pack2(o[0], o[1]), pack2(o[2], o[3]), pack2(o[4], o[5]), pack2(o[6], o[7])};
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (j * 32 + 16 + q * 8 + e < cols_left) dst[e] = from_float<bf16_t>(o[e]);
      }
    }
  } else if (EPI == EPI_BF16) {
    bf16_t* out = reinterpret_cast<bf16_t*>(C);
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int id = pass * 64 + lane, r = id / 8, c = (id % 8) * 8;
      if (row0 + r >= rows_left || c >= cols_left) continue;
      const float* src = patch + r * PATCH_LD + c;
      const f32x4_t a = *reinterpret_cast<const f32x4_t*>(src), b = *reinterpret_cast<const f32x4_t*>(src + 4);
      bf16_t* dst = out + (row0 + r) * ld + c;
      if (wide && c + 8 <= cols_left) {
        *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{pack2(a[0], a[1]), pack2(a[2], a[3]), pack2(b[0], b[1]), pack2(b[2], b[3])};
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c + e < cols_left) dst[e] = from_float<bf16_t>(e < 4 ? a[e] : b[e - 4]);
      }
    }
  } else {
    float* out = reinterpret_cast<float*>(C);
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
      const int id = pass * 64 + lane, r = id / 16, c = (id % 16) * 4;
      if (row0 + r >= rows_left || c >= cols_left) continue;
      f32x4_t a = *reinterpret_cast<const f32x4_t*>(patch + r * PATCH_LD + c);
      float* dst = out + (row0 + r) * ld + c;
      if (wide && c + 4 <= cols_left) {
        if (EPI == EPI_ACCUM) a += *reinterpret_cast<const f32x4_t*>(dst);
        *reinterpret_cast<f32x4_t*>(dst) = a;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c + e < cols_left) dst[e] = EPI == EPI_ACCUM ? dst[e] + a[e] : a[e];
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// Global loads go through buffer descriptors: a scalar base (the block's first row at its first
// k), a byte length, and per-lane 32-bit offsets.  An offset at or beyond the length reads
// zeros, which is how rows beyond the matrix and k beyond the range are filled, without a branch.
#if defined(__HIP_DEVICE_COMPILE__)
__device__ inline __amdgpu_buffer_rsrc_t operand_descriptor(const bf16_t* operand, addressing::Descriptor d) {
  // made scalar by hand so that the loads take the descriptor from scalar registers
  const long bytes = d.bytes;
  const uint64_t v = reinterpret_cast<uint64_t>(operand + d.base);
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
  constexpr int ROW = BK;                   // rows of 128 bytes, no padding (see the large-tile kernel)
  constexpr int TILE = BM * ROW;
  uint16_t* As = lds;                       // [2][BM][ROW], 16-byte pieces of a row turned by (row / 2) % 8
  uint16_t* Ws = lds + 2 * TILE;            // [2][BN][ROW]
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

  // global -> LDS without registers in between: load instruction p of wave w fills rows
  // (4 w + p) * 8 .. + 7 of a tile, lane l the 16-byte piece l % 8 of row l / 8, which is piece
  // (l % 8) ^ ((row / 2) % 8) of the row in memory.  Rows beyond the matrix and k beyond the
  // range take an offset outside the descriptor and arrive as zeros.
  const int a_rows = (int)min((long)BM, M - m0), w_rows = (int)min((long)BN, N - n0);
#if defined(__HIP_DEVICE_COMPILE__)
  const __amdgpu_buffer_rsrc_t a_src = operand_descriptor(A, addressing::tile_descriptor(m0, lda, k_lo, k_hi, a_rows));
  const __amdgpu_buffer_rsrc_t w_src = operand_descriptor(W, addressing::tile_descriptor(n0, ldw, k_lo, k_hi, w_rows));
#endif
  unsigned a_off[4], w_off[4];
  int piece_k[4];                           // the piece (8 k) of a slab's row that this lane fetches
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int row = (wave * 4 + p) * 8 + lane / 8;
    const int piece = addressing::tile_piece(lane, row);
    piece_k[p] = piece;
    a_off[p] = addressing::tile_lane_offset(row, a_rows, lda, piece);
    w_off[p] = addressing::tile_lane_offset(row, w_rows, ldw, piece);
  }
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto load_slab = [&](int k0, int buf) {
    // k0 is relative to k_lo; a lane's 8 k of the slab may lie beyond the range (last slab)
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_src, (lds_ptr_t)(As + buf * TILE + (wave * 4 + p) * 8 * ROW), 16,
                                               addressing::tile_slab_offset(a_off[p], k0, piece_k[p], k_hi - k_lo), 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_src, (lds_ptr_t)(Ws + buf * TILE + (wave * 4 + p) * 8 * ROW), 16,
                                               addressing::tile_slab_offset(w_off[p], k0, piece_k[p], k_hi - k_lo), 0, 0, 0);
    }
#endif
  };

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int slabs = (k_hi - k_lo + BK - 1) / BK;
  // 32 x 32 x 16 instruction: a lane reads row lane % 32, the 16 bytes of k = (lane / 32) * 8 of
  // every 16 k, at the place its row's turn puts them
  const int frow = lane % 32;
  int place[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) place[ks] = ((ks * 2 + lane / 32) ^ ((frow >> 1) & 7)) * 8;
  Frag fa[2][2], fb[2][2];
  auto read_frags = [&](int which, int buf, int ks) {   // ks: which 16 k of the slab
    const uint16_t* a_base = As + buf * TILE + (wm * 64 + frow) * ROW + place[ks];
    const uint16_t* w_base = Ws + buf * TILE + (wn * 64 + frow) * ROW + place[ks];
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[which][i].n = *reinterpret_cast<const u32x4_t*>(a_base + i * 32 * ROW);
#pragma unroll
    for (int j = 0; j < 2; ++j) fb[which][j].n = *reinterpret_cast<const u32x4_t*>(w_base + j * 32 * ROW);
  };
  auto products = [&](int which) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(fa[which][i], fb[which][j], acc[i][j]);
  };
  // The loop has no branch: a slab beyond the range loads zeros (offsets out of the
  // descriptor's range) into the buffer nobody reads.  Fragments of the next 16 k are read
  // while the matrix instructions of these 16 run; the hints deal one memory instruction of
  // each kind named after every matrix instruction.
  // The loop has no branch: a slab beyond the range arrives as zeros in the buffer nobody reads.
  // Fragments of the next 16 k are read while the matrix instructions of these 16 run; the hints
  // deal one memory instruction of each kind named after every matrix instruction.
#define PI_SCHED_MFMA 0x008
#define PI_SCHED_VMEM_READ 0x020
#define PI_SCHED_DS_READ 0x100
#define PI_SCHED_DS_WRITE 0x200
#define PI_DEAL4(kind_a, kind_b)                                                     \
  _Pragma("unroll") for (int d_ = 0; d_ < 4; ++d_) {                                 \
    __builtin_amdgcn_sched_group_barrier(PI_SCHED_MFMA, 1, 0);                       \
    if (kind_a) __builtin_amdgcn_sched_group_barrier(kind_a, 1, 0);                  \
    if (kind_b) __builtin_amdgcn_sched_group_barrier(kind_b, 2, 0);                  \
  }
  load_slab(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): this wave's pieces of the slab are in LDS
  __syncthreads();
  load_slab(BK, 1);
  read_frags(0, 0, 0);
  for (int s = 0; s < slabs; ++s) {
    const int buf = s & 1;
    read_frags(1, buf, 1);
    products(0);
    PI_DEAL4(PI_SCHED_DS_READ, 0)
    read_frags(0, buf, 2);
    products(1);
    PI_DEAL4(PI_SCHED_DS_READ, 0)
    read_frags(1, buf, 3);
    products(0);
    PI_DEAL4(PI_SCHED_DS_READ, 0)
    __builtin_amdgcn_s_waitcnt(0x0F70);     // slab s + 1 has landed (asked for a whole slab ago)
    __syncthreads();
    load_slab((s + 2) * BK, buf);           // into the buffer everybody has just left; beyond the range: zeros, unused
    read_frags(0, buf ^ 1, 0);
    products(1);
    PI_DEAL4(PI_SCHED_DS_READ, PI_SCHED_VMEM_READ)
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);       // nothing may still be on its way into LDS when the patches take it over
#undef PI_DEAL4
  __syncthreads();                  // the fragments read last belong to no slab; LDS is free for the patches

  // acc[i][j][v] is C[m0 + wm*64 + i*32 + 8*(v/4) + 4*(lane/32) + v%4][n0 + wn*64 + j*32 + lane%32].
  // Offsets inside the wave's corner are 32-bit (the host checks that 128 * ldc fits).
  {
    const long mw = m0 + wm * 64, nw = n0 + wn * 64;
    const int rows_left = (int)min((long)64, M - mw), cols_left = (int)min((long)64, N - nw);   // may be <= 0
    float* patch = reinterpret_cast<float*>(lds) + wave * PATCH_FLOATS;
    const int esize = EPI == EPI_BF16 || EPI == EPI_SWIGLU ? 2 : 4;
    char* corner = reinterpret_cast<char*>(Cv) + (mw * ldc + (EPI == EPI_SWIGLU ? nw / 2 : nw)) * esize;
    const bool wide = (ldc * esize) % 16 == 0 && reinterpret_cast<uintptr_t>(corner) % 16 == 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) store_rows32<EPI>(patch, acc[i][0], acc[i][1], corner, (int)ldc, i * 32, rows_left, cols_left, lane, wide);
  }
}

// ---------------------------------------------------------------------------------------------
// The same product with block tile 256 x 256 for problems that have enough of them to fill the
// chip and a k that is a multiple of the slab: eight waves in 2 x 4 (two per SIMD), each
// 128 x 64 as 4 x 2 tiles of v_mfma_f32_32x32x16_bf16.  Per 16 k a wave reads 6 fragments from
// LDS for 8 matrix-core instructions, three quarters of the LDS traffic per flop of the
// 128 x 128 kernel, and a block asks L2 for half the bytes per flop.  With one wave per SIMD
// (four waves of 128 x 128, the first form of this kernel) every barrier and every wait left
// the matrix pipe idle.  No branch in the loop (rows beyond the matrix are clamped on load and
// skipped on store), loads through a buffer descriptor (a scalar base that moves with k plus
// fixed 32-bit lane offsets, no vector arithmetic per slab) straight into the other LDS
// buffer, issued at the top of a slab and awaited at its one barrier, and scheduling hints that
// deal the memory instructions out between the matrix-core ones.
// Per output element the sum over k runs in ascending k, as in the small kernel.
#define GM 256
#define GN 256
#define BIG_TILE_ELEMS (GM * BK)

template <int EPI>
__global__ __launch_bounds__(512) void gemm_mfma_big_kernel(void* __restrict__ Cv, long ldc, const bf16_t* __restrict__ A, long lda,
                                                            const bf16_t* __restrict__ W, long ldw, int M, int N, int K,
                                                            int tiles_n, int k_per_split) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  constexpr int ROW = BK;                       // rows of 128 bytes, no padding: the loads write LDS themselves, lane after lane
  constexpr int TILE = GM * ROW;
  uint16_t* As = lds;                           // [2][GM][ROW], 16-byte pieces of a row turned by (row / 2) % 8
  uint16_t* Ws = lds + 2 * TILE;                // [2][GN][ROW]
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int wm = wave / 4, wn = wave % 4;       // a wave's corner: 128 rows x 64 columns
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

  // global -> LDS without registers in between: load instruction p of wave w fills rows
  // (4 w + p) * 8 .. + 7 of a tile, lane l the 16-byte piece l % 8 of row l / 8.  Which piece of
  // the row in memory that is depends on the row: piece c of row r lies at place c ^ ((r / 2) % 8),
  // so that the fragment reads of sixteen neighbouring rows fall on all 64 banks.
  const int a_rows = (int)min((long)GM, M - m0), w_rows = (int)min((long)GN, N - n0);
#if defined(__HIP_DEVICE_COMPILE__)
  const __amdgpu_buffer_rsrc_t a_src = operand_descriptor(A, addressing::tile_descriptor(m0, lda, k_lo, k_hi, a_rows));
  const __amdgpu_buffer_rsrc_t w_src = operand_descriptor(W, addressing::tile_descriptor(n0, ldw, k_lo, k_hi, w_rows));
#endif
  unsigned a_off[4], w_off[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int row = (wave * 4 + p) * 8 + lane / 8;
    const int piece = addressing::tile_piece(lane, row);
    a_off[p] = addressing::big_lane_offset(row, a_rows, lda, piece);
    w_off[p] = addressing::big_lane_offset(row, w_rows, ldw, piece);
  }
  const int slabs = (k_hi - k_lo) / BK;
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto load_slab = [&](int s, int buf) {
    const int kbytes = addressing::big_slab_bytes(s, slabs);     // past the last slab: read it again, unused
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_src, (lds_ptr_t)(As + buf * TILE + (wave * 4 + p) * 8 * ROW), 16, a_off[p], kbytes, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_src, (lds_ptr_t)(Ws + buf * TILE + (wave * 4 + p) * 8 * ROW), 16, w_off[p], kbytes, 0, 0);
    }
#endif
  };

  f32x16_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int frow = lane % 32;
  int place[4];                                  // where this lane's piece of each 16 k lies in its rows
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) place[ks] = ((ks * 2 + lane / 32) ^ ((frow >> 1) & 7)) * 8;
  Frag fa[2][4], fb[2][2];
  auto read_frags = [&](int which, int buf, int ks) {   // ks: which 16 k of the slab
    const uint16_t* a_base = As + buf * TILE + (wm * 128 + frow) * ROW + place[ks];
    const uint16_t* w_base = Ws + buf * TILE + (wn * 64 + frow) * ROW + place[ks];
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[which][i].n = *reinterpret_cast<const u32x4_t*>(a_base + i * 32 * ROW);
#pragma unroll
    for (int j = 0; j < 2; ++j) fb[which][j].n = *reinterpret_cast<const u32x4_t*>(w_base + j * 32 * ROW);
  };
  auto products = [&](int which) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(fa[which][i], fb[which][j], acc[i][j]);
  };

  load_slab(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): this wave's pieces of the slab are in LDS
  __syncthreads();
  read_frags(0, 0, 0);
  // the order wanted inside one scheduling region: one matrix-core instruction, then one of
  // each kind of memory instruction named, `n` times; the rest of the 8 after that
#define PI_DEAL(n, kind_a, kind_b)                                                   \
  _Pragma("unroll") for (int d_ = 0; d_ < n; ++d_) {                                 \
    __builtin_amdgcn_sched_group_barrier(PI_SCHED_MFMA, 1, 0);                       \
    if (kind_a) __builtin_amdgcn_sched_group_barrier(kind_a, 1, 0);                  \
    if (kind_b) __builtin_amdgcn_sched_group_barrier(kind_b, 1, 0);                  \
  }
  load_slab(1, 1);
  for (int s = 0; s < slabs; ++s) {
    const int buf = s & 1;
    read_frags(1, buf, 1);
    products(0);
    PI_DEAL(6, PI_SCHED_DS_READ, 0)
    PI_DEAL(2, 0, 0)
    read_frags(0, buf, 2);
    products(1);
    PI_DEAL(6, PI_SCHED_DS_READ, 0)
    PI_DEAL(2, 0, 0)
    read_frags(1, buf, 3);
    products(0);
    PI_DEAL(6, PI_SCHED_DS_READ, 0)
    PI_DEAL(2, 0, 0)
    __builtin_amdgcn_s_waitcnt(0x0F70);     // slab s + 1 has landed (asked for a whole slab ago)
    __syncthreads();
    load_slab(s + 2, buf);          // into the buffer everybody has just left
    read_frags(0, buf ^ 1, 0);
    products(1);
    PI_DEAL(6, PI_SCHED_DS_READ, PI_SCHED_VMEM_READ)
    PI_DEAL(2, PI_SCHED_VMEM_READ, 0)
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);       // nothing may still be on its way into LDS when the patches take it over
#undef PI_DEAL

  // acc[i][j][v] is C[m0 + wm*128 + i*32 + 8*(v/4) + 4*(lane/32) + v%4][n0 + wn*64 + j*32 + lane%32].
  // Offsets inside the wave's corner are 32-bit (the host checks that 128 * ldc fits).
  __syncthreads();                              // LDS is free for the waves' patches
  {
    const long mw = m0 + wm * 128, nw = n0 + wn * 64;
    const int rows_left = (int)min((long)128, M - mw), cols_left = (int)min((long)64, N - nw);   // may be <= 0
    float* patch = reinterpret_cast<float*>(lds) + wave * PATCH_FLOATS;
    const int esize = EPI == EPI_BF16 || EPI == EPI_SWIGLU ? 2 : 4;
    char* corner = reinterpret_cast<char*>(Cv) + (mw * ldc + (EPI == EPI_SWIGLU ? nw / 2 : nw)) * esize;
    const bool wide = (ldc * esize) % 16 == 0 && reinterpret_cast<uintptr_t>(corner) % 16 == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) store_rows32<EPI>(patch, acc[i][0], acc[i][1], corner, (int)ldc, i * 32, rows_left, cols_left, lane, wide);
  }
}

static const size_t kBigLdsBytes = 4 * BIG_TILE_ELEMS * sizeof(uint16_t);   // 131,072 bytes
// enough 256 x 256 tiles (times k pieces) to occupy most of the chip: three quarters of its compute units
static int big_min_tiles() {
  static int units = 0;
  if (units == 0) {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0)
      count = 256;
    units = count;
  }
  return units * 3 / 4;
}

static const size_t kLdsBytes = 4 * TILE_ELEMS * sizeof(uint16_t);   // 65,536 bytes

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
  const addressing::KSplit cut = addressing::cut_k(K, splits, BK);
  const int kps = cut.k_per_block;
  splits = cut.splits;
  const long big_tiles = (long)ceil_div(M, GM) * ceil_div(N, GN);
  if (big_tiles * splits >= big_min_tiles() && big_tiles < 2147483647L && K % BK == 0) {
    static bool big_configured = false;
    if (!big_configured) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_mfma_big_kernel<EPI>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLdsBytes);
      if (e != hipSuccess) return pi_fail("gemm_mfma: cannot reserve %zu bytes of LDS: %s", kBigLdsBytes, hipGetErrorString(e));
      big_configured = true;
    }
    hipLaunchKernelGGL((gemm_mfma_big_kernel<EPI>), dim3((unsigned)big_tiles, splits), dim3(512), kBigLdsBytes, stream, C, ldc,
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
  return addressing::cut_k(K, splits, BK).splits;
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
  PI_REQUIRE(ldc > 0 && ldc < (1L << 23), "gemm_mfma: the result's row stride (%ld) is too long for 32-bit offsets inside a tile", ldc);
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

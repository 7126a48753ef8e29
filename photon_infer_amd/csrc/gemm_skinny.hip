// bfloat16 matrix product for few rows (decoding and short prompt portions: 1..128 tokens), where the weights are read
// once from HBM and everything else is small:  C[M, N] (+)= X[M, K] . W[N, K]^T.
//
// The weights are the row operand of v_mfma_f32_16x16x32_bf16 and the activations the column
// operand, so a wave produces C^T for 32 weight rows (two row tiles) and up to 32 tokens (the
// second kernel below takes 33..128 tokens).
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
#include <type_traits>

#include "addressing.h"
#include "mfma.h"

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ACCUM = 2, EPI_SWIGLU = 3 };

#define ROWS_PER_BLOCK 32
#define RANGES_ROW_TILES 4      // row tiles per wave where the key ranges are merged on the way in (fewer blocks repeat the merge)
#define KSTEP addressing::KSTEP
#define SHARED_FROM_TOKENS 32   // more tokens than this: the kernel that shares an activation tile per block
#define SHARED_DEPTH 4          // k steps of loads a wave keeps in flight (measured: more is slower)

template <int EPI>
__device__ inline void epilogue_store(void* Cv, long ldc, long m, long n, float v) {
  if (EPI == EPI_BF16) reinterpret_cast<bf16_t*>(Cv)[m * ldc + n] = from_float<bf16_t>(v);
  if (EPI == EPI_F32) reinterpret_cast<float*>(Cv)[m * ldc + n] = v;
  if (EPI == EPI_ACCUM) reinterpret_cast<float*>(Cv)[m * ldc + n] += v;
}

// LDS of a block: while the k loop runs, each wave stages its activations there (the loads from
// memory follow the rows, eight lanes on a row's 128 bytes, which the cache serves at twice the
// rate of the operand's own pattern of sixteen rows per quarter wave); afterwards the same bytes
// hold the waves' partial tiles for the sum.
// Activations that are still the key ranges of a decode step's attention (one token per
// request, request r at row r): float32 [token, head, range, head_dim + 4] holding each range's
// un-normalised output, then its maximum and its sum of weights.  The product kernel merges
// them on the way in, which saves the merging kernel between attention and the o projection.
struct RangeSource {
  const float* ranges;
  int heads, head_dim, count;
};

// Lane group lg merges the key ranges of tokens lg, lg + 4, .. (TOK of them per round) for the
// lane's four features of one head and leaves them, rounded to bfloat16, where the product's
// operand reads expect them.  CNT > 0: up to CNT ranges, all loads of a round asked for before
// the first is used (one trip to memory); CNT == 0: any number, in two passes.  Ranges are added
// in range order with the shared arithmetic (range_weight / range_add / range_finish).
template <int CNT, int TOK>
__device__ inline void merge_ranges_of_tokens(const float* __restrict__ head_base, long token_stride, int count, int rec, int hd,
                                              int f0, int lg, int lr, int M, uint2* __restrict__ xs2) {
  const int piece = lr / 2;                              // the 16-byte piece of the k step the lane's features lie in
#pragma unroll 1
  for (int t0 = lg; t0 < M; t0 += 4 * TOK) {
    f32x4_t sum[TOK];
    float l_tot[TOK];
    if constexpr (CNT > 0) {
      float2 ml[TOK][CNT];
      f32x4_t o[TOK][CNT];
#pragma unroll
      for (int j = 0; j < TOK; ++j) {
        const float* base = head_base + (long)min(t0 + 4 * j, M - 1) * token_stride;
#pragma unroll
        for (int u = 0; u < CNT; ++u) {
          const int r = min(u, count - 1);
          ml[j][u] = *reinterpret_cast<const float2*>(base + r * rec + hd);
          o[j][u] = *reinterpret_cast<const f32x4_t*>(base + r * rec + f0);
        }
      }
#pragma unroll
      for (int j = 0; j < TOK; ++j) {
        float m_tot = -INFINITY;
#pragma unroll
        for (int u = 0; u < CNT; ++u) m_tot = fmaxf(m_tot, ml[j][u].x);
        sum[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        l_tot[j] = 0.f;
#pragma unroll
        for (int u = 0; u < CNT; ++u) {
          const float wgt = u < count ? range_weight(ml[j][u].x, m_tot) : 0.f;
          l_tot[j] = range_add(wgt, ml[j][u].y, l_tot[j]);
#pragma unroll
          for (int e = 0; e < 4; ++e) sum[j][e] = range_add(wgt, o[j][u][e], sum[j][e]);
        }
      }
    } else {
      static_assert(CNT > 0 || TOK == 1, "the two-pass merge takes one token per round");
      const float* base = head_base + (long)t0 * token_stride;
      float m_tot = -INFINITY;
#pragma unroll 8
      for (int r = 0; r < count; ++r) m_tot = fmaxf(m_tot, base[r * rec + hd]);
      sum[0] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      l_tot[0] = 0.f;
#pragma unroll 8
      for (int r = 0; r < count; ++r) {
        const float2 ml = *reinterpret_cast<const float2*>(base + r * rec + hd);
        const f32x4_t o = *reinterpret_cast<const f32x4_t*>(base + r * rec + f0);
        const float wgt = range_weight(ml.x, m_tot);
        l_tot[0] = range_add(wgt, ml.y, l_tot[0]);
#pragma unroll
        for (int e = 0; e < 4; ++e) sum[0][e] = range_add(wgt, o[e], sum[0][e]);
      }
    }
#pragma unroll
    for (int j = 0; j < TOK; ++j) {
      const int token = t0 + 4 * j;
      if (token >= M) break;
      uint2 packed;
      packed.x = pack_bf16x2(range_finish(sum[j][0], l_tot[j]), range_finish(sum[j][1], l_tot[j]));
      packed.y = pack_bf16x2(range_finish(sum[j][2], l_tot[j]), range_finish(sum[j][3], l_tot[j]));
      xs2[(piece * 16 + ((token + 2 * piece) & 15)) * 2 + (lr & 1)] = packed;
    }
  }
}

template <int MB, int RT>
union SkinnyLds {
  float red[4][RT * 16][MB * 16 + 1];
  u32x4_t xs[4][MB * 8 * 16];          // per wave: [token tile][16-byte piece of the k step][token], tokens turned by the piece
};

template <int MB, int EPI, bool RANGES = false, int RT = 2>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(void* __restrict__ Cv, long ldc, const bf16_t* __restrict__ X, long ldx,
                                                          const bf16_t* __restrict__ W, long ldw, int M, int N, int K,
                                                          int k_per_block, float* __restrict__ part, RangeSource rs, int tiled) {
  constexpr int ROWS = RT * 16;          // weight rows of a block: RT row tiles per wave
  static_assert(EPI != EPI_SWIGLU || RT == 2, "the SwiGLU epilogue pairs a wave's two row tiles");
  __shared__ SkinnyLds<MB, RT> lds;
  float (*red)[ROWS][MB * 16 + 1] = lds.red;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int lr = lane % 16, lg = lane / 16;
  const long n0 = (long)blockIdx.x * ROWS;
  const int splits = gridDim.y;

  // this wave's k-range: a quarter (rounded up to whole steps) of the block's range
  const addressing::WaveRange range = addressing::skinny_wave_range(K, k_per_block, blockIdx.y, wave);
  const int k0 = range.k0, k1 = range.k1;

  // rows beyond N read the last valid row; their results are never stored.  `tiled`: W is the
  // copy in the order this kernel reads (see pi_gemm_skinny): 16 rows x 64 k are 2 KB in a row,
  // one load instruction's 1 KB after the other, so a k step of 64 moves by 1,024 elements and
  // the step's second fragment lies 512 elements behind the first.
  const bf16_t* wrow[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) wrow[t] = W + addressing::skinny_w_base(tiled, n0, t, lr, lg, N, K, ldw);

  // Activations of a k step: load instruction i brings tokens 8i .. 8i+7, lane j the 16-byte
  // piece j % 8 of token 8i + j / 8.  Tokens beyond M are not loaded: what LDS holds for them
  // only reaches columns of the result that are never stored.
  const int x_loads = __builtin_amdgcn_readfirstlane((M + 7) / 8);
  const int xt = lane / 8, xp = lane % 8;
  const bf16_t* xsrc[MB * 2];
  int xdst[MB * 2];
#pragma unroll
  for (int i = 0; i < MB * 2; ++i) {
    const int token = i * 8 + xt;
    xsrc[i] = X + addressing::skinny_x_base(token, M, ldx, xp);
    xdst[i] = ((token / 16) * 8 + xp) * 16 + ((token + 2 * xp) & 15);
  }
  u32x4_t* xs = lds.xs[wave];
  int xfrag[MB][2];                     // where this lane's operand pieces lie: piece lg*2+h of token lr
#pragma unroll
  for (int c = 0; c < MB; ++c)
#pragma unroll
    for (int h = 0; h < 2; ++h) xfrag[c][h] = (c * 8 + lg * 2 + h) * 16 + ((lr + 2 * (lg * 2 + h)) & 15);

  f32x4_t acc[RT][MB];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int c = 0; c < MB; ++c) acc[t][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // one k step; in a last, partial one the 8-element pieces beyond k1 count as zero
  auto step = [&](const int kk, auto whole_step) {
    constexpr bool whole = decltype(whole_step)::value;
    Frag w[RT][2];
    u32x4_t xg[MB * 2];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // a piece beyond k1 is fetched from a stand-in address inside the row and counts as zero
        w[t][h] = load_frag(wrow[t] + addressing::skinny_w_step(tiled, whole, kk, h, lg, k0, k1));
        if (!addressing::skinny_w_used(whole, kk, h, lg, k1)) w[t][h] = zero_frag();
      }
    if constexpr (RANGES) {
      // The 64 features of this step belong to one head (head_dim is a multiple of 64).  Lane
      // group lg merges tokens lg, lg + 4, ..; a lane owns four features.  Every load is asked
      // for before the first is needed; the ranges are added in range order.
      static_assert(MB == 1, "merging on the way in serves up to 16 tokens");
      const int head = kk / rs.head_dim, f0 = kk - head * rs.head_dim + lr * 4;
      const int rec = rs.head_dim + 4;
      const float* head_base = rs.ranges + (long)head * rs.count * rec;
      const long token_stride = (long)rs.heads * rs.count * rec;
      uint2* xs2 = reinterpret_cast<uint2*>(xs);
      // tokens per lane group x ranges per token held in registers at once: about 16 either way
      if (rs.count <= 4) merge_ranges_of_tokens<4, 4>(head_base, token_stride, rs.count, rec, rs.head_dim, f0, lg, lr, M, xs2);
      else if (rs.count <= 8) merge_ranges_of_tokens<8, 2>(head_base, token_stride, rs.count, rec, rs.head_dim, f0, lg, lr, M, xs2);
      else if (rs.count <= 16) merge_ranges_of_tokens<16, 1>(head_base, token_stride, rs.count, rec, rs.head_dim, f0, lg, lr, M, xs2);
      else merge_ranges_of_tokens<0, 1>(head_base, token_stride, rs.count, rec, rs.head_dim, f0, lg, lr, M, xs2);
    } else {
      const bool x_ok = whole || kk + xp * 8 < k1;
#pragma unroll
      for (int i = 0; i < MB * 2; ++i)
        if (i == 0 || i < x_loads) {
          xg[i] = *reinterpret_cast<const u32x4_t*>(xsrc[i] + addressing::skinny_x_step(whole, kk, xp, k0, k1));
          if (!x_ok) xg[i] = u32x4_t{0u, 0u, 0u, 0u};
        }
#pragma unroll
      for (int i = 0; i < MB * 2; ++i)
        if (i == 0 || i < x_loads) xs[xdst[i]] = xg[i];
    }
    // the wave reads what its own lanes wrote: LDS serves one wave's accesses in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    Frag x[MB][2];
#pragma unroll
    for (int c = 0; c < MB; ++c)
#pragma unroll
      for (int h = 0; h < 2; ++h) x[c][h].n = xs[xfrag[c][h]];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int c = 0; c < MB; ++c) {
        acc[t][c] = mfma16(w[t][0], x[c][0], acc[t][c]);
        acc[t][c] = mfma16(w[t][1], x[c][1], acc[t][c]);
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };
  int kk = k0;
  for (; kk + KSTEP <= k1; kk += KSTEP) step(kk, std::true_type{});
  if (kk < k1) step(kk, std::false_type{});
  __syncthreads();                      // the partial tiles take the place of the staged activations

  // acc[t][c][r] is C^T[n0 + t*16 + lg*4 + r][c*16 + lr]; add the four waves through LDS
#pragma unroll
  for (int t = 0; t < RT; ++t)
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
      for (int idx = tid; idx < ROWS * cols; idx += 256) {
        const int nl = idx % ROWS, m = idx / ROWS;
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
  for (int idx = tid; idx < ROWS * cols; idx += 256) {
    const int nl = idx % ROWS, m = idx / ROWS;
    if (m >= M || n0 + nl >= N) continue;
    mine[(long)m * N + n0 + nl] = red[0][nl][m] + red[1][nl][m] + red[2][nl][m] + red[3][nl][m];
  }
}

// The same product for 33..128 tokens, where the activations are as many bytes as a block's
// weights: the four waves of a block take 16 weight rows each over the block's whole k-range
// and share one activation tile per k step through LDS (loaded once per block, not once per
// wave).  A block is alone on its compute unit, so every wave keeps DEPTH k steps of loads
// (weights and its share of the activation tile) in flight in registers; loads return in
// order, which is why both travel at the same distance.
#define SHARED_ROWS_PER_BLOCK 64

template <int MB, int EPI, int DEPTH>
__global__ __launch_bounds__(256) void gemm_skinny_shared_kernel(void* __restrict__ Cv, long ldc, const bf16_t* __restrict__ X, long ldx,
                                                                 const bf16_t* __restrict__ W, long ldw, int M, int N, int K,
                                                                 int k_per_block, float* __restrict__ part, int tiled) {
  constexpr int ROWS = SHARED_ROWS_PER_BLOCK;
  constexpr int XL = (MB + 1) / 2;      // 16-byte pieces of an activation tile per lane
  __shared__ union {
    u32x4_t xs[2][MB * 128];            // [token tile][piece of the k step][token], tokens turned by the piece
    float tile[ROWS][MB * 16 + 1];
  } lds;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int lr = lane % 16, lg = lane / 16;
  const long n0 = (long)blockIdx.x * ROWS;
  const int splits = gridDim.y;
  const int kb0 = blockIdx.y * k_per_block;
  const int kb1 = min(K, kb0 + k_per_block);
  const int steps = addressing::shared_steps(kb0, kb1);
  auto k_of = [&](const int s) { return addressing::shared_k_of(kb0, steps, s); };   // steps beyond the last are fetched, never used

  // rows beyond N and tokens beyond M read the last valid one; their results are never stored
  const bf16_t* wrow = W + addressing::shared_w_base(tiled, n0, wave, lr, lg, N, K, ldw);     // see gemm_skinny_kernel
  const int xp = tid % 8;
  const bf16_t* xsrc[XL];
  int xdst[XL];
  bool xmine[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int token = i * 32 + tid / 8;
    xsrc[i] = X + addressing::shared_x_base(token, M, ldx);
    xdst[i] = ((token / 16) * 8 + xp) * 16 + ((token + 2 * xp) & 15);
    xmine[i] = token < MB * 16;
  }
  int xfrag[MB][2];
#pragma unroll
  for (int c = 0; c < MB; ++c)
#pragma unroll
    for (int h = 0; h < 2; ++h) xfrag[c][h] = (c * 8 + lg * 2 + h) * 16 + ((lr + 2 * (lg * 2 + h)) & 15);

  f32x4_t acc[MB];
#pragma unroll
  for (int c = 0; c < MB; ++c) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  Frag wq[DEPTH][2];
  u32x4_t xq[DEPTH][XL];
  // every step issues the same loads, also beyond the range (clamped, never used): the count
  // of loads in flight is then a constant the compiler can wait on exactly
  auto fetch = [&](const int s, const int j) {
    const int kk = k_of(s);
#pragma unroll
    for (int i = 0; i < XL; ++i) xq[j][i] = *reinterpret_cast<const u32x4_t*>(xsrc[i] + addressing::shared_x_step(kk, xp, kb1));
#pragma unroll
    for (int h = 0; h < 2; ++h) wq[j][h] = load_frag(wrow + addressing::shared_w_step(tiled, kk, h, lg, kb1));
  };
#pragma unroll
  for (int j = 0; j < DEPTH; ++j) fetch(j, j);

  // the tile of step s + 1 goes to LDS (the other of two buffers) before step s computes, so
  // that the one barrier per step finds every wave's writes long done
  auto stage = [&](const int s, const int j) {
    const bool x_ok = k_of(s) + xp * 8 < kb1;          // 8-element pieces beyond the range count as zero
    u32x4_t* xs = lds.xs[s & 1];
#pragma unroll
    for (int i = 0; i < XL; ++i)
      if (xmine[i]) xs[xdst[i]] = x_ok ? xq[j][i] : u32x4_t{0u, 0u, 0u, 0u};
  };
  auto step = [&](const int s, const int j, auto more_to_fetch) {
    const int kk = k_of(s);
    stage(s + 1, (j + 1) % DEPTH);
    const u32x4_t* xs = lds.xs[s & 1];
    Frag x[MB][2], w[2];
#pragma unroll
    for (int c = 0; c < MB; ++c)
#pragma unroll
      for (int h = 0; h < 2; ++h) x[c][h].n = xs[xfrag[c][h]];
#pragma unroll
    for (int h = 0; h < 2; ++h) w[h].n = kk + lg * 16 + h * 8 < kb1 ? wq[j][h].n : u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int c = 0; c < MB; ++c) acc[c] = mfma16(w[h], x[c][h], acc[c]);
    if (decltype(more_to_fetch)::value) fetch(s + DEPTH, j);
    __syncthreads();
  };
  stage(0, 0);
  __syncthreads();
  // whole rounds of DEPTH steps have no branch, so that the waits stay exact; the last steps
  // fetch nothing more
  int s0 = 0;
  for (; s0 + DEPTH <= steps; s0 += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) step(s0 + j, j, std::true_type{});
  }
#pragma unroll
  for (int j = 0; j < DEPTH; ++j)
    if (s0 + j < steps) step(s0 + j, j, std::false_type{});
  // (the last step ended with a barrier: the result tile may take the place of the activation tiles)

  // acc[c][r] is C^T[n0 + wave*16 + lg*4 + r][c*16 + lr]
#pragma unroll
  for (int c = 0; c < MB; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) lds.tile[wave * 16 + lg * 4 + r][c * 16 + lr] = acc[c][r];
  __syncthreads();

  const int cols = MB * 16;
  if (splits == 1 && EPI == EPI_SWIGLU) {
    // rows [gate 16 | up 16 | gate 16 | up 16]: 32 features per block
    for (int idx = tid; idx < 32 * cols; idx += 256) {
      const int j = idx % 16, pair = (idx / 16) % 2, m = idx / 32;
      if (m >= M || n0 + pair * 32 + 16 + j >= N) continue;
      const float g = lds.tile[pair * 32 + j][m], u = lds.tile[pair * 32 + 16 + j][m];
      reinterpret_cast<bf16_t*>(Cv)[(long)m * ldc + n0 / 2 + pair * 16 + j] = from_float<bf16_t>(g / (1.0f + expf(-g)) * u);
    }
    return;
  }
  float* mine = part + (long)blockIdx.y * M * N;
  for (int idx = tid; idx < ROWS * cols; idx += 256) {
    const int nl = idx % ROWS, m = idx / ROWS;
    if (m >= M || n0 + nl >= N) continue;
    if (splits == 1) epilogue_store<EPI>(Cv, ldc, m, n0 + nl, lds.tile[nl][m]);
    else mine[(long)m * N + n0 + nl] = lds.tile[nl][m];   // the consumer adds the splits in split order
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
                     long ldw, int M, int N, int K, int kpb, float* part, int tiled) {
#define GO(E) hipLaunchKernelGGL((gemm_skinny_kernel<MB, E>), grid, dim3(256), 0, stream, C, ldc, X, ldx, W, ldw, M, N, K, kpb, part, RangeSource{}, tiled)
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

template <int MB>
static int launch_shared(int epi, dim3 grid, hipStream_t stream, void* C, long ldc, const bf16_t* X, long ldx, const bf16_t* W,
                         long ldw, int M, int N, int K, int kpb, float* part, int tiled) {
#define GO(E) hipLaunchKernelGGL((gemm_skinny_shared_kernel<MB, E, SHARED_DEPTH>), grid, dim3(256), 0, stream, C, ldc, X, ldx, W, ldw, M, N, K, kpb, part, tiled)
  switch (epi) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    case EPI_ACCUM: GO(EPI_ACCUM); break;
    case EPI_SWIGLU: GO(EPI_SWIGLU); break;
    default: return pi_fail("gemm_skinny: unknown epilogue %d", epi);
  }
#undef GO
  return pi_check_launch("gemm_skinny (shared activations)");
}

// Rows of the weight matrix per block for M tokens (the caller sizes its k-split by it).
extern "C" int pi_gemm_skinny_rows_per_block(int M) { return M > SHARED_FROM_TOKENS ? SHARED_ROWS_PER_BLOCK : ROWS_PER_BLOCK; }

// splits > 1: the partial products go to `part` (float32 [splits, M, N]) and C is not touched;
// *splits_out tells how many splits were made (no empty ones).
// `tiled` != 0: W is not [N, K] row after row but a copy in the order the kernels' loads want it,
// [N / 16][K / 64][2][4][16][8]: for 16 rows and 64 k, first the k of every lane's first
// fragment, then of its second; in each, lane group g's k = 16 g + 8 h .. + 7 of rows 0..15.
// A wave's load instruction then reads 1 KB in a row instead of 64 bytes from each of 16 rows.
// N must be a multiple of 16 and K of 64.
extern "C" int pi_gemm_skinny(void* C, int epilogue, long ldc, const void* X, long ldx, const void* W, long ldw, int M,
                              int N, int K, int splits, void* part, long part_elems, int* splits_out, int tiled,
                              hipStream_t stream) {
  PI_REQUIRE(!tiled || (N % 16 == 0 && K % 64 == 0), "gemm_skinny: a tiled weight matrix needs N (%d) a multiple of 16 and K (%d) of 64", N, K);
  PI_REQUIRE(M > 0 && M <= 128 && N > 0 && K > 0, "gemm_skinny: takes 1..128 rows, got M=%d N=%d K=%d", M, N, K);
  PI_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "gemm_skinny: K (%d) and row strides (%ld, %ld) must be multiples of 8", K, ldx, ldw);
  PI_REQUIRE(((uintptr_t)X % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_skinny: operands must be 16-byte aligned");
  PI_REQUIRE(splits >= 1 && splits <= 65535, "gemm_skinny: bad split count %d", splits);
  PI_REQUIRE(epilogue != EPI_SWIGLU || (splits == 1 && N % 32 == 0), "gemm_skinny: the SwiGLU epilogue needs one split and N (%d) a multiple of 32", N);
  const int groups = ceil_div(N, pi_gemm_skinny_rows_per_block(M));
  const addressing::KSplit cut = addressing::cut_k(K, splits, KSTEP);
  const int kpb = cut.k_per_block;
  splits = cut.splits;                            // no empty splits
  if (splits > 1)
    PI_REQUIRE(part && part_elems >= (long)splits * M * N, "gemm_skinny: workspace too small (%ld floats for %ld)", part_elems, (long)splits * M * N);
  if (splits_out) *splits_out = splits;
  const dim3 grid(groups, splits);
  const int mb = (M + 15) / 16;
  const bf16_t *x = (const bf16_t*)X, *w = (const bf16_t*)W;
  if (M > SHARED_FROM_TOKENS) {
#define SHARED(B) case B: return launch_shared<B>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part, tiled)
    switch (mb) {
      SHARED(3); SHARED(4); SHARED(5); SHARED(6); SHARED(7);
      default: return launch_shared<8>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part, tiled);
    }
#undef SHARED
  }
  switch (mb) {
    case 1: return launch_mb<1>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part, tiled);
    case 2: return launch_mb<2>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part, tiled);
    case 3: return launch_mb<3>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part, tiled);
    default: return launch_mb<4>(epilogue, grid, stream, C, ldc, x, ldx, w, ldw, M, N, K, kpb, (float*)part, tiled);
  }
}

// The same product for a decode step of up to 16 tokens whose activations are attention's key
// ranges not yet merged (`ranges`: float32 [M, heads, count, head_dim + 4], see RangeSource): K
// is heads * head_dim, and head_dim a multiple of the kernel's k step so that a step's features
// belong to one head.  Epilogues: store bf16, store f32, add into f32.
extern "C" int pi_gemm_skinny_ranges(void* C, int epilogue, long ldc, const void* ranges, int heads, int head_dim, int count,
                                     const void* W, long ldw, int M, int N, int splits, void* part, long part_elems,
                                     int* splits_out, int tiled, hipStream_t stream) {
  PI_REQUIRE(M > 0 && M <= 16 && N > 0 && heads > 0 && count >= 1 && count <= 64, "gemm_skinny_ranges: takes 1..16 tokens and 1..64 ranges, got M=%d N=%d heads=%d ranges=%d", M, N, heads, count);
  PI_REQUIRE(head_dim > 0 && head_dim % KSTEP == 0, "gemm_skinny_ranges: head_dim %d is no multiple of %d", head_dim, KSTEP);
  PI_REQUIRE(epilogue == EPI_BF16 || epilogue == EPI_F32 || epilogue == EPI_ACCUM, "gemm_skinny_ranges: unknown epilogue %d", epilogue);
  PI_REQUIRE(ldw % 8 == 0 && ((uintptr_t)W % 16 == 0) && ((uintptr_t)ranges % 16 == 0), "gemm_skinny_ranges: operands must be 16-byte aligned");
  PI_REQUIRE(splits >= 1 && splits <= 65535, "gemm_skinny_ranges: bad split count %d", splits);
  const long K = (long)heads * head_dim;
  PI_REQUIRE(K < (1L << 30), "gemm_skinny_ranges: k too long");
  PI_REQUIRE(!tiled || N % 16 == 0, "gemm_skinny_ranges: a tiled weight matrix needs N (%d) a multiple of 16", N);
  const addressing::KSplit cut = addressing::cut_k((int)K, splits, 4 * KSTEP);     // a block's four waves take whole steps
  const int kpb = cut.k_per_block;
  splits = cut.splits;
  if (splits > 1)
    PI_REQUIRE(part && part_elems >= (long)splits * M * N, "gemm_skinny_ranges: workspace too small (%ld floats for %ld)", part_elems, (long)splits * M * N);
  if (splits_out) *splits_out = splits;
  const dim3 grid(ceil_div(N, RANGES_ROW_TILES * 16), splits);
  const RangeSource rs{(const float*)ranges, heads, head_dim, count};
#define GO(E) hipLaunchKernelGGL((gemm_skinny_kernel<1, E, true, RANGES_ROW_TILES>), grid, dim3(256), 0, stream, C, ldc, (const bf16_t*)nullptr, 0L, \
                                 (const bf16_t*)W, ldw, M, N, (int)K, kpb, (float*)part, rs, tiled)
  switch (epilogue) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    default: GO(EPI_ACCUM); break;
  }
#undef GO
  return pi_check_launch("gemm_skinny (key ranges merged on the way in)");
}

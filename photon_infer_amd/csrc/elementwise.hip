// Embedding gather, RMS norm (optionally on gathered rows), SwiGLU, and the fused
// position-rotation + paged key/value write.  All sizes are run-time values.
#include "common.h"

PI_DEFINE_MODULE(core)

// ------------------------------------------------------------------ embedding
// out[t, :] = float(table[ids[t], :]).  An id outside [0, V) fills the row with NaN:
// loud in every later result, and no access outside the table.
template <typename TW>
__global__ void embedding_kernel(float* __restrict__ out, const TW* __restrict__ table,
                                 const int* __restrict__ ids, int D, int V) {
  const long t = blockIdx.x;
  const int id = ids[t];
  float* o = out + t * D;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = __builtin_nanf("");
    return;
  }
  const TW* row = table + (long)id * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = to_float(row[i]);
}

extern "C" int pi_embedding(float* out, const void* table, int table_dtype, const int* ids, int T, int D,
                            int V, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && D > 0 && V > 0, "embedding: bad sizes T=%d D=%d V=%d", T, D, V);
  if (T == 0) return 0;
  const int threads = D >= 256 ? 256 : 64;
  if (table_dtype == PI_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, dim3(T), dim3(threads), 0, stream, out, (const float*)table, ids, D, V);
  else if (table_dtype == PI_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, dim3(T), dim3(threads), 0, stream, out, (const bf16_t*)table, ids, D, V);
  else
    return pi_fail("embedding: unsupported table dtype %d", table_dtype);
  return pi_check_launch("embedding");
}

// ------------------------------------------------------------------ RMS norm
// y[m, :] = w * (x[r, :] * (1 / sqrt(mean(x[r, :]^2) + eps))), r = rows ? rows[m] : m.
// Sum of squares, root and scaling in float32; one rounding on store.
// With `part` (float32 [splits, x_rows, D]: the pieces of a matrix product that is still to be
// added to x), row r first becomes x[r, :] + sum_s part[s, r, :] (in split order), is written
// back to x, and is then normalised: the residual add, the split reduction and the norm in one pass.
template <typename TO, typename TW>
__global__ void rmsnorm_kernel(TO* __restrict__ out, float* __restrict__ x, const int* __restrict__ rows,
                               const TW* __restrict__ w, float eps, int D, const float* __restrict__ part, int splits,
                               long part_stride) {
  __shared__ float scratch[16];
  const long m = blockIdx.x;
  const long r = rows ? rows[m] : m;
  float* xr = x + r * D;
  float ss = 0.f;
  if (part) {
    const float* pr = part + r * D;
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
      float v = xr[i];
      // eight pieces at a time: the loads go out together, the adds keep the split order
      for (int s0 = 0; s0 < splits; s0 += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = (s0 + u < splits) ? pr[(s0 + u) * part_stride + i] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) v += t[u];
      }
      xr[i] = v;               // the same thread reads it back below
      ss += v * v;
    }
  } else {
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
      const float v = xr[i];
      ss += v * v;
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  TO* o = out + m * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) o[i] = from_float<TO>(to_float(w[i]) * (xr[i] * inv));
}

// The same for rows of a multiple of 4 floats, 16-byte aligned: a thread keeps its VPT groups of
// four values in registers between the two passes, and every access is 16 bytes wide (8 for
// bfloat16 output and weights).
template <typename T> struct Vec4Of;
template <> struct Vec4Of<float> {
  typedef float4 type;
  __device__ static inline void load(const float* p, float (&v)[4]) { const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
  __device__ static inline void store(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4Of<bf16_t> {
  __device__ static inline void load(const bf16_t* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
  }
  __device__ static inline void store(bf16_t* p, const float (&v)[4]) {
    *reinterpret_cast<uint2*>(p) = make_uint2(f32x2_to_bf16x2_bits(v[0], v[1]), f32x2_to_bf16x2_bits(v[2], v[3]));
  }
};

template <typename TO, typename TW, int VPT>
__global__ void rmsnorm_wide_kernel(TO* __restrict__ out, float* __restrict__ x, const int* __restrict__ rows,
                                    const TW* __restrict__ w, float eps, int D, const float* __restrict__ part, int splits,
                                    long part_stride) {
  __shared__ float scratch[16];
  const long m = blockIdx.x;
  const long r = rows ? rows[m] : m;
  float* xr = x + r * D;
  const int groups = D / 4;
  float v[VPT][4], ww[VPT][4];      // the weights come along with the row: one wait for memory, not two
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int gi = threadIdx.x + k * blockDim.x;
    if (gi < groups) {
      Vec4Of<float>::load(xr + gi * 4, v[k]);
      Vec4Of<TW>::load(w + gi * 4, ww[k]);
    } else {
      v[k][0] = v[k][1] = v[k][2] = v[k][3] = 0.f;
      ww[k][0] = ww[k][1] = ww[k][2] = ww[k][3] = 0.f;
    }
  }
  if (part) {
    const float* pr = part + r * D;
    // several pieces' loads go out together (eight where a thread holds few values: a decode
    // step's eight pieces are then one wait for memory, not two); the adds keep the split order
    constexpr int U = VPT <= 2 ? 8 : 4;
    for (int s0 = 0; s0 < splits; s0 += U) {
      float t[U][VPT][4];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
          const int gi = threadIdx.x + k * blockDim.x;
          if (s0 + u < splits && gi < groups) Vec4Of<float>::load(pr + (s0 + u) * part_stride + gi * 4, t[u][k]);
          else t[u][k][0] = t[u][k][1] = t[u][k][2] = t[u][k][3] = 0.f;
        }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int k = 0; k < VPT; ++k)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[k][e] += t[u][k][e];
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int gi = threadIdx.x + k * blockDim.x;
      if (gi < groups) Vec4Of<float>::store(xr + gi * 4, v[k]);
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k)
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += v[k][e] * v[k][e];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  TO* o = out + m * D;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int gi = threadIdx.x + k * blockDim.x;
    if (gi >= groups) continue;
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = ww[k][e] * (v[k][e] * inv);
    Vec4Of<TO>::store(o + gi * 4, y);
  }
}

// part == nullptr: plain norm.  Otherwise part is float32 [splits, x_rows, D].
extern "C" int pi_rmsnorm(void* out, int out_dtype, float* x, const int* rows, const void* w, int w_dtype, float eps, int M,
                          int D, const float* part, int splits, long x_rows, hipStream_t stream) {
  PI_REQUIRE(M >= 0 && D > 0, "rmsnorm: bad sizes M=%d D=%d", M, D);
  PI_REQUIRE(part == nullptr || (splits >= 1 && x_rows > 0), "rmsnorm: bad split description (%d splits, %ld rows)", splits, x_rows);
  if (M == 0) return 0;
  // few rows: many threads per row, so that a row's loads are all in flight at once
  int threads = (D >= 2048 && M <= 256) ? 1024 : (D >= 1024 ? 256 : (D >= 256 ? 128 : 64));
  const long stride = x_rows * (long)D;
  // rows of whole 16-byte groups, at most 8 groups per thread: the kernel with wide accesses
  // (no more threads than groups)
  bool wide = D % 4 == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)out % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
              (part == nullptr || (uintptr_t)part % 16 == 0);
  int per_thread = 0;
  if (wide) {
    const int groups = D / 4, most = threads;
    threads = groups >= most ? most : ((groups + 63) / 64) * 64;
    per_thread = (groups + threads - 1) / threads;
    if (per_thread > 8) { wide = false; threads = most; }
  }
#define WIDE(TO, TW, V) \
  hipLaunchKernelGGL((rmsnorm_wide_kernel<TO, TW, V>), dim3(M), dim3(threads), 0, stream, (TO*)out, x, rows, (const TW*)w, eps, D, part, splits, stride)
#define LAUNCH(TO, TW) \
  do { \
    if (wide && per_thread <= 1) WIDE(TO, TW, 1); \
    else if (wide && per_thread <= 2) WIDE(TO, TW, 2); \
    else if (wide && per_thread <= 4) WIDE(TO, TW, 4); \
    else if (wide) WIDE(TO, TW, 8); \
    else hipLaunchKernelGGL((rmsnorm_kernel<TO, TW>), dim3(M), dim3(threads), 0, stream, (TO*)out, x, rows, (const TW*)w, eps, D, part, splits, stride); \
  } while (0)
  if (out_dtype == PI_F32 && w_dtype == PI_F32) LAUNCH(float, float);
  else if (out_dtype == PI_F32 && w_dtype == PI_BF16) LAUNCH(float, bf16_t);
  else if (out_dtype == PI_BF16 && w_dtype == PI_F32) LAUNCH(bf16_t, float);
  else if (out_dtype == PI_BF16 && w_dtype == PI_BF16) LAUNCH(bf16_t, bf16_t);
  else return pi_fail("rmsnorm: unsupported dtypes out=%d weight=%d", out_dtype, w_dtype);
#undef LAUNCH
#undef WIDE
  return pi_check_launch("rmsnorm");
}

// ------------------------------------------------------------------ SwiGLU
// out[t, i] = g / (1 + exp(-g)) * u; float32 math.  Layout of gu [T, 2I]:
//   block == 0: gate in columns [0, I), up in [I, 2I);
//   block == b: gate and up interleaved in blocks of b columns (gate block, up block, ...).
template <typename T>
__global__ void swiglu_kernel(T* __restrict__ out, const T* __restrict__ gu, long total, int I, int block) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long t = idx / I;
  const int i = (int)(idx - t * I);
  const long gi = block ? (long)(i / block) * 2 * block + i % block : i;
  const long ui = block ? gi + block : (long)I + i;
  const float g = to_float(gu[t * 2 * I + gi]);
  const float u = to_float(gu[t * 2 * I + ui]);
  out[idx] = from_float<T>(g / (1.0f + expf(-g)) * u);
}

extern "C" int pi_swiglu(void* out, const void* gu, int dtype, int T, int I, int block, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  PI_REQUIRE(block >= 0 && (block == 0 || I % block == 0), "swiglu: interleave block %d does not divide %d", block, I);
  if (T == 0) return 0;
  const long total = (long)T * I;
  const int threads = 256;
  const long blocks = (total + threads - 1) / threads;
  PI_REQUIRE(blocks < 2147483647L, "swiglu: too many elements (%ld)", total);
  if (dtype == PI_F32)
    hipLaunchKernelGGL(swiglu_kernel<float>, dim3((unsigned)blocks), dim3(threads), 0, stream, (float*)out, (const float*)gu, total, I, block);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3((unsigned)blocks), dim3(threads), 0, stream, (bf16_t*)out, (const bf16_t*)gu, total, I, block);
  else
    return pi_fail("swiglu: unsupported dtype %d", dtype);
  return pi_check_launch("swiglu");
}

// ------------------------------------------------------------------ rotation + cache write
// One wave per (token, head).  Heads 0..nh-1 are queries (rotated in place); then, when
// the layer writes its cache, nkv key heads (rotated, stored to the page of the token's
// position) and nkv value heads (stored as they are).
// Cache layout: keys [page, kv_head, slot_in_page, head_dim]; values transposed,
// [page, kv_head, head_dim, slot_in_page], so that the keys of one page are contiguous for a
// fixed feature - the order in which the matrix-core attention kernels contract them.
// Pair j is (x[j], x[j + R/2]) or, interleaved, (x[2j], x[2j+1]);
// (a, b) <- (a cos - b sin, a sin + b cos) with cos / sin of the token's angle from the
// step's table (rope_table_kernel below).  Dims >= R are copied.
// table[t, j] = cos(angle), table[t, R/2 + j] = sin(angle), angle = float(pos[t]) * inv_freq[j]:
// float32 product, full-range sine and cosine.  Made once per step and read by every layer.
__global__ void rope_table_kernel(float* __restrict__ table, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int T, int half) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)T * half) return;
  const long t = idx / half;
  const int j = (int)(idx - t * half);
  const float angle = (float)positions[t] * inv_freq[j];
  float s, c;
  sincosf(angle, &s, &c);
  table[t * 2 * half + j] = c;
  table[t * 2 * half + half + j] = s;
}

extern "C" int pi_rope_table(float* table, const int* positions, const float* inv_freq, int T, int half, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && half > 0 && table && positions && inv_freq, "rope_table: bad arguments T=%d half=%d", T, half);
  if (T == 0) return 0;
  const long total = (long)T * half;
  hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, table, positions, inv_freq, T, half);
  return pi_check_launch("rope_table");
}

// The source of q, k, v is either the projection's output in the compute dtype (q is rotated in
// place) or, when `part` is given, the pieces of that projection still to be summed: float32
// [splits, T, ncols] with q at column q_col, k at k_col, v at v_col; the rotated q then goes to
// the q buffer, and nothing ever holds the unrotated values in reduced precision.
template <typename T>
__device__ inline float rope_source(const T* __restrict__ src, const float* __restrict__ part, int splits, long part_stride, int i) {
  if (!part) return to_float(src[i]);
  return split_sum(part, splits, part_stride, i);
}

// One wave per (token, head), four heads to a block; a lane owns whole pairs, so nothing is
// shared between lanes and every load of a lane is independent of the others.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride, const T* __restrict__ v, long v_stride,
    const int* __restrict__ positions, const int* __restrict__ req_of_token, const float* __restrict__ table,
    int rotary_dim, int interleaved, int nh, int nkv_write, int nkv, int hd, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int* __restrict__ block_table, int table_width, int page_size, long num_pages,
    const float* __restrict__ part, int splits, long part_stride, int ncols, int q_col, int k_col, int v_col) {
  const long t = blockIdx.x;
  const int h = blockIdx.y * 4 + threadIdx.x / PI_WAVE;
  const int lane = threadIdx.x % PI_WAVE;
  if (h >= nh + 2 * nkv_write) return;
  T* dst;
  long dst_stride = 1;        // element stride of the destination (values are stored transposed)
  const T* src = nullptr;
  int col = 0;
  bool rotate = rotary_dim > 0;
  if (h < nh) {
    dst = q + t * q_stride + (long)h * hd;
    src = dst;
    col = q_col + h * hd;
  } else {
    const int hh = h - nh;
    const bool is_v = hh >= nkv_write;
    const int g = is_v ? hh - nkv_write : hh;
    const int pos = positions[t];
    const int r = req_of_token[t];
    const int blk = pos / page_size;
    if (blk >= table_width) return;
    const long page = block_table[(long)r * table_width + blk];
    if (page < 0 || page >= num_pages) return;  // the host checks tables; never write outside the pool
    if (is_v) {
      src = v ? v + t * v_stride + (long)g * hd : nullptr;
      col = v_col + g * hd;
      dst = v_cache + (page * nkv + g) * (long)page_size * hd + (pos % page_size);
      dst_stride = page_size;
      rotate = false;
    } else {
      src = k ? k + t * k_stride + (long)g * hd : nullptr;
      col = k_col + g * hd;
      dst = k_cache + ((page * nkv + g) * page_size + (pos % page_size)) * hd;
    }
  }
  const float* pp = part ? part + t * ncols + col : nullptr;
  if (rotate) {
    const int half = rotary_dim / 2;
    for (int j = lane; j < half; j += PI_WAVE) {
      const int i0 = interleaved ? 2 * j : j;
      const int i1 = interleaved ? 2 * j + 1 : j + half;
      const float a = rope_source(src, pp, splits, part_stride, i0);
      const float b = rope_source(src, pp, splits, part_stride, i1);
      const float c = table[t * rotary_dim + j], s = table[t * rotary_dim + half + j];
      float lo, hi;
      rope_pair(a, b, c, s, lo, hi);
      dst[i0 * dst_stride] = from_float<T>(lo);
      dst[i1 * dst_stride] = from_float<T>(hi);
    }
    if (part || dst != src)
      for (int i = rotary_dim + lane; i < hd; i += PI_WAVE) dst[i * dst_stride] = from_float<T>(rope_source(src, pp, splits, part_stride, i));
  } else if (part || dst != src) {
    for (int i = lane; i < hd; i += PI_WAVE) dst[i * dst_stride] = from_float<T>(rope_source(src, pp, splits, part_stride, i));
  }
}

// The same for the common case, many tokens at a time (prompts): bfloat16 tensors or float32
// pieces, rotation over the whole head with halves paired, head size a multiple of 16.  Every memory
// access is wide: a thread turns 8 features and their 8 partners of one (token, head) (16-byte
// loads and stores, in place for queries, into the page for keys); for values a thread takes
// one feature of four consecutive tokens and, when the four are neighbours in one page,
// stores them with one 8-byte write into the transposed page.
__global__ __launch_bounds__(256) void rope_kv_write_wide_kernel(
    bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k, long k_stride, const bf16_t* __restrict__ v,
    long v_stride, const int* __restrict__ positions, const int* __restrict__ req_of_token, const float* __restrict__ table,
    int rotate, int T, int nh, int nkv_write, int nkv, int hd, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int table_width, int page_size, long num_pages, long rot_items,
    const float* __restrict__ part, int splits, long part_stride, int ncols, int q_col, int k_col, int v_col) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const int units = hd / 16, heads = nh + nkv_write;
  if (idx < rot_items) {
    const int unit = (int)(idx % units), head = (int)((idx / units) % heads);
    const long t = idx / ((long)units * heads);
    const int d = unit * 8;                      // features d .. d + 7 and their partners at + hd / 2
    const bf16_t* src;
    bf16_t* dst;
    int col;                                     // the head's first column among the pieces
    if (head < nh) {
      dst = q + t * q_stride + (long)head * hd;
      src = dst;
      col = q_col + head * hd;
    } else {
      const int g = head - nh, pos = positions[t], blk = pos / page_size;
      if (blk >= table_width) return;
      const long page = block_table[(long)req_of_token[t] * table_width + blk];
      if (page < 0 || page >= num_pages) return;   // the host checks tables; never write outside the pool
      src = k + t * k_stride + (long)g * hd;
      dst = k_cache + ((page * nkv + g) * page_size + (pos % page_size)) * hd;
      col = k_col + g * hd;
    }
    if (!part && !rotate && dst == src) return;
    typedef float quad_t __attribute__((ext_vector_type(4)));
    float a[8], b[8];                            // the features and their partners, float32
    if (part) {
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = b[e] = 0.f;
      const float* p = part + t * ncols + col + d;
      for (int s0 = 0; s0 < splits; s0 += 4) {   // four pieces' loads go out together, the adds keep the split order
        quad_t la[4][2], lb[4][2];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bool in = s0 + u < splits;
          const float* ps = p + (long)(in ? s0 + u : 0) * part_stride;
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            la[u][h] = in ? *reinterpret_cast<const quad_t*>(ps + 4 * h) : quad_t{0.f, 0.f, 0.f, 0.f};
            lb[u][h] = in ? *reinterpret_cast<const quad_t*>(ps + hd / 2 + 4 * h) : quad_t{0.f, 0.f, 0.f, 0.f};
          }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int e = 0; e < 8; ++e) { a[e] += la[u][e / 4][e % 4]; b[e] += lb[u][e / 4][e % 4]; }
      }
    } else {
      const uint4 lo = *reinterpret_cast<const uint4*>(src + d), hi = *reinterpret_cast<const uint4*>(src + d + hd / 2);
      const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w}, hw[4] = {hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int w = 0; w < 4; ++w) {              // two features per 32-bit word
        a[2 * w] = __uint_as_float(lw[w] << 16); a[2 * w + 1] = __uint_as_float(lw[w] & 0xffff0000u);
        b[2 * w] = __uint_as_float(hw[w] << 16); b[2 * w + 1] = __uint_as_float(hw[w] & 0xffff0000u);
      }
    }
    if (rotate) {
      const float* c = table + t * hd + d;
      const float* sn = c + hd / 2;
      const quad_t c0 = *reinterpret_cast<const quad_t*>(c), c1 = *reinterpret_cast<const quad_t*>(c + 4);
      const quad_t s0 = *reinterpret_cast<const quad_t*>(sn), s1 = *reinterpret_cast<const quad_t*>(sn + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float lo_e, hi_e;
        rope_pair(a[e], b[e], e < 4 ? c0[e] : c1[e - 4], e < 4 ? s0[e] : s1[e - 4], lo_e, hi_e);
        a[e] = lo_e;
        b[e] = hi_e;
      }
    }
    *reinterpret_cast<uint4*>(dst + d) = make_uint4(f32x2_to_bf16x2_bits(a[0], a[1]), f32x2_to_bf16x2_bits(a[2], a[3]),
                                                    f32x2_to_bf16x2_bits(a[4], a[5]), f32x2_to_bf16x2_bits(a[6], a[7]));
    *reinterpret_cast<uint4*>(dst + d + hd / 2) = make_uint4(f32x2_to_bf16x2_bits(b[0], b[1]), f32x2_to_bf16x2_bits(b[2], b[3]),
                                                             f32x2_to_bf16x2_bits(b[4], b[5]), f32x2_to_bf16x2_bits(b[6], b[7]));
    return;
  }
  // values: (four tokens, kv head, feature)
  const long j = idx - rot_items;
  const int d = (int)(j % hd), g = (int)((j / hd) % nkv);
  const long t0 = (j / ((long)hd * nkv)) * 4;
  if (nkv_write == 0 || t0 >= T) return;
  const int n = (int)min((long)4, T - t0);
  uint16_t val[4];
  int pos[4], req[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long t = t0 + (i < n ? i : 0);
    if (part) {
      const bf16_t r = from_float<bf16_t>(split_sum(part, splits, part_stride, t * ncols + v_col + g * hd + d));
      val[i] = *reinterpret_cast<const uint16_t*>(&r);
    } else {
      val[i] = *reinterpret_cast<const uint16_t*>(v + t * v_stride + (long)g * hd + d);
    }
    pos[i] = positions[t];
    req[i] = req_of_token[t];
  }
  const bool together = n == 4 && pos[0] % 4 == 0 && req[3] == req[0] && req[1] == req[0] && req[2] == req[0] &&
                        pos[1] == pos[0] + 1 && pos[2] == pos[0] + 2 && pos[3] == pos[0] + 3;
  if (together) {                                  // page sizes are multiples of 4 here: one page, four slots in a row
    const int blk = pos[0] / page_size;
    if (blk >= table_width) return;
    const long page = block_table[(long)req[0] * table_width + blk];
    if (page < 0 || page >= num_pages) return;
    uint2 w;
    w.x = (uint32_t)val[0] | ((uint32_t)val[1] << 16);
    w.y = (uint32_t)val[2] | ((uint32_t)val[3] << 16);
    *reinterpret_cast<uint2*>(v_cache + (page * nkv + g) * (long)page_size * hd + (long)d * page_size + pos[0] % page_size) = w;
    return;
  }
  for (int i = 0; i < n; ++i) {
    const int blk = pos[i] / page_size;
    if (blk >= table_width) continue;
    const long page = block_table[(long)req[i] * table_width + blk];
    if (page < 0 || page >= num_pages) continue;
    reinterpret_cast<uint16_t*>(v_cache)[(page * nkv + g) * (long)page_size * hd + (long)d * page_size + pos[i] % page_size] = val[i];
  }
}

extern "C" int pi_rope_kv_write(void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                                int dtype, const int* positions, const int* req_of_token, const float* table,
                                int rotary_dim, int interleaved, int T, int nh, int nkv, int hd, int write_kv,
                                void* k_cache, void* v_cache, const int* block_table, int table_width,
                                int page_size, long num_pages, const float* part, int splits, int ncols, int q_col,
                                int k_col, int v_col, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && nh >= 0 && nkv >= 0 && hd > 0 && hd <= 256, "rope_kv_write: bad sizes T=%d heads=%d kv_heads=%d head_dim=%d", T, nh, nkv, hd);
  PI_REQUIRE(rotary_dim >= 0 && rotary_dim <= hd && rotary_dim % 2 == 0, "rope_kv_write: rotary_dim %d must be even and <= head_dim %d", rotary_dim, hd);
  PI_REQUIRE(rotary_dim == 0 || table != nullptr, "rope_kv_write: rotation asked for without a cos / sin table");
  PI_REQUIRE(part == nullptr || (splits >= 1 && ncols > 0), "rope_kv_write: bad split description");
  if (write_kv) {
    PI_REQUIRE((part || (k && v)) && k_cache && v_cache && block_table && req_of_token, "rope_kv_write: cache write asked for without k/v/cache/table");
    PI_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0, "rope_kv_write: bad cache geometry page_size=%d table_width=%d pages=%ld", page_size, table_width, num_pages);
  }
  const int heads = nh + (write_kv ? 2 * nkv : 0);
  if (T == 0 || heads == 0) return 0;
  // many bfloat16 tokens with the usual rotation: the kernel with wide accesses
  const bool usual = rotary_dim == 0 || (rotary_dim == hd && !interleaved);
  const bool source_ok = part ? (ncols % 4 == 0 && ((uintptr_t)part % 16 == 0) && q_col % 4 == 0 && k_col % 4 == 0)
                              : (!write_kv || (k_stride % 8 == 0 && ((uintptr_t)k % 16 == 0)));
  const bool aligned = hd % 16 == 0 && q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && (!table || (uintptr_t)table % 16 == 0) &&
                       source_ok && (!write_kv || (((uintptr_t)k_cache % 16 == 0) && ((uintptr_t)v_cache % 8 == 0) && page_size % 4 == 0));
  if (dtype == PI_BF16 && usual && aligned && T >= 16) {
    const int nkv_w = write_kv ? nkv : 0;
    const long rot_items = (long)T * (nh + nkv_w) * (hd / 16);
    const long v_items = write_kv ? (long)((T + 3) / 4) * nkv * hd : 0;
    const long blocks = (rot_items + v_items + 255) / 256;
    PI_REQUIRE(blocks < 2147483647L, "rope_kv_write: too many tokens (%d)", T);
    hipLaunchKernelGGL(rope_kv_write_wide_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)q, q_stride,
                       (const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, positions, req_of_token, table,
                       rotary_dim > 0 ? 1 : 0, T, nh, nkv_w, nkv, hd, (bf16_t*)k_cache, (bf16_t*)v_cache, block_table,
                       table_width, page_size, num_pages, rot_items, part, splits, (long)T * ncols, ncols, q_col, k_col, v_col);
    return pi_check_launch("rope_kv_write_wide");
  }
  PI_REQUIRE(heads <= 65535, "rope_kv_write: too many heads (%d)", heads);
  const dim3 grid(T, (heads + 3) / 4), block(256);
  const int nkv_write = write_kv ? nkv : 0;
  const long part_stride = (long)T * ncols;
  if (dtype == PI_F32)
    hipLaunchKernelGGL(rope_kv_write_kernel<float>, grid, block, 0, stream, (float*)q, q_stride, (const float*)k, k_stride,
                       (const float*)v, v_stride, positions, req_of_token, table, rotary_dim, interleaved, nh, nkv_write,
                       nkv, hd, (float*)k_cache, (float*)v_cache, block_table, table_width, page_size, num_pages, part,
                       splits, part_stride, ncols, q_col, k_col, v_col);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(rope_kv_write_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)q, q_stride, (const bf16_t*)k, k_stride,
                       (const bf16_t*)v, v_stride, positions, req_of_token, table, rotary_dim, interleaved, nh, nkv_write,
                       nkv, hd, (bf16_t*)k_cache, (bf16_t*)v_cache, block_table, table_width, page_size, num_pages, part,
                       splits, part_stride, ncols, q_col, k_col, v_col);
  else
    return pi_fail("rope_kv_write: unsupported dtype %d", dtype);
  return pi_check_launch("rope_kv_write");
}

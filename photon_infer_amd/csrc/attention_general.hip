// Causal attention over the paged cache for any head size (multiple of 16, up to 256),
// any number of heads and groups, both storage types, prompts and single tokens alike.
// One wave per (token, head); scores, softmax and the weighted sum are float32.
//
// For the query at absolute position p (include/photon/ops/kernels/mha_kernel.hpp:174-230):
//   s_t = scale * <q, K[t]>, t = lo..p;  P = exp(s - max s) / sum exp(s - max s);
//   o = sum_t P_t V[t]
// with lo = 0, or p - window + 1 when a window is given.  Causality is the loop bound.
// The softmax is exact: no constant is added to the denominator (the reference's paged
// kernel adds 1e-6, src/ops/kernels/cuda/paged_attention.cu:71).
//
// Keys are visited 64 at a time with the usual running maximum / running sum, so the
// result for a token depends only on that token's position and its request's pages.
#include "common.h"

#define PI_MAX_HEAD_DIM 256

template <typename T>
__global__ __launch_bounds__(PI_WAVE) void paged_attention_general_kernel(
    T* __restrict__ out, long out_stride, const T* __restrict__ q, long q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ req_of_token, const int* __restrict__ positions, int nh, int nkv, int hd, int page_size,
    float scale, int window, long num_pages) {
  __shared__ float qs[PI_MAX_HEAD_DIM];
  __shared__ float ps[PI_WAVE];
  __shared__ long voff[PI_WAVE];   // values are stored [page, kv_head, head_dim, slot]
  const long t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int g = h / (nh / nkv);
  const T* qr = q + t * q_stride + (long)h * hd;
  for (int d = lane; d < hd; d += PI_WAVE) qs[d] = to_float(qr[d]);
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* bt = block_table + (long)req_of_token[t] * table_width;
  float m = -INFINITY, l = 0.f;
  float acc[PI_MAX_HEAD_DIM / PI_WAVE] = {0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  for (int k0 = lo; k0 <= p; k0 += PI_WAVE) {
    const int key = k0 + lane;
    float s = -INFINITY;
    long off = -1, vo = -1;
    if (key <= p) {
      const int blk = key / page_size;
      const long page = blk < table_width ? bt[blk] : -1;
      if (page >= 0 && page < num_pages) {
        off = ((page * nkv + g) * page_size + (key % page_size)) * hd;
        vo = (page * nkv + g) * (long)page_size * hd + (key % page_size);
        const T* kr = k_cache + off;
        float dot = 0.f;
        for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
        s = dot * scale;
      } else {
        s = __builtin_nanf("");  // a key without a page: make it visible, never read outside the pool
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pe = (key <= p) ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(pe);
    ps[lane] = pe;
    voff[lane] = vo;
#pragma unroll
    for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) acc[i] *= corr;
    __syncthreads();
    const int nk = (p - k0 + 1) < PI_WAVE ? (p - k0 + 1) : PI_WAVE;
    for (int kk = 0; kk < nk; ++kk) {
      const long o2 = voff[kk];
      if (o2 < 0) continue;
      const T* vr = v_cache + o2;
      const float pk = ps[kk];
#pragma unroll
      for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
        const int d = lane + i * PI_WAVE;
        if (d < hd) acc[i] = fmaf(pk, to_float(vr[(long)d * page_size]), acc[i]);
      }
    }
    m = m_new;
    __syncthreads();
  }
  T* o = out + t * out_stride + (long)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
    const int d = lane + i * PI_WAVE;
    if (d < hd) o[d] = from_float<T>(acc[i] * inv);
  }
}

extern "C" int pi_paged_attention_general(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                          const void* v_cache, int dtype, const int* block_table, int table_width,
                                          const int* req_of_token, const int* positions, int T, int nh, int nkv, int hd,
                                          int page_size, float scale, int window, long num_pages, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention: heads %d must be a positive multiple of kv heads %d", nh, nkv);
  PI_REQUIRE(hd > 0 && hd % 16 == 0 && hd <= PI_MAX_HEAD_DIM, "attention: head_dim %d must be a multiple of 16 up to %d", hd, PI_MAX_HEAD_DIM);
  PI_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0, "attention: bad cache geometry page_size=%d table_width=%d pages=%ld", page_size, table_width, num_pages);
  PI_REQUIRE(nh <= 65535, "attention: too many heads (%d)", nh);
  PI_REQUIRE(window >= 0, "attention: window must be >= 0, got %d", window);
  if (T == 0) return 0;
  const dim3 grid(T, nh), block(PI_WAVE);
  if (dtype == PI_F32)
    hipLaunchKernelGGL(paged_attention_general_kernel<float>, grid, block, 0, stream, (float*)out, out_stride, (const float*)q,
                       q_stride, (const float*)k_cache, (const float*)v_cache, block_table, table_width, req_of_token,
                       positions, nh, nkv, hd, page_size, scale, window, num_pages);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(paged_attention_general_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, out_stride,
                       (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width,
                       req_of_token, positions, nh, nkv, hd, page_size, scale, window, num_pages);
  else
    return pi_fail("attention: unsupported dtype %d", dtype);
  return pi_check_launch("paged_attention_general");
}

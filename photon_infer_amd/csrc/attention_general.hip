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
//
// A step of few tokens (decoding) has too few (token, head) pairs to fill the chip: its keys
// are then cut into `splits` ranges of whole 64-key groups, one wave each (grid z); every range
// leaves its un-normalised sum, maximum and sum of weights, and a second kernel merges the
// ranges in range order with the same exact exponentials.
#include "common.h"

#define PI_MAX_HEAD_DIM 256

template <typename T>
__global__ __launch_bounds__(PI_WAVE) void paged_attention_general_kernel(
    T* __restrict__ out, long out_stride, const T* __restrict__ q, long q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ req_of_token, const int* __restrict__ positions, int nh, int nkv, int hd, int page_size,
    float scale, int window, long num_pages, float* __restrict__ part) {
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
  // this wave's keys: all of lo..p, or the z-th of gridDim.z ranges of whole 64-key groups
  const int splits = gridDim.z;
  const int groups = (p - lo) / PI_WAVE + 1;
  const int per = (groups + splits - 1) / splits;
  const int first = lo + (int)blockIdx.z * per * PI_WAVE;
  const long last_l = (long)first + (long)per * PI_WAVE - 1;
  const int last = last_l < p ? (int)last_l : p;
  for (int k0 = first; k0 <= last; k0 += PI_WAVE) {
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
        for (int d = 0; d < hd; d += 4) {          // in ascending order of d, four features per load
          float kv[4];
          load4(kr + d, kv);
          dot = fmaf(qs[d], kv[0], dot);
          dot = fmaf(qs[d + 1], kv[1], dot);
          dot = fmaf(qs[d + 2], kv[2], dot);
          dot = fmaf(qs[d + 3], kv[3], dot);
        }
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
    // keys in ascending order; four at a time where they lie side by side in a page (values are
    // stored with the slot as the last axis), in the same order of additions
    for (int kk = 0; kk < nk;) {
      const long o2 = voff[kk];
      const bool four = page_size % 4 == 0 && ((k0 + kk) & 3) == 0 && kk + 3 < nk;
      if (o2 >= 0) {
        const T* vr = v_cache + o2;
        if (four) {
          const float p0 = ps[kk], p1 = ps[kk + 1], p2 = ps[kk + 2], p3 = ps[kk + 3];
#pragma unroll
          for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
            const int d = lane + i * PI_WAVE;
            if (d < hd) {
              float vv[4];
              load4(vr + (long)d * page_size, vv);
              acc[i] = fmaf(p0, vv[0], acc[i]);
              acc[i] = fmaf(p1, vv[1], acc[i]);
              acc[i] = fmaf(p2, vv[2], acc[i]);
              acc[i] = fmaf(p3, vv[3], acc[i]);
            }
          }
        } else {
          const float pk = ps[kk];
#pragma unroll
          for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
            const int d = lane + i * PI_WAVE;
            if (d < hd) acc[i] = fmaf(pk, to_float(vr[(long)d * page_size]), acc[i]);
          }
        }
      }
      kk += four ? 4 : 1;
    }
    m = m_new;
    __syncthreads();
  }
  if (splits > 1) {
    // [token, head, range, hd + 2]: the un-normalised sum, then the range's maximum and sum of weights
    float* mine = part + (((long)t * nh + h) * splits + blockIdx.z) * (hd + 2);
#pragma unroll
    for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
      const int d = lane + i * PI_WAVE;
      if (d < hd) mine[d] = acc[i];
    }
    if (lane == 0) {
      mine[hd] = m;
      mine[hd + 1] = l;
    }
    return;
  }
  T* o = out + t * out_stride + (long)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
    const int d = lane + i * PI_WAVE;
    if (d < hd) o[d] = from_float<T>(acc[i] * inv);
  }
}

// One wave per (token, head): o = sum_s e^(m_s - m) acc_s / sum_s e^(m_s - m) l_s, ranges in order;
// an empty range (m_s = -inf, l_s = 0) counts nothing.
template <typename T>
__global__ __launch_bounds__(PI_WAVE) void merge_key_ranges_kernel(T* __restrict__ out, long out_stride, const float* __restrict__ part,
                                                                   int nh, int hd, int splits) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* base = part + ((long)t * nh + h) * splits * (hd + 2);
  float m = -INFINITY;
  for (int s = 0; s < splits; ++s) m = fmaxf(m, base[s * (hd + 2) + hd]);
  float l = 0.f;
  float acc[PI_MAX_HEAD_DIM / PI_WAVE] = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < splits; ++s) {
    const float ms = base[s * (hd + 2) + hd];
    const float w = ms == -INFINITY ? 0.f : expf(ms - m);
    l = fmaf(w, base[s * (hd + 2) + hd + 1], l);
#pragma unroll
    for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
      const int d = lane + i * PI_WAVE;
      if (d < hd) acc[i] = fmaf(w, base[s * (hd + 2) + d], acc[i]);
    }
  }
  T* o = out + t * out_stride + (long)h * hd;
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < PI_MAX_HEAD_DIM / PI_WAVE; ++i) {
    const int d = lane + i * PI_WAVE;
    if (d < hd) o[d] = from_float<T>(acc[i] * inv);
  }
}

// Key ranges per (token, head) that pi_paged_attention_general makes for a step of T tokens whose
// longest context is max_kv_len: 1 unless the step's (token, head) pairs are too few for the chip
// and the contexts long; the caller provides float32 [T * nh * ranges * (hd + 2)] when it is more.
extern "C" int pi_paged_attention_general_ranges(int T, int nh, int max_kv_len) {
  const long pairs = (long)T * nh;
  if (pairs <= 0 || pairs >= 2048 || max_kv_len < 4 * PI_WAVE) return 1;
  long want = 4096 / pairs, most = max_kv_len / (2 * PI_WAVE);      // a range keeps at least 128 keys
  if (want > most) want = most;
  if (want > 64) want = 64;
  return want < 1 ? 1 : (int)want;
}

extern "C" int pi_paged_attention_general(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                          const void* v_cache, int dtype, const int* block_table, int table_width,
                                          const int* req_of_token, const int* positions, int T, int nh, int nkv, int hd,
                                          int page_size, float scale, int window, long num_pages, int splits, void* part,
                                          long part_elems, hipStream_t stream) {
  PI_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention: heads %d must be a positive multiple of kv heads %d", nh, nkv);
  PI_REQUIRE(hd > 0 && hd % 16 == 0 && hd <= PI_MAX_HEAD_DIM, "attention: head_dim %d must be a multiple of 16 up to %d", hd, PI_MAX_HEAD_DIM);
  PI_REQUIRE(page_size > 0 && table_width > 0 && num_pages > 0, "attention: bad cache geometry page_size=%d table_width=%d pages=%ld", page_size, table_width, num_pages);
  PI_REQUIRE(nh <= 65535, "attention: too many heads (%d)", nh);
  PI_REQUIRE(window >= 0, "attention: window must be >= 0, got %d", window);
  PI_REQUIRE(splits >= 1 && splits <= 65535, "attention: bad number of key ranges %d", splits);
  PI_REQUIRE(splits == 1 || (part && part_elems >= (long)T * nh * splits * (hd + 2)), "attention: workspace too small for %d key ranges", splits);
  if (T == 0) return 0;
  const dim3 grid(T, nh, splits), block(PI_WAVE);
  if (dtype == PI_F32)
    hipLaunchKernelGGL(paged_attention_general_kernel<float>, grid, block, 0, stream, (float*)out, out_stride, (const float*)q,
                       q_stride, (const float*)k_cache, (const float*)v_cache, block_table, table_width, req_of_token,
                       positions, nh, nkv, hd, page_size, scale, window, num_pages, (float*)part);
  else if (dtype == PI_BF16)
    hipLaunchKernelGGL(paged_attention_general_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, out_stride,
                       (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width,
                       req_of_token, positions, nh, nkv, hd, page_size, scale, window, num_pages, (float*)part);
  else
    return pi_fail("attention: unsupported dtype %d", dtype);
  if (pi_check_launch("paged_attention_general")) return -1;
  if (splits == 1) return 0;
  if (dtype == PI_F32)
    hipLaunchKernelGGL(merge_key_ranges_kernel<float>, dim3(T, nh), block, 0, stream, (float*)out, out_stride, (const float*)part, nh, hd, splits);
  else
    hipLaunchKernelGGL(merge_key_ranges_kernel<bf16_t>, dim3(T, nh), block, 0, stream, (bf16_t*)out, out_stride, (const float*)part, nh, hd, splits);
  return pi_check_launch("merge_key_ranges");
}

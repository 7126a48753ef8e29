// Decode attention over the paged cache, split over the keys (bfloat16, matrix cores).
//
// One wave per (key range, kv head, request).  The wave's 16 query columns are the heads of
// the kv group (up to 16; unused columns are padding), so a group's keys and values are read
// once.  Every range writes its un-normalised partial result with its running maximum and
// sum; the wave that arrives last at the (request, kv head) counter merges the ranges in range
// order (deterministic) and writes the output.  Counters reset themselves.  With one range
// the result is written directly.
//
// For the query at position p = kv_len - 1: keys lo..p with lo = max(0, p - window + 1)
// (window 0: all keys).  Ranges are cut at multiples of 32 keys.
#include "attention_mfma.h"

template <int HD>
__global__ __launch_bounds__(64) void attention_decode_kernel(
    bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q, long q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ q_start, const int* __restrict__ kv_len_of, int nh, int nkv, int page_size,
    float scale, int window, long num_pages, float* __restrict__ part, int* __restrict__ counters) {
  const int lane = threadIdx.x, lr = lane % 16, lg = lane / 16;
  const int split = blockIdx.x, splits = gridDim.x, g = blockIdx.y, r = blockIdx.z;
  const int G = nh / nkv;
  const int kv_len = kv_len_of[r];
  const int p = kv_len - 1;
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const long row = q_start[r];
  const int* bt = block_table + (long)r * table_width;

  AttnState<HD, 1> st;
  attn_init(st);
  const bool valid = lr < G;
  st.pos[0] = valid ? p : -1;
  st.lo[0] = lo;
  attn_load_q(st, 0, q, q_stride, row, g * G + lr, valid, lane);

  // this wave's keys: chunk `split` of the 32-key chunks between lo and p
  const int first_chunk = lo / 32, last_chunk = p / 32;
  const int chunks = last_chunk - first_chunk + 1;
  const int per = (chunks + splits - 1) / splits;
  const int c0 = first_chunk + split * per;
  const int c1 = min(last_chunk + 1, c0 + per);
  for (int c = c0; c < c1; ++c)
    attn_chunk<HD, 1>(st, c * 32, k_cache, v_cache, bt, table_width, kv_len, nkv, g, page_size, num_pages, scale, lane);

  const int head = g * G + lr;
  if (splits == 1) {
    if (valid) {
      const float inv = 1.0f / st.l[0];
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) {
        uint2 w;
        w.x = pack_bf16x2(st.o[db][0][0] * inv, st.o[db][0][1] * inv);
        w.y = pack_bf16x2(st.o[db][0][2] * inv, st.o[db][0][3] * inv);
        *reinterpret_cast<uint2*>(out + row * out_stride + (long)head * HD + db * 16 + lg * 4) = w;
      }
    }
    return;
  }

  // partial: [request, head, split, HD + 4] float32: O^T (un-normalised), then m, l
  const int rec = HD + 4;   // O^T, m, l, two floats of padding (keeps 16-byte alignment)
  if (valid) {
    float* mine = part + (((long)r * nh + head) * splits + split) * rec;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db)
      *reinterpret_cast<f32x4_t*>(mine + db * 16 + lg * 4) = st.o[db][0];
    if (lg == 0) {
      mine[HD] = st.m[0];
      mine[HD + 1] = st.l[0];
    }
  }
  __threadfence();
  int last = 0;
  if (lane == 0) last = (atomicAdd(&counters[r * nkv + g], 1) == splits - 1);
  last = __shfl(last, 0, 64);
  if (!last) return;
  __threadfence();
  // merge: lane (lr, lg) owns head lr, features lg*4 .. lg*4+3 of every 16-block
  if (valid) {
    const float* base = part + ((long)r * nh + head) * splits * rec;
    float m_tot = -INFINITY;
    for (int s = 0; s < splits; ++s) m_tot = fmaxf(m_tot, __builtin_nontemporal_load(base + s * rec + HD));
    float l_tot = 0.f;
    f32x4_t acc[HD / 16];
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) acc[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < splits; ++s) {
      const float ms = __builtin_nontemporal_load(base + s * rec + HD);
      if (ms == -INFINITY) continue;           // an empty range
      const float w = expf(ms - m_tot);
      l_tot += w * __builtin_nontemporal_load(base + s * rec + HD + 1);
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) {
        const f32x4_t o = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(base + s * rec + db * 16 + lg * 4));
        acc[db][0] += w * o[0]; acc[db][1] += w * o[1]; acc[db][2] += w * o[2]; acc[db][3] += w * o[3];
      }
    }
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
      uint2 w;
      w.x = pack_bf16x2(acc[db][0] * inv, acc[db][1] * inv);
      w.y = pack_bf16x2(acc[db][2] * inv, acc[db][3] * inv);
      *reinterpret_cast<uint2*>(out + row * out_stride + (long)head * HD + db * 16 + lg * 4) = w;
    }
  }
  if (lane == 0) counters[r * nkv + g] = 0;
}

// part: float32 [R * nh * splits * (hd + 4)], counters: int32 [R * nkv] (zero).
extern "C" int pi_attention_decode(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                   const void* v_cache, const int* block_table, int table_width, const int* q_start,
                                   const int* kv_len, int R, int nh, int nkv, int hd, int page_size, float scale, int window,
                                   long num_pages, int splits, void* part, long part_elems, void* counters,
                                   long num_counters, hipStream_t stream) {
  PI_REQUIRE(R > 0 && nh > 0 && nkv > 0 && nh % nkv == 0 && nh / nkv <= 16, "attention_decode: needs 1..16 heads per kv head, got %d / %d", nh, nkv);
  PI_REQUIRE(hd == 64 || hd == 128, "attention_decode: head_dim %d is not 64 or 128", hd);
  PI_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_decode: page size %d must be a multiple of 16", page_size);
  PI_REQUIRE(splits >= 1 && splits <= 1024 && R <= 65535 && nkv <= 65535, "attention_decode: bad grid (%d ranges, %d requests, %d kv heads)", splits, R, nkv);
  PI_REQUIRE(out_stride % 4 == 0 && q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 8 == 0), "attention_decode: q / out rows must be 16- / 8-byte aligned");
  if (splits > 1)
    PI_REQUIRE(part && counters && part_elems >= (long)R * nh * splits * (hd + 4) && num_counters >= (long)R * nkv,
               "attention_decode: workspace too small for %d ranges", splits);
  const dim3 grid(splits, nkv, R), block(64);
#define GO(H) hipLaunchKernelGGL(attention_decode_kernel<H>, grid, block, 0, stream, (bf16_t*)out, out_stride, (const bf16_t*)q, \
                                 q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width, q_start, \
                                 kv_len, nh, nkv, page_size, scale, window, num_pages, (float*)part, (int*)counters)
  if (hd == 64) GO(64); else GO(128);
#undef GO
  return pi_check_launch("attention_decode");
}

// Decode attention over the paged cache, split over the keys (bfloat16, matrix cores).
//
// One wave per (key range, kv head, request).  The wave's 16 query columns are the heads of
// the kv group (up to 16; unused columns are padding), so a group's keys and values are read
// once.  Every range writes its un-normalised partial result with its running maximum and
// sum; a second small kernel merges the ranges in range order (deterministic).  With one range
// the result is written directly.
//
// For the query at position p = kv_len - 1: keys lo..p with lo = max(0, p - window + 1)
// (window 0: all keys).  Ranges are cut at multiples of 32 keys.
#include "attention_mfma.h"

template <int HD>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 2 : 1))) void attention_decode_kernel(
    bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q, long q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ q_start, const int* __restrict__ kv_len_of, const int* __restrict__ req_ids,
    int nh, int nkv, int page_size, float scale, int window, long num_pages, float* __restrict__ part) {
  const int lane = threadIdx.x, lr = lane % 16, lg = lane / 16;
  const int split = blockIdx.x, splits = gridDim.x, g = blockIdx.y;
  // the z-th request of this launch: all of the step's requests, or the listed ones (a step
  // that also holds prompt portions sends only its single tokens here)
  const int r = req_ids ? req_ids[blockIdx.z] : (int)blockIdx.z;
  const int G = nh / nkv;
  const int kv_len = kv_len_of[r];
  const int p = kv_len - 1;
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const long row = q_start[r];
  const int* bt = block_table + (long)r * table_width;

  AttnState<HD, 1> st;
  attn_init(st);
  const bool valid = lr < G;     // the other columns are padding: computed on zeros, never stored
  st.pos[0] = p;
  st.lo[0] = lo;
  attn_load_q(st, 0, q, q_stride, row, g * G + lr, valid, lane);

  // this wave's keys: chunk `split` of the 32-key chunks between lo and p
  const int first_chunk = lo / 32, last_chunk = p / 32;
  const int chunks = last_chunk - first_chunk + 1;
  const int per = (chunks + splits - 1) / splits;
  const int c0 = first_chunk + split * per;
  const int c1 = min(last_chunk + 1, c0 + per);
  attn_walk<HD, 1>(st, c0, c1, (lo + 31) / 32, (p + 1) / 32 - 1, k_cache, v_cache, bt, table_width, kv_len, nkv, g,
                   page_size, num_pages, scale * PI_LOG2E, lane);
  attn_finish(st);

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
    float* mine = part + (((long)blockIdx.z * nh + head) * splits + split) * rec;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db)
      *reinterpret_cast<f32x4_t*>(mine + db * 16 + lg * 4) = st.o[db][0];
    if (lg == 0) {
      mine[HD] = st.m[0] * (scale * PI_LOG2E);   // base-2 scale; -inf stays -inf
      mine[HD + 1] = st.l[0];
    }
  }
}

// Merge the key ranges of every (request, head): one wave per pair, lane d owns feature d
// (and d + 64).  Ranges are added in range order; an empty range (m = -inf) counts nothing.
template <int HD>
__global__ __launch_bounds__(64) void attention_combine_kernel(bf16_t* __restrict__ out, long out_stride,
                                                               const int* __restrict__ q_start,
                                                               const int* __restrict__ req_ids,
                                                               const int* __restrict__ rows,
                                                               const float* __restrict__ part, int nh, int splits) {
  const int lane = threadIdx.x;
  const int head = blockIdx.x;
  // where the result goes: the token row of request r (decode), or a listed row (cut tiles)
  const int r = req_ids ? req_ids[blockIdx.y] : (int)blockIdx.y;
  const long out_row = rows ? rows[blockIdx.y] : q_start[r];
  const int rec = HD + 4;
  const float* base = part + ((long)blockIdx.y * nh + head) * splits * rec;
  // lane s holds range s (splits <= 64): maxima, weights and the total in parallel
  const float ms = lane < splits ? base[lane * rec + HD] : -INFINITY;
  const float ls = lane < splits ? base[lane * rec + HD + 1] : 0.f;
  const float m_tot = wave_max(ms);
  const float w = (ms == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ms - m_tot);   // maxima are in the base-2 scale
  float l_tot = 0.f;
  float acc[HD / 64];
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) acc[i] = 0.f;
  // ranges in order; eight loads in flight at a time
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float o[8][HD / 64], ws[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int s = s0 + u;
      ws[u] = __shfl(w, s < splits ? s : 0, 64);
      if (s >= splits) ws[u] = 0.f;
#pragma unroll
      for (int i = 0; i < HD / 64; ++i) o[u][i] = (s < splits) ? base[s * rec + lane + i * 64] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      l_tot += ws[u] * __shfl(ls, (s0 + u < splits) ? s0 + u : 0, 64);
#pragma unroll
      for (int i = 0; i < HD / 64; ++i) acc[i] += ws[u] * o[u][i];
    }
  }
  const float inv = 1.0f / l_tot;
  bf16_t* o = out + out_row * out_stride + (long)head * HD;
#pragma unroll
  for (int i = 0; i < HD / 64; ++i) o[lane + i * 64] = from_float<bf16_t>(acc[i] * inv);
}

// part: float32 [R * nh * splits * (hd + 4)], needed when splits > 1.
// req_ids: null (requests 0 .. R-1) or the R requests of the step that this launch serves; each
// has one query token, at row q_start[r], that sees kv_len[r] keys.
extern "C" int pi_attention_decode(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                   const void* v_cache, const int* block_table, int table_width, const int* q_start,
                                   const int* kv_len, const int* req_ids, int R, int nh, int nkv, int hd, int page_size,
                                   float scale, int window, long num_pages, int splits, void* part, long part_elems,
                                   hipStream_t stream) {
  PI_REQUIRE(R > 0 && nh > 0 && nkv > 0 && nh % nkv == 0 && nh / nkv <= 16, "attention_decode: needs 1..16 heads per kv head, got %d / %d", nh, nkv);
  PI_REQUIRE(hd == 64 || hd == 128, "attention_decode: head_dim %d is not 64 or 128", hd);
  PI_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_decode: page size %d must be a multiple of 16", page_size);
  PI_REQUIRE(splits >= 1 && splits <= 64 && R <= 65535 && nkv <= 65535, "attention_decode: bad grid (%d ranges, %d requests, %d kv heads)", splits, R, nkv);
  PI_REQUIRE(out_stride % 4 == 0 && q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 8 == 0), "attention_decode: q / out rows must be 16- / 8-byte aligned");
  if (splits > 1)
    PI_REQUIRE(part && part_elems >= (long)R * nh * splits * (hd + 4), "attention_decode: workspace too small for %d ranges", splits);
  const dim3 grid(splits, nkv, R), block(64);
#define GO(H) hipLaunchKernelGGL(attention_decode_kernel<H>, grid, block, 0, stream, (bf16_t*)out, out_stride, (const bf16_t*)q, \
                                 q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width, q_start, \
                                 kv_len, req_ids, nh, nkv, page_size, scale, window, num_pages, (float*)part)
  if (hd == 64) GO(64); else GO(128);
#undef GO
  if (pi_check_launch("attention_decode")) return -1;
  if (splits > 1) {
    const dim3 cgrid(nh, R);
    if (hd == 64)
      hipLaunchKernelGGL(attention_combine_kernel<64>, cgrid, block, 0, stream, (bf16_t*)out, out_stride, q_start, req_ids, (const int*)nullptr, (const float*)part, nh, splits);
    else
      hipLaunchKernelGGL(attention_combine_kernel<128>, cgrid, block, 0, stream, (bf16_t*)out, out_stride, q_start, req_ids, (const int*)nullptr, (const float*)part, nh, splits);
    return pi_check_launch("attention_combine");
  }
  return 0;
}

// Merge partial results that the tile kernel wrote for `Z` tokens whose tiles' keys were cut in
// `cuts` shares: part [Z, nh, cuts, hd + 4]; token z's result goes to row rows[z] of out.
extern "C" int pi_attention_combine_rows(void* out, long out_stride, const int* rows, int Z, const void* part, int nh, int hd,
                                         int cuts, hipStream_t stream) {
  PI_REQUIRE(Z > 0 && Z <= 65535 && nh > 0 && cuts >= 2 && cuts <= 64 && rows && part, "attention_combine_rows: bad arguments (%d tokens, %d heads, %d cuts)", Z, nh, cuts);
  PI_REQUIRE(hd == 64 || hd == 128, "attention_combine_rows: head_dim %d is not 64 or 128", hd);
  const dim3 grid(nh, Z), block(64);
  if (hd == 64)
    hipLaunchKernelGGL(attention_combine_kernel<64>, grid, block, 0, stream, (bf16_t*)out, out_stride, (const int*)nullptr,
                       (const int*)nullptr, rows, (const float*)part, nh, cuts);
  else
    hipLaunchKernelGGL(attention_combine_kernel<128>, grid, block, 0, stream, (bf16_t*)out, out_stride, (const int*)nullptr,
                       (const int*)nullptr, rows, (const float*)part, nh, cuts);
  return pi_check_launch("attention_combine_rows");
}

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
//
// FUSED: the kernel starts from the q|k|v projection as the product left it (a bfloat16 tensor
// or float32 pieces split over k) instead of rotated queries and a written cache: every wave
// rotates its own queries, and the wave whose range ends at the new token rotates that token's
// key, stores key and value into the page and waits for the stores before it walks.  A decode
// step then needs no kernel between the projection and the attention, and its results are, bit
// for bit, those of the separate kernels.
#include "attention_mfma.h"

struct DecodeSource {
  const bf16_t* qkv;      // [T, qkv_stride] or null
  long qkv_stride;
  const float* part;      // [splits, T, ncols] or null
  int splits;
  long part_stride;       // T * ncols
  int ncols;
  int q_col, k_col, v_col;
  const float* table;     // [T, HD]: cosines of the HD / 2 pair angles, then their sines; null: no rotation
  int write_kv;
  bf16_t* k_cache;
  bf16_t* v_cache;
};

// Values of a token's row of the projection: NO runs of eight consecutive columns (from
// ocol[i], multiples of 8; rows are 16-byte aligned) and NS single columns, zeros where the
// lane's flag says so.  Pieces are added in split order, several splits' loads in flight for
// all columns at once: a wave waits for memory once per group of splits, not once per column.
template <int NO, int NS>
__device__ inline void source_gather(const DecodeSource& src, long row, const int (&ocol)[NO], bool octets_wanted,
                                     float (&xo)[NO][8], const int (&scol)[NS > 0 ? NS : 1], bool singles_wanted,
                                     float (&xs)[NS > 0 ? NS : 1]) {
  typedef float quad_t __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int o = 0; o < NO; ++o)
#pragma unroll
    for (int e = 0; e < 8; ++e) xo[o][e] = 0.f;
#pragma unroll
  for (int i = 0; i < (NS > 0 ? NS : 1); ++i) xs[i] = 0.f;
  if (src.part) {
    const float* base = src.part + row * src.ncols;
    constexpr int U = NO <= 2 ? 8 : 4;     // splits in flight: as many as the registers hold
    for (int s0 = 0; s0 < src.splits; s0 += U) {
      quad_t lo[U][NO], hi[U][NO];
      float one[U][NS > 0 ? NS : 1];
      // every load is made (a split beyond the last reads the first again, a lane that wants
      // nothing reads column 0) and what is not wanted is zeroed afterwards: no branch around
      // each load, a fraction of the code
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bool in = s0 + u < src.splits;
        const float* p = base + (long)(in ? s0 + u : 0) * src.part_stride;
        const quad_t zero = quad_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int o = 0; o < NO; ++o) {
          const int c = octets_wanted ? ocol[o] : 0;
          const quad_t l = *reinterpret_cast<const quad_t*>(p + c), h = *reinterpret_cast<const quad_t*>(p + c + 4);
          lo[u][o] = (in && octets_wanted) ? l : zero;
          hi[u][o] = (in && octets_wanted) ? h : zero;
        }
#pragma unroll
        for (int i = 0; i < NS; ++i) {
          const float v = p[singles_wanted ? scol[i] : 0];
          one[u][i] = (in && singles_wanted) ? v : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int o = 0; o < NO; ++o)
#pragma unroll
          for (int e = 0; e < 4; ++e) { xo[o][e] += lo[u][o][e]; xo[o][4 + e] += hi[u][o][e]; }
#pragma unroll
        for (int i = 0; i < NS; ++i) xs[i] += one[u][i];
      }
    }
    return;
  }
  const bf16_t* base = src.qkv + row * src.qkv_stride;
#pragma unroll
  for (int o = 0; o < NO; ++o) {
    if (!octets_wanted) continue;
    const uint4 w = *reinterpret_cast<const uint4*>(base + ocol[o]);
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      xo[o][2 * e] = __uint_as_float(ws[e] << 16);
      xo[o][2 * e + 1] = __uint_as_float(ws[e] & 0xffff0000u);
    }
  }
#pragma unroll
  for (int i = 0; i < NS; ++i)
    if (singles_wanted) xs[i] = to_float(base[scol[i]]);
}

// The fragments of the HD features that start at column col0 of token row `row` (a query head
// or a key head), rotated and rounded to bfloat16 as the rotation kernel rounds them; zeros
// when valid is false.  A lane's features ks * 32 + lg * 8 .. + 7 pair with the same lane's
// features of fragment ks + HD / 64.  With them, NS single values (columns scol, for lanes with
// singles_wanted): the new token's values travel with its key.
template <int HD, int NS>
__device__ inline void rotated_fragments(Frag (&out)[HD / 32], const DecodeSource& src, long row, int col0, bool valid, int lane,
                                         const int (&scol)[NS > 0 ? NS : 1], bool singles_wanted, float (&xs)[NS > 0 ? NS : 1]) {
  typedef float quad_t __attribute__((ext_vector_type(4)));
  const int lg = lane / 16;
  constexpr int HALF = HD / 64;       // fragments per half of the head
  int ocol[2 * HALF];
  float x[2 * HALF][8];
#pragma unroll
  for (int ks = 0; ks < HALF; ++ks) {
    ocol[ks] = col0 + ks * 32 + lg * 8;
    ocol[HALF + ks] = ocol[ks] + HD / 2;
  }
  source_gather<2 * HALF, NS>(src, row, ocol, valid, x, scol, singles_wanted, xs);
#pragma unroll
  for (int ks = 0; ks < HALF; ++ks) {
    const float (&a)[8] = x[ks];
    const float (&b)[8] = x[HALF + ks];
    float lo[8], hi[8];
    if (src.table) {
      const float* c = src.table + row * HD + ks * 32 + lg * 8;
      const quad_t c0 = *reinterpret_cast<const quad_t*>(c), c1 = *reinterpret_cast<const quad_t*>(c + 4);
      const quad_t s0 = *reinterpret_cast<const quad_t*>(c + HD / 2), s1 = *reinterpret_cast<const quad_t*>(c + HD / 2 + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) rope_pair(a[e], b[e], e < 4 ? c0[e] : c1[e - 4], e < 4 ? s0[e] : s1[e - 4], lo[e], hi[e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) { lo[e] = a[e]; hi[e] = b[e]; }
    }
    out[ks].q = make_uint4(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(lo[4], lo[5]), pack_bf16x2(lo[6], lo[7]));
    out[ks + HALF].q = make_uint4(pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]), pack_bf16x2(hi[4], hi[5]), pack_bf16x2(hi[6], hi[7]));
  }
}

// The new token's key (rotated) and value of kv head g into their slot of the cache.  The key
// is formed as a fragment: lanes 0, 16, 32, 48 hold its features lg * 8 .. + 7 of every 32;
// lanes 0..15 take the values d = db * 16 + lane.
template <int HD>
__device__ inline void store_new_kv(const DecodeSource& src, long row, int g, int pos, const int* __restrict__ bt, int table_width,
                                    int nkv, int page_size, long num_pages, int lane) {
  const int lr = lane % 16, lg = lane / 16;
  const int blk = pos / page_size, slot = pos % page_size;
  if (blk >= table_width) return;
  const long page = bt[blk];
  if (page < 0 || page >= num_pages) return;   // the host checks tables; never write outside the pool
  Frag key[HD / 32];
  int vcol[HD / 16];
  float vals[HD / 16];
#pragma unroll
  for (int db = 0; db < HD / 16; ++db) vcol[db] = src.v_col + g * HD + db * 16 + lr;
  rotated_fragments<HD, HD / 16>(key, src, row, src.k_col + g * HD, lr == 0, lane, vcol, lg == 0, vals);
  bf16_t* kd = src.k_cache + ((page * nkv + g) * page_size + slot) * HD;
  bf16_t* vd = src.v_cache + (page * nkv + g) * (long)page_size * HD + slot;
  if (lr == 0) {
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks) *reinterpret_cast<u32x4_t*>(kd + ks * 32 + lg * 8) = key[ks].n;
  }
  if (lg == 0) {
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) vd[(long)(db * 16 + lr) * page_size] = from_float<bf16_t>(vals[db]);
  }
}

template <int HD, bool FUSED>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 2 : 1))) void attention_decode_kernel(
    bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q, long q_stride, DecodeSource src,
    const bf16_t* k_cache, const bf16_t* v_cache,   // not restrict: the fused kernel stores into them
    const int* __restrict__ block_table,
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
  // this wave's keys: chunk `split` of the 32-key chunks between lo and p
  const int first_chunk = lo / 32, last_chunk = p / 32;
  const int chunks = last_chunk - first_chunk + 1;
  const int per = (chunks + splits - 1) / splits;
  const int c0 = first_chunk + split * per;
  const int c1 = min(last_chunk + 1, c0 + per);
  // The wave whose keys end at the new token writes that token into the cache first and waits
  // for the stores; after that it reads the token like any other key, in the same order of
  // arithmetic as a kernel that finds the cache written: the same bits.
  if constexpr (FUSED) {
    if (src.write_kv && c0 < c1 && c1 == last_chunk + 1) {
      store_new_kv<HD>(src, row, g, p, bt, table_width, nkv, page_size, num_pages, lane);
      __threadfence_block();
    }
  }
  attn_walk<HD, 1>(st, c0, c1, (lo + 31) / 32, (p + 1) / 32 - 1, k_cache, v_cache, bt, table_width, kv_len, nkv, g,
                   page_size, num_pages, scale * PI_LOG2E, lane, [&]() {
                     // while the first keys and values are on their way
                     if constexpr (!FUSED) {
                       attn_load_q(st, 0, q, q_stride, row, g * G + lr, valid, lane);
                     } else {
                       const int none[1] = {0};
                       float unused[1];
                       rotated_fragments<HD, 0>(st.q[0], src, row, src.q_col + (g * G + lr) * HD, valid, lane, none, false, unused);
                     }
                   });
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

// Merge the key ranges of one (request, head) by one wave: lane d owns features d, d + 64, ..
// Ranges are added in range order; an empty range (m = -inf) counts nothing.
template <int HD>
__device__ inline void combine_ranges(bf16_t* __restrict__ o, const float* base, int splits, int lane) {
  const int rec = HD + 4;
  constexpr int NF = (HD + 63) / 64;     // features per lane
  // lane s holds range s (splits <= 64): maxima, weights and the total in parallel
  const float ms = lane < splits ? base[lane * rec + HD] : -INFINITY;
  const float ls = lane < splits ? base[lane * rec + HD + 1] : 0.f;
  const float m_tot = wave_max(ms);
  const float w = range_weight(ms, m_tot);
  float l_tot = 0.f;
  float acc[NF];
#pragma unroll
  for (int i = 0; i < NF; ++i) acc[i] = 0.f;
  // ranges in order; eight loads in flight at a time
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float ov[8][NF], ws[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int s = s0 + u;
      ws[u] = __shfl(w, s < splits ? s : 0, 64);
      if (s >= splits) ws[u] = 0.f;
#pragma unroll
      for (int i = 0; i < NF; ++i) ov[u][i] = (s < splits && lane + i * 64 < HD) ? base[s * rec + lane + i * 64] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      l_tot = range_add(ws[u], __shfl(ls, (s0 + u < splits) ? s0 + u : 0, 64), l_tot);
#pragma unroll
      for (int i = 0; i < NF; ++i) acc[i] = range_add(ws[u], ov[u][i], acc[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < NF; ++i)
    if (lane + i * 64 < HD) o[lane + i * 64] = from_float<bf16_t>(range_finish(acc[i], l_tot));
}

// One wave per (request, head).
template <int HD>
__global__ __launch_bounds__(64) void attention_combine_kernel(bf16_t* __restrict__ out, long out_stride,
                                                               const int* __restrict__ q_start,
                                                               const int* __restrict__ req_ids,
                                                               const int* __restrict__ rows,
                                                               const float* __restrict__ part, int nh, int splits) {
  const int head = blockIdx.x;
  // where the result goes: the token row of request r (decode), or a listed row (cut tiles)
  const int r = req_ids ? req_ids[blockIdx.y] : (int)blockIdx.y;
  const long out_row = rows ? rows[blockIdx.y] : q_start[r];
  combine_ranges<HD>(out + out_row * out_stride + (long)head * HD, part + ((long)blockIdx.y * nh + head) * splits * (HD + 4),
                     splits, threadIdx.x);
}

// One wave per (row of `part`, head): rows are a launch's requests (results to the requests'
// token rows) or listed token rows.
static int launch_combine(void* out, long out_stride, const int* q_start, const int* req_ids, const int* rows, int Z,
                          const void* part, int nh, int hd, int splits, hipStream_t stream) {
  const dim3 grid(nh, Z), block(64);
#define GO(H) hipLaunchKernelGGL(attention_combine_kernel<H>, grid, block, 0, stream, (bf16_t*)out, out_stride, q_start, req_ids, rows, \
                                 (const float*)part, nh, splits)
  switch (hd) {
    case 16: GO(16); break;
    case 32: GO(32); break;
    case 48: GO(48); break;
    case 64: GO(64); break;
    case 80: GO(80); break;
    case 96: GO(96); break;
    case 112: GO(112); break;
    case 128: GO(128); break;
    case 144: GO(144); break;
    case 160: GO(160); break;
    case 176: GO(176); break;
    case 192: GO(192); break;
    case 208: GO(208); break;
    case 224: GO(224); break;
    case 240: GO(240); break;
    case 256: GO(256); break;
    default: return pi_fail("attention_combine: head_dim %d is not a multiple of 16 up to 256", hd);
  }
#undef GO
  return pi_check_launch("attention_combine");
}

// part: float32 [R * nh * splits * (hd + 4)], needed when splits > 1.
// req_ids: null (requests 0 .. R-1) or the R requests of the step that this launch serves; each
// has one query token, at row q_start[r], that sees kv_len[r] keys.
static int launch_decode(bool fused, const DecodeSource& src, void* out, long out_stride, const void* q, long q_stride,
                         const void* k_cache, const void* v_cache, const int* block_table, int table_width,
                         const int* q_start, const int* kv_len, const int* req_ids, int R, int nh, int nkv, int hd,
                         int page_size, float scale, int window, long num_pages, int splits, void* part, long part_elems,
                         bool merge, hipStream_t stream) {
  PI_REQUIRE(R > 0 && nh > 0 && nkv > 0 && nh % nkv == 0 && nh / nkv <= 16, "attention_decode: needs 1..16 heads per kv head, got %d / %d", nh, nkv);
  PI_REQUIRE(hd >= 16 && hd <= 256 && hd % 16 == 0, "attention_decode: head_dim %d is not a multiple of 16 up to 256", hd);
  PI_REQUIRE(!fused || hd == 64 || hd == 128, "attention_decode: the kernel that starts from the projection takes head_dim 64 or 128, not %d", hd);
  PI_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_decode: page size %d must be a multiple of 16", page_size);
  PI_REQUIRE(splits >= 1 && splits <= 64 && R <= 65535 && nkv <= 65535, "attention_decode: bad grid (%d ranges, %d requests, %d kv heads)", splits, R, nkv);
  PI_REQUIRE(out_stride % 4 == 0 && ((uintptr_t)out % 8 == 0), "attention_decode: out rows must be 8-byte aligned");
  if (!fused)
    PI_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0), "attention_decode: q rows must be 16-byte aligned");
  if (splits > 1)
    PI_REQUIRE(part && part_elems >= (long)R * nh * splits * (hd + 4), "attention_decode: workspace too small for %d ranges", splits);
  const dim3 grid(splits, nkv, R), block(64);
#define GO(H, F) hipLaunchKernelGGL((attention_decode_kernel<H, F>), grid, block, 0, stream, (bf16_t*)out, out_stride, (const bf16_t*)q, \
                                    q_stride, src, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width, q_start, \
                                    kv_len, req_ids, nh, nkv, page_size, scale, window, num_pages, (float*)part)
  if (fused) { if (hd == 64) GO(64, true); else GO(128, true); }
  else {
    switch (hd) {
      case 16: GO(16, false); break;
      case 32: GO(32, false); break;
      case 48: GO(48, false); break;
      case 64: GO(64, false); break;
      case 80: GO(80, false); break;
      case 96: GO(96, false); break;
      case 112: GO(112, false); break;
      case 128: GO(128, false); break;
      case 144: GO(144, false); break;
      case 160: GO(160, false); break;
      case 176: GO(176, false); break;
      case 192: GO(192, false); break;
      case 208: GO(208, false); break;
      case 224: GO(224, false); break;
      case 240: GO(240, false); break;
      default: GO(256, false); break;
    }
  }
#undef GO
  if (pi_check_launch("attention_decode")) return -1;
  // merge == false: the caller's next kernel merges the ranges itself (nothing is in `out` then)
  if (splits > 1 && merge) return launch_combine(out, out_stride, q_start, req_ids, nullptr, R, part, nh, hd, splits, stream);
  return 0;
}

extern "C" int pi_attention_decode(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                   const void* v_cache, const int* block_table, int table_width, const int* q_start,
                                   const int* kv_len, const int* req_ids, int R, int nh, int nkv, int hd, int page_size,
                                   float scale, int window, long num_pages, int splits, void* part, long part_elems,
                                   hipStream_t stream) {
  return launch_decode(false, DecodeSource{}, out, out_stride, q, q_stride, k_cache, v_cache, block_table, table_width, q_start,
                       kv_len, req_ids, R, nh, nkv, hd, page_size, scale, window, num_pages, splits, part, part_elems, true, stream);
}

// The same for a step of single tokens only (T == R tokens, request r at row q_start[r]),
// straight from the q|k|v projection: `qkv` bfloat16 [T, qkv_stride] or `qkv_part` float32
// [qkv_splits, T, ncols] (one of the two), columns [q heads | k heads | v heads].  `table`:
// float32 [T, hd] cosines and sines of the tokens' angles (rotation over the whole head, halves
// paired), or null for no rotation.  write_kv: store the tokens' keys and values into the cache.
// merge == 0 (with splits > 1): leave the key ranges in `part` ([R, nh, splits, hd + 4]: output
// not yet normalised, maximum, sum of weights) for a consumer that merges them; `out` stays untouched.
extern "C" int pi_attention_decode_fused(void* out, long out_stride, const void* qkv, long qkv_stride, const void* qkv_part,
                                         int qkv_splits, int ncols, int T, const float* table, int write_kv, void* k_cache,
                                         void* v_cache, const int* block_table, int table_width, const int* q_start,
                                         const int* kv_len, int R, int nh, int nkv, int hd, int page_size, float scale,
                                         int window, long num_pages, int splits, void* part, long part_elems,
                                         int merge, hipStream_t stream) {
  PI_REQUIRE((qkv != nullptr) != (qkv_part != nullptr), "attention_decode_fused: give the projection as a tensor or as pieces");
  PI_REQUIRE(T == R, "attention_decode_fused: %d tokens for %d requests (single tokens only)", T, R);
  PI_REQUIRE(nh > 0 && nkv > 0 && hd > 0, "attention_decode_fused: bad sizes");
  const int need = (nh + (write_kv ? 2 * nkv : 0)) * hd;
  if (qkv) {
    PI_REQUIRE(qkv_stride >= need, "attention_decode_fused: projection rows of %ld hold no %d columns", qkv_stride, need);
    PI_REQUIRE(qkv_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0, "attention_decode_fused: projection rows must be 16-byte aligned");
  } else {
    PI_REQUIRE(qkv_splits >= 1 && ncols >= need, "attention_decode_fused: pieces [%d x %d columns] hold no %d columns", qkv_splits, ncols, need);
    PI_REQUIRE(ncols % 4 == 0 && (uintptr_t)qkv_part % 16 == 0, "attention_decode_fused: rows of the pieces must be 16-byte aligned");
  }
  PI_REQUIRE(table == nullptr || (uintptr_t)table % 16 == 0, "attention_decode_fused: the cos / sin table must be 16-byte aligned");
  DecodeSource src{};
  src.qkv = (const bf16_t*)qkv;
  src.qkv_stride = qkv_stride;
  src.part = (const float*)qkv_part;
  src.splits = qkv_splits;
  src.part_stride = (long)T * ncols;
  src.ncols = ncols;
  src.q_col = 0;
  src.k_col = nh * hd;
  src.v_col = (nh + nkv) * hd;
  src.table = table;
  src.write_kv = write_kv;
  src.k_cache = (bf16_t*)k_cache;
  src.v_cache = (bf16_t*)v_cache;
  return launch_decode(true, src, out, out_stride, nullptr, 0, k_cache, v_cache, block_table, table_width, q_start, kv_len,
                       nullptr, R, nh, nkv, hd, page_size, scale, window, num_pages, splits, part, part_elems, merge != 0, stream);
}

// Merge partial results that the tile kernel wrote for `Z` tokens whose tiles' keys were cut in
// `cuts` shares: part [Z, nh, cuts, hd + 4]; token z's result goes to row rows[z] of out.
extern "C" int pi_attention_combine_rows(void* out, long out_stride, const int* rows, int Z, const void* part, int nh, int hd,
                                         int cuts, hipStream_t stream) {
  PI_REQUIRE(Z > 0 && Z <= 65535 && nh > 0 && cuts >= 2 && cuts <= 64 && rows && part, "attention_combine_rows: bad arguments (%d tokens, %d heads, %d cuts)", Z, nh, cuts);
  return launch_combine(out, out_stride, nullptr, nullptr, rows, Z, part, nh, hd, cuts, stream);
}

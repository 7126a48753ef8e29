// The wave-level core of the matrix-core attention kernels (bfloat16, gfx950).
//
// A wave owns CB blocks of 16 query columns; a column is one (token, head) pair, all heads
// of one kv group, so keys and values are read once for the whole group.  Keys are visited
// 32 at a time (two tiles of 16).  Everything is computed transposed so that no value ever
// leaves its lane between the two products:
//   S^T[key, col] = K[key, :] . Q[col, :]      row operand: K tile,  column operand: Q
//   O^T[d,  col] += V^T[d, key] . P^T[key, col] row operand: V^T,     column operand: P^T
// The S^T result of a lane (4 keys of tile 0 and 4 keys of tile 1, one column) is, after the
// softmax, exactly the column-operand fragment of the second product, given that the row
// operand V^T is loaded with the same key assignment: lane group g holds keys 4g..4g+3 of
// tile 0 and of tile 1.  Values are cached transposed ([.., head_dim, slot]) so these are two
// 8-byte loads.  Running maximum, running sum and the rescaling factor belong to a column,
// i.e. to lane % 16, replicated over the four lane groups.
//
// Scores, softmax and both accumulations are float32.  The exponential is taken in base 2
// (scores are scaled by scale * log2(e) once, then v_exp_f32), so the running maximum is kept
// in that scale too.  P is rounded to bfloat16 for the second product; the sum of P is taken
// before rounding.
//
// The keys and values of a chunk are loaded into registers by attn_load and consumed by
// attn_compute, so a caller can have the next chunk's loads in flight while it computes.
#pragma once
#include "mfma.h"

#define PI_LOG2E 1.4426950408889634f

template <int HD, int CB>
struct AttnState {
  Frag q[CB][HD / 32];
  f32x4_t o[HD / 16][CB];
  float m[CB], l[CB];   // running maximum (base-2 scale) and running sum per column
  int pos[CB];          // last visible key of the column
  int lo[CB];           // first visible key of the column
};

template <int HD>
struct KVChunk {
  Frag k[2][HD / 32];   // key tiles: rows key0 + lane % 16
  Frag v[HD / 16];      // value rows d = db*16 + lane % 16; keys (lane/16)*4..+3 of both tiles
  bool have[2];
};

template <int HD, int CB>
__device__ inline void attn_init(AttnState<HD, CB>& st) {
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    st.m[c] = -INFINITY;
    st.l[c] = 0.f;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) st.o[db][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
}

// Issue the loads of the 32 keys starting at k0 (a multiple of 32).  `bt` is the request's
// block-table row, `kv_len` the number of keys its pages hold; page_size is a multiple of 16.
// A tile whose page is missing (beyond the length, or given back by a window) loads zeros.
// Page ids of a request, 64 consecutive block-table entries at a time in one register per lane
// (lane i holds block base + i), read out with v_readlane: the loads of a chunk then depend on
// no other load, and the table is read once per 64 pages instead of once per tile.
struct PageCache {
  int base = -(1 << 30);
  int ids = -1;
  __device__ inline int get(int blk, const int* __restrict__ bt, int table_width, int lane) {
    if (blk < base || blk >= base + 64) {          // uniform: blk and base are the same in every lane
      base = blk;
      const int b = blk + lane;
      ids = b < table_width ? bt[b] : -1;
    }
    return __builtin_amdgcn_readlane(ids, blk - base);
  }
};

// The loads are unconditional (a missing tile reads page 0 and is zeroed by attn_compute), so
// that the compiler can count them and wait for one chunk while the next is still in flight.
template <int HD>
__device__ inline void attn_load(KVChunk<HD>& kv, int k0, const bf16_t* __restrict__ k_cache,
                                 const bf16_t* __restrict__ v_cache, PageCache& pages, const int* __restrict__ bt,
                                 int table_width, int kv_len, int nkv, int g, int page_size, long num_pages, int lane) {
  const int lr = lane % 16, lg = lane / 16;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key0 = k0 + t * 16;
    const int page = key0 < kv_len ? pages.get(key0 / page_size, bt, table_width, lane) : -1;
    kv.have[t] = page >= 0 && page < num_pages;
    const long pg = kv.have[t] ? page : 0;
    const int slot = key0 % page_size;
    const bf16_t* kp = k_cache + ((pg * nkv + g) * page_size + slot + lr) * HD + lg * 8;
    const bf16_t* vp = v_cache + (pg * nkv + g) * (long)page_size * HD + slot + (long)lr * page_size + lg * 4;
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks) kv.k[t][ks] = load_frag(kp + ks * 32);
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) kv.v[db].d[t] = *reinterpret_cast<const uint2*>(vp + (long)db * 16 * page_size);
  }
}

// Fold one loaded chunk into the state.  `masked`: some key of the chunk may be invisible to
// some column (causal edge, window edge, missing tile); otherwise the per-key tests are skipped.
template <int HD, int CB>
__device__ inline void attn_compute(AttnState<HD, CB>& st, const KVChunk<HD>& kv, int k0, float scale_log2, bool masked,
                                    int lane) {
  const int lg = lane / 16;
  f32x4_t s[2][CB];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < HD / 32; ++ks) acc = mfma16(kv.k[t][ks], st.q[c][ks], acc);
      s[t][c] = acc;
    }

#pragma unroll
  for (int c = 0; c < CB; ++c) {
    float p[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = s[t][c][i] * scale_log2;
        if (masked) {
          const int key = k0 + t * 16 + lg * 4 + i;
          if (!(kv.have[t] && key <= st.pos[c] && key >= st.lo[c])) v = -INFINITY;
        }
        p[t][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = column_max(mx);
    const float m_new = fmaxf(st.m[c], mx);
    float alpha = 1.f, sum = 0.f;
    if (m_new == -INFINITY) {          // nothing visible yet in this column
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) p[t][i] = 0.f;
    } else {
      alpha = __builtin_amdgcn_exp2f(st.m[c] - m_new);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[t][i] = __builtin_amdgcn_exp2f(p[t][i] - m_new);
          sum += p[t][i];
        }
    }
    sum = column_sum(sum);
    st.l[c] = st.l[c] * alpha + sum;
    st.m[c] = m_new;
    Frag pb;
    pb.q.x = pack_bf16x2(p[0][0], p[0][1]);
    pb.q.y = pack_bf16x2(p[0][2], p[0][3]);
    pb.q.z = pack_bf16x2(p[1][0], p[1][1]);
    pb.q.w = pack_bf16x2(p[1][2], p[1][3]);
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
      f32x4_t o = st.o[db][c];
      o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
      Frag va = kv.v[db];
      if (masked) {   // a missing tile was read from page 0: its values must not meet even a zero weight
        if (!kv.have[0]) va.d[0] = make_uint2(0u, 0u);
        if (!kv.have[1]) va.d[1] = make_uint2(0u, 0u);
      }
      st.o[db][c] = mfma16(va, pb, o);
    }
  }
}

// Walk chunks c0 .. c1-1 (32 keys each) with the next chunk's loads in flight during the
// current chunk's arithmetic.  Chunks from `first_unmasked` up to `last_unmasked` (inclusive)
// are known to be fully visible to every column.
template <int HD, int CB>
__device__ inline void attn_walk(AttnState<HD, CB>& st, int c0, int c1, int first_unmasked, int last_unmasked,
                                 const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                 const int* __restrict__ bt, int table_width, int kv_len, int nkv, int g, int page_size,
                                 long num_pages, float scale_log2, int lane) {
  if (c0 >= c1) return;
  KVChunk<HD> a, b;
  PageCache pages;
  // the chunk after the last one is loaded too (its tiles lie beyond the keys and read page 0):
  // one load per compute, no branch between them
  attn_load<HD>(a, c0 * 32, k_cache, v_cache, pages, bt, table_width, kv_len, nkv, g, page_size, num_pages, lane);
  int c = c0;
  while (true) {
    attn_load<HD>(b, (c + 1 < c1 ? c + 1 : c) * 32, k_cache, v_cache, pages, bt, table_width, kv_len, nkv, g, page_size, num_pages, lane);
    attn_compute<HD, CB>(st, a, c * 32, scale_log2, c < first_unmasked || c > last_unmasked, lane);
    if (++c >= c1) break;
    attn_load<HD>(a, (c + 1 < c1 ? c + 1 : c) * 32, k_cache, v_cache, pages, bt, table_width, kv_len, nkv, g, page_size, num_pages, lane);
    attn_compute<HD, CB>(st, b, c * 32, scale_log2, c < first_unmasked || c > last_unmasked, lane);
    if (++c >= c1) break;
  }
}

// Load the query fragment of column block c: the lane's column is (token row `row`, head `head`),
// or padding (zeros) when valid is false.
template <int HD, int CB>
__device__ inline void attn_load_q(AttnState<HD, CB>& st, int c, const bf16_t* __restrict__ q, long q_stride, long row,
                                   int head, bool valid, int lane) {
  const int lg = lane / 16;
#pragma unroll
  for (int ks = 0; ks < HD / 32; ++ks)
    st.q[c][ks] = valid ? load_frag(q + row * q_stride + (long)head * HD + ks * 32 + lg * 8) : zero_frag();
}

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
// Scores, softmax and both accumulations are float32; P is rounded to bfloat16 for the
// second product, the sum of P is taken before rounding.
#pragma once
#include "mfma.h"

template <int HD, int CB>
struct AttnState {
  Frag q[CB][HD / 32];
  f32x4_t o[HD / 16][CB];
  float m[CB], l[CB];
  int pos[CB];   // last visible key of the column; -1: the column is padding
  int lo[CB];    // first visible key of the column
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

// One chunk of 32 keys starting at k0 (a multiple of 32).  `bt` is the request's block-table
// row, `kv_len` the number of keys its pages hold.  page_size is a multiple of 16.
template <int HD, int CB>
__device__ inline void attn_chunk(AttnState<HD, CB>& st, int k0, const bf16_t* __restrict__ k_cache,
                                  const bf16_t* __restrict__ v_cache, const int* __restrict__ bt, int table_width,
                                  int kv_len, int nkv, int g, int page_size, long num_pages, float scale, int lane) {
  const int lr = lane % 16, lg = lane / 16;
  long kbase[2], vbase[2];
  bool have[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key0 = k0 + t * 16;
    const int blk = key0 / page_size;
    long page = -1;
    if (key0 < kv_len && blk < table_width) page = bt[blk];
    have[t] = page >= 0 && page < num_pages;
    const long pg = have[t] ? page : 0;
    const int slot = key0 % page_size;
    kbase[t] = ((pg * nkv + g) * page_size + slot) * HD;
    vbase[t] = (pg * nkv + g) * (long)page_size * HD + slot;
  }

  // S^T = K . Q^T
  f32x4_t s[2][CB];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    Frag a[HD / 32];
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks)
      a[ks] = have[t] ? load_frag(k_cache + kbase[t] + (long)lr * HD + ks * 32 + lg * 8) : zero_frag();
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < HD / 32; ++ks) acc = mfma16(a[ks], st.q[c][ks], acc);
      s[t][c] = acc;
    }
  }

  // V^T fragments: rows d = db*16 + lr, keys lg*4..lg*4+3 of each tile
  Frag va[HD / 16];
#pragma unroll
  for (int db = 0; db < HD / 16; ++db) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (have[t])
        va[db].d[t] = *reinterpret_cast<const uint2*>(v_cache + vbase[t] + (long)(db * 16 + lr) * page_size + lg * 4);
      else
        va[db].d[t] = make_uint2(0u, 0u);
    }
  }

  // softmax update per column, then O^T += V^T . P^T
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    float p[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + t * 16 + lg * 4 + i;
        const bool visible = have[t] && key <= st.pos[c] && key >= st.lo[c];
        p[t][i] = visible ? s[t][c][i] * scale : -INFINITY;
        mx = fmaxf(mx, p[t][i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(st.m[c], mx);
    float alpha = 1.f, sum = 0.f;
    if (m_new == -INFINITY) {          // nothing visible yet in this column
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) p[t][i] = 0.f;
    } else {
      alpha = expf(st.m[c] - m_new);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[t][i] = expf(p[t][i] - m_new);
          sum += p[t][i];
        }
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
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
      st.o[db][c] = mfma16(va[db], pb, o);
    }
  }
}

// Load the query fragment of column block c: the lane's column is (token row `row`, head `head`),
// or padding when valid is false.
template <int HD, int CB>
__device__ inline void attn_load_q(AttnState<HD, CB>& st, int c, const bf16_t* __restrict__ q, long q_stride, long row,
                                   int head, bool valid, int lane) {
  const int lg = lane / 16;
#pragma unroll
  for (int ks = 0; ks < HD / 32; ++ks)
    st.q[c][ks] = valid ? load_frag(q + row * q_stride + (long)head * HD + ks * 32 + lg * 8) : zero_frag();
}

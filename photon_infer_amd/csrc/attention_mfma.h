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
// Scores, softmax and both accumulations are float32.  The exponential is taken in base 2:
// a weight is 2^((score - reference) * scale * log2(e)), one fused multiply-add and v_exp_f32.
// P is rounded to bfloat16 for the second product; the sum of P is a matrix product too (value
// rows of ones), so it is the sum of the weights as rounded.
//
// The keys and values of a chunk are loaded into registers by attn_load and consumed by
// attn_compute, so a caller can have the next chunk's loads in flight while it computes.
#pragma once
#include "addressing.h"
#include "mfma.h"

#define PI_LOG2E 1.4426950408889634f

// A head of HD features (a multiple of 16) is contracted in KS fragments of 32; when HD is no
// multiple of 32 the upper half of the last fragment (the lanes of groups 2 and 3) is zero in
// the queries and in the keys.
template <int HD>
struct HeadFrags {
  static constexpr int KS = (HD + 31) / 32;
  __device__ static inline bool holds(int ks, int lane) { return addressing::kv_lane_holds(HD, ks, lane); }   // false only in a half fragment
};

template <int HD, int CB>
struct AttnState {
  Frag q[CB][HeadFrags<HD>::KS];
  f32x4_t o[HD / 16][CB];
  float m[CB];          // reference score of the column (raw units, see attn_compute)
  f32x4_t ls[CB];       // the column's sum of weights, four times over (see weight_sum)
  float l[CB];          // the same as a scalar, set by attn_finish
  int pos[CB];          // last visible key of the column
  int lo[CB];           // first visible key of the column
};

template <int HD>
struct KVChunk {
  Frag k[2][HeadFrags<HD>::KS];   // key tiles: rows key0 + lane % 16
  Frag v[HD / 16];      // value rows d = db*16 + lane % 16; keys (lane/16)*4..+3 of both tiles
  bool have[2];
  __device__ inline Frag key(int t, int ks) const { return k[t][ks]; }
  __device__ inline Frag val(int db) const { return v[db]; }
};

// The same chunk lying in LDS in operand order ([fragment][lane], keys first): a fragment is
// read when the arithmetic wants it, so that a chunk never occupies registers as a whole.
template <int HD>
struct StagedChunk {
  const u32x4_t* from;  // this lane's first fragment
  bool have[2];
  __device__ inline Frag key(int t, int ks) const { Frag f; f.n = from[(t * HeadFrags<HD>::KS + ks) * 64]; return f; }
  __device__ inline Frag val(int db) const { Frag f; f.n = from[(2 * HeadFrags<HD>::KS + db) * 64]; return f; }
};

template <int HD, int CB>
__device__ inline void attn_init(AttnState<HD, CB>& st) {
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    st.m[c] = -INFINITY;
    st.l[c] = 0.f;
    st.ls[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) st.o[db][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
}

// The sum of a column's weights is left to the matrix unit: a product with sixteen value rows
// of ones adds the 32 weights of a chunk, exactly as rounded for the product with the values,
// and gives every lane of the column the whole sum.  The vector unit, which the weights keep
// busy, is spared eight additions per column and chunk and the exchange between lanes.
__device__ inline f32x4_t weight_sum(const Frag& weights, f32x4_t acc) {
  Frag ones;
  ones.n = u32x4_t{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  return mfma16(ones, weights, acc);
}

// After the last chunk.
template <int HD, int CB>
__device__ inline void attn_finish(AttnState<HD, CB>& st) {
#pragma unroll
  for (int c = 0; c < CB; ++c) st.l[c] = st.ls[c][0];
}

// Where the two key tiles of a chunk lie: page id (-1: none) and first slot in the page.  The
// same in every lane, so they live in scalar registers and are fetched by scalar loads, which
// the vector memory counter does not see: a table lookup never makes a wave wait for the keys
// and values that are still in flight.
struct ChunkPages {
  int page[2];
  int slot[2];
};

// Walks a request's block-table row tile by tile (16 keys; page_size is a multiple of 16).
struct PageCursor {
  typedef const int __attribute__((address_space(4)))* ScalarIntPtr;   // constant address space: scalar loads
  ScalarIntPtr bt;    // block-table row, uniform
  int table_width, kv_len, page_size;
  int key, blk, slot; // next tile
  __device__ inline void start(const int* row, int width, int len, int psize, int key0) {
    const uint64_t v = reinterpret_cast<uint64_t>(row);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    bt = (ScalarIntPtr)((static_cast<uint64_t>(hi) << 32) | lo);
    table_width = __builtin_amdgcn_readfirstlane(width);
    kv_len = __builtin_amdgcn_readfirstlane(len);
    page_size = __builtin_amdgcn_readfirstlane(psize);
    key = __builtin_amdgcn_readfirstlane(key0);
    blk = __builtin_amdgcn_readfirstlane(key0 / psize);
    slot = key - blk * page_size;
  }
  // A tile beyond the keys or beyond the table has no page.
  __device__ inline ChunkPages next() {
    ChunkPages cp;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const bool ok = key < kv_len && blk < table_width;
      const int id = bt[ok ? blk : 0];
      cp.page[t] = ok ? id : -1;
      cp.slot[t] = slot;
      key += 16;
      slot += 16;
      if (slot >= page_size) { slot = 0; ++blk; }
    }
    return cp;
  }
};

// What a lane adds to a tile's base address: fixed for a whole walk (bytes, 32 bits).
template <int HD>
struct KVLaneOffsets {
  uint32_t k;              // key row lane % 16, features (lane / 16) * 8 ..
  uint32_t k0;             // the row's first features (what a lane without features of its own reads)
  bool tail;               // the lane holds features of the last fragment (always, unless HD % 32 == 16)
  uint32_t v[HD / 16];     // value row db * 16 + lane % 16, keys (lane / 16) * 4 ..
  __device__ inline void set(int page_size, int lane) {
    k = addressing::kv_key_lane(lane, HD);
    k0 = addressing::kv_key_lane_first(lane, HD);
    tail = HeadFrags<HD>::holds(HeadFrags<HD>::KS - 1, lane);
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) v[db] = addressing::kv_value_lane(lane, db, page_size);
  }
};

// Issue the loads of a chunk of 32 keys.  The loads are unconditional (a missing tile reads
// page 0 and is zeroed by attn_compute), so that the compiler can count them and wait for one
// chunk while the next is still in flight.  A tile's base address is the same in every lane
// (scalar arithmetic); the lane's part is a 32-bit offset.
template <int HD>
__device__ inline void attn_load(KVChunk<HD>& kv, const ChunkPages& cp, const bf16_t* __restrict__ k_cache,
                                 const bf16_t* __restrict__ v_cache, const KVLaneOffsets<HD>& off, int nkv, int g,
                                 int page_size, int num_pages) {
  const long page_elems = addressing::kv_page_elems(nkv, page_size, HD);
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    kv.have[t] = addressing::kv_page_there(cp.page[t], num_pages);
    const long pg = addressing::kv_page_or_first(cp.page[t], num_pages);
    const char* kp = reinterpret_cast<const char*>(k_cache + addressing::kv_key_tile(pg, page_elems, g, page_size, cp.slot[t], HD));
    const char* vp = reinterpret_cast<const char*>(v_cache + addressing::kv_value_tile(pg, page_elems, g, page_size, cp.slot[t], HD));
#pragma unroll
    for (int ks = 0; ks < HeadFrags<HD>::KS; ++ks) {
      // a half fragment's upper lanes read their row's first features again and count as zero
      const bool held = HD % 32 == 0 || ks + 1 < HeadFrags<HD>::KS || off.tail;
      kv.k[t][ks].n = *reinterpret_cast<const u32x4_t*>(kp + (held ? off.k + ks * 64 : off.k0));
      if (!held) kv.k[t][ks].n = u32x4_t{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) kv.v[db].d[t] = *reinterpret_cast<const uint2*>(vp + off.v[db]);
  }
}

// How far (in powers of two) a column's scores may rise above its reference before the
// reference is moved and the column rescaled.  Weights then stay below 2^8, sums far inside
// float32; the reference cancels in the final division, so the result is the same softmax.
#define PI_RESCALE_SLACK 8.0f

// Fold one loaded chunk into the state.  MASKED: some key of the chunk may be invisible to
// some column (causal edge, window edge, missing tile); otherwise the per-key tests are left out.
// st.m is a column's reference score (raw, before the softmax scale): at least the largest
// score seen minus the slack.  Moving it costs a pass over the accumulators, so it only moves
// when some column of the wave needs it.
template <int HD, int CB, bool MASKED, class KV>
__device__ inline void attn_compute(AttnState<HD, CB>& st, const KV& kv, int k0, float scale_log2, int lane) {
  const int lg = lane / 16;
  f32x4_t s[2][CB];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < HeadFrags<HD>::KS; ++ks) acc = mfma16(kv.key(t, ks), st.q[c][ks], acc);
      s[t][c] = acc;
    }
  const float slack = PI_RESCALE_SLACK / scale_log2;

#pragma unroll
  for (int c = 0; c < CB; ++c) {
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (MASKED) {
          const int key = k0 + t * 16 + lg * 4 + i;
          if (!(kv.have[t] && key <= st.pos[c] && key >= st.lo[c])) s[t][c][i] = -INFINITY;
        }
        mx = fmaxf(mx, s[t][c][i]);
      }
    // weights 2^((score - reference) * scale), summed and folded into the accumulators; a column
    // that has seen nothing yet has only -inf scores
    auto fold = [&](float m_ref) {
      float mc = m_ref * scale_log2;
      if (MASKED) mc = (m_ref == -INFINITY) ? 0.f : mc;
      float p[2][4];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) p[t][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][c][i], scale_log2, -mc));
      Frag pb;
      pb.q.x = pack_bf16x2(p[0][0], p[0][1]);
      pb.q.y = pack_bf16x2(p[0][2], p[0][3]);
      pb.q.z = pack_bf16x2(p[1][0], p[1][1]);
      pb.q.w = pack_bf16x2(p[1][2], p[1][3]);
      st.ls[c] = weight_sum(pb, st.ls[c]);
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) {
        Frag va = kv.val(db);
        if (MASKED) {   // a missing tile was read from page 0: its values must not meet even a zero weight
          if (!kv.have[0]) va.d[0] = make_uint2(0u, 0u);
          if (!kv.have[1]) va.d[1] = make_uint2(0u, 0u);
        }
        st.o[db][c] = mfma16(va, pb, st.o[db][c]);
      }
    };
    // the cheap test first: does any lane hold a score that far above its column's reference?
    const float m_ref = st.m[c];
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m_ref + slack) != 0, 0)) {   // also at the first visible key: m_ref is -inf then
      mx = column_max(mx);
      const bool move = mx > m_ref + slack;
      const float alpha = move ? __builtin_amdgcn_exp2f((m_ref - mx) * scale_log2) : 1.f;
      const float m_new = move ? mx : m_ref;
      st.m[c] = m_new;
      st.ls[c][0] *= alpha; st.ls[c][1] *= alpha; st.ls[c][2] *= alpha; st.ls[c][3] *= alpha;
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) {
        st.o[db][c][0] *= alpha; st.o[db][c][1] *= alpha; st.o[db][c][2] *= alpha; st.o[db][c][3] *= alpha;
      }
      // The fold is written out on both paths, and the marker keeps the compiler from joining
      // them again: joined, the accumulators of the common path would be copied to where the
      // rescaled ones lie, 16 registers per column and chunk.
      fold(m_new);
      asm volatile("" ::: "memory");
    } else {
      fold(m_ref);
    }
  }
}

// Fold NJ staged chunks that every column sees whole (no per-key tests, every page there).
// `from`: this lane's first fragment of the first chunk in LDS (StagedChunk's order);
// `chunk_stride`: 16-byte units from one chunk to the next.  All scores of the group are
// formed first, then one test decides whether any column's reference has to move, then the
// weights and the accumulation run as straight-line code: matrix and vector instructions of
// different chunks and columns can overlap, and the test costs one branch per group.
template <int HD, int CB, int NJ>
__device__ inline void attn_compute_plain(AttnState<HD, CB>& st, const u32x4_t* from, int chunk_stride, float scale_log2) {
  // The key fragments of a chunk are read from LDS while the products of the chunk before it
  // run; the scheduler is told so, or it reads each fragment right before its use to save
  // registers and the wave waits for LDS sixteen times per group.
  constexpr int KS = HeadFrags<HD>::KS;
  constexpr int KF = 2 * KS;
  Frag kf[2][KF];
  f32x4_t s[NJ][2][CB];
#pragma unroll
  for (int f = 0; f < KF; ++f) kf[0][f].n = from[f * 64];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    if (j + 1 < NJ) {
#pragma unroll
      for (int f = 0; f < KF; ++f) kf[(j + 1) & 1][f].n = from[(j + 1) * chunk_stride + f * 64];
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int c = 0; c < CB; ++c) s[j][t][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int c = 0; c < CB; ++c) s[j][t][c] = mfma16(kf[j & 1][t * KS + ks], st.q[c][ks], s[j][t][c]);
    }
    if (j + 1 < NJ) __builtin_amdgcn_sched_group_barrier(0x100, KF, 0);   // LDS reads of the next chunk
    __builtin_amdgcn_sched_group_barrier(0x008, KF * CB, 0);               // this chunk's products
  }
  const float slack = PI_RESCALE_SLACK / scale_log2;
  float mx[CB];
  bool rise = false;
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    mx[c] = -INFINITY;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx[c] = fmaxf(mx[c], s[j][t][c][i]);
    rise = rise || mx[c] > st.m[c] + slack;
  }
  auto fold = [&]() {
    float mc[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) mc[c] = st.m[c] * scale_log2;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      Frag va[HD / 16];
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) va[db].n = from[j * chunk_stride + (KF + db) * 64];
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        float p[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) p[t][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][t][c][i], scale_log2, -mc[c]));
        Frag pb;
        pb.q.x = pack_bf16x2(p[0][0], p[0][1]);
        pb.q.y = pack_bf16x2(p[0][2], p[0][3]);
        pb.q.z = pack_bf16x2(p[1][0], p[1][1]);
        pb.q.w = pack_bf16x2(p[1][2], p[1][3]);
      st.ls[c] = weight_sum(pb, st.ls[c]);
#pragma unroll
        for (int db = 0; db < HD / 16; ++db) st.o[db][c] = mfma16(va[db], pb, st.o[db][c]);
      }
    }
  };
  if (__builtin_expect(__builtin_amdgcn_ballot_w64(rise) != 0, 0)) {   // also at the first keys: the references are -inf then
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const float top = column_max(mx[c]);
      const bool move = top > st.m[c] + slack;
      const float alpha = move ? __builtin_amdgcn_exp2f((st.m[c] - top) * scale_log2) : 1.f;
      st.m[c] = move ? top : st.m[c];
      st.ls[c][0] *= alpha; st.ls[c][1] *= alpha; st.ls[c][2] *= alpha; st.ls[c][3] *= alpha;
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) {
        st.o[db][c][0] *= alpha; st.o[db][c][1] *= alpha; st.o[db][c][2] *= alpha; st.o[db][c][3] *= alpha;
      }
    }
    fold();                          // written out on both paths, see attn_compute
    asm volatile("" ::: "memory");
  } else {
    fold();
  }
}

template <int HD, int CB, class KV>
__device__ inline void attn_compute(AttnState<HD, CB>& st, const KV& kv, int k0, float scale_log2, bool masked, int lane) {
  if (masked) attn_compute<HD, CB, true, KV>(st, kv, k0, scale_log2, lane);
  else attn_compute<HD, CB, false, KV>(st, kv, k0, scale_log2, lane);
}

// Walk chunks c0 .. c1-1 (32 keys each) with the next chunk's loads in flight during the
// current chunk's arithmetic.  Chunks from `first_unmasked` up to `last_unmasked` (inclusive)
// are known to be fully visible to every column.
// `meanwhile` is called once the first chunk's loads are on their way (also when the range is
// empty): work that the walk needs but the loads do not, such as fetching the queries.
template <int HD, int CB, class Meanwhile>
__device__ inline void attn_walk(AttnState<HD, CB>& st, int c0, int c1, int first_unmasked, int last_unmasked,
                                 const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                 const int* __restrict__ bt, int table_width, int kv_len, int nkv, int g, int page_size,
                                 long num_pages_l, float scale_log2, int lane, Meanwhile&& meanwhile) {
  // the range is the same in every lane; saying so keeps the loop's branches scalar, and a
  // divergent break would make the compiler wait for every load at the loop's head
  c0 = __builtin_amdgcn_readfirstlane(c0);
  c1 = __builtin_amdgcn_readfirstlane(c1);
  first_unmasked = __builtin_amdgcn_readfirstlane(first_unmasked);
  last_unmasked = __builtin_amdgcn_readfirstlane(last_unmasked);
  if (c0 >= c1) {
    meanwhile();
    return;
  }
  KVChunk<HD> a, b;
  KVLaneOffsets<HD> off;
  off.set(page_size, lane);
  const int num_pages = (int)(num_pages_l < 0x7fffffffL ? num_pages_l : 0x7fffffffL);
  PageCursor cur;
  cur.start(bt, table_width, kv_len, page_size, c0 * 32);
  // Page ids run two chunks ahead, keys and values one chunk ahead of the arithmetic.  Two
  // chunks per turn with fixed roles for the two buffers and no way out of the loop between
  // them: the loads of one buffer are then always the youngest in flight when the other is
  // consumed, which lets the compiler wait by count.  Up to two chunks beyond the range are
  // loaded and never used.
  ChunkPages pa = cur.next(), pb = cur.next();
  attn_load<HD>(a, pa, k_cache, v_cache, off, nkv, g, page_size, num_pages);
  meanwhile();
  for (int c = c0; c < c1; c += 2) {
    pa = cur.next();
    attn_load<HD>(b, pb, k_cache, v_cache, off, nkv, g, page_size, num_pages);
    attn_compute<HD, CB>(st, a, c * 32, scale_log2, c < first_unmasked || c > last_unmasked, lane);
    pb = cur.next();
    attn_load<HD>(a, pa, k_cache, v_cache, off, nkv, g, page_size, num_pages);
    if (c + 1 < c1) attn_compute<HD, CB>(st, b, (c + 1) * 32, scale_log2, c + 1 < first_unmasked || c + 1 > last_unmasked, lane);
  }
}

// Load the query fragment of column block c: the lane's column is (token row `row`, head `head`),
// or padding (zeros) when valid is false.
template <int HD, int CB>
__device__ inline void attn_load_q(AttnState<HD, CB>& st, int c, const bf16_t* __restrict__ q, long q_stride, long row,
                                   int head, bool valid, int lane) {
  const int lg = lane / 16;
#pragma unroll
  for (int ks = 0; ks < HeadFrags<HD>::KS; ++ks)
    st.q[c][ks].n = (valid && HeadFrags<HD>::holds(ks, lane))
                        ? *reinterpret_cast<const u32x4_t*>(q + row * q_stride + (long)head * HD + ks * 32 + lg * 8)
                        : u32x4_t{0u, 0u, 0u, 0u};
}

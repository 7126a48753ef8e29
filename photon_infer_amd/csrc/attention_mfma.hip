// Causal attention of prompt portions (and whatever else shares their batch) over the paged
// cache, bfloat16 on the matrix cores.
//
// The step's tokens are cut into tiles of TQ consecutive tokens of one request (work list made
// on the host).  A block of four waves handles one (tile, kv head) at a time: its 4 * CB * 16
// query columns are the tile's tokens times the heads of the kv group, so keys and values are
// read once for the whole group.  The block walks the keys 128 at a time: each wave fetches 32
// of them from the pages into registers while all four compute on the previous 128, which
// they share through LDS (stored in the very order the matrix-core operands want them, so
// both the writes and the reads are 16 bytes per lane, lane after lane).  One barrier per 128
// keys.  Heads of more than 128 features take 64 keys at a time (two of the waves fetch) and
// 16 columns per wave: two rounds of 128 would not fit the LDS, nor the state the registers.  A token at absolute position p sees keys lo..p only (lo = 0, or p - window + 1),
// whatever portion it arrived in; a wave skips the 32-key chunks none of its columns sees.
//
// The host sorts the tiles by the number of keys they walk and deals them out to the blocks
// of a kv head in rounds, back and forth, so that every block gets about the same work.
#include "attention_mfma.h"

#ifndef PLAIN_NJ
#define PLAIN_NJ 4   // chunks of a fully visible round that are folded as one group (2 or 4)
#endif

// NCH: chunks of 32 keys per round (4, or 2 for the large heads)
template <int HD, int CB, int NCH>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 2 : 1))) void attention_tiles_kernel(
    bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q, long q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ q_start, const int* __restrict__ kv_len_of,
    const int* __restrict__ tile_req, const int* __restrict__ tile_q0, const int* __restrict__ tile_cut,
    const int* __restrict__ tile_z0, float* __restrict__ part, const int* __restrict__ order, int rounds, int nh,
    int nkv, int page_size, float scale, int window, long num_pages_l, int TQ) {
  constexpr int KS = HeadFrags<HD>::KS;
  constexpr int F = 2 * KS + HD / 16;             // 16-byte operand fragments per lane and 32 keys: keys, then values
  constexpr int KEYS_PER_ROUND = NCH * 32;
  static_assert(NCH == 2 || NCH == 4, "a round is two or four chunks");
  extern __shared__ __attribute__((aligned(16))) u32x4_t staged[];   // [2 buffers][NCH chunks][F][64 lanes]
  __shared__ int present[2][4][2];                // is the page of a 16-key tile there
  const int lane = threadIdx.x % 64;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int lr = lane % 16, lg = lane / 16;
  // kv head in x: with 8 kv heads (or a multiple) a die, which takes every eighth block, walks
  // the keys of one kv head only and its L2 serves all tiles of that head
  const int g = blockIdx.x, G = nh / nkv, B = gridDim.y;
  // The host deals long tiles to low seats.  A die's 32 compute units take its blocks in turn,
  // so blocks y and y + 32 meet on one unit: every other run of 32 takes its seats in reverse,
  // and a long tile sits beside a short one.
  const int run = blockIdx.y / 32, run_len = min(32, B - run * 32);
  const int seat = run * 32 + ((run & 1) ? run_len - 1 - (int)(blockIdx.y % 32) : (int)(blockIdx.y % 32));
  const int num_pages = (int)(num_pages_l < 0x7fffffffL ? num_pages_l : 0x7fffffffL);
  const float scale_log2 = scale * PI_LOG2E;
  KVLaneOffsets<HD> off;
  off.set(page_size, lane);
  const int step_blk = KEYS_PER_ROUND / page_size, step_slot = KEYS_PER_ROUND % page_size;

  for (int round = 0; round < rounds; ++round) {
    const int tile = order[round * B + seat];
    if (tile < 0) continue;                        // same for the whole block
    const int r = tile_req[tile], q0 = tile_q0[tile];
    const int qs = q_start[r];
    const int q_len = q_start[r + 1] - qs;
    const int kv_len = kv_len_of[r];
    const int n_tok = min(TQ, q_len - q0);
    const int pos0 = kv_len - q_len + q0;          // position of the tile's first token
    auto first_key = [&](int pos) { return (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0; };
    // keys the block walks: the tile's, or one of `cuts` equal shares of them in rounds of 128
    // (the host cuts the key range of tiles when a step has too few tiles for the chip; the
    // shares' results are merged by the combine kernel, as for decode attention)
    const int cut = tile_cut[tile] & 0xff, cuts = tile_cut[tile] >> 8;
    const int all0 = first_key(pos0) / KEYS_PER_ROUND, all1 = (pos0 + n_tok - 1) / KEYS_PER_ROUND + 1;
    const int share = (all1 - all0 + cuts - 1) / cuts;
    const int sc0 = all0 + cut * share, sc1 = min(all1, sc0 + share);   // may be empty: nothing seen, m stays -inf
    // tokens of this wave's columns, and the keys all / any of them see
    const int tok_a = (wave * CB * 16) / G, tok_b = min(((wave + 1) * CB * 16 - 1) / G, n_tok - 1);
    const bool active = tok_a < n_tok;
    const int see_any_lo = first_key(pos0 + tok_a), see_any_hi = pos0 + tok_b;
    const int see_all_lo = first_key(pos0 + tok_b), see_all_hi = pos0 + tok_a;

    AttnState<HD, CB> st;
    attn_init(st);
    long rows[CB];
    int heads[CB];
    bool valid[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const int col = (wave * CB + c) * 16 + lr;
      const int tok = col / G;
      valid[c] = tok < n_tok;
      rows[c] = qs + q0 + tok;
      heads[c] = g * G + col % G;
      // padding columns are computed on zeros, see everything and are never stored
      st.pos[c] = valid[c] ? pos0 + tok : 0x7fffffff;
      st.lo[c] = valid[c] ? first_key(pos0 + tok) : 0;
      attn_load_q(st, c, q, q_stride, rows[c], heads[c], valid[c], lane);
    }

    // this wave's 32 keys of every round (the first NCH waves fetch): where they lie
    // (a constant where every wave fetches: behind a branch the compiler waits for the loads at
    // the branch's end instead of at their first use, and the round loses its overlap: 63 us
    // instead of 53 for a 2,048-token prompt at head size 64)
    const bool fetches = NCH == 4 || wave < NCH;
    PageCursor cur;
    cur.start(block_table + (long)r * table_width, table_width, kv_len, page_size, sc0 * KEYS_PER_ROUND + wave * 32);
    KVChunk<HD> pre;
    auto fetch = [&]() {
      if (!fetches) return;
      PageCursor two = cur;                        // the chunk's two tiles
      const ChunkPages cp = two.next();
      attn_load<HD>(pre, cp, k_cache, v_cache, off, nkv, g, page_size, num_pages);
      cur.key += KEYS_PER_ROUND;
      cur.blk += step_blk;
      cur.slot += step_slot;
      if (cur.slot >= page_size) { cur.slot -= page_size; ++cur.blk; }
    };
    auto stash = [&](int buf) {
      if (!fetches) return;
      u32x4_t* mine = staged + ((buf * NCH + wave) * F) * 64 + lane;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) mine[(t * KS + ks) * 64] = pre.k[t][ks].n;
#pragma unroll
      for (int db = 0; db < HD / 16; ++db)
        mine[(2 * KS + db) * 64] = u32x4_t{pre.v[db].d[0].x, pre.v[db].d[0].y, pre.v[db].d[1].x, pre.v[db].d[1].y};
      if (lane < 2) present[buf][wave][lane] = lane == 0 ? pre.have[0] : pre.have[1];
    };

    fetch();
    stash(0);
    __syncthreads();
    for (int sc = sc0; sc < sc1; ++sc) {
      const int buf = (sc - sc0) & 1;
      fetch();                                     // the next 128 keys (past the end: no pages, page 0 is read)
      // a round that every column of the wave sees whole, with every page there: straight-line
      // code without the per-key tests (the accumulators then stay in place from chunk to chunk)
      const int round0 = sc * KEYS_PER_ROUND;
      const bool missing = __builtin_amdgcn_ballot_w64(lane < 2 * NCH && !(&present[buf][0][0])[lane % 8]) != 0;
      constexpr int NJ = NCH < PLAIN_NJ ? NCH : PLAIN_NJ;
      if (active && !missing && round0 >= see_all_lo && round0 + KEYS_PER_ROUND - 1 <= see_all_hi) {
        attn_compute_plain<HD, CB, NJ>(st, staged + (buf * NCH * F) * 64 + lane, F * 64, scale_log2);
        if (NJ < NCH) attn_compute_plain<HD, CB, NJ>(st, staged + ((buf * NCH + 2) * F) * 64 + lane, F * 64, scale_log2);
      } else if (active) {
#pragma unroll 1
        for (int j = 0; j < NCH; ++j) {
          const int key0 = sc * KEYS_PER_ROUND + j * 32;
          if (key0 > see_any_hi || key0 + 31 < see_any_lo) continue;
          StagedChunk<HD> kv;
          kv.from = staged + ((buf * NCH + j) * F) * 64 + lane;
          kv.have[0] = __builtin_amdgcn_readfirstlane(present[buf][j][0]) != 0;
          kv.have[1] = __builtin_amdgcn_readfirstlane(present[buf][j][1]) != 0;
          const bool masked = key0 < see_all_lo || key0 + 31 > see_all_hi || !kv.have[0] || !kv.have[1];
          attn_compute<HD, CB, StagedChunk<HD>>(st, kv, key0, scale_log2, masked, lane);
        }
      }
      stash(buf ^ 1);
      __syncthreads();
    }
    attn_finish(st);

    if (cuts > 1) {
      // partial result [token of the cut tiles, head, cut, HD + 4] float32: O^T un-normalised, m, l
      const int rec = HD + 4;
      const float to_log2 = scale * PI_LOG2E;
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        if (!valid[c]) continue;
        const int tok = ((wave * CB + c) * 16 + lr) / G;
        float* mine = part + (((long)(tile_z0[tile] + tok) * nh + heads[c]) * cuts + cut) * rec;
#pragma unroll
        for (int db = 0; db < HD / 16; ++db) *reinterpret_cast<f32x4_t*>(mine + db * 16 + lg * 4) = st.o[db][c];
        if (lg == 0) {
          mine[HD] = st.m[c] * to_log2;        // base-2 scale; -inf stays -inf
          mine[HD + 1] = st.l[c];
        }
      }
      continue;
    }
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      if (!valid[c]) continue;
      const float inv = 1.0f / st.l[c];
      bf16_t* o = out + rows[c] * out_stride + (long)heads[c] * HD + lg * 4;
#pragma unroll
      for (int db = 0; db < HD / 16; ++db) {
        uint2 w;
        w.x = pack_bf16x2(st.o[db][c][0] * inv, st.o[db][c][1] * inv);
        w.y = pack_bf16x2(st.o[db][c][2] * inv, st.o[db][c][3] * inv);
        *reinterpret_cast<uint2*>(o + db * 16) = w;
      }
    }
  }
}

// Tokens per tile for a head layout: the block's columns divided among the heads of a group.
extern "C" int pi_attention_tile_rows(int nh, int nkv, int hd) {
  if (nkv <= 0 || nh <= 0 || nh % nkv) return 0;
  const int cols = 4 * (hd > 128 ? 1 : 2) * 16;   // four waves of two column blocks, one for the large heads
  return cols / (nh / nkv);
}

// Shared memory of one block: two buffers of a round's keys and values (128 keys, or 64 for the large heads).
static size_t tiles_lds_bytes(int hd) { return (size_t)2 * (hd > 128 ? 2 : 4) * (2 * ((hd + 31) / 32) + hd / 16) * 64 * 16; }

// `order`: [rounds, seats] tile indices (-1: none), the host's deal of the tiles to `seats`
// blocks per kv head.  tile_cut[t] = cut | cuts << 8: which of how many shares of its keys entry
// t walks; entries with cuts > 1 write partial results for token tile_z0[t] + i to `part`
// ([tokens, heads, cuts, hd + 4] float32), which pi_attention_combine_rows merges.
extern "C" int pi_attention_prefill_mfma(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                         const void* v_cache, const int* block_table, int table_width, const int* q_start,
                                         const int* kv_len, const int* tile_req, const int* tile_q0, const int* tile_cut,
                                         const int* tile_z0, void* part, const int* order, int rounds, int seats, int nh,
                                         int nkv, int hd, int page_size, float scale, int window, long num_pages,
                                         hipStream_t stream) {
  PI_REQUIRE(rounds > 0 && seats > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_prefill: bad sizes rounds=%d seats=%d heads=%d kv_heads=%d", rounds, seats, nh, nkv);
  PI_REQUIRE(hd >= 16 && hd <= 256 && hd % 16 == 0, "attention_prefill: head_dim %d is not a multiple of 16 up to 256", hd);
  PI_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_prefill: page size %d must be a multiple of 16", page_size);
  PI_REQUIRE(table_width >= 1, "attention_prefill: empty block table");
  const int TQ = pi_attention_tile_rows(nh, nkv, hd);
  PI_REQUIRE(TQ >= 1, "attention_prefill: %d heads per kv head do not fit a block", nh / nkv);
  PI_REQUIRE(seats <= 65535, "attention_prefill: too many blocks per kv head (%d)", seats);
  PI_REQUIRE(out_stride % 4 == 0 && q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 8 == 0), "attention_prefill: q / out rows must be 16- / 8-byte aligned");
  const size_t lds = tiles_lds_bytes(hd);
  const dim3 grid(nkv, seats), block(256);
#define GO(H, C, N)                                                                                                                          \
  do {                                                                                                                                     \
    static bool configured = false;                                                                                                        \
    if (!configured) {                                                                                                                     \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_tiles_kernel<H, C, N>),                                      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                            \
      if (e != hipSuccess) return pi_fail("attention_prefill: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));            \
      configured = true;                                                                                                                   \
    }                                                                                                                                      \
    hipLaunchKernelGGL((attention_tiles_kernel<H, C, N>), grid, block, lds, stream, (bf16_t*)out, out_stride, (const bf16_t*)q, q_stride,     \
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width, q_start, kv_len, tile_req, tile_q0,       \
                       tile_cut, tile_z0, (float*)part, order, rounds, nh, nkv, page_size, scale, window, num_pages, TQ);                  \
  } while (0)
  switch (hd) {
    case 16: GO(16, 2, 4); break;
    case 32: GO(32, 2, 4); break;
    case 48: GO(48, 2, 4); break;
    case 64: GO(64, 2, 4); break;
    case 80: GO(80, 2, 4); break;
    case 96: GO(96, 2, 4); break;
    case 112: GO(112, 2, 4); break;
    case 128: GO(128, 2, 4); break;
    case 144: GO(144, 1, 2); break;
    case 160: GO(160, 1, 2); break;
    case 176: GO(176, 1, 2); break;
    case 192: GO(192, 1, 2); break;
    case 208: GO(208, 1, 2); break;
    case 224: GO(224, 1, 2); break;
    case 240: GO(240, 1, 2); break;
    default: GO(256, 1, 2); break;
  }
#undef GO
  return pi_check_launch("attention_prefill_mfma");
}

// Causal attention of prompt portions (and whatever else shares their batch) over the paged
// cache, bfloat16 on the matrix cores.
//
// The step's tokens are cut into tiles of TQ consecutive tokens of one request (work list made
// on the host).  A block of four waves handles one (tile, kv head): its 4 * CB * 16 query
// columns are the tile's tokens times the heads of the kv group, so keys and values are read
// once for the whole group.  Tiles are small (CB = 2) so that a prompt makes more blocks than
// the chip has compute units and the short early tiles fill in around the long late ones.
// Each wave walks the keys its own columns can see, 32 at a time,
// with a running softmax per column; a token at absolute position p sees keys lo..p only
// (lo = 0, or p - window + 1), whatever portion it arrived in.
#include "attention_mfma.h"

template <int HD, int CB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(HD <= 64 ? 2 : 1))) void attention_tiles_kernel(
    bf16_t* __restrict__ out, long out_stride, const bf16_t* __restrict__ q, long q_stride,
    const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ q_start, const int* __restrict__ kv_len_of,
    const int* __restrict__ tile_req, const int* __restrict__ tile_q0, int nh, int nkv, int page_size, float scale,
    int window, long num_pages, int TQ) {
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int lr = lane % 16, lg = lane / 16;
  const int tile = gridDim.x - 1 - blockIdx.x, g = blockIdx.y;   // later tiles see more keys: start them first
  const int G = nh / nkv;
  const int r = tile_req[tile], q0 = tile_q0[tile];
  const int qs = q_start[r];
  const int q_len = q_start[r + 1] - qs;
  const int kv_len = kv_len_of[r];
  const int* bt = block_table + (long)r * table_width;

  AttnState<HD, CB> st;
  attn_init(st);
  long rows[CB];
  int heads[CB];
  bool valid[CB];
  // over the wave's real columns: the first and last key any of them sees (the walk), and the
  // keys all of them see (no masking needed there)
  int lo_min = 0x7fffffff, lo_max = 0, pos_min = 0x7fffffff, pos_max = -1;
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    const int col = (wave * CB + c) * 16 + lr;
    const int tok = col / G;
    valid[c] = tok < TQ && q0 + tok < q_len;
    const int pos = kv_len - q_len + q0 + tok;
    rows[c] = qs + q0 + tok;
    heads[c] = g * G + col % G;
    // padding columns are computed on zeros, see everything and are never stored
    st.pos[c] = valid[c] ? pos : 0x7fffffff;
    st.lo[c] = (valid[c] && window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    attn_load_q(st, c, q, q_stride, rows[c], heads[c], valid[c], lane);
    if (valid[c]) {
      lo_min = min(lo_min, st.lo[c]);
      lo_max = max(lo_max, st.lo[c]);
      pos_min = min(pos_min, pos);
      pos_max = max(pos_max, pos);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    lo_min = min(lo_min, __shfl_xor(lo_min, off, 64));
    lo_max = max(lo_max, __shfl_xor(lo_max, off, 64));
    pos_min = min(pos_min, __shfl_xor(pos_min, off, 64));
    pos_max = max(pos_max, __shfl_xor(pos_max, off, 64));
  }
  if (pos_max < 0) return;   // no column of this wave is a real query

  attn_walk<HD, CB>(st, lo_min / 32, pos_max / 32 + 1, (lo_max + 31) / 32, (pos_min + 1) / 32 - 1, k_cache, v_cache, bt,
                    table_width, kv_len, nkv, g, page_size, num_pages, scale * PI_LOG2E, lane);
  attn_finish(st);

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

// Tokens per tile for a head layout: the block's columns divided among the heads of a group.
extern "C" int pi_attention_tile_rows(int nh, int nkv, int hd) {
  if (nkv <= 0 || nh <= 0 || nh % nkv) return 0;
  const int cols = 4 * 2 * 16;
  return cols / (nh / nkv);
}

extern "C" int pi_attention_prefill_mfma(void* out, long out_stride, const void* q, long q_stride, const void* k_cache,
                                         const void* v_cache, const int* block_table, int table_width, const int* q_start,
                                         const int* kv_len, const int* tile_req, const int* tile_q0, int num_tiles, int nh,
                                         int nkv, int hd, int page_size, float scale, int window, long num_pages,
                                         hipStream_t stream) {
  PI_REQUIRE(num_tiles > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_prefill: bad sizes tiles=%d heads=%d kv_heads=%d", num_tiles, nh, nkv);
  PI_REQUIRE(hd == 64 || hd == 128, "attention_prefill: head_dim %d is not 64 or 128", hd);
  PI_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_prefill: page size %d must be a multiple of 16", page_size);
  const int TQ = pi_attention_tile_rows(nh, nkv, hd);
  PI_REQUIRE(TQ >= 1, "attention_prefill: %d heads per kv head do not fit a block", nh / nkv);
  PI_REQUIRE(nkv <= 65535, "attention_prefill: too many kv heads (%d)", nkv);
  PI_REQUIRE(out_stride % 4 == 0 && q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 8 == 0), "attention_prefill: q / out rows must be 16- / 8-byte aligned");
  const dim3 grid(num_tiles, nkv), block(256);
#define GO(H, C) hipLaunchKernelGGL((attention_tiles_kernel<H, C>), grid, block, 0, stream, (bf16_t*)out, out_stride, (const bf16_t*)q, \
                                    q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_width, q_start, \
                                    kv_len, tile_req, tile_q0, nh, nkv, page_size, scale, window, num_pages, TQ)
  if (hd == 64) GO(64, 2); else GO(128, 2);
#undef GO
  return pi_check_launch("attention_prefill_mfma");
}

// Where the matrix-product kernels fetch from: the address arithmetic of their global loads as
// plain integer functions, so that the kernels and a host-side test use the same code.
//
// A lane often fetches something it will not use (a row beyond the matrix, k beyond its range,
// a step beyond the last) from a stand-in address, so that every lane issues the same loads and
// the waits can be counted.  A stand-in that lies outside its tensor is invisible to every
// comparison of values and faults only when the tensor ends where its mapping ends; the test
// that includes this header (tests/cpp/load_bounds.cpp) enumerates every fetch of every lane
// for many shapes and checks that it lies inside the operand.
//
// All offsets are in bfloat16 elements from the operand's first element unless said otherwise; a fetch
// covers 8 elements (16 bytes).
#pragma once

#if defined(__HIPCC__)
#define PI_ADDR __host__ __device__ inline
#else
#define PI_ADDR inline
#endif

namespace addressing {

constexpr int KSTEP = 64;              // k per step of the weight-streaming kernels

PI_ADDR int imin(int a, int b) { return a < b ? a : b; }
PI_ADDR long lmin(long a, long b) { return a < b ? a : b; }

// ---------------------------------------------------------------- launch arithmetic (host)
// How a k-range of K is cut for `splits` blocks: k per block in whole steps (of `quantum`), and
// the number of non-empty splits that leaves.
struct KSplit {
  int k_per_block, splits;
};
PI_ADDR KSplit cut_k(int K, int splits, int quantum) {
  int kpb = (K + splits - 1) / splits;
  kpb = (kpb + quantum - 1) / quantum * quantum;
  return KSplit{kpb, (K + kpb - 1) / kpb};
}

// ---------------------------------------------------------------- gemm_skinny_kernel (1..32 tokens)
// A block is four waves on the same rows; wave w takes the w-th quarter, rounded up to whole
// steps, of the block's k-range [kb0, kb1).  k1 <= k0: the wave has nothing to do.
struct WaveRange {
  int k0, k1;
};
PI_ADDR WaveRange skinny_wave_range(int K, int k_per_block, int split, int wave) {
  const int kb0 = split * k_per_block;
  const int kb1 = imin(K, kb0 + k_per_block);
  const int per_wave = ((kb1 - kb0 + 4 * KSTEP - 1) / (4 * KSTEP)) * KSTEP;
  const int k0 = kb0 + wave * per_wave;
  return WaveRange{k0, imin(kb1, k0 + per_wave)};
}

// Row part of a lane's weight address for row tile t of the block whose first row is n0 (lane
// lr = lane % 16, lg = lane / 16).  Rows beyond N read the last row.  `tiled`: the matrix is the
// copy [N / 16][K / 64][2][4][16][8] (16 rows x 64 k are 1,024 elements in a row).
PI_ADDR long skinny_w_base(int tiled, long n0, int t, int lr, int lg, int N, int K, long ldw) {
  return tiled ? lmin(n0 / 16 + t, (long)N / 16 - 1) * (K / 64) * 1024 + lg * 128 + lr * 8
               : lmin(n0 + t * 16 + lr, (long)N - 1) * ldw + lg * 16;
}
// What step kk adds for the lane's fragment h (0, 1).  In a whole step every lane's 8 k lie
// inside the wave's range.  In the last, partial step (row-major matrices only: a tiled one has
// whole steps) a piece beyond k1 is fetched from the range's first 8 elements instead (k0 + 8 <=
// k1, both multiples of 8), which lie inside the row whatever the lane's own offset.
PI_ADDR long skinny_w_step(int tiled, bool whole, int kk, int h, int lg, int k0, int k1) {
  if (whole) return tiled ? (long)kk * 16 + h * 512 : (long)kk + h * 8;
  return kk + lg * 16 + h * 8 < k1 ? kk + h * 8 : k0 - lg * 16;
}
PI_ADDR bool skinny_w_used(bool whole, int kk, int h, int lg, int k1) { return whole || kk + lg * 16 + h * 8 < k1; }

// Activations: load i of a step brings tokens 8i .. 8i+7, lane j the piece xp = j % 8 of token
// 8i + j / 8; tokens beyond M read the last token.
PI_ADDR long skinny_x_base(int token, int M, long ldx, int xp) { return (long)imin(token, M - 1) * ldx + xp * 8; }
PI_ADDR long skinny_x_step(bool whole, int kk, int xp, int k0, int k1) { return (whole || kk + xp * 8 < k1) ? kk : k0 - xp * 8; }

// ---------------------------------------------------------------- gemm_skinny_shared_kernel (33..128 tokens)
// A block's waves take 16 rows each over the block's whole k-range [kb0, kb1) in steps of 64;
// steps beyond the last are fetched again (never used) so that every step issues the same loads.
PI_ADDR int shared_steps(int kb0, int kb1) { return (kb1 - kb0 + KSTEP - 1) / KSTEP; }
PI_ADDR int shared_k_of(int kb0, int steps, int s) { return kb0 + imin(s, steps - 1) * KSTEP; }
PI_ADDR long shared_w_base(int tiled, long n0, int wave, int lr, int lg, int N, int K, long ldw) {
  return tiled ? lmin(n0 / 16 + wave, (long)N / 16 - 1) * (K / 64) * 1024 + lg * 128 + lr * 8
               : lmin(n0 + wave * 16 + lr, (long)N - 1) * ldw;
}
// a piece beyond the range is fetched from the range's last 8 elements
PI_ADDR long shared_w_step(int tiled, int kk, int h, int lg, int kb1) {
  return tiled ? (long)kk * 16 + h * 512 : (long)imin(kk + lg * 16 + h * 8, kb1 - 8);
}
PI_ADDR long shared_x_base(int token, int M, long ldx) { return (long)imin(token, M - 1) * ldx; }
PI_ADDR long shared_x_step(int kk, int xp, int kb1) { return imin(kk + xp * 8, kb1 - 8); }

// ---------------------------------------------------------------- tile kernels (buffer descriptors)
// A block's operand is read through a buffer descriptor: a base (the block's first row at its
// first k) and a byte length; a lane's byte offset at or beyond the length reads zeros.  The
// descriptor must lie inside the operand, and a fetch that is used must lie inside the
// descriptor with all of its 16 bytes.
struct Descriptor {
  long base;        // elements from the operand's first
  long bytes;
};
PI_ADDR Descriptor tile_descriptor(long row0, long ld, int k_lo, int k_hi, int rows) {
  return Descriptor{row0 * ld + k_lo, ((long)(rows - 1) * ld + (k_hi - k_lo)) * 2};
}
constexpr unsigned OUT_OF_RANGE = 0x7ffffff0u;
// which 16-byte piece of its row in memory the lane fetches (the pieces of a row are turned by
// (row / 2) % 8 on their way into LDS)
PI_ADDR int tile_piece(int lane, int row) { return (lane % 8) ^ ((row >> 1) & 7); }
// 128 x 128 kernel: rows beyond the operand take an offset outside the descriptor
PI_ADDR unsigned tile_lane_offset(int row, int rows, long ld, int piece) {
  return row < rows ? (unsigned)(row * (int)ld + piece * 8) * 2u : OUT_OF_RANGE;
}
// ... and so does a piece whose k lies beyond the block's range (k0 relative to k_lo)
PI_ADDR unsigned tile_slab_offset(unsigned lane_offset, int k0, int piece, int k_range) {
  return k0 + piece * 8 < k_range ? lane_offset + (unsigned)k0 * 2u : OUT_OF_RANGE;
}
// 256 x 256 kernel (K a multiple of 64, whole slabs only): rows beyond the operand read the last row
PI_ADDR unsigned big_lane_offset(int row, int rows, long ld, int piece) {
  return (unsigned)(imin(row, rows - 1) * (int)ld + piece * 8) * 2u;
}
PI_ADDR int big_slab_bytes(int s, int slabs) { return imin(s, slabs - 1) * 64 * 2; }   // past the last slab: read it again, unused

// ---------------------------------------------------------------- attention over the paged cache
// Keys [pages, kv_heads, page, HD], values transposed [pages, kv_heads, HD, page], bfloat16.  A
// chunk is two tiles of 16 keys; a tile lies in one page (pages hold a multiple of 16 tokens) at
// slot .. slot + 15.  A tile whose page is missing (or whose id is no page of the pool) is read
// from page 0 instead and counts as zero.  Bases in elements, a lane's part in bytes.
PI_ADDR long kv_page_elems(int nkv, int page_size, int hd) { return (long)nkv * page_size * hd; }
PI_ADDR bool kv_page_there(long page, long num_pages) { return page >= 0 && page < num_pages; }
PI_ADDR long kv_page_or_first(long page, long num_pages) { return kv_page_there(page, num_pages) ? page : 0; }
PI_ADDR long kv_key_tile(long page, long page_elems, int g, int page_size, int slot, int hd) {
  return page * page_elems + (long)(g * page_size + slot) * hd;
}
PI_ADDR long kv_value_tile(long page, long page_elems, int g, int page_size, int slot, int hd) {
  return page * page_elems + (long)g * page_size * hd + slot;
}
// key row lane % 16 of the tile, features (lane / 16) * 8 .. + 7 of a fragment of 32 (fragment ks lies ks * 64 bytes on)
PI_ADDR unsigned kv_key_lane(int lane, int hd) { return (unsigned)((lane % 16) * hd + (lane / 16) * 8) * 2u; }
// what a lane without features of its own reads (a head of 16, 48, .. features: the last fragment is half empty)
PI_ADDR unsigned kv_key_lane_first(int lane, int hd) { return (unsigned)((lane % 16) * hd) * 2u; }
PI_ADDR bool kv_lane_holds(int hd, int ks, int lane) { return ks * 32 + (lane / 16) * 8 < hd; }
// value row db * 16 + lane % 16, keys (lane / 16) * 4 .. + 3 of the tile (8 bytes)
PI_ADDR unsigned kv_value_lane(int lane, int db, int page_size) { return (unsigned)((db * 16 + lane % 16) * page_size + (lane / 16) * 4) * 2u; }

}  // namespace addressing

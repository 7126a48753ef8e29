// Every global fetch of the matrix-product kernels, enumerated on the host from the kernels' own
// address arithmetic (csrc/addressing.h), checked to lie inside its operand.
//
//   load_bounds [old-standin] [only] [M N K splits]...
//
// Walks the built-in sweep of shapes (and any given as arguments) through the lanes, waves,
// blocks and steps of gemm_skinny_kernel, gemm_skinny_shared_kernel, gemm_mfma_kernel and
// gemm_mfma_big_kernel exactly as the kernels walk them (and, in the built-in sweep, through the
// key and value fetches of the attention kernels' chunks for every head size and several page sizes), with the matrices row by row (two row
// strides) and, where the sizes allow, in the weight-streaming kernels' tiled order.  Prints
// "ok <fetches>" or the first fetch that leaves its operand (exit status 1).
// "only" leaves the built-in sweep out.  "old-standin" replaces the stand-in address of a lane beyond a partial k step by the formula
// the kernel once had (the range's start plus the lane's own offset): the sweep must then fail.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "addressing.h"

namespace A = addressing;

static bool old_standin = false;
static long fetches = 0;

struct Shape {
  int M, N, K, splits;
};

static bool fail(const char* kernel, const char* operand, const Shape& s, long ld, int tiled, long off, const char* why) {
  std::printf("out of bounds: %s %s M=%d N=%d K=%d splits=%d ld=%ld tiled=%d offset=%ld: %s\n", kernel, operand, s.M, s.N, s.K,
              s.splits, ld, tiled, off, why);
  return false;
}

// an 8-element fetch at `off` of a row-major operand [rows, cols] with row stride ld must lie in row `row`
static bool in_row(long off, long row, long ld, int cols) { return off >= row * ld && off + 8 <= row * ld + cols; }

// ------------------------------------------------------------------ 1..32 tokens
static bool skinny(const Shape& s, long ldx, long ldw, int tiled, int RT, int quantum) {
  const int M = s.M, N = s.N, K = s.K;
  const A::KSplit cut = A::cut_k(K, s.splits, quantum);
  const int rows_per_block = RT * 16, MB = (M + 15) / 16;
  const int groups = (N + rows_per_block - 1) / rows_per_block;
  const int x_loads = (M + 7) / 8;
  for (int by = 0; by < cut.splits; ++by)
    for (int bx = 0; bx < groups; ++bx)
      for (int wave = 0; wave < 4; ++wave) {
        const A::WaveRange r = A::skinny_wave_range(K, cut.k_per_block, by, wave);
        for (int lane = 0; lane < 64; ++lane) {
          const int lr = lane % 16, lg = lane / 16, xt = lane / 8, xp = lane % 8;
          const long n0 = (long)bx * rows_per_block;
          int kk = r.k0;
          for (;; kk += A::KSTEP) {
            const bool whole = kk + A::KSTEP <= r.k1;
            if (!whole && kk >= r.k1) break;
            if (tiled && !whole) return fail("gemm_skinny", "W", s, ldw, tiled, kk, "a tiled matrix met a partial step");
            for (int t = 0; t < RT; ++t)
              for (int h = 0; h < 2; ++h) {
                long off = A::skinny_w_base(tiled, n0, t, lr, lg, N, K, ldw) + A::skinny_w_step(tiled, whole, kk, h, lg, r.k0, r.k1);
                if (old_standin && !whole && !A::skinny_w_used(whole, kk, h, lg, r.k1))
                  off = A::skinny_w_base(tiled, n0, t, lr, lg, N, K, ldw) + r.k0;
                ++fetches;
                if (tiled) {
                  if (off < 0 || off + 8 > (long)N * K) return fail("gemm_skinny", "W", s, ldw, tiled, off, "outside the matrix");
                } else {
                  const long row = A::lmin(n0 + t * 16 + lr, (long)N - 1);
                  if (!in_row(off, row, ldw, K)) return fail("gemm_skinny", "W", s, ldw, tiled, off, "outside its row");
                  if (A::skinny_w_used(whole, kk, h, lg, r.k1) && off != row * ldw + kk + lg * 16 + h * 8)
                    return fail("gemm_skinny", "W", s, ldw, tiled, off, "a used fetch is not the lane's k");
                }
              }
            for (int i = 0; i < MB * 2; ++i)
              if (i == 0 || i < x_loads) {
                const int token = i * 8 + xt;
                long off = A::skinny_x_base(token, M, ldx, xp) + A::skinny_x_step(whole, kk, xp, r.k0, r.k1);
                if (old_standin && !(whole || kk + xp * 8 < r.k1)) off = A::skinny_x_base(token, M, ldx, xp) + r.k0;
                ++fetches;
                if (!in_row(off, A::imin(token, M - 1), ldx, K)) return fail("gemm_skinny", "X", s, ldx, tiled, off, "outside its row");
              }
            if (!whole) break;
          }
        }
      }
  return true;
}

// ------------------------------------------------------------------ 33..128 tokens
static bool shared(const Shape& s, long ldx, long ldw, int tiled, int depth) {
  const int M = s.M, N = s.N, K = s.K;
  const A::KSplit cut = A::cut_k(K, s.splits, A::KSTEP);
  const int MB = (M + 15) / 16, XL = (MB + 1) / 2;
  const int groups = (N + 63) / 64;
  for (int by = 0; by < cut.splits; ++by) {
    const int kb0 = by * cut.k_per_block, kb1 = A::imin(K, kb0 + cut.k_per_block);
    const int steps = A::shared_steps(kb0, kb1);
    for (int bx = 0; bx < groups; ++bx)
      for (int tid = 0; tid < 256; ++tid) {
        const int wave = tid / 64, lane = tid % 64, lr = lane % 16, lg = lane / 16, xp = tid % 8;
        const long n0 = (long)bx * 64;
        for (int st = 0; st < steps + depth; ++st) {
          const int kk = A::shared_k_of(kb0, steps, st);
          for (int h = 0; h < 2; ++h) {
            const long off = A::shared_w_base(tiled, n0, wave, lr, lg, N, K, ldw) + A::shared_w_step(tiled, kk, h, lg, kb1);
            ++fetches;
            if (tiled) {
              if (off < 0 || off + 8 > (long)N * K) return fail("gemm_skinny_shared", "W", s, ldw, tiled, off, "outside the matrix");
            } else if (!in_row(off, A::lmin(n0 + wave * 16 + lr, (long)N - 1), ldw, K)) {
              return fail("gemm_skinny_shared", "W", s, ldw, tiled, off, "outside its row");
            }
          }
          for (int i = 0; i < XL; ++i) {
            const int token = i * 32 + tid / 8;
            const long off = A::shared_x_base(token, M, ldx) + A::shared_x_step(kk, xp, kb1);
            ++fetches;
            if (!in_row(off, A::imin(token, M - 1), ldx, K)) return fail("gemm_skinny_shared", "X", s, ldx, tiled, off, "outside its row");
          }
        }
      }
  }
  return true;
}

// ------------------------------------------------------------------ tile kernels
// One operand of one block: rows [row0, row0 + tile) of [R, K] with stride ld, k in [k_lo, k_hi).
static bool tile_operand(const char* kernel, const char* operand, const Shape& s, long R, long ld, long row0, int tile, int waves,
                         int k_lo, int k_hi, bool big) {
  const int rows = (int)A::lmin(tile, R - row0);
  const A::Descriptor d = A::tile_descriptor(row0, ld, k_lo, k_hi, rows);
  const long operand_bytes = ((R - 1) * ld + s.K) * 2;
  if (d.base < 0 || d.bytes <= 0 || d.base * 2 + d.bytes > operand_bytes || d.bytes >= 0x7ffffff0L)
    return fail(kernel, operand, s, ld, 0, d.base, "the descriptor leaves the operand");
  const int k_range = k_hi - k_lo, slabs = (k_range + 63) / 64;
  for (int wave = 0; wave < waves; ++wave)
    for (int p = 0; p < 4; ++p)
      for (int lane = 0; lane < 64; ++lane) {
        const int row = (wave * 4 + p) * 8 + lane / 8, piece = A::tile_piece(lane, row);
        for (int sl = 0; sl < slabs + 2; ++sl) {       // the kernels ask for up to two slabs past the last
          ++fetches;
          long off;      // bytes inside the descriptor
          bool used;
          if (big) {
            off = (long)A::big_lane_offset(row, rows, ld, piece) + A::big_slab_bytes(sl, slabs);
            used = row < rows && sl < slabs;
            if (off + 16 > d.bytes) return fail(kernel, operand, s, ld, 0, off, "a fetch of the large-tile kernel leaves its descriptor");
          } else {
            if (sl >= slabs) continue;                 // this kernel asks for existing slabs only
            off = A::tile_slab_offset(A::tile_lane_offset(row, rows, ld, piece), sl * 64, piece, k_range);
            used = row < rows && sl * 64 + piece * 8 < k_range;
            if (!used && off < d.bytes) return fail(kernel, operand, s, ld, 0, off, "a fetch that should read zeros lies inside the descriptor");
            if (used && off + 16 > d.bytes) return fail(kernel, operand, s, ld, 0, off, "a used fetch leaves its descriptor");
          }
          if (used && d.base * 2 + off != ((row0 + row) * ld + k_lo + A::imin(sl, slabs - 1) * 64 + piece * 8) * 2)
            return fail(kernel, operand, s, ld, 0, off, "a used fetch is not the lane's row and k");
        }
      }
  return true;
}

static bool tiles(const Shape& s, long lda, long ldw, bool big) {
  const int tile = big ? 256 : 128, waves = big ? 8 : 4;
  if (big && s.K % 64) return true;                    // the large-tile kernel takes whole slabs only
  const A::KSplit cut = A::cut_k(s.K, s.splits, 64);
  const char* kernel = big ? "gemm_mfma_big" : "gemm_mfma";
  for (int by = 0; by < cut.splits; ++by) {
    const int k_lo = by * cut.k_per_block, k_hi = A::imin(s.K, k_lo + cut.k_per_block);
    for (long m0 = 0; m0 < s.M; m0 += tile)
      if (!tile_operand(kernel, "A", s, s.M, lda, m0, tile, waves, k_lo, k_hi, big)) return false;
    for (long n0 = 0; n0 < s.N; n0 += tile)
      if (!tile_operand(kernel, "W", s, s.N, ldw, n0, tile, waves, k_lo, k_hi, big)) return false;
  }
  return true;
}

// ------------------------------------------------------------------ attention over the paged cache
// Every fetch of a chunk's two tiles (attn_load): the keys' fragments (16 bytes) and the values'
// (8 bytes) of every lane, for a page that is there, one that is missing and one whose id is no
// page of the pool (both read page 0 instead), lie inside the (page, kv head) block of their pool.
static bool attention(int hd, int page_size, int nkv, long num_pages) {
  const long page_elems = A::kv_page_elems(nkv, page_size, hd);
  const long pool_bytes = num_pages * page_elems * 2;
  const int KS = (hd + 31) / 32;
  const long ids[] = {0, num_pages - 1, -1, num_pages, num_pages + 5};
  for (long id : ids)
    for (int g = 0; g < nkv; ++g)
      for (int slot = 0; slot + 16 <= page_size; slot += 16) {
        const long pg = A::kv_page_or_first(id, num_pages);
        if (A::kv_page_there(id, num_pages) != (id >= 0 && id < num_pages) || pg < 0 || pg >= num_pages) {
          std::printf("out of bounds: attention page id %ld of %ld pages becomes %ld\n", id, num_pages, pg);
          return false;
        }
        const long block0 = ((pg * nkv + g) * (long)page_size) * hd * 2, block1 = block0 + (long)page_size * hd * 2;   // bytes of this (page, kv head)
        for (int lane = 0; lane < 64; ++lane) {
          for (int ks = 0; ks < KS; ++ks) {
            const bool held = hd % 32 == 0 || ks + 1 < KS || A::kv_lane_holds(hd, KS - 1, lane);
            const long at = A::kv_key_tile(pg, page_elems, g, page_size, slot, hd) * 2 + (held ? A::kv_key_lane(lane, hd) + ks * 64 : A::kv_key_lane_first(lane, hd));
            ++fetches;
            if (at < block0 || at + 16 > block1 || at + 16 > pool_bytes) {
              std::printf("out of bounds: attention key fetch hd=%d page=%d kv heads=%d g=%d slot=%d lane=%d ks=%d at %ld\n", hd, page_size, nkv, g, slot, lane, ks, at);
              return false;
            }
            const long row = (at - block0) / (hd * 2);        // the key it belongs to: one of the tile's sixteen
            if (row != slot + lane % 16) {
              std::printf("out of bounds: attention key fetch of lane %d reads key %ld of the page, not %d\n", lane, row, slot + lane % 16);
              return false;
            }
          }
          for (int db = 0; db < hd / 16; ++db) {
            const long at = A::kv_value_tile(pg, page_elems, g, page_size, slot, hd) * 2 + A::kv_value_lane(lane, db, page_size);
            ++fetches;
            if (at < block0 || at + 8 > block1) {
              std::printf("out of bounds: attention value fetch hd=%d page=%d kv heads=%d g=%d slot=%d lane=%d db=%d at %ld\n", hd, page_size, nkv, g, slot, lane, db, at);
              return false;
            }
            const long col = ((at - block0) / 2) % page_size;  // its first key: four of the tile's sixteen per lane group
            if (col != slot + (lane / 16) * 4) {
              std::printf("out of bounds: attention value fetch of lane %d starts at key %ld, not %d\n", lane, col, slot + (lane / 16) * 4);
              return false;
            }
          }
        }
      }
  return true;
}

static bool check(const Shape& s) {
  for (int pad = 0; pad <= 16; pad += 8) {             // row strides K, K + 8, K + 16
    const long ld = s.K + pad;
    if (s.M <= 32) {
      if (!skinny(s, ld, ld, 0, 2, A::KSTEP)) return false;
      if (s.M <= 16 && s.K % 64 == 0 && !skinny(s, ld, ld, 0, 4, 4 * A::KSTEP)) return false;     // the form that merges key ranges
    } else if (s.M <= 128) {
      if (!shared(s, ld, ld, 0, 4)) return false;
    }
    if (!tiles(s, ld, ld, false) || !tiles(s, ld, ld, true)) return false;
  }
  if (s.N % 16 == 0 && s.K % 64 == 0) {                // the streaming copy of the weights
    if (s.M <= 32 && !skinny(s, s.K, s.K, 1, 2, A::KSTEP)) return false;
    if (s.M <= 16 && !skinny(s, s.K, s.K, 1, 4, 4 * A::KSTEP)) return false;
    if (s.M > 32 && s.M <= 128 && !shared(s, s.K, s.K, 1, 4)) return false;
  }
  return true;
}

int main(int argc, char** argv) {
  std::vector<Shape> shapes;
  int a = 1;
  bool sweep = true;
  if (a < argc && !std::strcmp(argv[a], "old-standin")) { old_standin = true; ++a; }
  if (a < argc && !std::strcmp(argv[a], "only")) { sweep = false; ++a; }
  for (; a + 3 < argc; a += 4) shapes.push_back(Shape{std::atoi(argv[a]), std::atoi(argv[a + 1]), std::atoi(argv[a + 2]), std::atoi(argv[a + 3])});
  const int Ms[] = {1, 2, 7, 8, 9, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 129, 300};
  const int Ns[] = {1, 16, 31, 32, 33, 64, 100, 520, 2048};
  const int Ks[] = {8, 16, 64, 72, 96, 128, 160, 200, 256, 272, 344, 512, 1024, 2816};
  const int Ss[] = {1, 2, 3, 4, 8};
  for (int M : Ms)
    if (sweep)
    for (int N : Ns)
      for (int K : Ks)
        for (int S : Ss)
          if (S == 1 || K / S >= 8) shapes.push_back(Shape{M, N, K, S});
  for (const Shape& s : shapes)
    if (!check(s)) return 1;
  if (sweep)
    for (int hd = 16; hd <= 256; hd += 16)
      for (int page_size : {16, 32, 48, 64})
        for (int nkv : {1, 3, 8})
          if (!attention(hd, page_size, nkv, 7)) return 1;
  std::printf("ok %ld\n", fetches);
  return 0;
}

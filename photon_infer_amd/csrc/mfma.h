// Matrix-core helpers for gfx950 (CDNA4), wave64.
//
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] . B[32x16], float32 accumulate.
//   A operand: lane l holds 8 bf16 of row (l % 16); which 8 of the 32 k-values a lane group
//              (l / 16) holds does not matter as long as A and B use the same assignment,
//              because the instruction sums over k.
//   B operand: lane l holds 8 bf16 of column (l % 16), same k assignment as A.
//   D:         lane l holds D[(l / 16) * 4 + i][l % 16] for i = 0..3.
#pragma once
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

union Frag {          // 8 bf16 = 16 bytes, seen as the operand type or as raw words
  bf16x8_t v;
  uint4 q;
  u32x4_t n;          // the same words as a native vector (selects and copies stay in registers)
  uint2 d[2];
  uint16_t h[8];
};

__device__ inline f32x4_t mfma16(const Frag& a, const Frag& b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
}

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// 32 x 32 x 16: lane l holds row (column) l % 32 of the operand, k = (l / 32) * 8 .. + 8; of the
// result it holds column l % 32 and the 16 rows 8 * (v / 4) + 4 * (l / 32) + v % 4, v = 0..15.
__device__ inline f32x16_t mfma32(const Frag& a, const Frag& b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}

__device__ inline Frag zero_frag() {
  Frag f;
  f.q = make_uint4(0u, 0u, 0u, 0u);
  return f;
}

// 16-byte load of 8 consecutive bf16 (the address must be 16-byte aligned)
__device__ inline Frag load_frag(const bf16_t* p) {
  Frag f;
  f.q = *reinterpret_cast<const uint4*>(p);
  return f;
}

__device__ inline uint32_t pack_bf16x2(float lo, float hi) { return f32x2_to_bf16x2_bits(lo, hi); }

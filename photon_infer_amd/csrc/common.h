// Shared helpers of the gfx950 kernels: storage types, conversions, wave64 reductions,
// and the error channel of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define PI_WAVE 64

// dtype tags shared with the Python binding
enum PiDType : int { PI_F32 = 0, PI_BF16 = 1 };

// bfloat16 is stored as its 16 bits; arithmetic is always float.
struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float to_float(float v) { return v; }
__host__ __device__ inline float to_float(bf16_t v) {
  union { uint32_t u; float f; } c;
  c.u = ((uint32_t)v.bits) << 16;
  return c.f;
}

// round to nearest, ties to even; NaN stays NaN
__host__ __device__ inline uint16_t f32_to_bf16_bits(float f) {
  union { uint32_t u; float f; } c;
  c.f = f;
  uint32_t u = c.u;
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// on the device the conversion is one instruction (v_cvt_pk_bf16_f32, round to nearest even)
typedef __bf16 pi_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float pi_f32x2_t __attribute__((ext_vector_type(2)));
__host__ __device__ inline uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  pi_f32x2_t v = {lo, hi};
  pi_bf16x2_t b = __builtin_convertvector(v, pi_bf16x2_t);
  return *reinterpret_cast<uint32_t*>(&b);
#else
  return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
#endif
}

template <typename T> __host__ __device__ inline T from_float(float v);
template <> __host__ __device__ inline float from_float<float>(float v) { return v; }
template <> __host__ __device__ inline bf16_t from_float<bf16_t>(float v) {
  bf16_t r;
#if defined(__HIP_DEVICE_COMPILE__)
  r.bits = (uint16_t)(f32x2_to_bf16x2_bits(v, 0.f) & 0xffffu);
#else
  r.bits = f32_to_bf16_bits(v);
#endif
  return r;
}

// four consecutive elements as float32 (16-byte aligned float32, 8-byte aligned bfloat16)
__device__ inline void load4(const float* p, float v[4]) {
  const float4 q = *reinterpret_cast<const float4*>(p);
  v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
}
__device__ inline void load4(const bf16_t* p, float v[4]) {
  const uint2 q = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
  v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
}

// ---- wave64 reductions (every lane gets the result)
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = PI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PI_WAVE);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = PI_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PI_WAVE));
  return v;
}

// A rotated pair: (a, b) turned by the angle whose cosine and sine are c and s.  One spelling
// for every kernel that rotates, with the roundings fixed, so that a query or key comes out the
// same wherever it is rotated.
__device__ inline void rope_pair(float a, float b, float c, float s, float& lo, float& hi) {
  lo = __builtin_fmaf(a, c, -(b * s));
  hi = __builtin_fmaf(a, s, b * c);
}

// Element i of a product that is still split over k: the sum of its float32 pieces
// ([splits] planes of part_stride floats), added in split order, eight loads in flight.
__device__ inline float split_sum(const float* __restrict__ part, int splits, long part_stride, long i) {
  float val = 0.f;
  const float* p = part + i;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float tmp[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) tmp[u] = (s0 + u < splits) ? p[(s0 + u) * part_stride] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) val += tmp[u];
  }
  return val;
}

// ---- merging the key ranges of one (token, head): range s brings its un-normalised output,
// its maximum m (base-2 scale) and its sum of weights l.  One spelling of the arithmetic for
// every kernel that merges, so that the merged output is the same bits wherever it is made:
// weights against the overall maximum, sums in range order with fused multiply-adds, one
// division, one rounding.
__device__ inline float range_weight(float m, float m_tot) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_tot);
#else
  return 0.f;
#endif
}
__device__ inline float range_add(float w, float v, float sum) { return __builtin_fmaf(w, v, sum); }
__device__ inline float range_finish(float acc, float l_tot) { return acc * (1.0f / l_tot); }

// ---- reductions over the four lanes l, l+16, l+32, l+48 (one column of a matrix-core tile),
// with the gfx950 row / half swaps instead of a trip through the LDS crossbar:
// v_permlane16_swap exchanges the odd 16-lane rows of one register with the even rows of the
// other, v_permlane32_swap the upper half of one with the lower half of the other; fed the
// same value twice, the two results hold a lane's own value and its partner's.
__device__ inline float column_max(float v) {
#if defined(__HIP_DEVICE_COMPILE__)
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
#endif
  return v;
}
__device__ inline float column_sum(float v) {
#if defined(__HIP_DEVICE_COMPILE__)
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(b[0]) + __uint_as_float(b[1]);
#endif
  return v;
}

// Block-wide sum for blocks of up to 1024 threads (16 waves); `scratch` holds 16 floats.
__device__ inline float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / PI_WAVE, lane = threadIdx.x % PI_WAVE;
  const int nwaves = (blockDim.x + PI_WAVE - 1) / PI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

// ---- error channel: entry points return 0 or a negative code and leave a message
inline thread_local char pi_error_message[1024] = {0};

// Each shared library defines its own accessor: PI_DEFINE_MODULE(core) gives
// `const char* pi_core_last_error()`.
#define PI_DEFINE_MODULE(name) \
  extern "C" const char* pi_##name##_last_error() { return pi_error_message; }

inline int pi_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(pi_error_message, sizeof(pi_error_message), fmt, ap);
  va_end(ap);
  return -1;
}

inline int pi_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return pi_fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

#define PI_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return pi_fail(__VA_ARGS__); \
  } while (0)

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }
